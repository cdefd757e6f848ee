// Data gradient of stride-2 convolutions with at most four input channels and a large filter
// (the 7x7 stem), computed directly: no column matrix in memory, no gather pass.
//
//   dx[n][c][h][w] = sum_{k,r,s} dy[n][k][(h + ph - r)/2][(w + pw - s)/2] * W[k][c][r][s]
//                    over the (r, s) for which both quotients are exact.
//
// With h = 2i + a and w = 2j + b the element (c, a, b) of the 2x2 output block (i, j) is a dense
// stride-1 correlation over offsets dp, dq in a window of four:
//   out[(c,a,b)][i][j] = sum_{k,dp,dq} A[(c,a,b)][(dp,dq,k)] * dy[k][i + dp][j + dq],
//   A = W[k][c][a + ph - 2 dp][b + pw - 2 dq]  (zero where that tap does not exist).
// That is a GEMM with M = 4C <= 16 rows, so it runs on v_mfma_f32_16x16x4_f32: M = 16 rows
// (c, a, b), N = 16 consecutive j of one class row, K = 4 output channels k.  A wavefront owns one
// class row i (up to 8 N tiles, 4 accumulator registers each); the 8 wavefronts of a workgroup own
// 8 consecutive rows and share, per chunk of 8 channels k,
//   dyS[k][row][col]   the 11 dy rows x (Q + 3) columns their windows touch (zero padding
//                      materialised), so every (dp, dq) is a compile-time LDS offset,
//   aS[dp,dq][k][m]    the 16 x 8 x 16 slice of A.
// The next chunk is loaded with 128-bit loads while the current one is multiplied.  A lane ends up
// holding the 2x2 output block of one (c, i, j) and stores it as two 8-byte writes.
#include <stdlib.h>

#include "common.h"
#include "storage.h"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr int NT = 512;
constexpr int TI = 8;              // class rows per workgroup (one per wavefront)
constexpr int ND = 4;              // offsets per dimension
constexpr int SROWS = TI + ND - 1; // dy rows staged per channel
constexpr int KC = 8;              // channels k per chunk
constexpr int kOOB = int(0x80000000u);

__device__ __forceinline__ rsrc_t make_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, bytes, 0x00020000);
}

struct DFArgs {
  const void *dy;         // fp32, or 16-bit storage (template parameter S of the kernel)
  const float *aw;        // A re-laid as [dp,dq (16)][K][16], always fp32
  void *dx;
  int N, C, H, W, K, P, Q;
  int dp0, dq0;           // smallest row / column offset
};

// A[(dpi*4 + dqi)][k][m], m = c*4 + a*2 + b
__global__ __launch_bounds__(256) void k_dgrad_fewc_weights(const float *__restrict__ W, float *__restrict__ aw, int K, int C,
                                                           int R, int S, int ph, int pw, int dp0, int dq0) {
  const int total = ND * ND * K * 16;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
    const int m = i & 15, k = (i >> 4) % K, off = (i >> 4) / K;
    const int c = m >> 2, a = (m >> 1) & 1, b = m & 1;
    const int r = a + ph - 2 * (dp0 + off / ND), s = b + pw - 2 * (dq0 + off % ND);
    const bool ok = c < C && unsigned(r) < unsigned(R) && unsigned(s) < unsigned(S);
    aw[i] = ok ? W[((long(k) * C + c) * R + r) * S + s] : 0.f;
  }
}

// QT: 16-column tiles per class row (Q <= 16 * QT); S: storage type of dy and dx (storage.h) -- the
// slab in LDS, the weights and the arithmetic are fp32 in every case, a 16-bit dx is rounded once.
template <int QT, class S>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_dgrad_fewc(DFArgs a) {
  typedef typename S::elem elem;
  constexpr int ES = int(sizeof(elem));
  constexpr int PITCH = QT * 16 + 8;                       // slab column of dy column q is q + 4
  constexpr int CHS0 = SROWS * PITCH;
  constexpr int CHS = CHS0 + ((16 - CHS0 % 32) + 32) % 32;  // = 16 mod 32: the four k of a B fragment hit disjoint banks
  constexpr int SBUF = KC * CHS, ABUF = ND * ND * KC * 16;
  constexpr int SSLOTS = (KC * SROWS * QT * 4 + NT - 1) / NT;  // 128-bit slab loads per thread per chunk (upper bound)
  constexpr int NSTEP = ND * ND * (KC / 4);

  extern __shared__ float smem[];
  float *dyS = smem;               // [2][KC][CHS]
  float *aS = smem + 2 * SBUF;     // [2][16][KC][16]

  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int i0 = blockIdx.x * TI, n = blockIdx.y;
  const int PQ = a.P * a.Q, HW = a.H * a.W, Q4 = a.Q >> 2;
  const rsrc_t rdy = make_rsrc(static_cast<const elem *>(a.dy) + size_t(n) * a.K * PQ, unsigned(a.K) * PQ * unsigned(ES));
  const rsrc_t ra = make_rsrc(a.aw, unsigned(ND * ND) * a.K * 16 * 4u);

  // pad columns and rows outside the image stay zero: only image columns are (re)written
  for (int i = t; i < 2 * SBUF; i += NT) dyS[i] = 0.f;

  // ---- staging roles (the tile is fixed, so row validity is a thread constant) ------------------
  // slab float4 index f = e*NT + t over [KC][SROWS][Q/4]
  int sg[SSLOTS], sl[SSLOTS];
#pragma unroll
  for (int e = 0; e < SSLOTS; ++e) {
    const int f = e * NT + t, kc = f / (SROWS * Q4), rem = f - kc * (SROWS * Q4), sr = rem / Q4, c4 = rem - sr * Q4;
    const int p = i0 + a.dp0 + sr;
    const bool ok = kc < KC && unsigned(p) < unsigned(a.P);
    sg[e] = ok ? ((kc * a.P + p) * a.Q + c4 * 4) * ES : kOOB;
    sl[e] = kc < KC ? kc * CHS + sr * PITCH + 4 + c4 * 4 : -1;
  }
  const int ag = ((t >> 5) * a.K * 16 + (t & 31) * 4) * 4;   // A float4 index t: offset t / 32, (k, m) slice t % 32
  auto ldv = [&](rsrc_t r, int voff) -> v4f {
    return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
  };
  auto ld_dy = [&](int voff) -> v4f {   // four consecutive dy elements as floats
    if constexpr (ES == 4) {
      return ldv(rdy, voff);
    } else {
      typedef unsigned int v2u __attribute__((ext_vector_type(2)));
      const v2u w = __builtin_bit_cast(v2u, __builtin_amdgcn_raw_buffer_load_b64(rdy, voff, 0, 0));
      const elem h[4] = {elem(w[0] & 0xffffu), elem(w[0] >> 16), elem(w[1] & 0xffffu), elem(w[1] >> 16)};
      return v4f{S::ld(h), S::ld(h + 1), S::ld(h + 2), S::ld(h + 3)};
    }
  };

  // ---- operand lane constants -------------------------------------------------------------------
  // B: lane -> (k = lane / 16, j = lane % 16); slab row of class row i0 + wave at offset dpi is wave + dpi,
  //    slab column of j + dq0 + dqi is j + dq0 + dqi + 4
  const int bconst = (lane >> 4) * CHS + wave * PITCH + (lane & 15) + 4 + a.dq0;
  // A: lane -> (k = lane / 16, m = lane % 16) = aS[..][k][m] contiguous

  v4f acc[QT];
#pragma unroll
  for (int i = 0; i < QT; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};

  const int nchunks = a.K / KC;
  __syncthreads();  // zero fill done
#pragma unroll
  for (int e = 0; e < SSLOTS; ++e) {
    const v4f v = ld_dy(sg[e]);
    if (sl[e] >= 0) *reinterpret_cast<v4f *>(dyS + sl[e]) = v;
  }
  *reinterpret_cast<v4f *>(aS + t * 4) = ldv(ra, ag);
  __syncthreads();

  int cur = 0;
  for (int ch = 0; ch < nchunks; ++ch) {
    const float *bs = dyS + cur * SBUF + bconst;
    const float *as = aS + cur * ABUF + lane;
    // next chunk's loads (past the last chunk they fall outside the descriptors and return zero)
    const int k1 = (ch + 1) * KC;
    v4f ns[SSLOTS];
#pragma unroll
    for (int e = 0; e < SSLOTS; ++e) ns[e] = ld_dy(sg[e] + k1 * PQ * ES);
    const v4f na = ldv(ra, ag + k1 * 16 * 4);

    float av[2], bv[2][QT];
    auto frag = [&](int st, int buf) {
      const int off = st / (KC / 4), k4 = st % (KC / 4), dpi = off / ND, dqi = off % ND;
      av[buf] = as[(off * KC + k4 * 4) * 16];
#pragma unroll
      for (int j = 0; j < QT; ++j) bv[buf][j] = bs[(k4 * 4) * CHS + dpi * PITCH + j * 16 + dqi];
    };
    frag(0, 0);
#pragma unroll
    for (int st = 0; st < NSTEP; ++st) {
      if (st + 1 < NSTEP) frag(st + 1, (st + 1) & 1);
#pragma unroll
      for (int j = 0; j < QT; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[st & 1], bv[st & 1][j], acc[j], 0, 0, 0);
    }
    float *dn = dyS + (cur ^ 1) * SBUF;
#pragma unroll
    for (int e = 0; e < SSLOTS; ++e)
      if (sl[e] >= 0) *reinterpret_cast<v4f *>(dn + sl[e]) = ns[e];
    *reinterpret_cast<v4f *>(aS + (cur ^ 1) * ABUF + t * 4) = na;
    __syncthreads();
    cur ^= 1;
  }

  // epilogue: lane group lane / 16 is the channel, register v = a*2 + b the position in the 2x2 block
  const int c = lane >> 4, i = i0 + wave;
  if (c < a.C && i < a.P) {
    elem *o = static_cast<elem *>(a.dx) + (size_t(n) * a.C + c) * HW + size_t(2 * i) * a.W;
#pragma unroll
    for (int j = 0; j < QT; ++j) {
      const int q = j * 16 + (lane & 15);
      if (q < a.Q) {
        if constexpr (ES == 4) {
          *reinterpret_cast<v2f *>(o + 2 * q) = v2f{acc[j][0], acc[j][1]};
          *reinterpret_cast<v2f *>(o + a.W + 2 * q) = v2f{acc[j][2], acc[j][3]};
        } else {   // two 16-bit elements per 4-byte store (W is even: the pairs are aligned)
          elem r0[2], r1[2];
          S::st(r0, acc[j][0]), S::st(r0 + 1, acc[j][1]), S::st(r1, acc[j][2]), S::st(r1 + 1, acc[j][3]);
          *reinterpret_cast<unsigned *>(o + 2 * q) = unsigned(r0[0]) | (unsigned(r0[1]) << 16);
          *reinterpret_cast<unsigned *>(o + a.W + 2 * q) = unsigned(r1[0]) | (unsigned(r1[1]) << 16);
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// The same data gradient on 16-bit tensors with the 16-bit matrix instruction
// (v_mfma_f32_16x16x32_{f16,bf16}: M = 16 rows (c, a, b), N = 16 block columns j, 32 reduction indices per
// instruction, fp32 accumulation).  The reduction is ordered (offset (dp, dq), k) with k fastest, so one
// instruction consumes 32 channels k of one offset and a lane supplies eight consecutive k of its pixel:
// the gradient slab sits in LDS pixel-major, slab[row][col][k] (80-byte pitch: the 64 lanes of a fragment
// read spread evenly over the banks), transposed once per 32 channels while it is staged (dword = two
// pixels of one k; eight k and two v_perm give two 16-byte octets) and then read by all 16 offsets.  The
// weight fragments A[off][m][k] come straight from global memory (32 KB per layer, cache resident), all 16
// of a chunk before its first matrix instruction.  One wavefront per class row, four rows per workgroup,
// two workgroups per CU.  Every fragment read is 1 KB of LDS for 16 cycles of matrix work, so the kernel is
// bound by LDS bandwidth, at several times the fp32 instruction's rate.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int TI16 = 4, SR16 = TI16 + ND - 1, KC16 = 32, KP16 = KC16 + 8;

struct DF16Args {
  const uint16_t *dy;
  const uint16_t *aw;     // A re-laid as [dp,dq (16)][m (16)][KA], 16-bit, KA = K rounded up to 32
  uint16_t *dx;
  int N, C, H, W, K, KA, P, Q;
  int dp0, dq0;
};

// aw[(off * 16 + m) * KA + k], m = c*4 + a*2 + b; W holds the 16-bit weights widened to fp32 (exact)
template <bool BF16>
__global__ __launch_bounds__(256) void k_dgrad_fewc16_weights(const float *__restrict__ W, uint16_t *__restrict__ aw, int K,
                                                             int KA, int C, int R, int S, int ph, int pw, int dp0,
                                                             int dq0) {
  const int total = ND * ND * 16 * KA;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
    const int k = i % KA, m = (i / KA) & 15, off = i / (KA * 16);
    const int c = m >> 2, a = (m >> 1) & 1, b = m & 1;
    const int r = a + ph - 2 * (dp0 + off / ND), s = b + pw - 2 * (dq0 + off % ND);
    const bool ok = k < K && c < C && unsigned(r) < unsigned(R) && unsigned(s) < unsigned(S);
    const float v = ok ? W[((long(k) * C + c) * R + r) * S + s] : 0.f;
    aw[i] = BF16 ? sgh_f32_to_bf16(v) : sgh_f32_to_f16(v);
  }
}

template <int QT, bool BF16>
__global__ __launch_bounds__(256) void k_dgrad_fewc16(DF16Args a) {
  constexpr int COLS = QT * 16 + 8;                      // slab column of dy column q is q + 4
  constexpr int UN = (SR16 * QT * 8 * 4 + 255) / 256;    // staging units per thread (upper bound): (row, pixel pair, k octet)
  extern __shared__ __align__(16) uint16_t slab[];       // [SR16][COLS][KP16]
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int i0 = blockIdx.x * TI16, n = blockIdx.y;
  const int PQ = a.P * a.Q, HW = a.H * a.W, Q2 = a.Q >> 1, npair = SR16 * Q2;
  const rsrc_t rdy = make_rsrc(a.dy + size_t(n) * a.K * PQ, unsigned(a.K) * PQ * 2u);
  const rsrc_t raw = make_rsrc(a.aw, unsigned(ND * ND * 16) * a.KA * 2u);

  // rows outside the image and the pad columns stay zero: only image pixels are (re)written
  for (int i = t; i < SR16 * COLS * KP16 / 8; i += 256) reinterpret_cast<u32x4 *>(slab)[i] = u32x4{0u, 0u, 0u, 0u};

  int sg[UN], sl[UN];
#pragma unroll
  for (int e = 0; e < UN; ++e) {
    const int u = e * 256 + t, ko = u / npair, pr = u - ko * npair, sr = pr / Q2, pp = pr - sr * Q2;
    const int p = i0 + a.dp0 + sr;
    const bool ok = ko < 4 && unsigned(p) < unsigned(a.P);
    sg[e] = ok ? ((ko * 8 * a.P + p) * a.Q + 2 * pp) * 2 : kOOB;
    sl[e] = ok ? (sr * COLS + 2 * pp + 4) * KP16 + ko * 8 : -1;
  }
  const int m = lane & 15, g = lane >> 4;
  const int aoff = (m * a.KA + 8 * g) * 2;                                   // + off * 16 * KA * 2 + chunk
  const int boff = (wave * COLS + m + 4 + a.dq0) * KP16 + 8 * g;             // + (dpi * COLS + j * 16 + dqi) * KP16

  v4f acc[QT];
#pragma unroll
  for (int i = 0; i < QT; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};

  const int nchunks = a.KA / KC16;
  for (int ch = 0; ch < nchunks; ++ch) {
    const int k0 = ch * KC16;
    u32x4 af[ND * ND];
#pragma unroll
    for (int o = 0; o < ND * ND; ++o)
      af[o] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(raw, aoff + o * 16 * a.KA * 2, k0 * 2, 0));
    unsigned rd[UN][8];
#pragma unroll
    for (int e = 0; e < UN; ++e)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        rd[e][j] = unsigned(__builtin_amdgcn_raw_buffer_load_b32(rdy, sg[e], (k0 + j) * PQ * 2, 0));
    __syncthreads();   // the zero fill / every wavefront has finished reading the previous chunk
#pragma unroll
    for (int e = 0; e < UN; ++e) {
      if (sl[e] < 0) continue;
      u32x4 vA, vB;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        vA[d] = __builtin_amdgcn_perm(rd[e][2 * d + 1], rd[e][2 * d], 0x05040100u);
        vB[d] = __builtin_amdgcn_perm(rd[e][2 * d + 1], rd[e][2 * d], 0x07060302u);
      }
      *reinterpret_cast<u32x4 *>(slab + sl[e]) = vA;
      *reinterpret_cast<u32x4 *>(slab + sl[e] + KP16) = vB;
    }
    __syncthreads();
#pragma unroll
    for (int o = 0; o < ND * ND; ++o) {
      const int dpi = o / ND, dqi = o % ND;
      u32x4 bf[QT];
#pragma unroll
      for (int j = 0; j < QT; ++j)
        bf[j] = *reinterpret_cast<const u32x4 *>(slab + boff + (dpi * COLS + j * 16 + dqi) * KP16);
#pragma unroll
      for (int j = 0; j < QT; ++j) {
        if constexpr (BF16)
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[o]), __builtin_bit_cast(bf16x8, bf[j]),
                                                           acc[j], 0, 0, 0);
        else
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af[o]), __builtin_bit_cast(f16x8, bf[j]),
                                                          acc[j], 0, 0, 0);
      }
    }
  }

  // epilogue: lane group lane / 16 is the channel, register v = a*2 + b the position in the 2x2 block
  const int c = lane >> 4, i = i0 + wave;
  if (c < a.C && i < a.P) {
    uint16_t *o = a.dx + (size_t(n) * a.C + c) * HW + size_t(2 * i) * a.W;
#pragma unroll
    for (int j = 0; j < QT; ++j) {
      const int q = j * 16 + (lane & 15);
      if (q < a.Q) {
        const unsigned r00 = BF16 ? sgh_f32_to_bf16(acc[j][0]) : sgh_f32_to_f16(acc[j][0]);
        const unsigned r01 = BF16 ? sgh_f32_to_bf16(acc[j][1]) : sgh_f32_to_f16(acc[j][1]);
        const unsigned r10 = BF16 ? sgh_f32_to_bf16(acc[j][2]) : sgh_f32_to_f16(acc[j][2]);
        const unsigned r11 = BF16 ? sgh_f32_to_bf16(acc[j][3]) : sgh_f32_to_f16(acc[j][3]);
        *reinterpret_cast<unsigned *>(o + 2 * q) = r00 | (r01 << 16);
        *reinterpret_cast<unsigned *>(o + a.W + 2 * q) = r10 | (r11 << 16);
      }
    }
  }
}

struct DFPlan {
  bool ok;
  int qt, dp0, dq0;
  size_t lds;
};

// offsets dp = (a + pad - r) / 2 over a in {0, 1} and the taps r of matching parity
inline bool offset_range(int R, int pad, int *d0, int *cnt) {
  int lo = 1 << 30, hi = -(1 << 30);
  for (int a = 0; a < 2; ++a)
    for (int r = 0; r < R; ++r)
      if (((a + pad - r) & 1) == 0) {
        const int d = (a + pad - r) / 2;  // exact: the numerator is even (C++ division of a negative even number is exact too)
        if (d < lo) lo = d;
        if (d > hi) hi = d;
      }
  if (hi < lo) return false;
  *d0 = lo;
  *cnt = hi - lo + 1;
  return true;
}

inline DFPlan plan(const sgh_conv_geom *g) {
  DFPlan p{};
  p.ok = false;
  if (sgh_env().dgrad_fewc_off) return p;
  if (g->stride_h != 2 || g->stride_w != 2 || g->C > 4) return p;
  if (g->H != 2 * g->P || g->W != 2 * g->Q) return p;          // even image: 2x2 output blocks tile it exactly
  if (g->K % KC != 0 || g->Q % 4 != 0 || g->Q > 128 || g->Q < 4) return p;
  if (g->R * g->S < 16) return p;                               // small filters: the column GEMM is already cheap
  int ndp, ndq;
  if (!offset_range(g->R, g->pad_h, &p.dp0, &ndp) || !offset_range(g->S, g->pad_w, &p.dq0, &ndq)) return p;
  if (ndp > ND || ndq > ND) return p;
  if (p.dq0 < -4 || p.dq0 + ND - 1 > 4) return p;               // slab pad columns: 4 left of the image, 4 right
  p.qt = (g->Q + 15) / 16;
  const int pitch = p.qt * 16 + 8, chs0 = SROWS * pitch, chs = chs0 + ((16 - chs0 % 32) + 32) % 32;
  p.lds = (size_t(2) * KC * chs + size_t(2) * ND * ND * KC * 16) * sizeof(float);
  if (p.lds > 160 * 1024) return p;
  if (size_t(g->K) * g->P * g->Q * 4 >= (size_t(1) << 31)) return p;
  p.ok = true;
  return p;
}

template <int QT, class S>
int launch(const DFArgs &a, const DFPlan &p, dim3 grid, hipStream_t s) {
  auto kern = k_dgrad_fewc<QT, S>;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024) != hipSuccess)
      return SGH_EUNSUPPORTED;
    attr_set = true;
  }
  SGH_LAUNCH_TIMED(kern, grid, dim3(NT), p.lds, s, a);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

}  // namespace

bool sgh_dgrad_fewc_supported(const sgh_conv_geom *g) { return plan(g).ok; }

size_t sgh_dgrad_fewc_workspace_bytes(const sgh_conv_geom *g) {
  return plan(g).ok ? size_t(ND * ND) * g->K * 16 * sizeof(float) : 0;
}

// dy / dx in storage type S (fp32 weights W in every case)
template <class S>
static int dgrad_fewc_run(const sgh_conv_geom *g, const void *dy, const float *W, void *dx, void *workspace,
                          size_t ws_bytes, hipStream_t s, const char *tag) {
  const DFPlan p = plan(g);
  if (!p.ok) return SGH_EUNSUPPORTED;
  if (!workspace || ws_bytes < sgh_dgrad_fewc_workspace_bytes(g)) return SGH_EWORKSPACE;
  float *aw = static_cast<float *>(workspace);
  const int total = ND * ND * g->K * 16;
  hipLaunchKernelGGL(k_dgrad_fewc_weights, dim3((total + 255) / 256), dim3(256), 0, s, W, aw, g->K, g->C, g->R, g->S,
                     g->pad_h, g->pad_w, p.dp0, p.dq0);
  DFArgs a;
  a.dy = dy;
  a.aw = aw;
  a.dx = dx;
  a.N = g->N;
  a.C = g->C;
  a.H = g->H;
  a.W = g->W;
  a.K = g->K;
  a.P = g->P;
  a.Q = g->Q;
  a.dp0 = p.dp0;
  a.dq0 = p.dq0;
  dim3 grid((g->P + TI - 1) / TI, g->N, 1);
  if (grid.y > 65535u) return SGH_EUNSUPPORTED;
  int rc = SGH_EUNSUPPORTED;
  sgh_prof_kernel_begin(tag, 2.0 * g->N * g->K * g->P * g->Q * g->C * g->R * g->S);
  switch (p.qt) {
    case 1: rc = launch<1, S>(a, p, grid, s); break;
    case 2: rc = launch<2, S>(a, p, grid, s); break;
    case 3: rc = launch<3, S>(a, p, grid, s); break;
    case 4: rc = launch<4, S>(a, p, grid, s); break;
    case 5: rc = launch<5, S>(a, p, grid, s); break;
    case 6: rc = launch<6, S>(a, p, grid, s); break;
    case 7: rc = launch<7, S>(a, p, grid, s); break;
    case 8: rc = launch<8, S>(a, p, grid, s); break;
    default: break;
  }
  sgh_prof_kernel_end(s);
  return rc;
}

int sgh_dgrad_fewc_run(const sgh_conv_geom *g, const float *dy, const float *W, float *dx, void *workspace,
                       size_t ws_bytes, hipStream_t s) {
  return dgrad_fewc_run<StF32>(g, dy, W, dx, workspace, ws_bytes, s, "conv_dgrad/k_dgrad_fewc");
}

namespace {

template <int QT, bool BF16>
int launch16(const DF16Args &a, size_t lds, dim3 grid, hipStream_t s) {
  auto kern = k_dgrad_fewc16<QT, BF16>;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024) != hipSuccess)
      return SGH_EUNSUPPORTED;
    attr_set = true;
  }
  SGH_LAUNCH_TIMED(kern, grid, dim3(256), lds, s, a);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

template <bool BF16>
int dgrad_fewc16_mfma(const sgh_conv_geom *g, const DFPlan &p, const uint16_t *dy, const float *W, uint16_t *dx,
                      void *workspace, hipStream_t s) {
  const int KA = (g->K + KC16 - 1) / KC16 * KC16;
  uint16_t *aw = static_cast<uint16_t *>(workspace);   // (half the bytes of the fp32 table the workspace is sized for)
  const int total = ND * ND * 16 * KA;
  hipLaunchKernelGGL(k_dgrad_fewc16_weights<BF16>, dim3((total + 255) / 256), dim3(256), 0, s, W, aw, g->K, KA, g->C, g->R,
                     g->S, g->pad_h, g->pad_w, p.dp0, p.dq0);
  DF16Args a{};
  a.dy = dy, a.aw = aw, a.dx = dx;
  a.N = g->N, a.C = g->C, a.H = g->H, a.W = g->W, a.K = g->K, a.KA = KA, a.P = g->P, a.Q = g->Q;
  a.dp0 = p.dp0, a.dq0 = p.dq0;
  const dim3 grid((g->P + TI16 - 1) / TI16, g->N, 1);
  const size_t lds = size_t(SR16) * (p.qt * 16 + 8) * KP16 * sizeof(uint16_t);
  int rc = SGH_EUNSUPPORTED;
  sgh_prof_kernel_begin("conv_dgrad16/k_dgrad_fewc16", 2.0 * g->N * g->K * g->P * g->Q * g->C * g->R * g->S);
  switch (p.qt) {
    case 1: rc = launch16<1, BF16>(a, lds, grid, s); break;
    case 2: rc = launch16<2, BF16>(a, lds, grid, s); break;
    case 3: rc = launch16<3, BF16>(a, lds, grid, s); break;
    case 4: rc = launch16<4, BF16>(a, lds, grid, s); break;
    case 5: rc = launch16<5, BF16>(a, lds, grid, s); break;
    case 6: rc = launch16<6, BF16>(a, lds, grid, s); break;
    case 7: rc = launch16<7, BF16>(a, lds, grid, s); break;
    case 8: rc = launch16<8, BF16>(a, lds, grid, s); break;
    default: break;
  }
  sgh_prof_kernel_end(s);
  return rc;
}

}  // namespace

int sgh_dgrad_fewc_run16(const sgh_conv_geom *g, const uint16_t *dy, const float *W, uint16_t *dx, void *workspace,
                         size_t ws_bytes, bool bf16, hipStream_t s) {
  {
    // the 16-bit matrix instruction: K in whole chunks of 32, even Q (pixel pairs), offsets of the slab
    const DFPlan p = plan(g);
    if (p.ok && g->K % KC16 == 0 && g->Q % 2 == 0 && g->N <= 65535 && !sgh_env().dgrad_fewc16_off) {
      if (!workspace || ws_bytes < sgh_dgrad_fewc_workspace_bytes(g)) return SGH_EWORKSPACE;
      return bf16 ? dgrad_fewc16_mfma<true>(g, p, dy, W, dx, workspace, s)
                  : dgrad_fewc16_mfma<false>(g, p, dy, W, dx, workspace, s);
    }
  }
  return bf16 ? dgrad_fewc_run<StBF16>(g, dy, W, dx, workspace, ws_bytes, s, "conv_dgrad16/k_dgrad_fewc")
              : dgrad_fewc_run<StF16>(g, dy, W, dx, workspace, ws_bytes, s, "conv_dgrad16/k_dgrad_fewc");
}
