// fp32 MFMA GEMM core and the implicit-GEMM convolution passes built on it
// (conv forward, dgrad, wgrad) plus the Linear-layer GEMM.
//
// One workgroup = 256 threads = 4 wavefronts in a WGM x WGN grid; the workgroup computes a
// BM x BN tile of C, each wavefront a (BM/WGM) x (BN/WGN) sub-tile out of 32x32x2 fp32 MFMAs
// (v_mfma_f32_32x32x2_f32: lane l feeds A[l%32][l/32] and B[l/32][l%32]; its 16 accumulators
// hold C[8*(v/4) + 4*(l/32) + v%4][l%32]).
//
// Operands are staged through LDS in [k][m] / [k][n] order with a row pitch of (tile + 4)
// floats: the MFMA operand reads (32 consecutive m for two consecutive k) and both kinds of
// staging writes (threads consecutive in m, or consecutive in k) then touch every bank at most
// twice per 64-lane access, which is the minimum.
//
// Software pipeline of one BK-chunk (8 MFMA k-steps):
//   - the LDS operand fragments of k-step s+1 are fetched into a second register set before the
//     MFMAs of k-step s are issued;
//   - the global loads of the NEXT chunk (address arithmetic included) are spread over the
//     k-steps and issued right behind each step's MFMAs, so their VALU work and latency hide
//     under the matrix pipeline;
//   - after the last k-step the loaded registers go to the other LDS buffer (one barrier per chunk).
//
// A "problem" supplies two loaders (how to fetch element (row, k) of A and (k, col) of B,
// zero outside the valid range) and an epilogue (where C[m][n] goes).  The convolution loaders
// perform im2col on the fly: no column matrix is ever materialised.
#include <stdlib.h>

#include "common.h"
#include "storage.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int NT = 256;
constexpr int BK = 16;
constexpr int KSTEPS = BK / 2;

// Global operands are read through buffer loads: the hardware range check makes an out-of-range
// byte offset return 0, which gives zero padding / tile tails without a branch per element.
// Every operand tensor is therefore limited to < 2 GiB (SINGA's Device::Malloc(int) caps a Block
// at that size anyway: include/singa/core/device.h:142).
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int kOOB = int(0x80000000u);
__device__ __forceinline__ rsrc_t make_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, bytes, 0x00020000);
}
// `ok` must be built with bitwise '&' (no short-circuit) so that the load stays straight-line code.
__device__ __forceinline__ float buf_ld(rsrc_t r, int elem_off, int ok) {
  const int m = -ok;  // all ones when valid
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, ((elem_off << 2) & m) | (kOOB & ~m), 0, 0));
}

// ------------------------------------------------------------------------------------------
// Thread -> staged element mapping.
//   K-contiguous operand (consecutive k are consecutive in memory):
//       kk = t % BK, row = t / BK + e * (NT / BK)
//   M/N-contiguous operand (consecutive rows are consecutive in memory):
//       row = t % ROWS, kk = t / ROWS + e * (NT / ROWS)
// e = 0 .. ROWS * BK / NT - 1.
// ------------------------------------------------------------------------------------------
template <int ROWS, bool KCONTIG>
struct StageMap {
  static constexpr int E = ROWS * BK / NT;
  static constexpr int ROW_STEP = KCONTIG ? NT / BK : 0;
  static constexpr int K_STEP = KCONTIG ? 0 : NT / ROWS;
  __device__ static __forceinline__ int row0(int t) { return KCONTIG ? t / BK : t % ROWS; }
  __device__ static __forceinline__ int kk0(int t) { return KCONTIG ? t % BK : t / ROWS; }
};

template <int ROWS, bool KCONTIG>
__device__ __forceinline__ void stage_store(float *lds /* [BK][ROWS + 4] */, const float (&r)[ROWS * BK / NT], int t) {
  using M = StageMap<ROWS, KCONTIG>;
  const int row0 = M::row0(t), kk0 = M::kk0(t);
#pragma unroll
  for (int e = 0; e < M::E; ++e) lds[(kk0 + e * M::K_STEP) * (ROWS + 4) + row0 + e * M::ROW_STEP] = r[e];
}

// Every loader has:   init(tile0, t)          once per kernel (per-thread constants)
//                     prepare(tile0, k0, k_end, t)   once per chunk (per-chunk index arithmetic)
//                     get(e)                   element e of the chunk prepared last

// ------------------------------------------------------------------------------------------
// Loader 1: dense strided matrix.  element(row, k) = base[row * rs + k * ks]; whichever of
// rs / ks is 1 decides KCONTIG.
// ------------------------------------------------------------------------------------------
template <int ROWS, bool KCONTIG>
struct DenseLoader {
  using M = StageMap<ROWS, KCONTIG>;
  const float *base;
  int rs, ks;
  int rows, K;
  unsigned bytes;
  int row0_, kk0_, kend_;
  __device__ __forceinline__ void init(int, int) {}
  __device__ __forceinline__ void prepare(int tile_row0, int k0, int k_end, int t) {
    row0_ = tile_row0 + M::row0(t);
    kk0_ = k0 + M::kk0(t);
    kend_ = k_end;
  }
  __device__ __forceinline__ float get(int e) const {
    const int row = row0_ + e * M::ROW_STEP, k = kk0_ + e * M::K_STEP;
    return buf_ld(make_rsrc(base, bytes), row * rs + k * ks, int(row < rows) & int(k < kend_));
  }
};

// ------------------------------------------------------------------------------------------
// Convolution geometry shared by the gather loaders.
// ------------------------------------------------------------------------------------------
struct ConvG {
  int N, C, H, W, K, R, S, sh, sw, ph, pw, P, Q;
};

// ------------------------------------------------------------------------------------------
// Loader 2: pixel gather for forward and dgrad (N-contiguous: a thread owns ONE pixel column of
// the tile for the whole kernel and walks k).
//   k index = tap * CP + ch, tap = r * S + s, CP = channel count rounded up to BK, so one
//   BK-chunk has a single tap and the tap's validity test is done once per chunk per thread.
//   FWD:   column = (n, p, q) of y;  source = x[n][ch][p*sh - ph + r][q*sw - pw + s]
//   DGRAD: column = (n, h, w) of dx; source = dy[n][ch][(h + ph - r)/sh][(w + pw - s)/sw]
//          (only where both divisions are exact and in range)
// ------------------------------------------------------------------------------------------
template <int ROWS, bool DGRAD>
struct PixelGatherLoader {
  using M = StageMap<ROWS, false>;
  const float *src;
  ConvG g;
  int CP;        // padded channel count of the k index
  int src_ch;    // channels of the source tensor (C for fwd, K for dgrad)
  int src_h, src_w;
  int cols;      // valid columns (N * P * Q or N * H * W)
  unsigned bytes;
  // per-thread state
  int img_base;  // offset of image n in src
  int a, b;      // (p, q) for fwd, (h, w) for dgrad
  bool col_ok;
  // per-chunk state
  int p_, ch0_, ok_;

  __device__ __forceinline__ void init(int tile_col0, int t) {
    const int col = tile_col0 + M::row0(t);
    col_ok = col < cols;
    const int plane = DGRAD ? g.H * g.W : g.P * g.Q;
    const int wdt = DGRAD ? g.W : g.Q;
    const int n = col / plane, rem = col - n * plane;
    a = rem / wdt;
    b = rem - a * wdt;
    img_base = n * src_ch * src_h * src_w;
  }

  __device__ __forceinline__ void prepare(int, int k0, int, int t) {
    const int tap = k0 / CP;
    ch0_ = k0 - tap * CP + M::kk0(t);
    const int fr = tap / g.S, fs = tap - fr * g.S;
    int y, x;
    int ok = col_ok;
    if (DGRAD) {
      const int hp = a + g.ph - fr, wp = b + g.pw - fs;
      y = hp / g.sh;
      x = wp / g.sw;
      ok = ok & (hp >= 0) & (wp >= 0) & (y * g.sh == hp) & (x * g.sw == wp) & (y < g.P) & (x < g.Q);
    } else {
      y = a * g.sh - g.ph + fr;
      x = b * g.sw - g.pw + fs;
      ok = ok & (unsigned(y) < unsigned(g.H)) & (unsigned(x) < unsigned(g.W));
    }
    ok_ = ok;
    p_ = img_base + y * src_w + x;
  }

  __device__ __forceinline__ float get(int e) const {
    const int ch = ch0_ + e * M::K_STEP;
    return buf_ld(make_rsrc(src, bytes), p_ + ch * (src_h * src_w), ok_ & int(ch < src_ch));
  }
};

// ------------------------------------------------------------------------------------------
// Loaders 3 and 4: wgrad.  The reduction index g = n * PQ + p * Q + q is contiguous in memory
// for both operands, so both are K-contiguous.
//   A(m = k_out, g) = dy[n][m][pq]
//   B(g, j = (c, r, s) in KCRS order) = x[n][c][p*sh - ph + r][q*sw - pw + s]
// ------------------------------------------------------------------------------------------
template <int ROWS>
struct WgradDyLoader {
  using M = StageMap<ROWS, true>;
  const float *dy;
  int K, PQ, G;  // G = N * PQ
  unsigned bytes;
  int row0_, p_, ok_;
  __device__ __forceinline__ void init(int, int) {}
  __device__ __forceinline__ void prepare(int tile_row0, int k0, int k_end, int t) {
    const int gi = k0 + M::kk0(t);
    ok_ = gi < k_end;
    const int n = gi / PQ, pq = gi - n * PQ;
    p_ = n * K * PQ + pq;
    row0_ = tile_row0 + M::row0(t);
  }
  __device__ __forceinline__ float get(int e) const {
    const int row = row0_ + e * M::ROW_STEP;
    return buf_ld(make_rsrc(dy, bytes), p_ + row * PQ, ok_ & int(row < K));
  }
};

template <int ROWS>
struct WgradXLoader {
  using M = StageMap<ROWS, true>;
  const float *x;
  ConvG g;
  int CRS;
  unsigned bytes;
  // per-thread, per staged row: offset of (c, r - ph, s - pw) inside an image, and the tap shifts
  int off[ROWS * BK / NT];
  short dr[ROWS * BK / NT], ds[ROWS * BK / NT];
  int h0_, w0_, base_, ok_;
  // Column `ones_col` (CRS when the bias gradient rides along, else -1) is a column of ones over the
  // valid pixels: its dot product with a dy row is that row's sum, i.e. db[k], from the same MFMAs.
  int ones_col;
  unsigned ones_mask;   // staged rows of this thread that are that column
  __device__ __forceinline__ void init(int tile_col0, int t) {
    const int RS = g.R * g.S;
    ones_mask = 0u;
#pragma unroll
    for (int e = 0; e < M::E; ++e) {
      const int j = tile_col0 + M::row0(t) + e * M::ROW_STEP;
      if (j == ones_col) ones_mask |= 1u << e;
      if (j < CRS) {
        const int c = j / RS, rs = j - c * RS, fr = rs / g.S, fs = rs - fr * g.S;
        dr[e] = short(fr - g.ph);
        ds[e] = short(fs - g.pw);
        off[e] = (c * g.H + (fr - g.ph)) * g.W + (fs - g.pw);
      } else {
        dr[e] = short(-30000);  // fails the row test below for every p
        ds[e] = 0;
        off[e] = 0;
      }
    }
  }
  __device__ __forceinline__ void prepare(int, int k0, int k_end, int t) {
    const int gi = k0 + M::kk0(t);
    ok_ = gi < k_end;
    const int PQ = g.P * g.Q;
    const int n = gi / PQ, pq = gi - n * PQ;
    const int p = pq / g.Q, q = pq - p * g.Q;
    h0_ = p * g.sh;
    w0_ = q * g.sw;
    base_ = n * g.C * g.H * g.W + h0_ * g.W + w0_;
  }
  __device__ __forceinline__ float get(int e) const {
    const int h = h0_ + dr[e], w = w0_ + ds[e];
    // unsigned compares fold the two-sided range checks
    const int v = ok_ & int(unsigned(h) < unsigned(g.H)) & int(unsigned(w) < unsigned(g.W));
    const float xv = buf_ld(make_rsrc(x, bytes), base_ + off[e], v);
    return (ones_mask >> e) & 1u ? (ok_ ? 1.f : 0.f) : xv;
  }
};

// ------------------------------------------------------------------------------------------
// Loaders 5 and 6 + epilogue: dgrad decomposed by output-pixel residue class.
// With stride (sh, sw) the pixels h = ch + sh*hh, w = cw + sw*ww of class (ch, cw) receive
// contributions only from the taps r = r0 + i*sh, s = s0 + j*sw (r0 = (ch + ph) % sh), and for
// those p = hh + bh - i, q = ww + bw - j are exact.  Each class is therefore a dense stride-1
// problem over its own tap subset: no MFMA work is spent on taps that cannot contribute
// (a plain gather wastes 1 - 1/(sh*sw) of it).  blockIdx.z selects the class.
//   k index inside a class = (i * ns + j) * KP + k_out
//   class weights Wc[(tap_off + i*ns + j) * KP + k_out][c]  (k_weight_relayout_classes)
// ------------------------------------------------------------------------------------------
constexpr int kMaxClasses = 9;
constexpr int kMaxTaps = 128;

struct DgCls {
  short ch, cw, r0, s0, nr, ns, bh, bw;
  int Hc, Wc, tap_off;
};
struct DgClsTable {
  DgCls c[kMaxClasses];
};
struct TapTable {  // class-ordered tap list: rs[t] = r * S + s
  short rs[kMaxTaps];
};

template <int ROWS>
struct DgradWLoader {  // A(m = c, k) = Wc[class][k][c], M-contiguous
  using M = StageMap<ROWS, false>;
  const float *Wc;
  int C, KP;
  const DgCls *tab;  // class table in device memory (written by k_weight_relayout_classes)
  unsigned bytes;
  int base;
  int row_, kk0_, kend_;
  __device__ __forceinline__ void init(int, int) { base = tab[blockIdx.z].tap_off * KP * C; }
  __device__ __forceinline__ void prepare(int tile_row0, int k0, int k_end, int t) {
    row_ = tile_row0 + M::row0(t);
    kk0_ = k0 + M::kk0(t);
    kend_ = k_end;
  }
  __device__ __forceinline__ float get(int e) const {
    const int k = kk0_ + e * M::K_STEP;
    return buf_ld(make_rsrc(Wc, bytes), base + k * C + row_, int(row_ < C) & int(k < kend_));
  }
};

template <int ROWS>
struct DgradDyLoader {  // B(k, col = (n, hh, ww) of the class), N-contiguous
  using M = StageMap<ROWS, false>;
  const float *dy;
  ConvG g;
  int KP;
  const DgCls *tab;
  unsigned bytes;
  int img_base;
  int hh, ww, cols;
  bool col_ok;
  DgCls c;
  int src_, ch0_, ok_;
  __device__ __forceinline__ void init(int tile_col0, int t) {
    c = tab[blockIdx.z];
    const int plane = c.Hc * c.Wc;
    cols = g.N * plane;
    const int col = tile_col0 + M::row0(t);
    col_ok = col < cols;
    const int pl = plane > 0 ? plane : 1, wd = c.Wc > 0 ? c.Wc : 1;
    const int n = col / pl, rem = col - n * pl;
    hh = rem / wd;
    ww = rem - hh * wd;
    img_base = n * g.K * g.P * g.Q;
  }
  __device__ __forceinline__ int ktotal() const { return int(c.nr) * c.ns * KP; }
  __device__ __forceinline__ bool block_empty(int tile_col0) const { return tile_col0 >= cols; }
  __device__ __forceinline__ void prepare(int, int k0, int, int t) {
    const int tap = k0 / KP;
    ch0_ = k0 - tap * KP + M::kk0(t);
    const int ns = c.ns > 0 ? c.ns : 1;
    const int i = tap / ns, j = tap - i * ns;
    const int p = hh + c.bh - i, q = ww + c.bw - j;
    ok_ = int(col_ok) & int(unsigned(p) < unsigned(g.P)) & int(unsigned(q) < unsigned(g.Q));
    src_ = img_base + p * g.Q + q;
  }
  __device__ __forceinline__ float get(int e) const {
    const int ch = ch0_ + e * M::K_STEP;
    return buf_ld(make_rsrc(dy, bytes), src_ + ch * (g.P * g.Q), ok_ & int(ch < g.K));
  }
};

struct DgradStore {  // dx[n][m][ch + sh*hh][cw + sw*ww]
  float *dx;
  ConvG g;
  const DgCls *tab;
  __device__ __forceinline__ void operator()(int m, int col, float v) const {
    const DgCls c = tab[blockIdx.z];
    const int plane = c.Hc * c.Wc;
    if (m < g.C && col < g.N * plane) {
      const int n = col / plane, rem = col - n * plane;
      const int hh = rem / c.Wc, ww = rem - hh * c.Wc;
      dx[((long(n) * g.C + m) * g.H + c.ch + g.sh * hh) * g.W + c.cw + g.sw * ww] = v;
    }
  }
};

// ------------------------------------------------------------------------------------------
// Epilogues
// ------------------------------------------------------------------------------------------
struct DenseStore {  // C[m * ldc + n] = alpha * acc + beta * C
  float *C;
  long ldc;
  int M, N;
  float alpha, beta;
  __device__ __forceinline__ void operator()(int m, int n, float v) const {
    if (m < M && n < N) {
      float *p = C + m * ldc + n;
      *p = beta == 0.f ? alpha * v : alpha * v + beta * *p;
    }
  }
};

struct NchwStore {  // out[(img * CH + m) * plane + rem] (+ bias[m]), column = img * plane + rem
  float *out;
  const float *bias;
  int CH, plane, cols;
  __device__ __forceinline__ void operator()(int m, int col, float v) const {
    if (m < CH && col < cols) {
      const int img = col / plane, rem = col - img * plane;
      out[(long(img) * CH + m) * plane + rem] = bias ? v + bias[m] : v;
    }
  }
};

// Data gradient of a 1x1, pad-0, stride-s convolution: GEMM column (img, p, q) lands on
// dx[img][m][s*p][s*q] and the other positions of its s x s block are zero.  A lane writes the
// whole block, so dx is produced in one pass without a separate zero fill.
struct DilateStore {
  float *dx;
  int C, H, W, P, Q, sh, sw, cols;
  __device__ __forceinline__ void operator()(int m, int col, float v) const {
    if (m < C && col < cols) {
      const int PQ = P * Q;
      const int img = col / PQ, rem = col - img * PQ, p = rem / Q, q = rem - p * Q;
      float *o = dx + ((long(img) * C + m) * H + p * sh) * W + q * sw;
      if (sh == 2 && sw == 2 && p * 2 + 1 < H && q * 2 + 1 < W && (reinterpret_cast<uintptr_t>(o) & 7u) == 0 &&
          (W & 1) == 0) {
        typedef float v2f __attribute__((ext_vector_type(2)));
        *reinterpret_cast<v2f *>(o) = v2f{v, 0.f};
        *reinterpret_cast<v2f *>(o + W) = v2f{0.f, 0.f};
      } else {
        // rows / columns of the block that fall outside the image (odd sizes) are skipped; the
        // last block of a row / column also covers the remainder beyond s * Q (s * P)
        const int he = p == P - 1 ? H - p * sh : sh, we = q == Q - 1 ? W - q * sw : sw;
        for (int a = 0; a < he; ++a)
          for (int b = 0; b < we; ++b) o[a * W + b] = (a == 0 && b == 0) ? v : 0.f;
      }
    }
  }
};

struct SplitStore {  // partial[split][m * N + n]; column N, if wanted, goes to bpart[split][m]
  float *part;
  int M, N;
  float *bpart;
  __device__ __forceinline__ void operator()(int m, int n, float v) const {
    if (m < M && n < N) part[long(blockIdx.z) * M * N + long(m) * N + n] = v;
    else if (bpart && m < M && n == N) bpart[long(blockIdx.z) * M + m] = v;
  }
};

// ------------------------------------------------------------------------------------------
// The kernel.  grid = (M tiles, N tiles, K splits); split z covers chunks
// [z * chunks_per_split, (z + 1) * chunks_per_split) of the reduction.
// With ZCLASS, blockIdx.z is a problem class instead (the B loader reports its reduction length
// and whether this tile lies outside the class).
// ------------------------------------------------------------------------------------------
template <int BM, int BN, class LA, class LB, class ST, bool A_KCONTIG, bool B_KCONTIG, bool ZCLASS = false,
          int WGM = 2, int PF = 1>
__global__ __launch_bounds__(NT) void k_igemm(LA la, LB lb, ST st, int Ktotal, int chunks_per_split) {
  // the four wavefronts form a WGM x WGN grid over the tile
  constexpr int WGN = 4 / WGM;
  constexpr int PA = BM + 4, PB = BN + 4;
  constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
  static_assert(TM >= 1 && TN >= 1 && WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
  constexpr int EA = BM * BK / NT, EB = BN * BK / NT, ET = EA + EB;
  __shared__ float As[2][BK * PA];
  __shared__ float Bs[2][BK * PB];

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  const int m0 = blockIdx.x * BM, n0 = blockIdx.y * BN;
  int k_begin = blockIdx.z * chunks_per_split * BK;
  int k_end = k_begin + chunks_per_split * BK;
  if (k_end > Ktotal) k_end = Ktotal;

  la.init(m0, t);
  lb.init(n0, t);
  if constexpr (ZCLASS) {
    if (lb.block_empty(n0)) return;  // uniform over the workgroup, before any barrier
    k_begin = 0;
    k_end = lb.ktotal();
  }

  v16f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // PF chunks of loads are in flight in registers (set c % PF holds chunk c until it is written to LDS): a
  // chunk of a small tile holds far fewer MFMA cycles than a load takes to return, so one chunk ahead leaves
  // the loop waiting for memory; the loop is unrolled PF times so that the sets are addressed statically.
  float ra[PF][EA], rb[PF][EB];
  if (k_begin < k_end) {
#pragma unroll
    for (int d = 0; d < PF; ++d) {
      la.prepare(m0, k_begin + d * BK, k_end, t);
      lb.prepare(n0, k_begin + d * BK, k_end, t);
#pragma unroll
      for (int e = 0; e < EA; ++e) ra[d][e] = la.get(e);
#pragma unroll
      for (int e = 0; e < EB; ++e) rb[d][e] = lb.get(e);
    }
    stage_store<BM, A_KCONTIG>(As[0], ra[0], t);
    stage_store<BN, B_KCONTIG>(Bs[0], rb[0], t);
  }
  __syncthreads();

  int cur = 0;
  for (int kb = k_begin; kb < k_end; kb += PF * BK) {
#pragma unroll
    for (int d = 0; d < PF; ++d) {
      const int k0 = kb + d * BK;
      if (k0 >= k_end) break;
      // chunk k0 / BK + PF is always fetched into the set this chunk has just left: past the end every loader
      // yields zeros (or, for the gather loaders, values that are never stored), which keeps this loop free
      // of branches
      la.prepare(m0, k0 + PF * BK, k_end, t);
      lb.prepare(n0, k0 + PF * BK, k_end, t);

      const float *as = As[cur] + (lane >> 5) * PA + wm * WM + (lane & 31);
      const float *bs = Bs[cur] + (lane >> 5) * PB + wn * WN + (lane & 31);
      float a[2][TM], b[2][TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[0][i] = as[i * 32];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[0][j] = bs[j * 32];
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        const int cb = s & 1, nb = cb ^ 1;
        if (s + 1 < KSTEPS) {
#pragma unroll
          for (int i = 0; i < TM; ++i) a[nb][i] = as[(2 * s + 2) * PA + i * 32];
#pragma unroll
          for (int j = 0; j < TN; ++j) b[nb][j] = bs[(2 * s + 2) * PB + j * 32];
        }
        __builtin_amdgcn_sched_barrier(0);  // operand prefetch stays ahead of this k-step's MFMAs
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cb][i], b[cb][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);  // this k-step's share of the global loads
        if (PF == 1) {
#pragma unroll
          for (int q = 0; q < ET; ++q) {
            if (q * KSTEPS / ET == s) {
              if (q < EA) ra[d][q] = la.get(q);
              else rb[d][q - EA] = lb.get(q - EA);
            }
          }
        }
      }
      if (k0 + BK < k_end) {
        // the next chunk's registers go to LDS before its set is reloaded (with one set, it was reloaded above)
        stage_store<BM, A_KCONTIG>(As[cur ^ 1], ra[(d + 1) % PF], t);
        stage_store<BN, B_KCONTIG>(Bs[cur ^ 1], rb[(d + 1) % PF], t);
      }
      if (PF > 1) {
#pragma unroll
        for (int e = 0; e < EA; ++e) ra[d][e] = la.get(e);
#pragma unroll
        for (int e = 0; e < EB; ++e) rb[d][e] = lb.get(e);
      }
      __syncthreads();
      cur ^= 1;
    }
  }

#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * WM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        const int n = n0 + wn * WN + j * 32 + (lane & 31);
        st(m, n, acc[i][j][v]);
      }
}

// Ordered reduction of split-K partials: out[i] = sum_s part[s][i], s ascending.
__global__ __launch_bounds__(NT) void k_split_reduce(const float *__restrict__ part, float *__restrict__ out, long n,
                                                    int splits) {
  const long stride = long(gridDim.x) * NT;
  for (long i = long(blockIdx.x) * NT + threadIdx.x; i < n; i += stride) {
    float s = 0.f;
    for (int z = 0; z < splits; ++z) s += part[z * n + i];
    out[i] = s;
  }
}

// The same sum for small outputs with many splits: 16 z-lanes x 16 elements per workgroup, lane zl
// sums z = zl, zl + 16, ... (ascending), the lane sums are added in lane order.  Which of the two
// kernels runs depends on the shape only, so results stay run-to-run identical.
__global__ __launch_bounds__(256) void k_split_reduce_lanes(const float *__restrict__ part, float *__restrict__ out,
                                                           long n, int splits) {
  __shared__ float lanes[16][16];
  const int e = threadIdx.x & 15, zl = threadIdx.x >> 4;
  const long i = long(blockIdx.x) * 16 + e;
  float s = 0.f;
  if (i < n)
    for (int z = zl; z < splits; z += 16) s += part[long(z) * n + i];
  lanes[zl][e] = s;
  __syncthreads();
  if (threadIdx.x < 16 && i < n) {
    float r = lanes[0][e];
#pragma unroll
    for (int l = 1; l < 16; ++l) r += lanes[l][e];
    out[i] = r;
  }
}

// Weight re-layout for the pixel-gather passes:  W[K][C][R][S]  ->  Wt[tap][chp][m]
//   forward (mode 0): ch = c (padded to CP), m = k   -> Wt[(tap * CP + c) * K + k]
//   dgrad   (mode 1): ch = k (padded to KP), m = c   -> Wt[(tap * KP + k) * C + c]
//   forward with the taps in reverse order (mode 2): as mode 0 from W[..][RS - 1 - tap]; a
//   correlation with the flipped filter is what the shared-tile data-gradient kernel computes,
//   so that kernel then evaluates the forward convolution
__global__ __launch_bounds__(NT) void k_weight_relayout(const float *__restrict__ W, float *__restrict__ Wt, int K, int C,
                                                       int RS, int CHP, int dgrad) {
  const bool flip = dgrad == 2;
  if (flip) dgrad = 0;
  const long total = long(RS) * CHP * (dgrad ? C : K);
  const long stride = long(gridDim.x) * NT;
  const int Mdim = dgrad ? C : K;
  for (long i = long(blockIdx.x) * NT + threadIdx.x; i < total; i += stride) {
    const int m = int(i % Mdim);
    const long rest = i / Mdim;
    const int ch = int(rest % CHP), tap = int(rest / CHP);
    float v = 0.f;
    if (dgrad) {
      if (ch < K) v = W[(long(ch) * C + m) * RS + tap];
    } else {
      if (ch < C) v = W[(long(m) * C + ch) * RS + (flip ? RS - 1 - tap : tap)];
    }
    Wt[i] = v;
  }
}

// Class-ordered weight re-layout for the decomposed dgrad:
//   Wc[(t * KP + k) * C + c] = W[k][c][taps.rs[t]],  t = position in the class-ordered tap list
__global__ __launch_bounds__(NT) void k_weight_relayout_classes(const float *__restrict__ W, float *__restrict__ Wc,
                                                               int K, int C, int RS, int KP, TapTable taps,
                                                               DgClsTable tab, DgCls *__restrict__ tab_out) {
  if (blockIdx.x == 0 && threadIdx.x < kMaxClasses) {
    // static indexing keeps the by-value table in SGPRs
    DgCls c = tab.c[0];
#pragma unroll
    for (int i = 1; i < kMaxClasses; ++i)
      if (int(threadIdx.x) == i) c = tab.c[i];
    tab_out[threadIdx.x] = c;
  }
  const long total = long(RS) * KP * C;
  const long stride = long(gridDim.x) * NT;
  for (long i = long(blockIdx.x) * NT + threadIdx.x; i < total; i += stride) {
    const int c = int(i % C);
    const long rest = i / C;
    const int k = int(rest % KP), tt = int(rest / KP);
    Wc[i] = k < K ? W[(long(k) * C + c) * RS + taps.rs[tt]] : 0.f;
  }
}

// Col2im as a gather (the scatter loop of the CPU algorithm turned inside out): one thread per
// dx element adds the column entries of every tap that maps onto it, in ascending (r, s) order.
//   dx[n][c][h][w] = sum_{r,s} dcol[(c*R + r)*S + s][n*PQ + p*Q + q],  p*sh = h + ph - r, q*sw = w + pw - s
// Only the taps of the element's residue class are visited (r = r0, r0 + sh, ...), and the
// threads of a wavefront take elements of ONE class along w (w = cw + sw * j, j consecutive), so
// that for a fixed tap they read consecutive q: coalesced reads of dcol, stride-sw writes of dx.
__global__ __launch_bounds__(NT) void k_col2im_gather(const float *__restrict__ dcol, float *__restrict__ dx, ConvG g,
                                                     long total) {
  const long stride = long(gridDim.x) * NT;
  const int PQ = g.P * g.Q;
  const long ncols = long(g.N) * PQ;
  const int WJ = (g.W + g.sw - 1) / g.sw;  // elements per class along w (the last class may be shorter)
  const long rowlen = long(WJ) * g.sw;      // iteration space per row: sw classes x WJ
  const long total_it = long(g.N) * g.C * g.H * rowlen;
  (void)total;
  for (long i = long(blockIdx.x) * NT + threadIdx.x; i < total_it; i += stride) {
    const int it = int(i % rowlen);
    const long row = i / rowlen;
    const int cw = it / WJ, j = it - cw * WJ;
    const int w = cw + g.sw * j;
    if (w >= g.W) continue;
    const int h = int(row % g.H);
    const long t2 = row / g.H;
    const int c = int(t2 % g.C), n = int(t2 / g.C);
    const int r0 = (h + g.ph) % g.sh, s0 = (w + g.pw) % g.sw;
    float acc = 0.f;
    for (int r = r0; r < g.R; r += g.sh) {
      const int p = (h + g.ph - r) / g.sh;  // exact by construction
      if (h + g.ph - r < 0) break;
      if (p >= g.P) continue;
      const float *src = dcol + long((c * g.R + r) * g.S) * ncols + long(n) * PQ + p * g.Q;
      for (int s = s0; s < g.S; s += g.sw) {
        const int wq = w + g.pw - s;
        if (wq < 0) break;
        const int q = wq / g.sw;
        if (q < g.Q) acc += src[long(s) * ncols + q];
      }
    }
    dx[(row * g.W) + w] = acc;
  }
}

// One thread per (k), summing dy over n, p, q is too serial; use one workgroup per k.
template <class S>
__global__ __launch_bounds__(NT) void k_conv_bgrad(const typename S::elem *__restrict__ dy,
                                                  typename S::elem *__restrict__ db, int N, int K, int PQ) {
  __shared__ float red[16];
  const int k = blockIdx.x;
  float s = 0.f;
  const int total = N * PQ;
  for (int i = threadIdx.x; i < total; i += NT) {
    const int n = i / PQ, r = i - n * PQ;
    s += S::ld(dy + (long(n) * K + k) * PQ + r);
  }
  s = sgh_block_sum(s, red);
  if (threadIdx.x == 0) S::st(db + k, s);
}

inline int round_up(int v, int m) { return (v + m - 1) / m * m; }

inline ConvG to_g(const sgh_conv_geom *g) {
  return ConvG{g->N, g->C, g->H, g->W, g->K, g->R, g->S, g->stride_h, g->stride_w, g->pad_h, g->pad_w, g->P, g->Q};
}

constexpr size_t kMaxOperandBytes = size_t(1) << 31;  // buffer-load addressing limit per tensor

inline bool conv_ok(const sgh_conv_geom *g) {
  if (!g) return false;
  if (g->N <= 0 || g->C <= 0 || g->H <= 0 || g->W <= 0 || g->K <= 0 || g->R <= 0 || g->S <= 0 || g->stride_h <= 0 ||
      g->stride_w <= 0 || g->pad_h < 0 || g->pad_w < 0 || g->P <= 0 || g->Q <= 0)
    return false;
  if (g->P != (g->H + 2 * g->pad_h - g->R) / g->stride_h + 1) return false;
  if (g->Q != (g->W + 2 * g->pad_w - g->S) / g->stride_w + 1) return false;
  if (g->groups < 1 || g->C % g->groups != 0 || g->K % g->groups != 0) return false;
  if (g->pad_h > 16000 || g->pad_w > 16000 || g->R > 16000 || g->S > 16000) return false;
  // every tensor is addressed with 32-bit byte offsets inside the kernels
  const size_t lim = kMaxOperandBytes / sizeof(float);
  if (size_t(g->N) * g->C * g->H * g->W >= lim) return false;
  if (size_t(g->N) * g->K * g->P * g->Q >= lim) return false;
  if (size_t(g->R) * g->S * (size_t(g->C) + BK) * (size_t(g->K) + BK) >= lim) return false;
  return true;
}

inline unsigned bytes_of(size_t elems) { return unsigned(elems * sizeof(float)); }

// ---- loader factories (host) -------------------------------------------------------------
template <int ROWS, bool KC>
inline DenseLoader<ROWS, KC> dense_loader(const float *base, long rs, long ks, int rows, int K) {
  DenseLoader<ROWS, KC> l;
  l.base = base;
  l.rs = int(rs);
  l.ks = int(ks);
  l.rows = rows;
  l.K = K;
  const size_t extent = (rows > 0 && K > 0) ? size_t(rows - 1) * rs + size_t(K - 1) * ks + 1 : 0;
  l.bytes = bytes_of(extent);
  l.row0_ = l.kk0_ = l.kend_ = 0;
  return l;
}

template <int ROWS, bool DG>
inline PixelGatherLoader<ROWS, DG> gather_loader(const float *src, const ConvG &g, int CP, int src_ch, int src_h,
                                                 int src_w, int cols) {
  PixelGatherLoader<ROWS, DG> l;
  l.src = src;
  l.g = g;
  l.CP = CP;
  l.src_ch = src_ch;
  l.src_h = src_h;
  l.src_w = src_w;
  l.cols = cols;
  l.bytes = bytes_of(size_t(g.N) * src_ch * src_h * src_w);
  l.img_base = l.a = l.b = 0;
  l.col_ok = false;
  l.p_ = l.ch0_ = l.ok_ = 0;
  return l;
}

struct WgradPlan {
  int bm, bn, splits, chunks_per_split;
};

inline WgradPlan plan_wgrad(const sgh_conv_geom *g) {
  WgradPlan p;
  const int CRS = g->C * g->R * g->S;
  p.bm = g->K > 64 ? 128 : 64;
  p.bn = CRS > 64 ? 128 : 64;
  // 64 output channels: a 64 x 256 tile (wavefronts 1 x 4, 64 x 64 each) keeps four MFMAs per
  // operand fetch, which a 64 x 128 tile (32 x 64 per wavefront) cannot
  if (p.bm == 64 && CRS >= 256) p.bn = 256;
  // 576 = 64 channels x 9 taps is exactly three 192-wide tiles (a 128- or 256-wide tile would
  // spend 10 % / 25 % of its MFMAs on padding columns)
  if (p.bm == 64 && CRS % 192 == 0 && CRS % 256 != 0) p.bn = 192;
  if (sgh_env().wgrad_tile >= 0) {
    static const int bm[6] = {128, 64, 128, 64, 64, 64}, bn[6] = {128, 128, 64, 64, 256, 192};
    p.bm = bm[sgh_env().wgrad_tile];
    p.bn = bn[sgh_env().wgrad_tile];
  }
  const long tiles = long((g->K + p.bm - 1) / p.bm) * ((CRS + p.bn - 1) / p.bn);
  const long G = long(g->N) * g->P * g->Q;
  const long chunks = (G + BK - 1) / BK;
  long want = (long(sgh_num_cus()) * 2 + tiles - 1) / tiles;
  long max_splits = chunks / 8;  // at least 8 chunks per split
  if (max_splits < 1) max_splits = 1;
  long s = want < max_splits ? want : max_splits;
  if (s < 1) s = 1;
  if (s > 1024) s = 1024;
  p.chunks_per_split = int((chunks + s - 1) / s);
  p.splits = int((chunks + p.chunks_per_split - 1) / p.chunks_per_split);
  return p;
}

template <int BM, int BN, class LA, class LB, class ST, bool AK, bool BKc, bool ZCLASS = false, int WGM = 2, int PF = 1>
inline int launch_igemm(const LA &la, const LB &lb, const ST &st, int M, int N, int Ktotal, int splits,
                        int chunks_per_split, hipStream_t stream, const char *tag = nullptr, double flops = 0) {
  dim3 grid((M + BM - 1) / BM, (N + BN - 1) / BN, splits);
  if (grid.y > 65535u || grid.z > 65535u) return SGH_EUNSUPPORTED;
  if (tag) sgh_prof_kernel_begin(tag, flops);  // kernel-level record: this launch only
  SGH_LAUNCH_TIMED((k_igemm<BM, BN, LA, LB, ST, AK, BKc, ZCLASS, WGM, PF>), grid, dim3(NT), 0, stream, la, lb, st,
                     Ktotal, chunks_per_split);
  if (tag) sgh_prof_kernel_end(stream);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

// algorithmic FLOPs of one convolution pass: 2 * N * K * P * Q * C * R * S
inline double conv_flops(const sgh_conv_geom *g) {
  return 2.0 * g->N * g->K * g->P * g->Q * g->C * g->R * g->S;
}

// ---- dense GEMM dispatch over the four transpose combinations and two tile sizes -----------
template <int BM, int BN, bool AK, bool BKc>
inline int gemm_tile(int M, int N, int K, float alpha, const float *A, long a_rs, long a_ks, const float *B, long b_rs,
                     long b_ks, float beta, float *C, int ldc, hipStream_t stream) {
  auto la = dense_loader<BM, AK>(A, a_rs, a_ks, M, K);
  auto lb = dense_loader<BN, BKc>(B, b_rs, b_ks, N, K);
  DenseStore st{C, ldc, M, N, alpha, beta};
  const int chunks = (K + BK - 1) / BK;
  return launch_igemm<BM, BN, DenseLoader<BM, AK>, DenseLoader<BN, BKc>, DenseStore, AK, BKc, false, 2, (BM * BN <= 64 * 64 ? 4 : 2)>(
      la, lb, st, M, N, K, 1, chunks, stream);
}

// ---- C = alpha * A * B^T + beta * C with few output tiles and a long reduction (the data gradient of a
// classifier: batch x features, reduced over the classes) ------------------------------------------------
// Both operands have the reduction index contiguous -- the operand shape of v_mfma_f32_32x32x2_f32, whose lane
// (i, h) supplies A[i][h] and B[h][i] -- so the wavefronts feed the matrix instructions straight from global
// memory with 16-byte loads: lane (i, h) takes the reduction indices 8 j + 4 h + (0..3) of row i of each
// operand, which the four instructions of group j consume as the pairs (8 j + u, 8 j + 4 + u).  A workgroup
// owns a 32 x 32 tile of C; its four wavefronts each take a quarter of the reduction and the four partial
// tiles are added in wavefront order through LDS, so results are run-to-run identical.  The tiled kernel
// runs such a problem on 16 workgroups that walk the whole reduction one 16-index chunk at a time
// (128 x 512 x 1000: 33.8 us).
extern "C++" {
__global__ __launch_bounds__(256) void k_gemm_kk(const float *__restrict__ A, long lda, const float *__restrict__ B,
                                                 long ldb, float *__restrict__ C, long ldc, int M, int N, int K, int kq,
                                                 float alpha, float beta) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef float f32x16 __attribute__((ext_vector_type(16)));
  __shared__ float part[4][32 * 32];
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63, i = lane & 31, h = lane >> 5;
  const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
  const int kb = wave * kq, ke = kb + kq < K ? kb + kq : K;   // (kq is a multiple of 8)
  const bool am = m0 + i < M, bn = n0 + i < N;
  const float *ap = A + size_t(am ? m0 + i : 0) * lda + 4 * h;
  const float *bp = B + size_t(bn ? n0 + i : 0) * ldb + 4 * h;
  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  constexpr int U = 4;   // groups of eight reduction indices requested before the first is used
  int k = kb;
  for (; k + 8 * U <= ke; k += 8 * U) {
    f32x4 a[U], b[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      a[u] = *reinterpret_cast<const f32x4 *>(ap + k + 8 * u);
      b[u] = *reinterpret_cast<const f32x4 *>(bp + k + 8 * u);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (!am) a[u] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (!bn) b[u] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][e], b[u][e], acc, 0, 0, 0);
    }
  }
  for (; k < ke; k += 8) {   // the last groups, element by element
    f32x4 a = {0.f, 0.f, 0.f, 0.f}, b = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (k + 4 * h + e < ke) {
        if (am) a[e] = ap[k + e];
        if (bn) b[e] = bp[k + e];
      }
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0);
  }
  // lane (i, h) holds column i, rows 8 (v / 4) + 4 h + v % 4
#pragma unroll
  for (int v = 0; v < 16; ++v) part[wave][(8 * (v >> 2) + 4 * h + (v & 3)) * 32 + i] = acc[v];
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int e = t + 256 * r, row = e >> 5, col = e & 31;
    const float v = ((part[0][e] + part[1][e]) + part[2][e]) + part[3][e];
    if (m0 + row < M && n0 + col < N) {
      float *p = C + size_t(m0 + row) * ldc + n0 + col;
      *p = beta == 0.f ? alpha * v : alpha * v + beta * *p;
    }
  }
}
}  // extern "C++"

// (used when the 64 x 64 tiles of the tiled kernel would leave more than half of the CUs without a workgroup)
inline bool gemm_kk_ok(int M, int N, int K, const float *A, long lda, const float *B, long ldb) {
  const long tiles64 = long((M + 63) / 64) * ((N + 63) / 64);
  return K >= 256 && tiles64 * 2 <= sgh_num_cus() && lda % 4 == 0 && ldb % 4 == 0 && sgh_aligned16(A) && sgh_aligned16(B) &&
         (N + 31) / 32 <= 65535 && (M + 31) / 32 <= 65535;
}

template <bool AK, bool BKc>
inline int gemm_pick(int M, int N, int K, float alpha, const float *A, long a_rs, long a_ks, const float *B, long b_rs,
                     long b_ks, float beta, float *C, int ldc, hipStream_t stream) {
  const long tiles128 = long((M + 127) / 128) * ((N + 127) / 128);
  if (M > 64 && N > 64 && tiles128 >= sgh_num_cus())
    return gemm_tile<128, 128, AK, BKc>(M, N, K, alpha, A, a_rs, a_ks, B, b_rs, b_ks, beta, C, ldc, stream);
  return gemm_tile<64, 64, AK, BKc>(M, N, K, alpha, A, a_rs, a_ks, B, b_rs, b_ks, beta, C, ldc, stream);
}

// Tile choice for an M x N problem launched `z` times: 0 = 128x128, 1 = 64x128, 2 = 128x64,
// 3 = 64x64.  The largest tile that still yields at least two workgroups per CU wins; a small
// problem takes the smallest tile.  An environment variable (value 0..3) overrides the choice,
// the counterpart of the reference's CUDNN_CONV_ALG switch
// (reference: src/model/operation/convolution.cc:453-457).
inline int pick_tile(int forced, int M, int N, int z) {
  if (forced >= 0) return forced;
  static const int bm[4] = {128, 64, 128, 64}, bn[4] = {128, 128, 64, 64};
  const long want = 2L * sgh_num_cus();
  for (int i = 0; i < 4; ++i) {
    if (bm[i] == 128 && M <= 64) continue;
    if (bn[i] == 128 && N <= 64) continue;
    const long blocks = long((M + bm[i] - 1) / bm[i]) * ((N + bn[i] - 1) / bn[i]) * z;
    if (blocks >= want) return i;
  }
  return (M <= 64) ? (N <= 64 ? 3 : 1) : 3;
}

// Which algorithm a dgrad of this geometry uses.
enum DgradPath { kDgradFewC, kDgradPointwise, kDgradColumns, kDgradTile3x3, kDgradClasses, kDgradGather };

inline DgradPath dgrad_path(const sgh_conv_geom *g) {
  const size_t RS = size_t(g->R) * g->S;
  // at most four input channels, stride 2, large filter (the stem): direct 16-row MFMA kernel
  if (sgh_dgrad_fewc_supported(g)) return kDgradFewC;
  // 1x1 without padding: a plain GEMM over the output pixels whose store dilates by the stride
  if (RS == 1 && g->pad_h == 0 && g->pad_w == 0 && g->C >= 32 && !sgh_env().dgrad_pointwise_off)
    return kDgradPointwise;
  // few input channels: the C x pixels output tile would waste most of a 64-row MFMA tile, so run
  // the dense GEMM dcol = W^T * dy (CRS rows) and fold the columns back with a gather
  if (g->C < 32 && RS * g->C * size_t(g->N) * g->P * g->Q * sizeof(float) < kMaxOperandBytes) return kDgradColumns;
  if (sgh_dgrad3x3_supported(g)) return kDgradTile3x3;
  if (g->stride_h * g->stride_w <= kMaxClasses && RS <= size_t(kMaxTaps)) return kDgradClasses;
  return kDgradGather;
}

inline size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

// A 3x3 stride-1 pad-1 forward convolution is the data gradient of the channel-swapped problem
// with the filter taps reversed; `gt` receives that problem when the shared-tile kernel covers it.
inline bool fwd_as_dgrad(const sgh_conv_geom *g, sgh_conv_geom *gt) {
  if (g->R != 3 || g->S != 3 || g->stride_h != 1 || g->stride_w != 1 || g->pad_h != 1 || g->pad_w != 1) return false;
  if (g->C % BK != 0) return false;  // the reduction (input channels) runs in whole chunks
  *gt = *g;
  gt->C = g->K;
  gt->K = g->C;
  return sgh_dgrad3x3_supported(gt);
}

}  // namespace

// ---- grouped convolution (cudnnSetConvolutionGroupCount in the reference, src/model/operation/convolution.cc
// :486-490): group i convolves input channels [i C/G, (i+1) C/G) with filters [i K/G, (i+1) K/G) of the
// [K, C/G, R, S] weight tensor.  Each group runs as a dense convolution of its own: its channel slices are
// gathered into dense tensors in the workspace (strided device-to-device copies, one row per image), the
// ordinary entry point runs on the sub-geometry, and the result is scattered back; a group's weight gradient
// is a dense block of dW and needs no copy.  Workspace: [x slice | y slice | workspace of the sub-geometry].
namespace {

struct GroupPlan {
  sgh_conv_geom sg;          // one group's geometry
  size_t xe, ye, we;         // elements of a group's x / y slice per image, and of its weights
  size_t x_bytes, y_bytes;   // the gathered slices
};

GroupPlan group_plan(const sgh_conv_geom *g, size_t elem) {
  GroupPlan p{};
  p.sg = *g;
  p.sg.C = g->C / g->groups, p.sg.K = g->K / g->groups, p.sg.groups = 1;
  sgh_prelaid_clear(&p.sg);
  p.xe = size_t(p.sg.C) * g->H * g->W, p.ye = size_t(p.sg.K) * g->P * g->Q;
  p.we = size_t(p.sg.K) * p.sg.C * g->R * g->S;
  p.x_bytes = align256(p.xe * g->N * elem), p.y_bytes = align256(p.ye * g->N * elem);
  return p;
}

// `sub(sg, which, a, b, bias, out, workspace, ws_bytes)` runs one dense pass; T is the element type.
template <typename T, typename Sub>
int conv_grouped(const sgh_conv_geom *g, int which, const T *a, const T *b, const T *bias, T *out, void *workspace,
                 size_t ws_bytes, size_t sub_ws, hipStream_t s, Sub sub) {
  if (!conv_ok(g) || !a || !b || !out) return SGH_EINVAL;
  GroupPlan p = group_plan(g, sizeof(T));
  if (!workspace || ws_bytes < p.x_bytes + p.y_bytes + sub_ws) return SGH_EWORKSPACE;
  char *w = static_cast<char *>(workspace);
  T *xg = reinterpret_cast<T *>(w), *yg = reinterpret_cast<T *>(w + p.x_bytes);
  void *inner = w + p.x_bytes + p.y_bytes;
  const size_t xfull = size_t(g->C) * g->H * g->W, yfull = size_t(g->K) * g->P * g->Q;
  auto gather = [&](T *dst, const T *src, size_t per, size_t full, int gi) {
    return hipMemcpy2DAsync(dst, per * sizeof(T), src + gi * per, full * sizeof(T), per * sizeof(T), size_t(g->N),
                            hipMemcpyDeviceToDevice, s);
  };
  auto scatter = [&](T *dst, const T *src, size_t per, size_t full, int gi) {
    return hipMemcpy2DAsync(dst + gi * per, full * sizeof(T), src, per * sizeof(T), per * sizeof(T), size_t(g->N),
                            hipMemcpyDeviceToDevice, s);
  };
  for (int gi = 0; gi < g->groups; ++gi) {
    int rc;
    if (which == SGH_CONV_FWD) {           // a = x, b = W, out = y
      SGH_HIP_TRY(gather(xg, a, p.xe, xfull, gi));
      rc = sub(&p.sg, which, xg, b + gi * p.we, bias ? bias + gi * p.sg.K : nullptr, yg, inner, sub_ws);
      if (rc == SGH_OK) SGH_HIP_TRY(scatter(out, yg, p.ye, yfull, gi));
    } else if (which == SGH_CONV_DGRAD) {  // a = dy, b = W, out = dx
      SGH_HIP_TRY(gather(yg, a, p.ye, yfull, gi));
      rc = sub(&p.sg, which, yg, b + gi * p.we, nullptr, xg, inner, sub_ws);
      if (rc == SGH_OK) SGH_HIP_TRY(scatter(out, xg, p.xe, xfull, gi));
    } else {                               // a = dy, b = x, out = dW
      SGH_HIP_TRY(gather(yg, a, p.ye, yfull, gi));
      SGH_HIP_TRY(gather(xg, b, p.xe, xfull, gi));
      rc = sub(&p.sg, which, yg, xg, nullptr, out + gi * p.we, inner, sub_ws);
    }
    if (rc != SGH_OK) return rc;
  }
  return SGH_OK;
}

}  // namespace

extern "C" {

int sgh_conv_geom_init(sgh_conv_geom *g, int N, int C, int H, int W, int K, int R, int S, int stride_h, int stride_w,
                       int pad_h, int pad_w) {
  if (!g) return SGH_EINVAL;
  if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || K <= 0 || R <= 0 || S <= 0 || stride_h <= 0 || stride_w <= 0 ||
      pad_h < 0 || pad_w < 0)
    return SGH_EINVAL;
  if (H + 2 * pad_h < R || W + 2 * pad_w < S) return SGH_EINVAL;
  g->N = N;
  g->C = C;
  g->H = H;
  g->W = W;
  g->K = K;
  g->R = R;
  g->S = S;
  g->stride_h = stride_h;
  g->stride_w = stride_w;
  g->pad_h = pad_h;
  g->pad_w = pad_w;
  // ConvHandle's integer division (reference: src/model/operation/convolution.cc:56-59)
  g->P = (H + 2 * pad_h - R) / stride_h + 1;
  g->Q = (W + 2 * pad_w - S) / stride_w + 1;
  g->groups = 1;
  sgh_prelaid_clear(g);
  return conv_ok(g) ? SGH_OK : SGH_EINVAL;
}

int sgh_conv_geom_init_grouped(sgh_conv_geom *g, int N, int C, int H, int W, int K, int R, int S, int stride_h,
                               int stride_w, int pad_h, int pad_w, int groups) {
  if (groups < 1 || C <= 0 || K <= 0 || C % groups != 0 || K % groups != 0) return SGH_EINVAL;
  const int rc = sgh_conv_geom_init(g, N, C, H, W, K, R, S, stride_h, stride_w, pad_h, pad_w);
  if (rc != SGH_OK) return rc;
  g->groups = groups;
  return SGH_OK;
}

namespace {

int conv_dense_f32(sgh_conv_geom *sg, int which, const float *a, const float *b, const float *bias, float *out,
                   void *ws, size_t ws_bytes, void *stream) {
  if (which == SGH_CONV_FWD) return sgh_conv_fwd_f32(sg, a, b, bias, out, ws, ws_bytes, stream);
  if (which == SGH_CONV_DGRAD) return sgh_conv_dgrad_f32(sg, a, b, out, ws, ws_bytes, stream);
  return sgh_conv_wgrad_f32(sg, a, b, out, ws, ws_bytes, stream);
}

int conv_grouped_f32(const sgh_conv_geom *g, int which, const float *a, const float *b, const float *bias, float *out,
                     void *workspace, size_t ws_bytes, void *stream) {
  GroupPlan p = group_plan(g, sizeof(float));
  const size_t sub_ws = sgh_conv_workspace_bytes(&p.sg, which);
  return conv_grouped<float>(g, which, a, b, bias, out, workspace, ws_bytes, sub_ws, sgh_stream_of(stream),
                             [&](sgh_conv_geom *sg, int wh, const float *a_, const float *b_, const float *bias_,
                                 float *out_, void *ws, size_t wsb) {
                               return conv_dense_f32(sg, wh, a_, b_, bias_, out_, ws, wsb, stream);
                             });
}

}  // namespace

size_t sgh_conv_workspace_bytes(const sgh_conv_geom *g, int which) {
  if (!conv_ok(g)) return 0;
  if (g->groups > 1) {
    if (which < 0 || which > 2) return 0;
    const GroupPlan p = group_plan(g, sizeof(float));
    return p.x_bytes + p.y_bytes + sgh_conv_workspace_bytes(&p.sg, which);
  }
  const size_t RS = size_t(g->R) * g->S;
  switch (which) {
    case SGH_CONV_FWD: {
      sgh_conv_geom gt;
      const size_t wt = RS * round_up(g->C, BK) * g->K * sizeof(float);
      const size_t need = fwd_as_dgrad(g, &gt) ? align256(wt) + sgh_dgrad3x3_partial_bytes(&gt) : wt;
      return need > sgh_fwd_fewc_workspace_bytes(g) ? need : sgh_fwd_fewc_workspace_bytes(g);
    }
    case SGH_CONV_DGRAD:
      if (dgrad_path(g) == kDgradFewC) return sgh_dgrad_fewc_workspace_bytes(g);
      if (dgrad_path(g) == kDgradPointwise) return 0;
      if (dgrad_path(g) == kDgradColumns) return RS * g->C * size_t(g->N) * g->P * g->Q * sizeof(float);
      return align256(RS * round_up(g->K, BK) * g->C * sizeof(float)) + align256(sizeof(DgClsTable)) +
             sgh_dgrad3x3_partial_bytes(g);
    case SGH_CONV_WGRAD: {
      const size_t tiled = sgh_wgrad3x3_workspace_bytes(g);
      if (tiled) return tiled;
      const size_t fewc = sgh_wgrad_fewc_workspace_bytes(g);
      if (fewc) return fewc;
      const size_t pw = sgh_env().pw_wgrad_off ? 0 : sgh_pw_wgrad_workspace_bytes(g);
      if (pw) return pw;
      const WgradPlan p = plan_wgrad(g);
      // split partials of dW, then those of the bias gradient that may ride along (sgh_conv_wgrad_bias_f32)
      return p.splits > 1 ? align256(size_t(p.splits) * g->K * g->C * RS * sizeof(float)) + size_t(p.splits) * g->K * sizeof(float) : 0;
    }
    default: return 0;
  }
}

// `prelaid`: the workspace already holds this layer's re-laid weights (sgh_conv_dgrad_prepare_multi)
static int conv_dgrad(const sgh_conv_geom *g, const float *dy, const float *W, float *dx, void *workspace,
                      size_t ws_bytes, void *stream, bool accumulate, bool prelaid) {
  if (!conv_ok(g) || !dy || !W || !dx) return SGH_EINVAL;
  const size_t need = sgh_conv_workspace_bytes(g, SGH_CONV_DGRAD);
  if (need && (!workspace || ws_bytes < need)) return SGH_EWORKSPACE;
  hipStream_t s = sgh_stream_of(stream);
  const int RS = g->R * g->S, KP = round_up(g->K, BK);
  const DgradPath path = dgrad_path(g);
  if (accumulate && path != kDgradTile3x3) return SGH_EUNSUPPORTED;  // only the shared-tile kernels add into dx
  int rc = SGH_OK;
  sgh_prof_start("conv_dgrad_op", conv_flops(g), s);

  if (path == kDgradFewC) {
    rc = sgh_dgrad_fewc_run(g, dy, W, dx, workspace, ws_bytes, s);
  } else if (path == kDgradPointwise && sgh_pw_dgrad_supported(g) && !sgh_env().pw_dgrad_off) {
    rc = sgh_pw_dgrad_run(g, dy, W, dx, s);
  } else if (path == kDgradPointwise) {
    // dx block (img, m, p, q) = sum_k W[k][m] * dy[img][k][p][q]: A(m, k) = W[k * C + m] in its native layout
    const int Ncols = g->N * g->P * g->Q;
    ConvG fake{g->N, g->K, g->P, g->Q, g->K, 1, 1, 1, 1, 0, 0, g->P, g->Q};
    DilateStore st{dx, g->C, g->H, g->W, g->P, g->Q, g->stride_h, g->stride_w, Ncols};
    const int chunks = (g->K + BK - 1) / BK;
    const long tiles128 = long((g->C + 127) / 128) * ((Ncols + 127) / 128);
    // (this GEMM has a short reduction and a large store: it wants many workgroups in flight, so the
    // larger tiles are only taken when they still give two workgroups per CU)
    const long need = long(sgh_num_cus()) * 2;
    if (g->C > 64 && tiles128 >= need) {
      auto la = dense_loader<128, false>(W, 1, g->C, g->C, g->K);
      auto lb = gather_loader<128, false>(dy, fake, KP, g->K, g->P, g->Q, Ncols);
      rc = launch_igemm<128, 128, DenseLoader<128, false>, PixelGatherLoader<128, false>, DilateStore, false, false, false, 2, 2>(
          la, lb, st, g->C, Ncols, g->K, 1, chunks, s, "conv_dgrad/k_igemm", conv_flops(g));
    } else if (long((g->C + 63) / 64) * ((Ncols + 127) / 128) >= need) {
      auto la = dense_loader<64, false>(W, 1, g->C, g->C, g->K);
      auto lb = gather_loader<128, false>(dy, fake, KP, g->K, g->P, g->Q, Ncols);
      rc = launch_igemm<64, 128, DenseLoader<64, false>, PixelGatherLoader<128, false>, DilateStore, false, false, false, 2, 4>(
          la, lb, st, g->C, Ncols, g->K, 1, chunks, s, "conv_dgrad/k_igemm", conv_flops(g));
    } else {
      auto la = dense_loader<64, false>(W, 1, g->C, g->C, g->K);
      auto lb = gather_loader<64, false>(dy, fake, KP, g->K, g->P, g->Q, Ncols);
      rc = launch_igemm<64, 64, DenseLoader<64, false>, PixelGatherLoader<64, false>, DilateStore, false, false, false, 2, 4>(
          la, lb, st, g->C, Ncols, g->K, 1, chunks, s, "conv_dgrad/k_igemm", conv_flops(g));
    }
  } else if (path == kDgradColumns) {
    float *dcol = static_cast<float *>(workspace);
    const int CRS = g->C * RS, Ncols = g->N * g->P * g->Q;
    auto la = dense_loader<64, false>(W, 1, CRS, CRS, g->K);
    ConvG fake{g->N, g->K, g->P, g->Q, g->K, 1, 1, 1, 1, 0, 0, g->P, g->Q};
    auto lb = gather_loader<128, false>(dy, fake, KP, g->K, g->P, g->Q, Ncols);
    DenseStore st{dcol, long(Ncols), CRS, Ncols, 1.f, 0.f};
    rc = launch_igemm<64, 128, DenseLoader<64, false>, PixelGatherLoader<128, false>, DenseStore, false, false>(
        la, lb, st, CRS, Ncols, g->K, 1, (g->K + BK - 1) / BK, s, "conv_dgrad/k_igemm", conv_flops(g));
    if (rc == SGH_OK) {
      const long total = long(g->N) * g->C * g->H * (long((g->W + g->stride_w - 1) / g->stride_w) * g->stride_w);
      long blocks = (total + NT - 1) / NT;
      const long cap = long(sgh_num_cus()) * 32;
      if (blocks > cap) blocks = cap;
      hipLaunchKernelGGL(k_col2im_gather, dim3(int(blocks)), dim3(NT), 0, s, dcol, dx, to_g(g), total);
    }
  } else if (path == kDgradTile3x3) {
    float *Wt = static_cast<float *>(workspace);
    const long total = long(RS) * KP * g->C;
    long blocks = (total + NT - 1) / NT;
    if (blocks > 4096) blocks = 4096;
    if (!prelaid)
      hipLaunchKernelGGL(k_weight_relayout, dim3(int(blocks)), dim3(NT), 0, s, W, Wt, g->K, g->C, RS, KP, 1);
    float *partials = reinterpret_cast<float *>(static_cast<char *>(workspace) +
                                                align256(size_t(RS) * KP * g->C * sizeof(float)) +
                                                align256(sizeof(DgClsTable)));
    rc = sgh_dgrad3x3_run(g, dy, Wt, KP, dx, partials, s, "conv_dgrad/k_dgrad3x3", nullptr, accumulate);
  } else if (path == kDgradClasses) {
    float *Wc = static_cast<float *>(workspace);
    const size_t wc_bytes = size_t(RS) * KP * g->C * sizeof(float);
    DgCls *tab_dev = reinterpret_cast<DgCls *>(static_cast<char *>(workspace) + align256(wc_bytes));
    DgClsTable tab;
    TapTable taps;
    int ncls = 0, tap_off = 0, max_cols = 0;
    for (int ch = 0; ch < g->stride_h; ++ch)
      for (int cw = 0; cw < g->stride_w; ++cw) {
        DgCls &c = tab.c[ncls++];
        const int r0 = (ch + g->pad_h) % g->stride_h, s0 = (cw + g->pad_w) % g->stride_w;
        c.ch = short(ch);
        c.cw = short(cw);
        c.r0 = short(r0);
        c.s0 = short(s0);
        c.nr = short(r0 < g->R ? (g->R - r0 + g->stride_h - 1) / g->stride_h : 0);
        c.ns = short(s0 < g->S ? (g->S - s0 + g->stride_w - 1) / g->stride_w : 0);
        if (c.nr == 0 || c.ns == 0) c.nr = c.ns = 0;
        c.bh = short((ch + g->pad_h - r0) / g->stride_h);
        c.bw = short((cw + g->pad_w - s0) / g->stride_w);
        c.Hc = ch < g->H ? (g->H - ch + g->stride_h - 1) / g->stride_h : 0;
        c.Wc = cw < g->W ? (g->W - cw + g->stride_w - 1) / g->stride_w : 0;
        c.tap_off = tap_off;
        for (int i = 0; i < c.nr; ++i)
          for (int j = 0; j < c.ns; ++j)
            taps.rs[tap_off + i * c.ns + j] = short((r0 + i * g->stride_h) * g->S + (s0 + j * g->stride_w));
        tap_off += c.nr * c.ns;
        const int cols = g->N * c.Hc * c.Wc;
        if (cols > max_cols) max_cols = cols;
      }
    for (int i = tap_off; i < kMaxTaps; ++i) taps.rs[i] = 0;
    for (int i = ncls; i < kMaxClasses; ++i) tab.c[i] = tab.c[0];
    {
      const long total = long(tap_off) * KP * g->C;
      long blocks = (total + NT - 1) / NT;
      if (blocks > 4096) blocks = 4096;
      if (blocks < 1) blocks = 1;  // the class table is written even when no tap survives
      hipLaunchKernelGGL(k_weight_relayout_classes, dim3(int(blocks)), dim3(NT), 0, s, W, Wc, g->K, g->C, RS, KP, taps,
                         tab, tab_dev);
    }
    const int M = g->C;
    DgradStore st{dx, to_g(g), tab_dev};
    const int tile = pick_tile(sgh_env().dgrad_tile, M, max_cols, ncls);
#define SGH_DGRAD_CASE(BM_, BN_)                                                                              \
  {                                                                                                           \
    DgradWLoader<BM_> la{Wc, g->C, KP, tab_dev, unsigned(wc_bytes), 0, 0, 0, 0};                              \
    DgradDyLoader<BN_> lb;                                                                                    \
    lb.dy = dy;                                                                                               \
    lb.g = to_g(g);                                                                                           \
    lb.KP = KP;                                                                                               \
    lb.tab = tab_dev;                                                                                         \
    lb.bytes = bytes_of(size_t(g->N) * g->K * g->P * g->Q);                                                   \
    rc = launch_igemm<BM_, BN_, DgradWLoader<BM_>, DgradDyLoader<BN_>, DgradStore, false, false, true>(       \
        la, lb, st, M, max_cols, 0, ncls, 0, s, "conv_dgrad/k_igemm", conv_flops(g));                                 \
  }
    if (tile == 0) SGH_DGRAD_CASE(128, 128)
    else if (tile == 1) SGH_DGRAD_CASE(64, 128)
    else if (tile == 2) SGH_DGRAD_CASE(128, 64)
    else SGH_DGRAD_CASE(64, 64)
#undef SGH_DGRAD_CASE
  } else {
    float *Wt = static_cast<float *>(workspace);
    const long total = long(RS) * KP * g->C;
    long blocks = (total + NT - 1) / NT;
    if (blocks > 4096) blocks = 4096;
    if (!prelaid)
      hipLaunchKernelGGL(k_weight_relayout, dim3(int(blocks)), dim3(NT), 0, s, W, Wt, g->K, g->C, RS, KP, 1);
    const int M = g->C, Ncols = g->N * g->H * g->W, Ktot = RS * KP;
    NchwStore st{dx, nullptr, g->C, g->H * g->W, Ncols};
    auto la = dense_loader<128, false>(Wt, 1, g->C, M, Ktot);
    auto lb = gather_loader<128, true>(dy, to_g(g), KP, g->K, g->P, g->Q, Ncols);
    rc = launch_igemm<128, 128, DenseLoader<128, false>, PixelGatherLoader<128, true>, NchwStore, false, false>(
        la, lb, st, M, Ncols, Ktot, 1, Ktot / BK, s, "conv_dgrad/k_igemm", conv_flops(g));
  }
  sgh_prof_stop(s);
  if (rc != SGH_OK) return rc;
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

// The note of a prepare call is read once: whether it held or not, this pass leaves none behind.
static bool take_prelaid(sgh_conv_geom *g, int dtype, const void *W, const void *workspace) {
  if (!g) return false;
  const bool ok = sgh_prelaid_valid(g, dtype, W, workspace);
  sgh_prelaid_clear(g);
  return ok;
}

int sgh_conv_dgrad_f32(sgh_conv_geom *g, const float *dy, const float *W, float *dx, void *workspace,
                       size_t ws_bytes, void *stream) {
  if (g && conv_ok(g) && g->groups > 1)
    return conv_grouped_f32(g, SGH_CONV_DGRAD, dy, W, nullptr, dx, workspace, ws_bytes, stream);
  const bool prelaid = take_prelaid(g, 0, W, workspace);
  return conv_dgrad(g, dy, W, dx, workspace, ws_bytes, stream, false, prelaid);
}

void sgh_conv_weights_changed(void) { sgh_weights_epoch_bump(); }

// ---- all data-gradient weight re-layouts of a backward pass in one launch ----------------------
namespace {

constexpr int kMaxRelayouts = 56;   // per launch: the table travels as a kernel argument

struct RelayoutTable {
  int count;
  int block0[kMaxRelayouts + 1];   // first workgroup of each item, then the total
  struct Item {
    const void *W;
    void *Wt;
    int K, C, RS, A, B;   // destination [tap][A][B]: fp32 A = KP (k), B = C;  16-bit A = CP (c), B = KP (k)
  } it[kMaxRelayouts];
};

constexpr int kRelayoutPerBlock = NT * 8, kRelayoutTile = 32, kRelayoutMaxTaps = 9;

// One 32 (k) x 32 (c) x RS tile of a re-layout through LDS: the source rows W[k][c0 .. c0+31][taps] are
// contiguous runs, the destination rows [tap][.][32 contiguous] are too.
extern "C++" {
template <class T>
__device__ __forceinline__ void relayout_tile(const T *__restrict__ W, T *__restrict__ Wt, int K, int C, int RS, int A,
                                              int B, bool k_fastest, int tile) {
  __shared__ T lds[kRelayoutTile][kRelayoutTile * kRelayoutMaxTaps + 1];
  // destination [tap][A][B]; k_fastest: (A, B) = (c, k), else (k, c)
  const int kdim = k_fastest ? B : A, cdim = k_fastest ? A : B;
  const int ctiles = (cdim + kRelayoutTile - 1) / kRelayoutTile;
  const int k0 = (tile / ctiles) * kRelayoutTile, c0 = (tile % ctiles) * kRelayoutTile;
  const int run = kRelayoutTile * RS, t = threadIdx.x;
  const int cvalid = C - c0 < kRelayoutTile ? C - c0 : kRelayoutTile, rlen = cvalid > 0 ? cvalid * RS : 0;
  // (source rows are contiguous runs; eight loads in flight per thread -- with one, a launch over the 11 M weights
  // of ResNet-18 took 38 us, the time of its 36 loads per thread one after the other)
  constexpr int U = 8;
  for (int i0 = t; i0 < kRelayoutTile * run; i0 += NT * U) {
    T v[U];
    int kk[U], r[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * NT;
      kk[u] = i / run, r[u] = i - kk[u] * run;
      const int k = k0 + kk[u];
      v[u] = (kk[u] < kRelayoutTile && k < K && r[u] < rlen) ? W[(long(k) * C + c0) * RS + r[u]] : T(0);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (kk[u] < kRelayoutTile) lds[kk[u]][r[u]] = v[u];
  }
  __syncthreads();
  const int f = t & 31;   // position along the destination's contiguous dimension
  for (int o = t >> 5; o < kRelayoutTile * RS; o += NT / 32) {
    const int tap = o / kRelayoutTile, s_ = o - tap * kRelayoutTile;   // s_: position along the other tile dimension
    const int kk = k_fastest ? f : s_, cc = k_fastest ? s_ : f;
    const int k = k0 + kk, c = c0 + cc;
    if (k < kdim && c < cdim) {
      const long dst = k_fastest ? (long(tap) * A + c) * B + k : (long(tap) * A + k) * B + c;
      Wt[dst] = lds[kk][cc * RS + tap];
    }
  }
}
}  // extern "C++"

extern "C++" {
// T = float: destination [tap][KP][C]; T = uint16_t: destination [tap][CP][KP] (see RelayoutTable)
template <class T>
__global__ __launch_bounds__(NT) void k_weight_relayout_multi(const RelayoutTable t) {
  constexpr bool k_fastest = sizeof(T) == 2;
  int lo = 0, hi = t.count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (int(blockIdx.x) >= t.block0[mid]) lo = mid;
    else hi = mid - 1;
  }
  const int K = t.it[lo].K, C = t.it[lo].C, RS = t.it[lo].RS, A = t.it[lo].A, B = t.it[lo].B;
  const int blk = int(blockIdx.x) - t.block0[lo];
  const T *W = static_cast<const T *>(t.it[lo].W);
  T *Wt = static_cast<T *>(t.it[lo].Wt);
  if (RS <= kRelayoutMaxTaps) {
    relayout_tile<T>(W, Wt, K, C, RS, A, B, k_fastest, blk);
    return;
  }
  // large filters: element by element
  const long total = long(RS) * A * B;
  const long base = long(blk) * kRelayoutPerBlock + threadIdx.x;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const long i = base + u * NT;
    if (i < total) {
      const int f = int(i % B), s_ = int((i / B) % A), tap = int(i / (long(A) * B));
      const int k = k_fastest ? f : s_, c = k_fastest ? s_ : f;
      Wt[i] = (k < K && c < C) ? W[(long(k) * C + c) * RS + tap] : T(0);
    }
  }
}
}  // extern "C++"

}  // namespace

int sgh_conv_dgrad_prepare_multi(const sgh_conv_prepare_item *items, int count, int dtype, void *stream) {
  if (count < 0 || (count > 0 && !items) || dtype < 0 || dtype > 2) return SGH_EINVAL;
  hipStream_t s = sgh_stream_of(stream);
  RelayoutTable t;
  t.count = 0, t.block0[0] = 0;
  sgh_conv_geom *batch[kMaxRelayouts];
  size_t batch_bytes[kMaxRelayouts];
  auto flush = [&]() -> int {
    if (t.count == 0) return SGH_OK;
    if (dtype == 0) hipLaunchKernelGGL(k_weight_relayout_multi<float>, dim3(unsigned(t.block0[t.count])), dim3(NT), 0, s, t);
    else hipLaunchKernelGGL(k_weight_relayout_multi<uint16_t>, dim3(unsigned(t.block0[t.count])), dim3(NT), 0, s, t);
    if (hipGetLastError() != hipSuccess) return SGH_EINVAL;
    for (int i = 0; i < t.count; ++i) {
      sgh_conv_geom *g = batch[i];
      g->prelaid_dtype = dtype, g->prelaid_W = t.it[i].W, g->prelaid_ws = t.it[i].Wt;
      g->prelaid_ws_bytes = batch_bytes[i], g->prelaid_epoch = sgh_weights_epoch();
      sgh_prepared_weights_add(t.it[i].W, size_t(g->K) * g->C * g->R * g->S * (dtype == 0 ? 4 : 2));
    }
    t.count = 0;
    return SGH_OK;
  };
  for (int i = 0; i < count; ++i) {
    sgh_conv_geom *g = items[i].g;
    if (!g || !conv_ok(g) || !items[i].W) return SGH_EINVAL;
    sgh_prelaid_clear(g);
    if (g->groups > 1) continue;   // (a grouped layer re-lays each group's weights when its data gradient runs)
    RelayoutTable::Item it{};
    it.W = items[i].W, it.Wt = items[i].workspace, it.K = g->K, it.C = g->C, it.RS = g->R * g->S;
    size_t need;
    if (dtype == 0) {
      const DgradPath path = dgrad_path(g);
      if (path != kDgradTile3x3 && path != kDgradGather) continue;   // the other kernels read W as it is or re-lay it their own way
      it.A = round_up(g->K, BK), it.B = g->C;
      need = sgh_conv_workspace_bytes(g, SGH_CONV_DGRAD);
    } else {
      if (sgh_env().conv16_off || !sgh_conv16_dgrad_relayout_dims(g, &it.A, &it.B)) continue;
      need = sgh_conv16_workspace_bytes(g, SGH_CONV_DGRAD);
    }
    if (!items[i].workspace || items[i].ws_bytes < need) return SGH_EWORKSPACE;
    const long total = long(it.RS) * it.A * it.B;
    const long blocks = it.RS <= kRelayoutMaxTaps
                            ? long((it.A + kRelayoutTile - 1) / kRelayoutTile) * ((it.B + kRelayoutTile - 1) / kRelayoutTile)
                            : (total + kRelayoutPerBlock - 1) / kRelayoutPerBlock;
    if (t.count == kMaxRelayouts || long(t.block0[t.count]) + blocks >= (long(1) << 30)) {
      const int rc = flush();
      if (rc != SGH_OK) return rc;
    }
    t.it[t.count] = it;
    batch[t.count] = g;
    batch_bytes[t.count] = items[i].ws_bytes;
    t.block0[t.count + 1] = t.block0[t.count] + int(blocks);
    ++t.count;
  }
  return flush();
}

int sgh_conv_dgrad_acc_supported(const sgh_conv_geom *g) {
  return g && conv_ok(g) && g->groups == 1 && dgrad_path(g) == kDgradTile3x3 ? 1 : 0;
}

int sgh_conv_dgrad_acc_f32(sgh_conv_geom *g, const float *dy, const float *W, float *dx, void *workspace,
                           size_t ws_bytes, void *stream) {
  if (g && conv_ok(g) && !sgh_conv_dgrad_acc_supported(g)) return SGH_EUNSUPPORTED;   // (the note stays for the fallback call)
  const bool prelaid = take_prelaid(g, 0, W, workspace);
  return conv_dgrad(g, dy, W, dx, workspace, ws_bytes, stream, true, prelaid);
}

int sgh_conv_fwd_f32(sgh_conv_geom *g, const float *x, const float *W, const float *bias, float *y,
                     void *workspace, size_t ws_bytes, void *stream) {
  if (!conv_ok(g) || !x || !W || !y) return SGH_EINVAL;
  if (g->groups > 1) return conv_grouped_f32(g, SGH_CONV_FWD, x, W, bias, y, workspace, ws_bytes, stream);
  sgh_prelaid_clear_if_overlap(g, workspace, ws_bytes);
  const size_t need = sgh_conv_workspace_bytes(g, SGH_CONV_FWD);
  if (!workspace || ws_bytes < need) return SGH_EWORKSPACE;
  hipStream_t s = sgh_stream_of(stream);
  float *Wt = static_cast<float *>(workspace);
  const int RS = g->R * g->S, CP = round_up(g->C, BK);
  sgh_prof_start("conv_fwd_op", conv_flops(g), s);
  if (!sgh_env().fwd_fewc_off) {   // the stem
    const int rcf = sgh_fwd_fewc_run(g, x, W, bias, y, workspace, ws_bytes, s);
    if (rcf != SGH_EUNSUPPORTED) {
      sgh_prof_stop(s);
      return rcf;
    }
  }
  sgh_conv_geom gt;
  if (fwd_as_dgrad(g, &gt)) {
    // 3x3 stride 1 pad 1: the shared-tile kernel on the channel-swapped problem with reversed taps
    const long total = long(RS) * CP * g->K;
    long blocks = (total + NT - 1) / NT;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(k_weight_relayout, dim3(int(blocks)), dim3(NT), 0, s, W, Wt, g->K, g->C, RS, CP, 2);
    float *partials = reinterpret_cast<float *>(static_cast<char *>(workspace) +
                                                align256(size_t(RS) * CP * g->K * sizeof(float)));
    const int rc3 = sgh_dgrad3x3_run(&gt, x, Wt, CP, y, partials, s, "conv_fwd/k_dgrad3x3", bias, false);
    sgh_prof_stop(s);
    return rc3;
  }
  {
    const long total = long(RS) * CP * g->K;
    long blocks = (total + NT - 1) / NT;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(k_weight_relayout, dim3(int(blocks)), dim3(NT), 0, s, W, Wt, g->K, g->C, RS, CP, 0);
  }
  const int M = g->K, Ncols = g->N * g->P * g->Q, Ktot = RS * CP;
  const int chunks = Ktot / BK;
  NchwStore st{y, bias, g->K, g->P * g->Q, Ncols};
  int rc;
  // the largest tile that still gives every CU a workgroup (the late, small layers: 98 tiles of 128 x 128 at
  // 512 filters on 7 x 7 planes, N = 64)
  const long cus = sgh_num_cus();
  const long t128 = long((M + 127) / 128) * ((Ncols + 127) / 128), t64x128 = long((M + 63) / 64) * ((Ncols + 127) / 128);
  if (M > 64 && t128 >= cus) {
    auto la = dense_loader<128, false>(Wt, 1, g->K, M, Ktot);
    auto lb = gather_loader<128, false>(x, to_g(g), CP, g->C, g->H, g->W, Ncols);
    rc = launch_igemm<128, 128, DenseLoader<128, false>, PixelGatherLoader<128, false>, NchwStore, false, false>(
        la, lb, st, M, Ncols, Ktot, 1, chunks, s, "conv_fwd/k_igemm", conv_flops(g));
  } else if (M <= 64 || t64x128 >= cus) {
    auto la = dense_loader<64, false>(Wt, 1, g->K, M, Ktot);
    auto lb = gather_loader<128, false>(x, to_g(g), CP, g->C, g->H, g->W, Ncols);
    rc = launch_igemm<64, 128, DenseLoader<64, false>, PixelGatherLoader<128, false>, NchwStore, false, false>(
        la, lb, st, M, Ncols, Ktot, 1, chunks, s, "conv_fwd/k_igemm", conv_flops(g));
  } else {
    auto la = dense_loader<64, false>(Wt, 1, g->K, M, Ktot);
    auto lb = gather_loader<64, false>(x, to_g(g), CP, g->C, g->H, g->W, Ncols);
    rc = launch_igemm<64, 64, DenseLoader<64, false>, PixelGatherLoader<64, false>, NchwStore, false, false, false, 2, 4>(
        la, lb, st, M, Ncols, Ktot, 1, chunks, s, "conv_fwd/k_igemm", conv_flops(g));
  }
  sgh_prof_stop(s);
  if (rc != SGH_OK) return rc;
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

static int bgrad_launch(const sgh_conv_geom *g, const float *dy, float *db, hipStream_t s) {
  hipLaunchKernelGGL(k_conv_bgrad<StF32>, dim3(g->K), dim3(NT), 0, s, dy, db, g->N, g->K, g->P * g->Q);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

// `db` (may be null): the bias gradient as well.  In the generic kernel it rides along as one more column
// of the x operand (a column of ones) whenever the last column tile has a spare column; the shared-tile
// and few-channel kernels are followed by the reduction kernel of sgh_conv_bgrad_f32.
static int conv_wgrad(sgh_conv_geom *g, const float *dy, const float *x, float *dW, float *db, void *workspace,
                      size_t ws_bytes, void *stream) {
  if (!conv_ok(g) || !dy || !x || !dW) return SGH_EINVAL;
  if (g->groups > 1) {   // (the bias gradient does not depend on the grouping)
    const int rc = conv_grouped_f32(g, SGH_CONV_WGRAD, dy, x, nullptr, dW, workspace, ws_bytes, stream);
    return rc == SGH_OK && db ? bgrad_launch(g, dy, db, sgh_stream_of(stream)) : rc;
  }
  sgh_prelaid_clear_if_overlap(g, workspace, ws_bytes);
  if (sgh_wgrad3x3_workspace_bytes(g)) {  // 3x3, stride 1 or 2: shared-input-tile kernel
    sgh_prof_start("conv_wgrad_op", conv_flops(g), sgh_stream_of(stream));
    const int rc3 = sgh_wgrad3x3_run(g, dy, x, dW, workspace, ws_bytes, sgh_stream_of(stream));
    sgh_prof_stop(sgh_stream_of(stream));
    return rc3 == SGH_OK && db ? bgrad_launch(g, dy, db, sgh_stream_of(stream)) : rc3;
  }
  if (sgh_wgrad_fewc_workspace_bytes(g)) {  // few input channels, large filter (the stem)
    sgh_prof_start("conv_wgrad_op", conv_flops(g), sgh_stream_of(stream));
    const int rcf = sgh_wgrad_fewc_run(g, dy, x, dW, workspace, ws_bytes, sgh_stream_of(stream));
    sgh_prof_stop(sgh_stream_of(stream));
    return rcf == SGH_OK && db ? bgrad_launch(g, dy, db, sgh_stream_of(stream)) : rcf;
  }
  if (!sgh_env().pw_wgrad_off && sgh_pw_wgrad_workspace_bytes(g)) {  // 1x1 strided (the downsample layers)
    sgh_prof_start("conv_wgrad_op", conv_flops(g), sgh_stream_of(stream));
    const int rcp = sgh_pw_wgrad_run(g, dy, x, dW, workspace, ws_bytes, sgh_stream_of(stream));
    sgh_prof_stop(sgh_stream_of(stream));
    return rcp == SGH_OK && db ? bgrad_launch(g, dy, db, sgh_stream_of(stream)) : rcp;
  }
  const WgradPlan p = plan_wgrad(g);
  const size_t need = sgh_conv_workspace_bytes(g, SGH_CONV_WGRAD);
  if (need && (!workspace || ws_bytes < need)) return SGH_EWORKSPACE;
  hipStream_t s = sgh_stream_of(stream);
  const int CRS = g->C * g->R * g->S, PQ = g->P * g->Q;
  const long G = long(g->N) * PQ;
  float *part = p.splits > 1 ? static_cast<float *>(workspace) : dW;
  const bool ride = db && CRS % p.bn != 0;   // a spare column in the last column tile
  float *bpart = !ride ? nullptr
                 : p.splits > 1 ? reinterpret_cast<float *>(static_cast<char *>(workspace) +
                                                            align256(size_t(p.splits) * g->K * CRS * sizeof(float)))
                                : db;
  SplitStore st{part, g->K, CRS, bpart};
  int rc;
  sgh_prof_start("conv_wgrad_op", conv_flops(g), s);
#define SGH_WGRAD_CASE(BM_, BN_, WGM_, PF_)                                                                          \
  {                                                                                                                \
    WgradDyLoader<BM_> la{dy, g->K, PQ, int(G), bytes_of(size_t(G) * g->K), 0, 0, 0};                              \
    WgradXLoader<BN_> lb;                                                                                          \
    lb.x = x;                                                                                                      \
    lb.g = to_g(g);                                                                                                \
    lb.CRS = CRS;                                                                                                  \
    lb.ones_col = ride ? CRS : -1;                                                                                 \
    lb.bytes = bytes_of(size_t(g->N) * g->C * g->H * g->W);                                                        \
    rc = launch_igemm<BM_, BN_, WgradDyLoader<BM_>, WgradXLoader<BN_>, SplitStore, true, true, false, WGM_, PF_>(  \
        la, lb, st, g->K, CRS, int(G), p.splits, p.chunks_per_split, s, "conv_wgrad/k_igemm", conv_flops(g));              \
  }
  // (chunks in flight: see k_igemm; the smaller the tile, the fewer MFMA cycles a chunk holds)
  if (p.bm == 128 && p.bn == 128) SGH_WGRAD_CASE(128, 128, 2, 2)
  else if (p.bm == 64 && p.bn == 256) SGH_WGRAD_CASE(64, 256, 1, 2)
  else if (p.bm == 64 && p.bn == 192) SGH_WGRAD_CASE(64, 192, 2, 2)
  else if (p.bm == 64 && p.bn == 128) SGH_WGRAD_CASE(64, 128, 2, 3)
  else if (p.bm == 128 && p.bn == 64) SGH_WGRAD_CASE(128, 64, 2, 3)
  else SGH_WGRAD_CASE(64, 64, 2, 4)
#undef SGH_WGRAD_CASE
  if (rc == SGH_OK && p.splits > 1) {
    const long n = long(g->K) * CRS;
    if (p.splits >= 32 && n <= long(sgh_num_cus()) * 16 * 64) {
      hipLaunchKernelGGL(k_split_reduce_lanes, dim3(int((n + 15) / 16)), dim3(256), 0, s, part, dW, n, p.splits);
    } else {
      long blocks = (n + NT - 1) / NT;
      if (blocks > 2048) blocks = 2048;
      hipLaunchKernelGGL(k_split_reduce, dim3(int(blocks)), dim3(NT), 0, s, part, dW, n, p.splits);
    }
    if (ride) hipLaunchKernelGGL(k_split_reduce, dim3((g->K + NT - 1) / NT), dim3(NT), 0, s, bpart, db, long(g->K), p.splits);
  }
  sgh_prof_stop(s);
  if (rc != SGH_OK) return rc;
  SGH_LAUNCH_CHECK();
  return db && !ride ? bgrad_launch(g, dy, db, s) : SGH_OK;
}

int sgh_conv_wgrad_f32(sgh_conv_geom *g, const float *dy, const float *x, float *dW, void *workspace,
                       size_t ws_bytes, void *stream) {
  return conv_wgrad(g, dy, x, dW, nullptr, workspace, ws_bytes, stream);
}

int sgh_conv_wgrad_bias_f32(sgh_conv_geom *g, const float *dy, const float *x, float *dW, float *db, void *workspace,
                            size_t ws_bytes, void *stream) {
  if (!db) return SGH_EINVAL;
  return conv_wgrad(g, dy, x, dW, db, workspace, ws_bytes, stream);
}


int sgh_conv_bgrad_f32(const sgh_conv_geom *g, const float *dy, float *db, void *stream) {
  if (!conv_ok(g) || !dy || !db) return SGH_EINVAL;
  hipLaunchKernelGGL(k_conv_bgrad<StF32>, dim3(g->K), dim3(NT), 0, sgh_stream_of(stream), dy, db, g->N, g->K,
                     g->P * g->Q);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_gemm_f32(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda, const float *B,
                 int ldb, float beta, float *C, int ldc, void *stream) {
  if (M < 0 || N < 0 || K < 0) return SGH_EINVAL;
  if (M == 0 || N == 0) return SGH_OK;
  if (!C || ldc < N) return SGH_EINVAL;
  if (K > 0 && (!A || !B)) return SGH_EINVAL;
  if (K > 0 && (lda < (transA ? M : K) || ldb < (transB ? K : N))) return SGH_EINVAL;
  // operands are addressed with 32-bit byte offsets
  const size_t a_ext = size_t(transA ? K : M) * lda, b_ext = size_t(transB ? N : K) * ldb;
  if (a_ext * sizeof(float) >= kMaxOperandBytes || b_ext * sizeof(float) >= kMaxOperandBytes) return SGH_EUNSUPPORTED;
  hipStream_t s = sgh_stream_of(stream);
  // element(row, k) strides of each operand
  const long a_rs = transA ? 1 : lda, a_ks = transA ? lda : 1;  // A(m, k)
  const long b_rs = transB ? ldb : 1, b_ks = transB ? 1 : ldb;  // B(k, n) addressed as (n, k)
  int rc;
  sgh_prof_start("gemm", 2.0 * M * N * K, s);
  if (!transA && transB && gemm_kk_ok(M, N, K, A, lda, B, ldb)) {
    const int kq = ((K + 3) / 4 + 7) / 8 * 8;
    hipLaunchKernelGGL(k_gemm_kk, dim3(unsigned((N + 31) / 32), unsigned((M + 31) / 32)), dim3(256), 0, s, A, long(lda), B,
                       long(ldb), C, long(ldc), M, N, K, kq, alpha, beta);
    rc = hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
  } else if (!transA && transB) rc = gemm_pick<true, true>(M, N, K, alpha, A, a_rs, a_ks, B, b_rs, b_ks, beta, C, ldc, s);
  else if (!transA && !transB) rc = gemm_pick<true, false>(M, N, K, alpha, A, a_rs, a_ks, B, b_rs, b_ks, beta, C, ldc, s);
  else if (transA && transB) rc = gemm_pick<false, true>(M, N, K, alpha, A, a_rs, a_ks, B, b_rs, b_ks, beta, C, ldc, s);
  else rc = gemm_pick<false, false>(M, N, K, alpha, A, a_rs, a_ks, B, b_rs, b_ks, beta, C, ldc, s);
  sgh_prof_stop(s);
  return rc;
}


// ---- 16-bit storage (binary16 / bfloat16) --------------------------------------------------
// The tensors are converted to fp32 in the workspace, the fp32 kernels above do the arithmetic
// (fp32 MFMA, fp32 accumulation) and the result is rounded once on the way out.  The workspace
// holds the three fp32 copies followed by the fp32 pass's own workspace.
namespace {

struct HalfPlan {
  size_t a_elems, b_elems, out_elems, inner;  // the two inputs, the output, the fp32 pass's workspace
  size_t total() const { return align256(a_elems * 4) + align256(b_elems * 4) + align256(out_elems * 4) + inner; }
};

inline HalfPlan half_plan(const sgh_conv_geom *g, int which) {
  const size_t x = size_t(g->N) * g->C * g->H * g->W, y = size_t(g->N) * g->K * g->P * g->Q;
  const size_t w = size_t(g->K) * g->C * g->R * g->S;
  HalfPlan p{};
  p.inner = sgh_conv_workspace_bytes(g, which);
  if (which == SGH_CONV_DGRAD) p.a_elems = y, p.b_elems = w, p.out_elems = x;
  else if (which == SGH_CONV_WGRAD) p.a_elems = y, p.b_elems = x, p.out_elems = w;
  else p.a_elems = x, p.b_elems = w, p.out_elems = y;
  return p;
}

typedef int (*cast_in_fn)(const uint16_t *, float *, size_t, void *);
typedef int (*cast_out_fn)(const float *, uint16_t *, size_t, void *);

// which: SGH_CONV_*; (a, b) are the pass's two tensor inputs in the order of its fp32 entry point
int conv_half(sgh_conv_geom *g, int which, const uint16_t *a, const uint16_t *b, const uint16_t *bias,
              uint16_t *out, void *workspace, size_t ws_bytes, void *stream, cast_in_fn in, cast_out_fn outc) {
  if (!conv_ok(g) || !a || !b || !out) return SGH_EINVAL;
  if (g->groups > 1) {
    GroupPlan p = group_plan(g, sizeof(uint16_t));
    const size_t sub_ws = sgh_conv_workspace_bytes_h(&p.sg, which);
    return conv_grouped<uint16_t>(g, which, a, b, bias, out, workspace, ws_bytes, sub_ws, sgh_stream_of(stream),
                                  [&](sgh_conv_geom *sg, int wh, const uint16_t *a_, const uint16_t *b_,
                                      const uint16_t *bias_, uint16_t *out_, void *ws, size_t wsb) {
                                    return conv_half(sg, wh, a_, b_, bias_, out_, ws, wsb, stream, in, outc);
                                  });
  }
  bool prelaid = false;
  if (which == SGH_CONV_DGRAD) prelaid = take_prelaid(g, in == sgh_cast_bf16_to_f32 ? 2 : 1, b, workspace);
  else sgh_prelaid_clear_if_overlap(g, workspace, ws_bytes);
  // the gradients and the forward pass (strides 1 and 2) run on the 16-bit matrix instructions where
  // conv16.hip covers the geometry; everything else computes in fp32 on widened copies
  if (which == SGH_CONV_FWD && !sgh_env().conv16_off && !sgh_env().fwd_fewc_off) {   // the stem
    const int rc = sgh_fwd_fewc16_run(g, a, b, bias, out, workspace, ws_bytes, in == sgh_cast_bf16_to_f32,
                                      sgh_stream_of(stream));
    if (rc != SGH_EUNSUPPORTED) return rc;
  }
  if (sgh_conv16_workspace_bytes(g, which) != 0 && !sgh_env().conv16_off) {
    const bool bf16 = in == sgh_cast_bf16_to_f32;
    hipStream_t s = sgh_stream_of(stream);
    const int rc = which == SGH_CONV_DGRAD   ? sgh_conv16_dgrad(g, a, b, out, workspace, ws_bytes, bf16, s, prelaid)
                   : which == SGH_CONV_WGRAD ? sgh_conv16_wgrad(g, a, b, out, workspace, ws_bytes, bf16, s)
                                             : sgh_conv16_fwd(g, a, b, bias, out, workspace, ws_bytes, bf16, s);
    if (rc != SGH_EUNSUPPORTED) return rc;
  }
  // the stem's data gradient (few input channels, large filter): the fp32 kernel reads the 16-bit
  // gradient and writes the 16-bit result itself; only the small weight tensor is widened
  if (which == SGH_CONV_DGRAD && sgh_dgrad_fewc_supported(g) && !sgh_env().conv16_off) {
    const size_t w_elems = size_t(g->K) * g->C * g->R * g->S, w_bytes = align256(w_elems * 4);
    if (!workspace || ws_bytes < w_bytes + sgh_dgrad_fewc_workspace_bytes(g)) return SGH_EWORKSPACE;
    float *w32 = static_cast<float *>(workspace);
    int rc = in(b, w32, w_elems, stream);
    if (rc != SGH_OK) return rc;
    rc = sgh_dgrad_fewc_run16(g, a, w32, out, static_cast<char *>(workspace) + w_bytes, ws_bytes - w_bytes,
                              in == sgh_cast_bf16_to_f32, sgh_stream_of(stream));
    if (rc != SGH_EUNSUPPORTED) return rc;
  }
  const HalfPlan p = half_plan(g, which);
  if (!workspace || ws_bytes < p.total() + (bias ? align256(size_t(g->K) * 4) : 0)) return SGH_EWORKSPACE;
  char *w = static_cast<char *>(workspace);
  float *a32 = reinterpret_cast<float *>(w);
  float *b32 = reinterpret_cast<float *>(w + align256(p.a_elems * 4));
  float *o32 = reinterpret_cast<float *>(w + align256(p.a_elems * 4) + align256(p.b_elems * 4));
  char *inner = w + align256(p.a_elems * 4) + align256(p.b_elems * 4) + align256(p.out_elems * 4);
  float *bias32 = nullptr;
  int rc = in(a, a32, p.a_elems, stream);
  if (rc == SGH_OK) rc = in(b, b32, p.b_elems, stream);
  if (rc == SGH_OK && bias) {
    bias32 = reinterpret_cast<float *>(inner + p.inner);
    rc = in(bias, bias32, size_t(g->K), stream);
  }
  if (rc != SGH_OK) return rc;
  if (which == SGH_CONV_DGRAD) rc = sgh_conv_dgrad_f32(g, a32, b32, o32, inner, p.inner, stream);
  else if (which == SGH_CONV_WGRAD) rc = sgh_conv_wgrad_f32(g, a32, b32, o32, inner, p.inner, stream);
  else rc = sgh_conv_fwd_f32(g, a32, b32, bias32, o32, inner, p.inner, stream);
  if (rc != SGH_OK) return rc;
  return outc(o32, out, p.out_elems, stream);
}

}  // namespace

int sgh_conv_bgrad_f16(const sgh_conv_geom *g, const uint16_t *dy, uint16_t *db, void *stream) {
  if (!conv_ok(g) || !dy || !db) return SGH_EINVAL;
  hipLaunchKernelGGL(k_conv_bgrad<StF16>, dim3(g->K), dim3(NT), 0, sgh_stream_of(stream), dy, db, g->N, g->K,
                     g->P * g->Q);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}
int sgh_conv_bgrad_bf16(const sgh_conv_geom *g, const uint16_t *dy, uint16_t *db, void *stream) {
  if (!conv_ok(g) || !dy || !db) return SGH_EINVAL;
  hipLaunchKernelGGL(k_conv_bgrad<StBF16>, dim3(g->K), dim3(NT), 0, sgh_stream_of(stream), dy, db, g->N, g->K,
                     g->P * g->Q);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

size_t sgh_conv_workspace_bytes_h(const sgh_conv_geom *g, int which) {
  if (!conv_ok(g) || which < 0 || which > 2) return 0;
  if (g->groups > 1) {
    const GroupPlan p = group_plan(g, sizeof(uint16_t));
    return p.x_bytes + p.y_bytes + sgh_conv_workspace_bytes_h(&p.sg, which);
  }
  const size_t wide = half_plan(g, which).total() + (which == SGH_CONV_FWD ? align256(size_t(g->K) * 4) : 0);
  size_t native = sgh_conv16_workspace_bytes(g, which);
  if (which == SGH_CONV_FWD && sgh_fwd_fewc16_workspace_bytes(g) > native) native = sgh_fwd_fewc16_workspace_bytes(g);
  return wide > native ? wide : native;
}

int sgh_conv_dgrad_f16(sgh_conv_geom *g, const uint16_t *dy, const uint16_t *W, uint16_t *dx, void *workspace,
                       size_t ws_bytes, void *stream) {
  return conv_half(g, SGH_CONV_DGRAD, dy, W, nullptr, dx, workspace, ws_bytes, stream, sgh_cast_f16_to_f32,
                   sgh_cast_f32_to_f16);
}
int sgh_conv_dgrad_bf16(sgh_conv_geom *g, const uint16_t *dy, const uint16_t *W, uint16_t *dx, void *workspace,
                        size_t ws_bytes, void *stream) {
  return conv_half(g, SGH_CONV_DGRAD, dy, W, nullptr, dx, workspace, ws_bytes, stream, sgh_cast_bf16_to_f32,
                   sgh_cast_f32_to_bf16);
}
int sgh_conv_wgrad_f16(sgh_conv_geom *g, const uint16_t *dy, const uint16_t *x, uint16_t *dW, void *workspace,
                       size_t ws_bytes, void *stream) {
  return conv_half(g, SGH_CONV_WGRAD, dy, x, nullptr, dW, workspace, ws_bytes, stream, sgh_cast_f16_to_f32,
                   sgh_cast_f32_to_f16);
}
int sgh_conv_wgrad_bf16(sgh_conv_geom *g, const uint16_t *dy, const uint16_t *x, uint16_t *dW, void *workspace,
                        size_t ws_bytes, void *stream) {
  return conv_half(g, SGH_CONV_WGRAD, dy, x, nullptr, dW, workspace, ws_bytes, stream, sgh_cast_bf16_to_f32,
                   sgh_cast_f32_to_bf16);
}
int sgh_conv_fwd_f16(sgh_conv_geom *g, const uint16_t *x, const uint16_t *W, const uint16_t *bias, uint16_t *y,
                     void *workspace, size_t ws_bytes, void *stream) {
  return conv_half(g, SGH_CONV_FWD, x, W, bias, y, workspace, ws_bytes, stream, sgh_cast_f16_to_f32,
                   sgh_cast_f32_to_f16);
}
int sgh_conv_fwd_bf16(sgh_conv_geom *g, const uint16_t *x, const uint16_t *W, const uint16_t *bias, uint16_t *y,
                      void *workspace, size_t ws_bytes, void *stream) {
  return conv_half(g, SGH_CONV_FWD, x, W, bias, y, workspace, ws_bytes, stream, sgh_cast_bf16_to_f32,
                   sgh_cast_f32_to_bf16);
}

}  // extern "C"
