// Convolution gradients on 16-bit tensors (IEEE binary16 / bfloat16, NCHW) with the 16-bit matrix
// instructions of gfx950: v_mfma_f32_32x32x16_{f16,bf16}, fp32 accumulation, one rounding at the
// store.  Reference entry points: ConvBackwardx / ConvBackwardW, src/model/operation/convolution.cc
// :634-681 (cuDNN with half tensors); formulas as in igemm.hip.
//
// Both MFMA operands hold, per lane, EIGHT CONSECUTIVE reduction indices of one tile row (lane l:
// row l % 32, indices 8 * (l / 32) .. + 7), so both LDS tiles are kept as [row][reduction] with the
// reduction index contiguous (pitch 64 + 8 halves: ds_read_b128, conflict-free).  Which eight
// indices share an octet is irrelevant as long as both operands agree, which is what makes NCHW
// usable without a layout change:
//
//   weight gradient  dW[k][(c,r,s)] = sum_{n,p,q} dy[n,k,p,q] * x[n,c,p*st-pad+r,q*st-pad+s]
//     The reduction runs over pixels, contiguous in memory for both operands.  An octet is 8
//     consecutive q of one output row (the last octet of a row is partly empty: at most 12.5 % of
//     the MFMA work for Q = 7, 14, 28, none for 56 and 112); 1x1 stride-1 layers are passed in with
//     the image plane as one row.  dy octets are 16-byte loads; an x octet is the 16 (stride 2: 32)
//     bytes at the tap's offset, loaded unaligned and masked at the image border.
//   data gradient    dx[c][(n,h,w)]  = sum_{r,s,k} W[k,c,r,s] * dy[n,k,(h+pad-r)/st,(w+pad-s)/st]
//     The reduction runs over k, strided in memory, while pixels are contiguous: a thread loads one
//     dword (two neighbouring pixels) for each of 8 consecutive k and transposes them into two
//     octets with v_perm_b32 (the selector also encodes which of the two pixels exist for the
//     tap, so border handling costs nothing extra).  Weights are re-laid as [tap][C][K] in 16 bits.
//     Stride 2 is handled by residue class: output pixels (2i+a, 2j+b) of one class form their own
//     pixel space with a stride-1 gradient window, and only the taps of that class are visited.
//
// 512 threads = two groups of 2 x 2 wavefronts on a workgroup tile of 128 (or 64) x 128; both groups
// tile the same outputs and take the first / second half of every 64-wide reduction chunk's MFMA
// steps, their accumulators are added through LDS at the end.  With two workgroups per CU that
// puts four wavefronts on every SIMD, so one wavefront's staging arithmetic and memory waits
// overlap the others' matrix work.  LDS and register double buffering.
#include <hip/hip_runtime.h>

#include <atomic>
#include <type_traits>

#include "common.h"
#include "storage.h"

namespace {

constexpr int NT = 512, BN = 128, KC = 64, PITCH = KC + 8;  // PITCH in 16-bit elements
constexpr int kOOB = int(0x80000000u);

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

__device__ __forceinline__ rsrc_t make_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, int(bytes), 0x00020000);
}

template <bool BF16>
__device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0,
                                                   0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                  0);
}

template <bool BF16>
__device__ __forceinline__ uint16_t round16(float v) {
  return BF16 ? sgh_f32_to_bf16(v) : sgh_f32_to_f16(v);
}

// keeps elements j in [lo, hi) of an octet, zeroes the others
__device__ __forceinline__ u32x4 mask_range(u32x4 v, int lo, int hi) {
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const unsigned m = ((2 * d >= lo && 2 * d < hi) ? 0xffffu : 0u) | ((2 * d + 1 >= lo && 2 * d + 1 < hi) ? 0xffff0000u : 0u);
    v[d] &= m;
  }
  return v;
}

// element-wise guarded load of elements j in [lo, hi) at p[off + j * STEP]
template <int STEP>
__device__ __forceinline__ u32x4 load_elems(const uint16_t *p, long off, int lo, int hi) {
  u32x4 v = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int j = 0; j < 8; ++j)
    if (j >= lo && j < hi) v[j >> 1] |= unsigned(p[off + long(j) * STEP]) << (16 * (j & 1));
  return v;
}

__device__ __forceinline__ u32x4 load16b(const uint16_t *p) {  // 16 bytes at any 2-byte alignment
  u32x4 v;
  __builtin_memcpy(&v, p, 16);
  return v;
}

// One wavefront group's half (two of the four MFMA steps) of a reduction chunk, on a wavefront's
// (TM*32) x 64 tile.  `koff` = element offset of the half within the chunk (0 or 32) + 8 * (lane / 32).
// acc[.][j] belongs to the 32-column block at B row brow + j * bstep: group 0 numbers its two blocks
// 0, 1 and group 1 numbers them 1, 0, so that for both groups acc[.][0] is the block the group keeps
// and acc[.][1] the one it hands over when the groups' sums are combined.
template <int TM, bool BF16>
__device__ __forceinline__ void mma_chunk(const uint16_t *As, const uint16_t *Bs, int arow, int brow, int bstep,
                                          int koff, f32x16 (&acc)[TM][2]) {
#pragma unroll
  for (int j = 0; j < KC / 32; ++j) {
    u32x4 av[TM], bv[2];
#pragma unroll
    for (int i = 0; i < TM; ++i) av[i] = *reinterpret_cast<const u32x4 *>(As + (arow + i * 32) * PITCH + koff + 16 * j);
#pragma unroll
    for (int i = 0; i < 2; ++i) bv[i] = *reinterpret_cast<const u32x4 *>(Bs + (brow + i * bstep) * PITCH + koff + 16 * j);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int jn = 0; jn < 2; ++jn) acc[i][jn] = mfma<BF16>(av[i], bv[jn], acc[i][jn]);
  }
}

// Sums the two wavefront groups' accumulators through LDS (after the last chunk; the tile buffers
// are free then).  Every wavefront hands over acc[.][1] and adds what its partner hands over to
// acc[.][0] (see mma_chunk for the numbering), so afterwards acc[.][0] is complete in both groups and
// both take part in the store.
template <int TM>
__device__ __forceinline__ void combine_halves(float *lds, int half, int w4, int lane, f32x16 (&acc)[TM][2]) {
  __syncthreads();
  float *send = lds + ((half * 4 + w4) * (TM * 16)) * 64 + lane;
  const float *recv = lds + (((half ^ 1) * 4 + w4) * (TM * 16)) * 64 + lane;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) send[(i * 16 + v) * 64] = acc[i][1][v];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][0][v] += recv[(i * 16 + v) * 64];
}

// ------------------------------------------------------------------------------------------------
// weight gradient
// ------------------------------------------------------------------------------------------------
struct W16Args {
  const uint16_t *dy, *x;
  float *partial;  // [splits][K][CRS]
  int N, C, H, W, K, P, Q, R, S, pad_h, pad_w;
  int QO;          // octets per output row: ceil(Q / 8)
  int CRS, mtiles, tiles, splits;
  int chunks, chunks_per_split;  // a chunk = 8 octets = 8 units (n, p, octet)
  long dy_elems, x_elems;
};

template <int BM, int STRIDE, bool BF16>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_wgrad16(W16Args a) {
  extern __shared__ __align__(16) uint16_t lds16[];
  constexpr int TM = BM / 64, ASLOTS = BM * 8 / NT, BSLOTS = BN * 8 / NT;
  uint16_t *const As0 = lds16, *const Bs0 = lds16 + BM * PITCH;
  uint16_t *const As1 = lds16 + (BM + BN) * PITCH, *const Bs1 = As1 + BM * PITCH;
  // octet masks by valid element range: lut[lo * 9 + hi] keeps elements lo <= j < hi (branch-free
  // border handling: one LDS read and four ANDs per octet)
  u32x4 *const lut = reinterpret_cast<u32x4 *>(lds16 + 2 * (BM + BN) * PITCH);
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int half = wave >> 2, w4 = wave & 3, wm = w4 >> 1, wn = w4 & 1;
  const int l32 = lane & 31, lh = lane >> 5;
  // Workgroup w runs on XCD w % 8 (each XCD has its own L2).  All tiles of one split of the
  // reduction read the same dy rows, so a split's tiles are given to one XCD: split = 8 * (slot /
  // tiles) + w % 8 with slot = w / 8.
  // (only when the split count is a multiple of 8: otherwise some XCDs would get more splits than
  // others, and the tiles are dealt round-robin instead)
  int tile, split;
  if ((a.splits & 7) == 0) {
    const int slot = int(blockIdx.x) >> 3;
    tile = slot % a.tiles;
    split = (slot / a.tiles) * 8 + (int(blockIdx.x) & 7);
  } else {
    tile = int(blockIdx.x) % a.tiles;
    split = int(blockIdx.x) / a.tiles;
  }
  if (split >= a.splits) return;
  if (t < 81) lut[t] = mask_range(u32x4{~0u, ~0u, ~0u, ~0u}, t / 9, t % 9);
  __syncthreads();
  const int m0 = (tile % a.mtiles) * BM, n0 = (tile / a.mtiles) * BN;
  const int c_begin = split * a.chunks_per_split;
  const int c_end = min(a.chunks, c_begin + a.chunks_per_split);
  const int oct = t & 7, rb = t >> 3;
  const int PQ = a.P * a.Q, HW = a.H * a.W, RS = a.R * a.S;

  // this thread's unit (n, p, qo) in the current chunk, and the step of 8 units to the next chunk
  const int PQO = a.P * a.QO;
  int n, p, qo;
  {
    const long unit = long(c_begin) * 8 + oct;
    n = int(unit / PQO);
    const int rem = int(unit - long(n) * PQO);
    p = rem / a.QO;
    qo = rem - p * a.QO;
  }
  const int dn = 8 / PQO, dp = (8 - dn * PQO) / a.QO, dq = 8 - dn * PQO - dp * a.QO;
  auto advance = [&]() {
    qo += dq;
    if (qo >= a.QO) qo -= a.QO, ++p;
    p += dp;
    if (p >= a.P) p -= a.P, ++n;
    n += dn;
  };

  // Loads are issued for the next chunk before the MFMA steps of the current one and only
  // touched (masked, compacted) when they are written to LDS afterwards, so their latency hides
  // behind the matrix work.  Offsets are bytes into buffer descriptors; kOOB reads as zero.
  const rsrc_t rdy = make_rsrc(a.dy, unsigned(a.dy_elems * 2)), rx = make_rsrc(a.x, unsigned(a.x_elems * 2));
  int aoff[ASLOTS];
#pragma unroll
  for (int i = 0; i < ASLOTS; ++i) {
    const int k = m0 + rb + 64 * i;
    aoff[i] = k < a.K && rb + 64 * i < BM ? k * PQ : -1;
  }
  int boff[BSLOTS], br[BSLOTS], bs[BSLOTS];
#pragma unroll
  for (int i = 0; i < BSLOTS; ++i) {
    const int col = n0 + rb + 64 * i;
    const int c = col / RS, tap = col - c * RS, r = tap / a.S;
    br[i] = r - a.pad_h;
    bs[i] = tap - r * a.S - a.pad_w;
    boff[i] = c * HW + br[i] * a.W + bs[i];
    if (col >= a.CRS) br[i] = -(1 << 28);  // (a row that is never inside the image)
  }

  struct Stage {                   // one chunk in flight
    u32x4 ra[ASLOTS], rbv[BSLOTS][STRIDE];
    int a_nv;                      // valid elements of the dy octet
    int b_lohi[BSLOTS];            // lo * 9 + hi for the valid element range [lo, hi) of each x octet
  };
  auto load = [&](Stage &g, auto tails) {
    const int nv = min(8, a.Q - 8 * qo);
    const bool unit_ok = n < a.N;
    g.a_nv = nv;
    const int abase = n * a.K * PQ + p * a.Q + 8 * qo;
    bool any_tail = false;
#pragma unroll
    for (int i = 0; i < ASLOTS; ++i) {
      const int off = abase + aoff[i];
      const bool ok = unit_ok && aoff[i] >= 0;
      const bool tail = ok && off + 8 > int(a.dy_elems);  // the 16 bytes would cross the end of the tensor
      any_tail |= tail;
      g.ra[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rdy, ok && !tail ? off * 2 : kOOB, 0, 0));
    }
    const int xbase = n * a.C * HW + p * STRIDE * a.W + 8 * STRIDE * qo;
#pragma unroll
    for (int i = 0; i < BSLOTS; ++i) {
      const int h = p * STRIDE + br[i], col0 = 8 * STRIDE * qo + bs[i];
      const int lo = col0 < 0 ? (-col0 + STRIDE - 1) / STRIDE : 0;
      const int hi = min(nv, (a.W - col0 + STRIDE - 1) / STRIDE);
      const bool ok = unit_ok && unsigned(h) < unsigned(a.H) && hi > lo;
      const int off = xbase + boff[i];
      const bool tail = ok && (off < 0 || off + 8 * STRIDE > int(a.x_elems));
      any_tail |= tail;
      g.b_lohi[i] = ok ? lo * 9 + hi : 0;
      const int voff = ok && !tail ? off * 2 : kOOB;
#pragma unroll
      for (int u = 0; u < STRIDE; ++u)
        g.rbv[i][u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, voff, 16 * u, 0));
    }
    // Octets whose 16 bytes would start before or end after the tensor (its first / last rows only)
    // are fetched element by element, so that no access leaves the tensor.  Rare, and the only
    // place where this function waits for memory.
    if (decltype(tails)::value && any_tail) {
#pragma unroll
      for (int i = 0; i < ASLOTS; ++i) {
        const int off = abase + aoff[i];
        if (unit_ok && aoff[i] >= 0 && off + 8 > int(a.dy_elems)) g.ra[i] = load_elems<1>(a.dy, off, 0, nv);
      }
#pragma unroll
      for (int i = 0; i < BSLOTS; ++i) {
        const int h = p * STRIDE + br[i], col0 = 8 * STRIDE * qo + bs[i];
        const int lo = col0 < 0 ? (-col0 + STRIDE - 1) / STRIDE : 0;
        const int hi = min(nv, (a.W - col0 + STRIDE - 1) / STRIDE);
        const int off = xbase + boff[i];
        if (unit_ok && unsigned(h) < unsigned(a.H) && hi > lo && (off < 0 || off + 8 * STRIDE > int(a.x_elems))) {
          const u32x4 v = load_elems<STRIDE>(a.x, off, lo, hi);  // already compacted and masked
          g.rbv[i][0] = v;
          if (STRIDE == 2) {  // (spread again so that the common compaction below reproduces v)
            g.rbv[i][0] = u32x4{v[0] & 0xffffu, v[0] >> 16, v[1] & 0xffffu, v[1] >> 16};
            g.rbv[i][STRIDE - 1] = u32x4{v[2] & 0xffffu, v[2] >> 16, v[3] & 0xffffu, v[3] >> 16};
          }
          g.b_lohi[i] = 8;
        }
      }
    }
    advance();
  };
  auto stage = [&](const Stage &g, uint16_t *As, uint16_t *Bs) {
    const u32x4 ma = lut[g.a_nv];
#pragma unroll
    for (int i = 0; i < ASLOTS; ++i)
      if (BM >= 128 || rb < BM) *reinterpret_cast<u32x4 *>(As + (rb + 64 * i) * PITCH + oct * 8) = g.ra[i] & ma;
#pragma unroll
    for (int i = 0; i < BSLOTS; ++i) {
      u32x4 v = g.rbv[i][0];
      if (STRIDE == 2) {  // 16 elements loaded, every other one wanted
        const u32x4 v1 = g.rbv[i][STRIDE - 1];
        const u32x4 v0 = v;
        v[0] = __builtin_amdgcn_perm(v0[1], v0[0], 0x05040100u);
        v[1] = __builtin_amdgcn_perm(v0[3], v0[2], 0x05040100u);
        v[2] = __builtin_amdgcn_perm(v1[1], v1[0], 0x05040100u);
        v[3] = __builtin_amdgcn_perm(v1[3], v1[2], 0x05040100u);
      }
      *reinterpret_cast<u32x4 *>(Bs + (rb + 64 * i) * PITCH + oct * 8) = v & lut[g.b_lohi[i]];
    }
  };

  f32x16 acc[TM][2];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int arow = wm * (TM * 32) + l32, brow = wn * 64 + half * 32 + l32, bstep = half ? -32 : 32;
  const int koff = half * 32 + lh * 8;
  // Chunk c is computed from LDS buffer c & 1 while the loads of chunk c + 1 are in flight; they are
  // written to the other buffer after the MFMA steps.
  auto run = [&](auto tails) {
    Stage g;
    load(g, tails);
    stage(g, As0, Bs0);
    __syncthreads();
    for (int c = c_begin; c < c_end; ++c) {
      const bool cur1 = (c - c_begin) & 1, more = c + 1 < c_end;
      if (more) load(g, tails);
      mma_chunk<TM, BF16>(cur1 ? As1 : As0, cur1 ? Bs1 : Bs0, arow, brow, bstep, koff, acc);
      if (more) stage(g, cur1 ? As0 : As1, cur1 ? Bs0 : Bs1);
      __syncthreads();
    }
  };
  // Only the first chunk (x rows before the first image) and the chunks of the last two output
  // rows of the last image can hold an octet that would reach outside a tensor; every other
  // workgroup runs the loop without that code.
  if (c_begin < c_end) {
    if (c_begin == 0 || c_end + (2 * a.QO + 7) / 8 + 1 >= a.chunks) run(std::true_type{});
    else run(std::false_type{});
  }

  combine_halves<TM>(reinterpret_cast<float *>(lds16), half, w4, lane, acc);
  float *out = a.partial + size_t(split) * a.K * a.CRS;
  const int col = n0 + wn * 64 + half * 32 + l32;   // the block this group kept
  if (col < a.CRS) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * (TM * 32) + i * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
        if (row < a.K) out[size_t(row) * a.CRS + col] = acc[i][0][v];
      }
  }
}

// dW = round16(sum over splits).  A workgroup takes EP consecutive elements; its 256 threads form
// ZL = 256 / EP z-lanes: lane zl sums the splits zl, zl + ZL, ... in ascending order and the lane
// sums are added in lane order, so the result depends on the shape only: run-to-run identical.
template <int EP, bool BF16>
__global__ __launch_bounds__(256) void k_wgrad16_reduce(const float *__restrict__ partial, int splits, size_t n,
                                                        uint16_t *__restrict__ dW) {
  constexpr int ZL = 256 / EP;
  __shared__ float lanes[ZL][EP];
  const int e = threadIdx.x % EP, zl = threadIdx.x / EP;
  const size_t i = size_t(blockIdx.x) * EP + e;
  float s = 0.f;
  if (i < n) {
    // (eight loads in flight, added in the same ascending order: one load per addition waited for each in turn)
    constexpr int U = 8;
    int z = zl;
    for (; z + (U - 1) * ZL < splits; z += U * ZL) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = partial[size_t(z + u * ZL) * n + i];
#pragma unroll
      for (int u = 0; u < U; ++u) s += v[u];
    }
    for (; z < splits; z += ZL) s += partial[size_t(z) * n + i];
  }
  lanes[zl][e] = s;
  __syncthreads();
  if (zl == 0 && i < n) {
    float r = lanes[0][e];
#pragma unroll
    for (int l = 1; l < ZL; ++l) r += lanes[l][e];
    dW[i] = round16<BF16>(r);
  }
}

// ------------------------------------------------------------------------------------------------
// data gradient
// ------------------------------------------------------------------------------------------------
struct D16Args {
  const uint16_t *dy, *wt;  // wt: [tap][CP][KP], zero-filled padding
  const uint16_t *dyT;      // pixel-major copy [n][p][q][k] of dy (PIXK kernels), else null
  uint16_t *dx;
  int N, C, H, W, K, P, Q, R, S, stride, pad_h, pad_w;
  int KP, CP, mtiles, ptiles;
  int cls_tile0[5];  // first pixel tile of each residue class (stride^2 classes), then the total
  unsigned dy_bytes, wt_bytes;
  const uint16_t *bias;  // per output row (channel c), or null: the forward pass run as a data gradient
  int fs;   // step of the gradient pixel per output pixel: 1, or the stride of a forward pass run on this kernel
            // (pixel-major loads only): tap (ti, tj) of output pixel (i, j) reads (fs * i + dr0 - ti, fs * j + ds0 - tj)
  int rowstore;   // the tile leaves as contiguous rows (stride 1, even width, planes of whole 8-byte groups, dx 16-byte aligned)
  int dilate, out_W, out_HW;   // 1x1 stride 2: the kernel sees the stride-1 problem on the P x Q grid and its store
                               // writes the 2 x 2 block (value, 0 / 0, 0) of the real out_HW image per pixel
};

constexpr unsigned kSelLo = 0x05040100u, kSelHi = 0x07060302u, kSelZero = 0x0c0c0c0cu;

// PIXK: the gradient is read from a pixel-major copy dyT[n][p][q][k] (k contiguous; made by
// k_pixel_major16 when a layer has several taps): an octet of the B tile is then one aligned 16-byte
// load at any tap offset, staged like the weights, instead of eight dword loads and a transposition.
template <int BM, bool BF16, bool PIXK>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_dgrad16(D16Args a) {
  extern __shared__ __align__(16) uint16_t lds16[];
  constexpr int TM = BM / 64, ASLOTS = BM * 8 / NT, BSLOTS = BN * 8 / NT;
  uint16_t *const As0 = lds16, *const Bs0 = lds16 + BM * PITCH;
  uint16_t *const As1 = lds16 + (BM + BN) * PITCH, *const Bs1 = As1 + BM * PITCH;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int half = wave >> 2, w4 = wave & 3, wm = w4 >> 1, wn = w4 & 1, l32 = lane & 31, lh = lane >> 5;
  // XCD-aware ids (workgroup w runs on XCD w % 8): the channel tiles of one pixel tile read the
  // same gradient pixels and share an XCD's L2.
  const int slot = int(blockIdx.x) >> 3, pt = (slot / a.mtiles) * 8 + (int(blockIdx.x) & 7);
  if (pt >= a.ptiles) return;
  const int m0 = (slot % a.mtiles) * BM;
  const int st = a.stride, PQ = a.P * a.Q, HW = a.H * a.W;
  int cls = 0;
  while (pt >= a.cls_tile0[cls + 1]) ++cls;
  const int ca = cls / st, cb = cls - ca * st;
  // the class's pixel space: rows are padded to an even width so that a pixel pair never
  // straddles two rows (an odd width costs one dummy pixel per row)
  const int Hc = (a.H - ca + st - 1) / st, Wreal = (a.W - cb + st - 1) / st, Wc = (Wreal + 1) & ~1, HWc = Hc * Wc;
  const long cnt = long(a.N) * HWc;
  const long pix0 = long(pt - a.cls_tile0[cls]) * BN;
  const rsrc_t rdy = make_rsrc(PIXK ? a.dyT : a.dy, a.dy_bytes);

  // The taps of this class are r = r0 + st * ti, s = s0 + st * tj (ti < nr, tj < ns): those with
  // (ca + pad_h - r) and (cb + pad_w - s) divisible by the stride; the gradient pixel of tap
  // (ti, tj) is (i + dr0 - ti, j + ds0 - tj).  (st is 1 or 2: shifts, no divisions.)
  const int sh = st - 1;
  const int r0 = (ca + a.pad_h) & sh, s0 = (cb + a.pad_w) & sh;
  const int nr = r0 < a.R ? (a.R - r0 + sh) >> sh : 0, ns = s0 < a.S ? (a.S - s0 + sh) >> sh : 0;
  const int dr0 = (ca + a.pad_h - r0) >> sh, ds0 = (cb + a.pad_w - s0) >> sh;

  const int oct = t & 7, rb = t >> 3;   // staging roles: octet of the chunk, tile row (0..63)
  // B loader, dword pairs: pixel pair pp of the tile, k octet kq of the chunk (one per wavefront)
  const int pp = lane, kq = wave;
  const long pixA = pix0 + 2 * pp, pixB = pixA + 1;
  const int nA = int(pixA / HWc), remA = int(pixA - long(nA) * HWc), iA = remA / Wc, jA = remA - iA * Wc;
  int voff = kOOB;  // byte offset of the dword holding both pixels (kOOB: neither exists)
  unsigned selA = kSelZero, selB = kSelZero;
  const bool pixA_ok = pixA < cnt, pixB_ok = pixB < cnt && jA + 1 < Wreal;
  // B loader, pixel-major copy: pixels rb and rb + 64 of the tile, octet `oct`
  int bn_[BSLOTS], bi_[BSLOTS], bj_[BSLOTS], bvoff[BSLOTS];
  if constexpr (PIXK) {
#pragma unroll
    for (int i = 0; i < BSLOTS; ++i) {
      const long pix = pix0 + rb + 64 * i;
      const bool live = pix < cnt;
      const int n = live ? int(pix / HWc) : 0, rem = live ? int(pix - long(n) * HWc) : 0;
      bn_[i] = n, bi_[i] = rem / Wc, bj_[i] = rem - bi_[i] * Wc;
      if (!live || bj_[i] >= Wreal) bi_[i] = -0x10000;   // no tap of a dummy pixel lands inside the image
      bvoff[i] = kOOB;
    }
  }
  auto set_tap = [&](int ti, int tj) {
    if constexpr (PIXK) {
#pragma unroll
      for (int i = 0; i < BSLOTS; ++i) {
        const int p = bi_[i] * a.fs + dr0 - ti, q = bj_[i] * a.fs + ds0 - tj;
        const bool in = unsigned(p) < unsigned(a.P) && unsigned(q) < unsigned(a.Q);
        bvoff[i] = in ? (((bn_[i] * a.P + p) * a.Q + q) * a.K + oct * 8) * 2 : kOOB;
      }
    } else {
      const int p = iA + dr0 - ti, q0 = jA + ds0 - tj;
      const bool row = unsigned(p) < unsigned(a.P);
      const bool memA = row && unsigned(q0) < unsigned(a.Q), memB = row && unsigned(q0 + 1) < unsigned(a.Q);
      const int base = ((nA * a.K) * a.P + p) * a.Q + q0;
      // both pixels exist: their dword; only A: the dword before (A in the high half); only B: the
      // dword after (B in the low half) -- the load never leaves the row
      voff = memA ? (memB ? base * 2 : (base - 1) * 2) : (memB ? (base + 1) * 2 : kOOB);
      selA = memA && pixA_ok ? (memB ? kSelLo : kSelHi) : kSelZero;
      selB = memB && pixB_ok ? (memA ? kSelHi : kSelLo) : kSelZero;
    }
  };
  const int nkc = a.KP / KC;

  // Two register sets: the chunk after next is requested before the next one is written to LDS, so a request has
  // two chunks of matrix work to arrive in (one chunk is 0.1 us of a wavefront's matrix work against a memory
  // latency of about 1 us: with one set the reduction loop ran at the speed of the loads).
  // (the 128-row tile has 64 accumulator registers and no room for a second set within the 128 registers of four
  // wavefronts per SIMD: it keeps one set)
  constexpr int NSETS = BM == 64 ? 2 : 1;
  u32x4 ra[NSETS][ASLOTS];
  u32x4 rbv[NSETS][BSLOTS];   // pixel-major copy: the octets of this thread's pixels
  unsigned rd[NSETS][8];      // dword pairs: the pair's dword for 8 consecutive k
  unsigned sel_a[NSETS], sel_b[NSETS];   // the selectors of the tap a set was requested for
  const rsrc_t rwt = make_rsrc(a.wt, a.wt_bytes);
  const int woff = ((m0 + rb) * a.KP + oct * 8) * 2;   // rb = t / 8 in 0..63
  // (`live` false: a request beyond the last chunk.  It issues the same loads at out-of-range offsets, which
  // return zeros without touching memory: the number of loads between a request and its use is then the same on
  // every path, so the wait in front of the use can leave the newer request in flight.  A request inside a
  // branch made every such wait a wait for all loads.)
  auto load = [&](auto SET, int tap, int kc, bool live) {
    constexpr int S = decltype(SET)::value;
    const int wso = (tap * a.CP * a.KP + kc * KC) * 2;
    const int wv = live ? woff : kOOB;
#pragma unroll
    for (int i = 0; i < ASLOTS; ++i)
      ra[S][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rwt, wv + 64 * i * a.KP * 2, wso, 0));
    if constexpr (PIXK) {
      const bool kin = live && kc * KC + oct * 8 < a.K;   // (K is a multiple of 8: an octet is inside or outside)
#pragma unroll
      for (int i = 0; i < BSLOTS; ++i)
        rbv[S][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rdy, kin ? bvoff[i] : kOOB, kc * KC * 2, 0));
    } else {
      sel_a[S] = selA, sel_b[S] = selB;
      const int kb = kc * KC + kq * 8;
      const int dv = live && kb < a.K ? voff : kOOB;
#pragma unroll
      for (int j = 0; j < 8; ++j) rd[S][j] = unsigned(__builtin_amdgcn_raw_buffer_load_b32(rdy, dv, (kb + j) * PQ * 2, 0));
    }
  };
  auto stage = [&](auto SET, uint16_t *As, uint16_t *Bs) {
    constexpr int S = decltype(SET)::value;
#pragma unroll
    for (int i = 0; i < ASLOTS; ++i) *reinterpret_cast<u32x4 *>(As + (rb + 64 * i) * PITCH + oct * 8) = ra[S][i];
    if constexpr (PIXK) {
#pragma unroll
      for (int i = 0; i < BSLOTS; ++i) *reinterpret_cast<u32x4 *>(Bs + (rb + 64 * i) * PITCH + oct * 8) = rbv[S][i];
    } else {
      u32x4 vA, vB;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        vA[d] = __builtin_amdgcn_perm(rd[S][2 * d + 1], rd[S][2 * d], sel_a[S]);
        vB[d] = __builtin_amdgcn_perm(rd[S][2 * d + 1], rd[S][2 * d], sel_b[S]);
      }
      *reinterpret_cast<u32x4 *>(Bs + (2 * pp) * PITCH + kq * 8) = vA;
      *reinterpret_cast<u32x4 *>(Bs + (2 * pp + 1) * PITCH + kq * 8) = vB;
    }
  };

  f32x16 acc[TM][2];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  if (nr > 0 && ns > 0) {
    typedef std::integral_constant<int, 0> Set0;
    typedef std::integral_constant<int, NSETS - 1> Set1;
    const int total = nr * ns * nkc;   // chunks: taps in (ti, tj) order, the k chunks of a tap in turn
    int ti = 0, tj = 0, kc = 0;        // the next chunk to request
    auto request = [&](auto SET) {
      const bool live = ti < nr;
      if (live && kc == 0) set_tap(ti, tj);
      load(SET, live ? (r0 + st * ti) * a.S + s0 + st * tj : 0, live ? kc : 0, live);
      if (live && ++kc == nkc) {
        kc = 0;
        if (++tj == ns) tj = 0, ++ti;
      }
    };
    auto mma = [&](const uint16_t *As, const uint16_t *Bs) {
      mma_chunk<TM, BF16>(As, Bs, wm * (TM * 32) + l32, wn * 64 + half * 32 + l32, half ? -32 : 32, half * 32 + lh * 8, acc);
    };
    request(Set0{});
    if constexpr (NSETS == 2) {
      request(Set1{});
      stage(Set0{}, As0, Bs0);
      __syncthreads();
      for (int c = 0;; c += 2) {
        // chunk c is in LDS buffer 0, chunk c + 1 on its way into register set 1
        request(Set0{});
        mma(As0, Bs0);
        if (c + 1 >= total) break;
        stage(Set1{}, As1, Bs1);
        __syncthreads();
        request(Set1{});
        mma(As1, Bs1);
        if (c + 2 >= total) break;
        stage(Set0{}, As0, Bs0);
        __syncthreads();
      }
    } else {
      stage(Set0{}, As0, Bs0);
      __syncthreads();
      bool cur1 = false;
      for (int c = 0;; ++c) {
        request(Set0{});
        mma(cur1 ? As1 : As0, cur1 ? Bs1 : Bs0);
        if (c + 1 >= total) break;
        stage(Set0{}, cur1 ? As0 : As1, cur1 ? Bs0 : Bs1);
        __syncthreads();
        cur1 = !cur1;
      }
    }
  }

  // epilogue: lane's pixel column, 16 channel rows per accumulator
  combine_halves<TM>(reinterpret_cast<float *>(lds16), half, w4, lane, acc);
  if (a.rowstore) {
    // Stride 1 on an even width with planes that are whole 8-byte groups: the tile is 128 consecutive pixels of
    // dx, so it goes through LDS as [channel][pixel] and leaves in 8- or 16-byte pieces of contiguous rows (a
    // wavefront's own layout, one pixel per lane and 2 bytes per store, kept the vector memory path busy
    // longer than the whole reduction on the layers with large outputs).
    constexpr int OP = BN + 8;
    uint16_t *ot = lds16;
    __syncthreads();   // the exchange above has been read
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = wm * (TM * 32) + i * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
        float r = acc[i][0][v];
        if (a.bias && m0 + row < a.C) r += BF16 ? sgh_bf16_to_f32(a.bias[m0 + row]) : sgh_f16_to_f32(a.bias[m0 + row]);
        ot[row * OP + wn * 64 + half * 32 + l32] = round16<BF16>(r);
      }
    __syncthreads();
    if ((HW & 7) == 0) {
      const int g = t & 15;
      const long p8 = pix0 + 8 * g;
      if (p8 < cnt) {
        const int n = int(p8 / HW), rem = int(p8 - long(n) * HW);
        uint16_t *o = a.dx + (size_t(n) * a.C + m0) * HW + rem;
        for (int row = t >> 4; row < BM && m0 + row < a.C; row += NT / 16)
          *reinterpret_cast<u32x4 *>(o + size_t(row) * HW) = *reinterpret_cast<const u32x4 *>(ot + row * OP + 8 * g);
      }
    } else {
      typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
      const int g = t & 31;
      const long p4 = pix0 + 4 * g;
      if (p4 < cnt) {
        const int n = int(p4 / HW), rem = int(p4 - long(n) * HW);
        uint16_t *o = a.dx + (size_t(n) * a.C + m0) * HW + rem;
        for (int row = t >> 5; row < BM && m0 + row < a.C; row += NT / 32)
          *reinterpret_cast<u32x2 *>(o + size_t(row) * HW) = *reinterpret_cast<const u32x2 *>(ot + row * OP + 4 * g);
      }
    }
    return;
  }
  const long pix = pix0 + wn * 64 + half * 32 + l32;   // the block this group kept
  if (pix >= cnt) return;
  const int n = int(pix / HWc), rem = int(pix - long(n) * HWc), i_ = rem / Wc, j_ = rem - i_ * Wc;
  if (j_ >= Wreal) return;
  if (a.dilate) {
    uint16_t *o2 = a.dx + (size_t(n) * a.C) * a.out_HW + (2 * i_) * a.out_W + 2 * j_;   // (even: dword aligned)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int c = m0 + wm * (TM * 32) + i * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
        if (c < a.C) {
          *reinterpret_cast<unsigned *>(o2 + size_t(c) * a.out_HW) = unsigned(round16<BF16>(acc[i][0][v]));
          *reinterpret_cast<unsigned *>(o2 + size_t(c) * a.out_HW + a.out_W) = 0u;
        }
      }
    return;
  }
  uint16_t *o = a.dx + (size_t(n) * a.C) * HW + (st * i_ + ca) * a.W + st * j_ + cb;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int c = m0 + wm * (TM * 32) + i * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
      if (c < a.C) {
        float r = acc[i][0][v];
        if (a.bias) r += BF16 ? sgh_bf16_to_f32(a.bias[c]) : sgh_f16_to_f32(a.bias[c]);
        o[size_t(c) * HW] = round16<BF16>(r);
      }
    }
}

// dst[n][pq][k] = src[n][k][pq]: the pixel-major copy of a gradient tensor that the multi-tap data
// gradient reads (64 x 64 tiles through LDS; K is even).  PAIR: PQ is even, the source is read as dwords.
template <bool PAIR>
__global__ __launch_bounds__(256) void k_pixel_major16(const uint16_t *__restrict__ src, uint16_t *__restrict__ dst, int K,
                                                      int PQ) {
  __shared__ __align__(4) uint16_t tile[64][66];   // [k][pq]
  const int t = threadIdx.x, n = blockIdx.z, k0 = blockIdx.y * 64, q0 = blockIdx.x * 64;
  const uint16_t *s = src + size_t(n) * K * PQ;
  if constexpr (PAIR) {
    const int c2 = t & 31;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int kr = (t >> 5) + 8 * i, k = k0 + kr, pq = q0 + 2 * c2;
      unsigned v = 0u;
      if (k < K && pq < PQ) v = *reinterpret_cast<const unsigned *>(s + size_t(k) * PQ + pq);
      *reinterpret_cast<unsigned *>(&tile[kr][2 * c2]) = v;
    }
  } else {
    const int c = t & 63;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int kr = (t >> 6) + 4 * i, k = k0 + kr, pq = q0 + c;
      tile[kr][c] = (k < K && pq < PQ) ? s[size_t(k) * PQ + pq] : uint16_t(0);
    }
  }
  __syncthreads();
  const int kd = 2 * (t & 31);
  if (k0 + kd >= K) return;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int pr = (t >> 5) + 8 * i, pq = q0 + pr;
    if (pq < PQ)
      *reinterpret_cast<unsigned *>(dst + (size_t(n) * PQ + pq) * K + k0 + kd) =
          unsigned(tile[kd][pr]) | (unsigned(tile[kd + 1][pr]) << 16);
  }
}

// wt[tap][c][k] (c < CP, k < KP; zero beyond C / K) from W[k][c][r][s]
__global__ __launch_bounds__(256) void k_relayout16(const uint16_t *W, uint16_t *wt, int K, int C, int RS, int KP, int CP) {
  const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x, n = size_t(RS) * CP * KP;
  if (i >= n) return;
  const int k = int(i % KP), c = int((i / KP) % CP), tap = int(i / (size_t(KP) * CP));
  wt[i] = (k < K && c < C) ? W[(size_t(k) * C + c) * RS + tap] : uint16_t(0);
}

// the forward pass as a data gradient: wt[tap][ko][c] = W[ko][c][RS - 1 - tap] (ko < KOP, c < CRP; zero beyond)
__global__ __launch_bounds__(256) void k_relayout16_fwd(const uint16_t *W, uint16_t *wt, int K, int C, int RS, int CRP,
                                                        int KOP) {
  const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x, n = size_t(RS) * KOP * CRP;
  if (i >= n) return;
  const int c = int(i % CRP), ko = int((i / CRP) % KOP), tap = int(i / (size_t(CRP) * KOP));
  wt[i] = (ko < K && c < C) ? W[(size_t(ko) * C + c) * RS + (RS - 1 - tap)] : uint16_t(0);
}

// ------------------------------------------------------------------------------------------------
// data gradient of 3x3 / stride 1 / padding 1 layers: gradient slab shared by the nine taps
// ------------------------------------------------------------------------------------------------
// The pixels of all images are laid on one line with ONE zero position behind every row and one
// zero row behind every image: position g = (n * (H + 1) + h) * (W + 1) + w.  The neighbour (h + dr,
// w + ds) of a pixel is then g + dr * (W + 1) + ds for every pixel, border or not -- what falls off
// an image lands on a zero position -- so a tap is a constant shift of the whole tile.  A workgroup
// takes MT consecutive positions x BMC channels.  Per 64 gradient channels it stages the positions
// [m0 - W - 2, m0 + MT + W + 2) ONCE as a pixel-major slab in LDS and all nine taps read their B
// fragments from it at their shift; only the 16 KB weight tile of a (tap, chunk) pair is streamed.
// That is a ninth of the gradient loads of the tap-by-tap kernel above and 9 x 4 matrix steps per
// slab instead of 4.
//   Staging: a thread owns EV (8 or 4) consecutive pixels of the NCHW tensor and 8 consecutive k (the lanes that
// share a pixel group take different k octets): it
// loads the 8 rows with 16- (8-) byte loads, transposes the 8 x EV block in registers (v_perm_b32) and
// writes one 16-byte octet per pixel to that pixel's slab row (planes are whole groups of EV pixels, so
// a group never straddles two images; it may straddle two rows, where the slab row skips the zero
// position).  Zero positions are written once, at the start.  (2-byte loads, one per element, kept the
// vector memory path busy for 10 us per slab: 47 cycles per wavefront instruction.)
//   Pipeline: the nine tap steps of a chunk are unrolled.  The loads of the next chunk's block are
// issued in steps 0-3 and written in steps 7-8; the weight tile of step s + 2 is loaded in step s into
// one of two register sets and written to LDS at the end of step s + 1 (a tile loaded and written within
// one step left every wavefront waiting 500 ns for L2 at the end of the step).  Every load is issued
// unconditionally (out-of-range ones through an offset beyond the buffer, which reads zero) so that the
// waits can count loads instead of draining them.
// 512 threads: two groups of four wavefronts tile the same outputs and take the first / second half of
// the matrix steps of every weight tile (summed through LDS at the end, as above); a wavefront holds
// TC x TP accumulator blocks (channels x positions).
struct S16Args {
  const uint16_t *dy, *wt;  // wt: [tap][CP][KP]
  uint16_t *dx;
  const uint16_t *bias;
  int N, C, H, W, K, KP, CP, mtiles, ptiles;
  int Wp, HpWp, SP;   // W + 1, (H + 1) * (W + 1), slab entries MT + 2 * Wp + 2
  int G;              // positions in all: N * HpWp
  unsigned dy_bytes, wt_bytes;
};

template <int EV> struct SlabVec;
template <> struct SlabVec<8> {
  typedef u32x4 type;
  static __device__ __forceinline__ type load(rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
  }
};
template <> struct SlabVec<4> {
  typedef unsigned int type __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ type load(rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(type, __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0));
  }
};

// MULTI: more than one chunk of 64 gradient channels (two slab buffers; the next chunk's block in flight)
template <int TC, int TP, int WC, int WP, int EV, bool MULTI, bool BF16>
__global__ __launch_bounds__(NT) void k_dgrad16_slab(S16Args a) {
  // SPLIT: two groups of four wavefronts share the outputs and split every tile's matrix steps; otherwise the
  // eight wavefronts tile the outputs and each takes all four steps
  constexpr bool SPLIT = WC * WP == 4;
  constexpr int KS = SPLIT ? 2 : 4;
  static_assert((WC * WP == 4 && TP % 2 == 0) || WC * WP == 8, "four wavefronts per group (each keeps half of the position blocks), or eight tiles");
  constexpr int BMC = WC * TC * 32, MT = WP * TP * 32, WSLOTS = BMC * 8 / NT;
  constexpr int NB = EV == 8 ? 1 : 2;   // blocks (8 k x EV pixels) per thread and chunk
  constexpr int KOL = 8 / NB;           // lanes per pixel group
  typedef typename SlabVec<EV>::type ev_t;
  extern __shared__ __align__(16) uint16_t lds16[];
  const int SPR = a.SP + 1;   // slab rows: the entries and a sink for octets that belong to no entry
  uint16_t *const slab0 = lds16, *const slab1 = slab0 + (MULTI ? SPR * PITCH : 0);
  uint16_t *const wts0 = slab1 + SPR * PITCH, *const wts1 = wts0 + BMC * PITCH;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int half = SPLIT ? wave >> 2 : 0, w4 = SPLIT ? wave & 3 : wave, wc = w4 / WP, wp = w4 % WP, l32 = lane & 31, lh = lane >> 5;
  // workgroup w runs on XCD w % 8: the channel tiles of one position tile share an XCD's L2
  const int slot = int(blockIdx.x) >> 3, pt = (slot / a.mtiles) * 8 + (int(blockIdx.x) & 7);
  if (pt >= a.ptiles) return;
  const int c0 = (slot % a.mtiles) * BMC, m0 = pt * MT, HW = a.H * a.W;
  const rsrc_t rdy = make_rsrc(a.dy, a.dy_bytes), rwt = make_rsrc(a.wt, a.wt_bytes);

  // This thread's pixel group: number gi among the groups of EV pixels (in tensor order, all images on one
  // line) from the one that holds the first pixel of the slab; its blocks are k octets ko[j] of a chunk.
  const int g_lo = m0 - a.Wp - 1;
  int voff = kOOB, row0 = a.SP, wrapat = EV, wrapinc = 0;
  {
    int n, h, w;
    {
      const int gs = g_lo > 0 ? g_lo : 0;
      n = gs / a.HpWp;
      const int rem = gs - n * a.HpWp;
      h = rem / a.Wp, w = rem - h * a.Wp;
      if (h == a.H) h = 0, w = 0, ++n;   // (a zero row: on to the next image)
      else if (w == a.W) {               // (a zero position: on to the next row)
        w = 0;
        if (++h == a.H) h = 0, ++n;
      }
    }
    const long f_lo = long(n) * HW + h * a.W + w;
    const long f0 = (f_lo / EV + wave * (8 * NB) + lane / KOL) * EV;
    if (f0 < long(a.N) * HW) {
      const int n0 = int(f0 / HW), pix = int(f0 - long(n0) * HW), h0 = pix / a.W, w0 = pix - h0 * a.W;
      row0 = n0 * a.HpWp + h0 * a.Wp + w0 - g_lo;
      wrapat = a.W - w0;
      wrapinc = 1 + (h0 + 1 == a.H ? a.Wp : 0);
      const int last = row0 + EV - 1 + (EV - 1 >= wrapat ? wrapinc : 0);
      if (last >= 0 && row0 < a.SP) voff = (n0 * a.K * HW + pix) * 2;
    }
  }
  // k octets of this thread's blocks.  The KOL lanes that share a pixel group take different octets, so that a
  // wavefront's LDS write covers whole slab rows (128 or 64 contiguous bytes per row, 4-way bank conflicts; with
  // one octet per wavefront and a row per lane, rows EV apart fell on 2 of the 16 bank groups: 32-way).
  int ko[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) ko[j] = lane % KOL + KOL * j;

  ev_t blk[NB][8];       // the block(s) in flight: row kk = EV pixels of gradient channel 8 * ko + kk
  u32x4 ra[2][WSLOTS];   // two weight tiles in flight
  const int oct = t & 7, rb = t >> 3;
  const int woff = ((c0 + rb) * a.KP + oct * 8) * 2;
  const int nkc = a.KP / KC, nsteps = 9 * nkc;

  auto load_rows = [&](int kc, int kk0, int count) {   // rows kk0 .. kk0 + count - 1 of the blocks of chunk kc
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int kb = kc * KC + ko[j] * 8;
      const int vo = (kc < nkc && kb < a.K ? voff : kOOB) + ko[j] * 8 * HW * 2;   // (K is a multiple of 8)
#pragma unroll
      for (int kk = 0; kk < 8; ++kk)
        if (kk >= kk0 && kk < kk0 + count) blk[j][kk] = SlabVec<EV>::load(rdy, vo, (kc * KC + kk) * HW * 2);
    }
  };
  auto stage_pixels = [&](uint16_t *slab, int p0, int count) {   // pixels p0 .. p0 + count - 1 of the blocks
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int p = 0; p < EV; ++p)
        if (p >= p0 && p < p0 + count) {
          u32x4 v;
#pragma unroll
          for (int d = 0; d < 4; ++d)
            v[d] = __builtin_amdgcn_perm(blk[j][2 * d + 1][p >> 1], blk[j][2 * d][p >> 1], (p & 1) ? kSelHi : kSelLo);
          int row = row0 + p + (p >= wrapat ? wrapinc : 0);
          row = unsigned(row) < unsigned(a.SP) ? row : a.SP;
          *reinterpret_cast<u32x4 *>(slab + row * PITCH + ko[j] * 8) = v;
        }
  };
  auto load_w = [&](int step, u32x4 (&r)[WSLOTS]) {
    const int kc = step / 9, tap = step - 9 * kc;
    const int wso = (tap * a.CP * a.KP + kc * KC) * 2;
    const int vo = step < nsteps ? woff : kOOB;
#pragma unroll
    for (int i = 0; i < WSLOTS; ++i)
      r[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rwt, vo + 64 * i * a.KP * 2, wso, 0));
  };
  auto stage_w = [&](uint16_t *wts, const u32x4 (&r)[WSLOTS]) {
#pragma unroll
    for (int i = 0; i < WSLOTS; ++i) *reinterpret_cast<u32x4 *>(wts + (rb + 64 * i) * PITCH + oct * 8) = r[i];
  };

  // prologue: the first chunk's block and the first two weight tiles on their way, the slabs zeroed meanwhile
  load_rows(0, 0, 8);
  load_w(0, ra[0]);
  load_w(1, ra[1]);
  {
    const u32x4 z = {0u, 0u, 0u, 0u};
    const int n16 = (MULTI ? 2 : 1) * SPR * PITCH / 8;
    for (int i = t; i < n16; i += NT) reinterpret_cast<u32x4 *>(slab0)[i] = z;
  }
  f32x16 acc[TC][TP];
#pragma unroll
  for (int i = 0; i < TC; ++i)
#pragma unroll
    for (int j = 0; j < TP; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  __syncthreads();
  stage_pixels(slab0, 0, EV);
  stage_w(wts0, ra[0]);
  __syncthreads();

  const int arow = (wc * TC * 32 + l32) * PITCH + half * 32 + lh * 8;
  const int brow = (wp * TP * 32 + l32 + a.Wp + 1) * PITCH + half * 32 + lh * 8;
  // step = 9 * kc + tap; PAR = step & 1 names the weight tile buffer in LDS that the step reads and the
  // register set that it loads
  auto step = [&](int kc, auto tapc, auto parc) {
    constexpr int TAP = decltype(tapc)::value, PAR = decltype(parc)::value, R_ = TAP / 3, S_ = TAP % 3;
    const uint16_t *const slab = (MULTI && (kc & 1)) ? slab1 : slab0;
    uint16_t *const slab_next = (MULTI && (kc & 1)) ? slab0 : slab1;
    load_w(9 * kc + TAP + 2, ra[PAR]);
    if (MULTI && TAP < 4) load_rows(kc + 1, 2 * TAP, 2);
    const uint16_t *As = (PAR ? wts1 : wts0) + arow;
    const uint16_t *Bs = slab + brow + ((1 - R_) * a.Wp + (1 - S_)) * PITCH;
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      u32x4 av[TC], bv[TP];
#pragma unroll
      for (int i = 0; i < TC; ++i) av[i] = *reinterpret_cast<const u32x4 *>(As + i * 32 * PITCH + 16 * j);
#pragma unroll
      for (int i = 0; i < TP; ++i) bv[i] = *reinterpret_cast<const u32x4 *>(Bs + i * 32 * PITCH + 16 * j);
#pragma unroll
      for (int i = 0; i < TC; ++i)
#pragma unroll
        for (int jp = 0; jp < TP; ++jp) acc[i][jp] = mfma<BF16>(av[i], bv[jp], acc[i][jp]);
    }
    stage_w(PAR ? wts0 : wts1, ra[PAR ^ 1]);   // the tile of step + 1, loaded during step - 1
    if (MULTI && TAP == 7) stage_pixels(slab_next, 0, EV / 2);
    if (MULTI && TAP == 8) stage_pixels(slab_next, EV / 2, EV / 2);
    __syncthreads();
  };
  auto chunk = [&](int kc, auto parc) {
    constexpr int P = decltype(parc)::value;
    typedef std::integral_constant<int, P> P0;
    typedef std::integral_constant<int, P ^ 1> P1;
    step(kc, std::integral_constant<int, 0>{}, P0{});
    step(kc, std::integral_constant<int, 1>{}, P1{});
    step(kc, std::integral_constant<int, 2>{}, P0{});
    step(kc, std::integral_constant<int, 3>{}, P1{});
    step(kc, std::integral_constant<int, 4>{}, P0{});
    step(kc, std::integral_constant<int, 5>{}, P1{});
    step(kc, std::integral_constant<int, 6>{}, P0{});
    step(kc, std::integral_constant<int, 7>{}, P1{});
    step(kc, std::integral_constant<int, 8>{}, P0{});
  };
  for (int kc = 0; kc < nkc; kc += 2) {
    chunk(kc, std::integral_constant<int, 0>{});
    if (!MULTI || kc + 1 >= nkc) break;
    chunk(kc + 1, std::integral_constant<int, 1>{});
  }

  // SPLIT: the two groups' sums meet in LDS, one channel block at a time: a wavefront hands over the position
  // blocks of the other group's half and adds what its partner hands over to the blocks it keeps.
  constexpr int TH = SPLIT ? TP / 2 : TP;
  if constexpr (SPLIT) {
    float *const xl = reinterpret_cast<float *>(lds16);
    float *send = xl + ((half * 4 + w4) * (TH * 16)) * 64 + lane;
    const float *recv = xl + (((half ^ 1) * 4 + w4) * (TH * 16)) * 64 + lane;
#pragma unroll
    for (int i = 0; i < TC; ++i) {
      if (i) __syncthreads();
#pragma unroll
      for (int j = 0; j < TH; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) send[(j * 16 + v) * 64] = half ? acc[i][j][v] : acc[i][TH + j][v];
      __syncthreads();
#pragma unroll
      for (int j = 0; j < TH; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          if (half) acc[i][TH + j][v] += recv[(j * 16 + v) * 64];
          else acc[i][j][v] += recv[(j * 16 + v) * 64];
        }
    }
  }
  // store: a lane owns one position per kept block, 16 channels per accumulator.  (Measured against this: the tile
  // taken through LDS as [channel][pixel in tensor order] and written in 16-byte groups, with and without
  // non-temporal stores -- 3 to 10 us slower per layer; the workgroups of a round reach their stores together
  // and the burst is bound by the write path either way.)
#pragma unroll
  for (int j = 0; j < TH; ++j) {
    const int g = m0 + (wp * TP + half * TH + j) * 32 + l32;
    if (g >= a.G) continue;
    const int n = g / a.HpWp, rem = g - n * a.HpWp, h = rem / a.Wp, w = rem - h * a.Wp;
    if (h >= a.H || w >= a.W) continue;
    uint16_t *o = a.dx + (size_t(n) * a.C) * HW + h * a.W + w;
#pragma unroll
    for (int i = 0; i < TC; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int c = c0 + (wc * TC + i) * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
        if (c < a.C) {
          float r = (SPLIT && half) ? acc[i][TP - TH + j][v] : acc[i][j][v];
          if (a.bias) r += BF16 ? sgh_bf16_to_f32(a.bias[c]) : sgh_f16_to_f32(a.bias[c]);
          o[size_t(c) * HW] = round16<BF16>(r);
        }
      }
  }
}

inline size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

constexpr size_t kLutBytes = 81 * 16;  // wgrad: octet mask table behind the tiles
constexpr size_t kLds128 = size_t(2) * (128 + BN) * PITCH * 2, kLds64 = size_t(2) * (64 + BN) * PITCH * 2;

template <typename Kern>
bool allow_lds(Kern kern, size_t bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                             int(bytes)) == hipSuccess;
}

struct W16Plan {
  bool ok;
  int bm, stride, mtiles, ntiles, chunks, splits, cps;
  sgh_conv_geom f;  // the geometry the kernel sees (1x1 stride-1 layers: image plane as one row)
  int QO;
};

// `shared`: the launch shares the chip with another stream's kernels (it runs on a device's auxiliary stream
// beside the data-gradient / BatchNorm chain): the split is planned for one workgroup per CU instead of two.
// Alone, the weight-gradient kernels are slower that way (6.1 -> 6.8 ms over the ResNet-50 step at N = 128);
// side by side with the main stream the step is faster (9.51 -> 9.27 ms): half the fp32 partials to write and
// sum, and workgroups that do not queue behind the other stream's for the same CUs.
W16Plan wplan(const sgh_conv_geom *g, bool shared) {
  W16Plan p{};
  if (g->stride_h != g->stride_w || (g->stride_h != 1 && g->stride_h != 2)) return p;
  const size_t lim = size_t(1) << 30;  // byte offsets into x and dy stay below 2^31
  const size_t xe = size_t(g->N) * g->C * g->H * g->W, ye = size_t(g->N) * g->K * g->P * g->Q;
  if (xe >= lim || ye >= lim || size_t(g->K) * g->C * g->R * g->S >= lim) return p;
  p.f = *g;
  if (g->R == 1 && g->S == 1 && g->stride_h == 1 && g->pad_h == 0 && g->pad_w == 0) {
    p.f.H = 1, p.f.W = g->H * g->W, p.f.P = 1, p.f.Q = g->P * g->Q;
  }
  p.stride = g->stride_h;
  p.bm = g->K <= 64 ? 64 : 128;
  p.mtiles = (g->K + p.bm - 1) / p.bm;
  p.ntiles = (g->C * g->R * g->S + BN - 1) / BN;
  p.QO = (p.f.Q + 7) / 8;
  const long units = long(p.f.N) * p.f.P * p.QO;
  p.chunks = int((units + 7) / 8);
  // Splits of the reduction: the chip holds 2 workgroups per CU at a time; among 1..4 such rounds
  // take the split count whose (rounds x chunks per split) is smallest, i.e. avoid a last round
  // that is mostly empty.  Every split gets at least 4 chunks.
  const int tiles = p.mtiles * p.ntiles, slots = (shared ? 1 : 2) * sgh_num_cus();
  // the split reduction reads splits x |dW| fp32 partials at about 5 TB/s; one chunk of a round takes
  // about 0.9 us -> its cost in chunk units per split
  const double reduce_chunks_per_split = double(g->K) * g->C * g->R * g->S * 4.0 / 5.0e6 / 0.9;
  double best = -1;
  for (int r = 1; r <= 4; ++r) {
    int s = slots * r / tiles;
    if (s < 1) s = 1;
    if (s > (p.chunks + 3) / 4) s = (p.chunks + 3) / 4;
    if (s < 1) s = 1;
    if (s >= 8) s &= ~7;   // a multiple of 8 lets every XCD take whole splits (see the kernel)
    const int cps = (p.chunks + s - 1) / s;
    // (with 8 or more splits the count stays the multiple of 8; the last splits may then be short or empty)
    const int s2 = s >= 8 ? s : (p.chunks + cps - 1) / cps;
    const long rounds = (long(tiles) * s2 + slots - 1) / slots;
    const double cost = double(rounds * (cps + 2)) + s2 * reduce_chunks_per_split;  // (+2: prologue, epilogue)
    if (best < 0 || cost < best) best = cost, p.cps = cps, p.splits = s2;
  }
  p.ok = true;
  return p;
}

struct D16Plan {
  bool ok;
  bool pixk;   // several taps: the kernel reads a pixel-major copy of the gradient (k_pixel_major16)
  int bm, mtiles, KP, CP, tiles;
  int cls_tile0[5];
  size_t wt_bytes, dyT_bytes;   // workspace: re-laid weights, then the pixel-major copy
  int fs;             // see D16Args::fs
  int slab;           // k_dgrad16_slab: 0 no, else the tile: 1 = 64 channels x 256 positions, 2 = 128 x 256, 3 = 128 x 128
  int slab_sp;        // slab entries
  int slab_ev;        // pixels per staging group: 8 or 4
  bool dilate;        // 1x1, stride 2, no padding, even image: see D16Args::dilate
  sgh_conv_geom kg;   // the geometry the kernel sees (the stride-1 problem on the P x Q grid when `dilate`)
};

D16Plan dplan(const sgh_conv_geom *real, int fs = 1) {
  D16Plan p{};
  p.fs = fs;
  if (real->stride_h != real->stride_w || (real->stride_h != 1 && real->stride_h != 2)) return p;
  if (real->K % 8 != 0 || real->Q < 2 || real->C < 16) return p;  // (a 64-row tile is mostly empty below 16 channels)
  const size_t lim = size_t(1) << 30;  // byte offsets of dy stay below 2^31
  if (size_t(real->N) * real->K * real->P * real->Q >= lim || size_t(real->N) * real->C * real->H * real->W >= 2 * lim)
    return p;
  // 1x1 stride 2: three of the four residue classes receive no tap; instead of workgroups that only
  // store zeros at every other position, the (0, 0) class is computed as a stride-1 problem and its
  // store writes whole 2 x 2 blocks
  p.kg = *real;
  p.dilate = real->R == 1 && real->S == 1 && real->stride_h == 2 && real->pad_h == 0 && real->pad_w == 0 &&
             real->H % 2 == 0 && real->W % 2 == 0;
  if (p.dilate) p.kg.H = real->P, p.kg.W = real->Q, p.kg.stride_h = p.kg.stride_w = 1;
  const sgh_conv_geom *g = &p.kg;
  const int st = g->stride_h;
  long tiles = 0;
  for (int cls = 0; cls < st * st; ++cls) {
    const int ca = cls / st, cb = cls % st;
    const int Hc = (g->H - ca + st - 1) / st, Wc = ((g->W - cb + st - 1) / st + 1) & ~1;  // rows padded to even
    p.cls_tile0[cls] = int(tiles);
    tiles += (long(g->N) * Hc * Wc + BN - 1) / BN;
  }
  for (int cls = st * st; cls < 5; ++cls) p.cls_tile0[cls] = int(tiles);
  // 3x3 / stride 1 / padding 1 on planes of whole 4- or 8-pixel groups: the slab kernel, when its slab fits beside
  // the weight tiles in the 160 KB of LDS and a thread per pixel group (two per group of 4) covers it
  if (fs == 1 && g->R == 3 && g->S == 3 && st == 1 && g->pad_h == 1 && g->pad_w == 1 && !sgh_env().slab16_off &&
      (g->H * g->W) % 4 == 0 && g->W >= 8) {
    const long G = long(g->N) * (g->H + 1) * (g->W + 1);
    const int ev = (g->H * g->W) % 8 == 0 ? 8 : 4;
    const int bmc = g->C <= 64 ? 64 : 128, mt_c = (g->C + bmc - 1) / bmc;
    const int KP = (g->K + KC - 1) / KC * KC;
    int mt = 256;
    if (bmc == 128 && ((G + 255) / 256) * mt_c < sgh_num_cus() * 3 / 4) mt = 128;
    for (; mt >= (bmc == 128 ? 128 : 256); mt /= 2) {
      const int sp = mt + 2 * (g->W + 1) + 2;
      const size_t lds = (size_t(KP > KC ? 2 : 1) * (sp + 1) + 2 * bmc) * PITCH * 2;
      if (G + 1024 >= (long(1) << 31) || sp / ev + 3 > (ev == 8 ? 64 : 128) || lds > size_t(160) * 1024) continue;
      p.slab = bmc == 64 ? 1 : (mt == 256 ? 2 : 3);
      p.slab_sp = sp, p.slab_ev = ev;
      p.bm = bmc, p.mtiles = mt_c, p.CP = mt_c * bmc, p.KP = KP;
      p.tiles = int((G + mt - 1) / mt);
      p.pixk = false;
      p.wt_bytes = align256(size_t(9) * p.CP * p.KP * sizeof(uint16_t));
      p.dyT_bytes = 0;
      p.ok = true;
      return p;
    }
  }
  // 64-row channel tiles when 128-row ones would leave CUs without a workgroup
  p.bm = (g->C <= 64 || tiles * ((g->C + 127) / 128) < sgh_num_cus() * 5 / 4) ? 64 : 128;
  p.mtiles = (g->C + p.bm - 1) / p.bm;
  p.CP = p.mtiles * p.bm;
  p.KP = (g->K + KC - 1) / KC * KC;
  if (tiles * p.mtiles >= (long(1) << 30) || size_t(g->R) * g->S * p.CP * p.KP >= lim) return p;
  p.tiles = int(tiles);
  // The copy pays where the dword-pair loads are at their worst: odd class widths (7 x 7 planes,
  // stride 2 on 14 x 14), where every pair row carries a dummy pixel.  (Elsewhere the kernel gains
  // 10-20 % from the aligned loads and the copy costs as much: measured at 56 x 56 .. 14 x 14.)
  p.pixk = fs > 1 || (g->R * g->S > 1 && ((g->W + st - 1) / st) % 2 == 1);
  p.wt_bytes = align256(size_t(g->R) * g->S * p.CP * p.KP * sizeof(uint16_t));
  p.dyT_bytes = p.pixk ? align256(size_t(g->N) * g->K * g->P * g->Q * sizeof(uint16_t)) : 0;
  p.ok = true;
  return p;
}

template <int BM, int STRIDE, bool BF16>
int launch_w(const W16Args &a, const W16Plan &p, hipStream_t s) {
  auto kern = k_wgrad16<BM, STRIDE, BF16>;
  const size_t lds = (BM == 128 ? kLds128 : kLds64) + kLutBytes;
  static bool attr = false;
  if (!attr) {
    if (!allow_lds(kern, lds)) return SGH_EUNSUPPORTED;
    attr = true;
  }
  SGH_LAUNCH_TIMED(kern, dim3(unsigned(p.mtiles * p.ntiles) * unsigned(p.splits)), dim3(NT), lds, s, a);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

template <int BM, bool BF16, bool PIXK>
int launch_d(const D16Args &a, const D16Plan &p, hipStream_t s) {
  auto kern = k_dgrad16<BM, BF16, PIXK>;
  const size_t lds = BM == 128 ? kLds128 : kLds64;
  static bool attr = false;
  if (!attr) {
    if (!allow_lds(kern, lds)) return SGH_EUNSUPPORTED;
    attr = true;
  }
  SGH_LAUNCH_TIMED(kern, dim3(unsigned((p.tiles + 7) / 8) * 8u * unsigned(p.mtiles)), dim3(NT), lds, s, a);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

template <int TC, int TP, int WC, int WP, int EV, bool MULTI, bool BF16>
int launch_slab2(const S16Args &a, const D16Plan &p, hipStream_t s) {
  auto kern = k_dgrad16_slab<TC, TP, WC, WP, EV, MULTI, BF16>;
  constexpr int BMC = WC * TC * 32;
  const size_t lds = (size_t(MULTI ? 2 : 1) * (p.slab_sp + 1) + 2 * BMC) * PITCH * 2;
  static size_t allowed = 0;
  if (lds > allowed) {
    if (!allow_lds(kern, lds)) return SGH_EUNSUPPORTED;
    allowed = lds;
  }
  SGH_LAUNCH_TIMED(kern, dim3(unsigned((p.tiles + 7) / 8) * 8u * unsigned(p.mtiles)), dim3(NT), lds, s, a);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

template <int TC, int TP, int WC, int WP>
int launch_slab(const S16Args &a, const D16Plan &p, bool bf16, hipStream_t s) {
  const bool multi = a.KP > KC;
  if (p.slab_ev == 8) {
    if (multi) return bf16 ? launch_slab2<TC, TP, WC, WP, 8, true, true>(a, p, s) : launch_slab2<TC, TP, WC, WP, 8, true, false>(a, p, s);
    return bf16 ? launch_slab2<TC, TP, WC, WP, 8, false, true>(a, p, s) : launch_slab2<TC, TP, WC, WP, 8, false, false>(a, p, s);
  }
  if (multi) return bf16 ? launch_slab2<TC, TP, WC, WP, 4, true, true>(a, p, s) : launch_slab2<TC, TP, WC, WP, 4, true, false>(a, p, s);
  return bf16 ? launch_slab2<TC, TP, WC, WP, 4, false, true>(a, p, s) : launch_slab2<TC, TP, WC, WP, 4, false, false>(a, p, s);
}

// A stride-1 forward convolution is the data gradient of the convolution with the channel roles
// swapped, the taps reversed and pad' = R - 1 - pad: y[ko][p,q] = sum_{c,r',s'} W[ko][c][R-1-r'][S-1-s']
// * x[c][p + pad' - r'][q + pad' - s'].  False when the geometry has no such twin.
bool fwd_twin(const sgh_conv_geom *g, sgh_conv_geom *t, int *fs) {
  // stride 2: the same twin with the input pixel of tap (r', s') at (2p + pad' - r', 2q + pad' - s'), which
  // the pixel-major loader reaches by stepping two gradient pixels per output pixel (D16Args::fs)
  if (g->stride_h != g->stride_w || (g->stride_h != 1 && g->stride_h != 2)) return false;
  if (g->pad_h > g->R - 1 || g->pad_w > g->S - 1) return false;
  *fs = g->stride_h;
  *t = *g;
  t->stride_h = t->stride_w = 1;
  t->C = g->K, t->K = g->C;
  t->H = g->P, t->W = g->Q, t->P = g->H, t->Q = g->W;
  t->pad_h = g->R - 1 - g->pad_h, t->pad_w = g->S - 1 - g->pad_w;
  return true;
}

}  // namespace

static std::atomic<int> g_wgrad16_split_mode{-1};

extern "C" void sgh_conv_wgrad16_split_mode(int mode) {
  g_wgrad16_split_mode.store(mode < 0 ? -1 : (mode ? 1 : 0), std::memory_order_relaxed);
}

size_t sgh_conv16_workspace_bytes(const sgh_conv_geom *g, int which) {
  if (which == SGH_CONV_FWD) {
    sgh_conv_geom t;
    int fs;
    if (!fwd_twin(g, &t, &fs)) return 0;
    const D16Plan p = dplan(&t, fs);
    return p.ok ? p.wt_bytes + p.dyT_bytes : 0;
  }
  if (which == SGH_CONV_WGRAD) {   // (room for either plan)
    const W16Plan p = wplan(g, false), q = wplan(g, true);
    return p.ok ? align256(size_t(p.splits > q.splits ? p.splits : q.splits) * g->K * g->C * g->R * g->S * sizeof(float)) : 0;
  }
  if (which == SGH_CONV_DGRAD) {
    const D16Plan p = dplan(g);
    return p.ok ? p.wt_bytes + p.dyT_bytes : 0;
  }
  return 0;
}

int sgh_conv16_wgrad(const sgh_conv_geom *g, const uint16_t *dy, const uint16_t *x, uint16_t *dW, void *workspace,
                     size_t ws_bytes, bool bf16, hipStream_t s) {
  const int mode = g_wgrad16_split_mode.load(std::memory_order_relaxed);
  const W16Plan p = wplan(g, mode < 0 ? sgh_stream_is_aux(s) : mode != 0);
  if (!p.ok) return SGH_EUNSUPPORTED;
  if (!workspace || ws_bytes < sgh_conv16_workspace_bytes(g, SGH_CONV_WGRAD)) return SGH_EWORKSPACE;
  W16Args a{};
  a.dy = dy, a.x = x, a.partial = static_cast<float *>(workspace);
  a.N = p.f.N, a.C = p.f.C, a.H = p.f.H, a.W = p.f.W, a.K = p.f.K, a.P = p.f.P, a.Q = p.f.Q;
  a.R = p.f.R, a.S = p.f.S, a.pad_h = p.f.pad_h, a.pad_w = p.f.pad_w;
  a.QO = p.QO, a.CRS = g->C * g->R * g->S, a.mtiles = p.mtiles, a.tiles = p.mtiles * p.ntiles, a.splits = p.splits;
  a.chunks = p.chunks, a.chunks_per_split = p.cps;
  a.dy_elems = long(g->N) * g->K * g->P * g->Q, a.x_elems = long(g->N) * g->C * g->H * g->W;
  const double flops = 2.0 * g->N * g->K * g->P * g->Q * double(g->C) * g->R * g->S;
  sgh_prof_kernel_begin("conv_wgrad16/k_wgrad16", flops);
  int rc;
  if (p.bm == 128) {
    if (p.stride == 1) rc = bf16 ? launch_w<128, 1, true>(a, p, s) : launch_w<128, 1, false>(a, p, s);
    else rc = bf16 ? launch_w<128, 2, true>(a, p, s) : launch_w<128, 2, false>(a, p, s);
  } else {
    if (p.stride == 1) rc = bf16 ? launch_w<64, 1, true>(a, p, s) : launch_w<64, 1, false>(a, p, s);
    else rc = bf16 ? launch_w<64, 2, true>(a, p, s) : launch_w<64, 2, false>(a, p, s);
  }
  sgh_prof_kernel_end(s);
  if (rc != SGH_OK) return rc;
  const size_t n = size_t(g->K) * a.CRS;
  if (n / 64 >= size_t(2 * sgh_num_cus()) || p.splits < 16) {
    const dim3 grid(unsigned((n + 63) / 64));
    if (bf16) hipLaunchKernelGGL((k_wgrad16_reduce<64, true>), grid, dim3(256), 0, s, a.partial, p.splits, n, dW);
    else hipLaunchKernelGGL((k_wgrad16_reduce<64, false>), grid, dim3(256), 0, s, a.partial, p.splits, n, dW);
  } else {  // few elements, many splits: more z-lanes
    const dim3 grid(unsigned((n + 15) / 16));
    if (bf16) hipLaunchKernelGGL((k_wgrad16_reduce<16, true>), grid, dim3(256), 0, s, a.partial, p.splits, n, dW);
    else hipLaunchKernelGGL((k_wgrad16_reduce<16, false>), grid, dim3(256), 0, s, a.partial, p.splits, n, dW);
  }
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

namespace {

// `fwd_of`: null for the data gradient of g; otherwise g is the twin (see fwd_twin) of the forward
// geometry *fwd_of, W is that convolution's weight tensor and `bias` its bias (or null)
int run_d16(const sgh_conv_geom *g, const sgh_conv_geom *fwd_of, const uint16_t *dy, const uint16_t *W,
            const uint16_t *bias, uint16_t *dx, void *workspace, size_t ws_bytes, bool bf16, hipStream_t s, int fs = 1,
            bool prelaid = false) {
  const D16Plan p = dplan(g, fs);
  if (!p.ok) return SGH_EUNSUPPORTED;
  const int RS = g->R * g->S;
  const size_t nw = size_t(RS) * p.CP * p.KP;
  if (!workspace || ws_bytes < p.wt_bytes + p.dyT_bytes) return SGH_EWORKSPACE;
  uint16_t *wt = static_cast<uint16_t *>(workspace);
  uint16_t *dyT = p.pixk ? reinterpret_cast<uint16_t *>(static_cast<char *>(workspace) + p.wt_bytes) : nullptr;
  if (p.pixk) {
    const int PQ = g->P * g->Q;
    const dim3 grid(unsigned((PQ + 63) / 64), unsigned((g->K + 63) / 64), unsigned(g->N));
    if (PQ % 2 == 0) hipLaunchKernelGGL(k_pixel_major16<true>, grid, dim3(256), 0, s, dy, dyT, g->K, PQ);
    else hipLaunchKernelGGL(k_pixel_major16<false>, grid, dim3(256), 0, s, dy, dyT, g->K, PQ);
    if (hipGetLastError() != hipSuccess) return SGH_EINVAL;
  }
  if (!fwd_of && prelaid) {
    // re-laid by sgh_conv_dgrad_prepare_multi
  } else if (fwd_of)
    hipLaunchKernelGGL(k_relayout16_fwd, dim3(unsigned((nw + 255) / 256)), dim3(256), 0, s, W, wt, fwd_of->K, fwd_of->C,
                       RS, p.KP, p.CP);
  else
    hipLaunchKernelGGL(k_relayout16, dim3(unsigned((nw + 255) / 256)), dim3(256), 0, s, W, wt, g->K, g->C, RS, p.KP,
                       p.CP);
  if (hipGetLastError() != hipSuccess) return SGH_EINVAL;
  if (p.slab) {
    S16Args b{};
    b.dy = dy, b.wt = wt, b.dx = dx, b.bias = bias;
    b.N = g->N, b.C = g->C, b.H = g->H, b.W = g->W, b.K = g->K, b.KP = p.KP, b.CP = p.CP;
    b.mtiles = p.mtiles, b.ptiles = p.tiles;
    b.Wp = g->W + 1, b.HpWp = (g->H + 1) * (g->W + 1), b.SP = p.slab_sp, b.G = g->N * b.HpWp;
    b.dy_bytes = unsigned(size_t(g->N) * g->K * g->P * g->Q * 2), b.wt_bytes = unsigned(nw * 2);
    const double fl = 2.0 * g->N * g->K * g->P * g->Q * double(g->C) * 9;
    sgh_prof_kernel_begin(fwd_of ? "conv_fwd16/k_dgrad16_slab" : "conv_dgrad16/k_dgrad16_slab", fl);
    int rc;
    if (p.slab == 1) rc = launch_slab<2, 2, 1, 4>(b, p, bf16, s);
    else if (p.slab == 2) rc = launch_slab<2, 2, 2, 4>(b, p, bf16, s);
    else rc = launch_slab<2, 2, 2, 2>(b, p, bf16, s);
    sgh_prof_kernel_end(s);
    return rc;
  }
  D16Args a{};
  a.dy = dy, a.dyT = dyT, a.wt = wt, a.dx = dx, a.bias = bias;
  const sgh_conv_geom *kg = &p.kg;
  a.N = kg->N, a.C = kg->C, a.H = kg->H, a.W = kg->W, a.K = kg->K, a.P = kg->P, a.Q = kg->Q, a.R = kg->R, a.S = kg->S;
  a.stride = kg->stride_h, a.pad_h = kg->pad_h, a.pad_w = kg->pad_w;
  a.dilate = p.dilate ? 1 : 0, a.out_W = g->W, a.out_HW = g->H * g->W;
  a.fs = p.fs;
  a.rowstore = (!p.dilate && kg->stride_h == 1 && kg->W % 2 == 0 && (kg->H * kg->W) % 4 == 0 &&
                (reinterpret_cast<uintptr_t>(dx) & 15u) == 0) ? 1 : 0;
  a.KP = p.KP, a.CP = p.CP, a.mtiles = p.mtiles, a.ptiles = p.tiles;
  for (int i = 0; i < 5; ++i) a.cls_tile0[i] = p.cls_tile0[i];
  a.dy_bytes = unsigned(size_t(g->N) * g->K * g->P * g->Q * 2);
  a.wt_bytes = unsigned(nw * 2);
  const double flops = 2.0 * g->N * g->K * g->P * g->Q * double(g->C) * g->R * g->S;
  sgh_prof_kernel_begin(fwd_of ? "conv_fwd16/k_dgrad16" : "conv_dgrad16/k_dgrad16", flops);
  int rc;
  if (p.pixk) {
    if (p.bm == 128) rc = bf16 ? launch_d<128, true, true>(a, p, s) : launch_d<128, false, true>(a, p, s);
    else rc = bf16 ? launch_d<64, true, true>(a, p, s) : launch_d<64, false, true>(a, p, s);
  } else {
    if (p.bm == 128) rc = bf16 ? launch_d<128, true, false>(a, p, s) : launch_d<128, false, false>(a, p, s);
    else rc = bf16 ? launch_d<64, true, false>(a, p, s) : launch_d<64, false, false>(a, p, s);
  }
  sgh_prof_kernel_end(s);
  return rc;
}

}  // namespace

bool sgh_conv16_dgrad_relayout_dims(const sgh_conv_geom *g, int *CP, int *KP) {
  const D16Plan p = dplan(g);
  if (!p.ok) return false;
  *CP = p.CP, *KP = p.KP;
  return true;
}

int sgh_conv16_dgrad(const sgh_conv_geom *g, const uint16_t *dy, const uint16_t *W, uint16_t *dx, void *workspace,
                     size_t ws_bytes, bool bf16, hipStream_t s, bool prelaid) {
  return run_d16(g, nullptr, dy, W, nullptr, dx, workspace, ws_bytes, bf16, s, 1, prelaid);
}

int sgh_conv16_fwd(const sgh_conv_geom *g, const uint16_t *x, const uint16_t *W, const uint16_t *bias, uint16_t *y,
                   void *workspace, size_t ws_bytes, bool bf16, hipStream_t s) {
  sgh_conv_geom t;
  int fs;
  if (!fwd_twin(g, &t, &fs)) return SGH_EUNSUPPORTED;
  return run_d16(&t, g, x, W, bias, y, workspace, ws_bytes, bf16, s, fs);
}
