// Data gradient of 3x3, pad-1 convolutions (stride 1; stride 2 on even images) with an LDS gradient
// tile shared by all nine taps.
//
//   dx[n][c][h][w] = sum_{k,r,s} dy[n][k][h + 1 - r][w + 1 - s] * W[k][c][r][s]
//
// GEMM view: M = C (128 per workgroup), N = 128 consecutive pixels of the flattened (n, h, w)
// index, reduction = (k, tap).  The reduction runs in chunks of 16 output channels k; per chunk
// the workgroup stages in LDS
//   dyS[kc][vrow][col]   the dy rows its 128 pixels touch (one halo row above / below, halo
//                        columns, zero padding materialised).  Rows are addressed in a "virtual
//                        row" space in which every image owns P + 2 rows (a zero row on top and
//                        at the bottom), so a tile may straddle image boundaries;
//   Ws[kc][m]            the 16 x 128 weight slice of ONE tap, double-buffered across taps.
// Every tap reads its B operand from the same dy tile at a compile-time offset, so the inner loop
// is nothing but LDS reads and MFMAs: no address arithmetic, no predicates, and each dy element is
// fetched from global memory once per chunk instead of nine times.
// 512 threads = 8 wavefronts in a 2 (M) x 4 (N) grid, 64 x 32 per wavefront
// (v_mfma_f32_32x32x2_f32).  The LDS footprint is at most 80 KB and the kernel needs fewer than
// 128 registers, so two workgroups (four wavefronts per SIMD) share a CU and one's staging work
// and barriers overlap the other's MFMAs.
#include <stdlib.h>

#include "common.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr int NT = 512;
constexpr int BN = 128, KC = 16;
constexpr int kOOB = int(0x80000000u);
#ifndef D3_LAT
#define D3_LAT 2
#endif

__device__ __forceinline__ rsrc_t make_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, bytes, 0x00020000);
}

struct D3Args {
  const float *dy, *wt;   // wt: re-laid weights [tap][KP][C]
  const float *bias;      // per output channel, added when a tile is finished (NULL: none)
  int accumulate;         // dx += result instead of dx = result (gradient fan-in folded into the store)
  float *dx;
  int N, C, H, W, K, KP;  // dx is N x C x H x W
  int P, Q;               // dy is N x K x P x Q (stride 1: P == H, Q == W; stride 2: H == 2P, W == 2Q)
  int total_pix;          // N * P * Q: pixels of the tile index space
  // Work assignment (1-D grid).  Tile t = (pixel tile t / ctiles, channel tile t % ctiles).  Workgroups
  // [0, dp_tiles) take one whole tile each; workgroup dp_tiles + g takes units
  // [g * sk_units / sk_wgs, (g + 1) * sk_units / sk_wgs) of the remaining tiles, a unit being one
  // reduction chunk of one tile (unit u = tile dp_tiles + u / nchunks, chunk u % nchunks).
  int ctiles, dp_tiles, sk_wgs;
  long sk_units;
  int xcd_runs;           // whole-tile workgroups take their tiles in runs per XCD (whole_tile_of)
  float *partials;        // [sk_wgs][2][classes * BM * BN]: a workgroup's first / last incomplete tile
  unsigned dy_bytes, wt_bytes;
};

// Tile of whole-tile workgroup w.  Workgroup w runs on XCD w % 8 and every XCD has an L2 of its own, so the
// j-th workgroup of XCD x takes tile ((j / 8) * 8 + x) * 8 + j % 8: an XCD works on runs of eight consecutive
// tiles at a time, which share the halo rows of their dy slabs (and, for several channel tiles per pixel
// tile, the whole slab) in its L2.  Measured on the ResNet-18 layers: the kernels fetch a third to a quarter of
// the bytes into L2 (C64 56x56: 246 -> 65 MB per launch) at the same speed; whole contiguous ranges per XCD, and
// the same treatment of the workgroups that share tiles, ran 1.5-3 % slower.  Only which hardware computes
// which tile changes: results are identical.
__device__ __forceinline__ int whole_tile_of(const D3Args &a, int w) {
  if (!a.xcd_runs) return w;
  const int x = w & 7, j = w >> 3;
  return (((j >> 3) << 3) + x) * 8 + (j & 7);
}

// LOGP: log2 of the LDS row pitch (>= W + 2); VR: virtual rows held per channel.
// BM: output channels per workgroup (64 or 128; the wavefront tile is (BM/2) x 32).
//
// The reduction is a flat sequence of tap steps (chunk, tap).  Global loads run LAT steps ahead of
// their LDS write: the data written at the end of step q (tap q+1's weights, a ninth of the next
// chunk's dy slab) was requested at the start of step q - LAT and waits in registers, so a
// request has LAT + 1 steps of MFMA time to return.  Every load address is "thread constant +
// scalar term" (one vector add); the thread constant is out of range for elements that must read
// as zero, and K is a multiple of 16, so no per-load predicate is left.
//
// S2 (stride 2, pad 1, even H and W): the tile index space is the P x Q grid of one residue class
// (h, w) = (2i + a, 2j + b); all four classes of a pixel block are accumulated by the same
// workgroup (tap (r, s) belongs to class a = (r != 1), b = (s != 1) and reads dy[i + (r == 0)]
// [j + (s == 0)]), so no MFMA is spent on the zeros of a dilated gradient, every tap is still a
// compile-time LDS offset, and a lane stores its 2 x 2 output block as two 8-byte writes.
template <int BM, int LOGP, int VR, bool S2>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(2, 4))) void k_dgrad3x3(D3Args a) {
  constexpr int NCLS = S2 ? 4 : 1;          // residue classes accumulated side by side
  constexpr int PA = BM;                    // weight tile pitch
  constexpr int TM = BM / 64;               // 32-row MFMA tiles per wavefront
  constexpr int PITCHP = 1 << LOGP;
  constexpr int VRP = VR * PITCHP;          // floats per channel slab
  constexpr int CHS = VRP;                   // channel stride in LDS (a wavefront's two 32-lane halves are served separately)
  constexpr int DSLOTS = KC * VRP / NT;     // dy elements per thread per chunk
  constexpr int SPT = (DSLOTS + 8) / 9;     // dy slots fetched per tap step
  constexpr int SUB = VRP > NT ? VRP / NT : 1;   // passes of the 512 threads over one channel slab
  constexpr int KPP = VRP > NT ? 1 : NT / VRP;   // channels covered by one pass
  constexpr int LAT = D3_LAT;               // tap steps between a load and its LDS write
  static_assert(KC * VRP % NT == 0 && (NT % VRP == 0 || VRP % NT == 0), "slab must tile over the threads");
  static_assert(9 % (LAT + 1) == 0, "the staging registers rotate with the tap index");

  extern __shared__ float smem[];
  float *Ws = smem;                         // [2][KC][PA]
  float *dyS = smem + 2 * KC * PA;          // [2][KC][CHS]

  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = wave >> 2, wn = wave & 3;  // 2 x 4 wavefronts, 64 x 32 each
  const int HW = a.H * a.W, PQ = a.P * a.Q;
  const int VH = S2 ? a.P + 1 : a.P + 2;    // virtual rows per image: its dy rows plus the zero rows a tap can reach
  const rsrc_t rdy = make_rsrc(a.dy, a.dy_bytes), rw = make_rsrc(a.wt, a.wt_bytes);
  const int nchunks = a.KP / KC;

  // ---- this workgroup's work: one whole tile, or a run of (tile, chunk) units that may span tiles
  const bool stream = int(blockIdx.x) >= a.dp_tiles;
  const int sk_g = int(blockIdx.x) - a.dp_tiles;
  long u = stream ? sk_g * a.sk_units / a.sk_wgs : 0;
  const long u_end = stream ? (sk_g + 1) * a.sk_units / a.sk_wgs : 0;
  const int first_tile = int(u / nchunks);
  for (bool again = true; again;) {
  int tile, ch_begin, ch_end, tile_rel = 0;
  if (!stream) {
    tile = whole_tile_of(a, int(blockIdx.x));
    ch_begin = 0;
    ch_end = nchunks;
    again = false;
  } else {
    if (u >= u_end) break;
    tile_rel = int(u / nchunks);
    tile = a.dp_tiles + tile_rel;
    ch_begin = int(u - long(tile_rel) * nchunks);
    ch_end = int(min(long(nchunks), ch_begin + (u_end - u)));
    u += ch_end - ch_begin;
  }
  const bool whole = ch_begin == 0 && ch_end == nchunks;
  const int c0 = (tile % a.ctiles) * BM;
  const int pix0 = (tile / a.ctiles) * BN;

  // first virtual row of the slab: the row above the tile's first pixel row
  const int n_first = pix0 / PQ, h_first = (pix0 - n_first * PQ) / a.Q;
  const int vbase = n_first * VH + h_first;  // stride 1: virtual row of dy row (h_first - 1); stride 2: of row h_first

  // ---- dy slab loader ------------------------------------------------------------------------
  // slot e covers channel kc = (e / SUB) * KPP + tkc and slab element within = (e % SUB) * NT + tw:
  // virtual row vr = within >> LOGP, column col = within % PITCHP; dy row p = (vbase + vr) % VH - 1
  // of image (vbase + vr) / VH, dy column q = col - 1.  The byte offset splits into a thread part
  // g0 (kOOB for halo / padding elements) and the scalar (k0 + (e / SUB) * KPP) * P * Q * 4.
  // (Stride 2: no halo row above or column to the left, p = (vbase + vr) % VH, q = col.)
  const int tkc = VRP > NT ? 0 : t / VRP, tw = VRP > NT ? t : t % VRP;
  int g0[SUB];
#pragma unroll
  for (int sub = 0; sub < SUB; ++sub) {
    const int within = sub * NT + tw, vr = within >> LOGP, col = within & (PITCHP - 1);
    const int v = vbase + vr, n = v / VH, p = v - n * VH - (S2 ? 0 : 1), q = col - (S2 ? 0 : 1);
    const bool ok = n < a.N && unsigned(p) < unsigned(a.P) && unsigned(q) < unsigned(a.Q);
    g0[sub] = ok ? (((n * a.K + tkc) * a.P + p) * a.Q + q) * 4 : kOOB;
  }
  const int l0 = tkc * CHS + tw;
  auto dy_get = [&](int e, int k0) -> float {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_raw_buffer_load_b32(rdy, g0[e % SUB] + (k0 + (e / SUB) * KPP) * PQ * 4, 0, 0));
  };
  auto dy_loff = [&](int e) -> int { return l0 + (e / SUB) * KPP * CHS + (e % SUB) * NT; };

  // ---- weight tile loader: one 128-bit load per thread per tap step ------------------------
  // (BM == 64: the upper half of the threads has no weight element to fetch)
  constexpr int WV = BM / 4;                     // float4 per weight row
  const int w_kc = t / WV, w_m = (t % WV) * 4;   // 16 rows x WV float4
  const int w0 = (c0 + w_m + 3 < a.C) && (w_kc < KC) ? (w_kc * a.C + c0 + w_m) * 4 : kOOB;
  auto w_get = [&](int tap, int k0) -> v4f {
    return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rw, w0 + (tap * a.KP + k0) * a.C * 4, 0, 0));
  };
  auto w_put = [&](v4f v, float *dst) {
    if (BM == 128 || wave < 4) *reinterpret_cast<v4f *>(dst + w_kc * PA + w_m) = v;
  };

  // ---- this lane's pixel (B operand column) ------------------------------------------------
  const int pix = pix0 + wn * 32 + (lane & 31);
  const int pixc = pix < a.total_pix ? pix : a.total_pix - 1;  // a tail lane computes a valid pixel, stores nothing
  const int pn = pixc / PQ, prem = pixc - pn * PQ, ph_ = prem / a.Q, pw_ = prem - ph_ * a.Q;
  // LDS offset of tap (r = 2, s = 2); tap (r, s) adds (2 - r) * PITCHP + (2 - s):
  //   dy row h + 1 - r  ->  virtual row pn*VH + h + 2 - r ; slab column of q = w + 1 - s is w + 2 - s
  const int boff = (pn * VH + ph_ - vbase) * PITCHP + pw_ + (lane >> 5) * CHS;
  const int aoff = (lane >> 5) * PA + wm * (BM / 2) + (lane & 31);

  v16f acc[NCLS * TM];
#pragma unroll
  for (int i = 0; i < NCLS * TM; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

  // Staging registers.  Step q (tap q % 9 of chunk q / 9) requests what step q + LAT writes: the
  // weights of step q + LAT + 1 and dy slots [td * SPT, (td + 1) * SPT) of the chunk after step
  // q + LAT's, td = (q + LAT) % 9.  Requests past the last chunk land in buffers nobody reads.
  v4f wst[LAT + 1];
  float dst[LAT + 1][SPT];
  auto request = [&](int tq, int ch) {  // tq: tap index relative to chunk ch (negative during warm-up)
    const int slot = ((tq % (LAT + 1)) + LAT + 1) % (LAT + 1);
    const int qw = tq + LAT + 1, qd = tq + LAT;
    wst[slot] = w_get(qw % 9, (ch + qw / 9) * KC);
#pragma unroll
    for (int j = 0; j < SPT; ++j) {
      const int e = (qd % 9) * SPT + j;
      if (e < DSLOTS) dst[slot][j] = dy_get(e, (ch + 1 + qd / 9) * KC);
    }
  };

  // prologue: the first chunk's dy slab and tap 0's weights, then the requests of the LAT steps
  // that would have preceded step 0
#pragma unroll
  for (int e = 0; e < DSLOTS; ++e) dyS[dy_loff(e)] = dy_get(e, ch_begin * KC);
  w_put(w_get(0, ch_begin * KC), Ws);
#pragma unroll
  for (int tq = -LAT; tq < 0; ++tq) request(tq, ch_begin);
  __syncthreads();

  int dcur = 0, wcur = 0;
  for (int ch = ch_begin; ch < ch_end; ++ch) {
    const float *dys = dyS + dcur * (KC * CHS) + boff;
    float *dyn = dyS + (dcur ^ 1) * (KC * CHS);
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) {
      const int r = tap / 3, s = tap - r * 3;
      const int toff = S2 ? (r == 0) * PITCHP + (s == 0) : (2 - r) * PITCHP + (2 - s);
      const int cls = S2 ? 2 * (r != 1) + (s != 1) : 0;
      const float *ws = Ws + wcur * (KC * PA) + aoff;
      request(tap, ch);
#pragma unroll
      for (int kk = 0; kk < KC; kk += 2) {
        const float b = dys[kk * CHS + toff];
#pragma unroll
        for (int i = 0; i < TM; ++i)
          acc[cls * TM + i] =
              __builtin_amdgcn_mfma_f32_32x32x2f32(ws[kk * PA + i * 32], b, acc[cls * TM + i], 0, 0, 0);
      }
      // what step (tap - LAT) requested: tap + 1's weights and this tap's share of the next slab
      const int slot = ((tap - LAT) % (LAT + 1) + LAT + 1) % (LAT + 1);
      w_put(wst[slot], Ws + (wcur ^ 1) * (KC * PA));
#pragma unroll
      for (int j = 0; j < SPT; ++j) {
        const int e = tap * SPT + j;
        if (e < DSLOTS) dyn[dy_loff(e)] = dst[slot][j];
      }
      __syncthreads();
      wcur ^= 1;
    }
    dcur ^= 1;
  }

  // epilogue.  A finished tile goes to dx[n][c][h][w] (this lane's pixel, rows c0 + wm*(BM/2) + i*32 +
  // 8*(v/4) + 4*(lane/32) + v%4); an incomplete one to this workgroup's partial slot as
  // [class][row][pixel], to be summed by k_dgrad3x3_fixup.
  // (the lane term is laundered through an empty asm so that the epilogue's address arithmetic is
  // not hoisted out of the segment loop, where it would occupy registers during the MFMA loop)
  int lhalf = lane >> 5;
  asm volatile("" : "+v"(lhalf));
  if (!whole) {
    float *ps = a.partials + (size_t(sk_g) * 2 + (tile_rel == first_tile ? 0 : 1)) * (NCLS * BM * BN) +
                (wm * (BM / 2) + 4 * lhalf) * BN + wn * 32 + (lane & 31);
#pragma unroll
    for (int cl = 0; cl < NCLS; ++cl)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) ps[(cl * BM + i * 32 + 8 * (v >> 2) + (v & 3)) * BN] = acc[cl * TM + i][v];
  } else if (pix < a.total_pix) {
    if (S2) {
      typedef float v2f __attribute__((ext_vector_type(2)));
      float *o = a.dx + size_t(pn) * a.C * HW + (2 * ph_) * a.W + 2 * pw_;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int c = c0 + wm * (BM / 2) + i * 32 + 8 * (v >> 2) + 4 * lhalf + (v & 3);
          if (c < a.C) {
            const float bb = a.bias ? a.bias[c] : 0.f;
            float *oc = o + size_t(c) * HW;
            v2f r0 = v2f{acc[0 * TM + i][v] + bb, acc[1 * TM + i][v] + bb};
            v2f r1 = v2f{acc[2 * TM + i][v] + bb, acc[3 * TM + i][v] + bb};
            if (a.accumulate) r0 += *reinterpret_cast<const v2f *>(oc), r1 += *reinterpret_cast<const v2f *>(oc + a.W);
            *reinterpret_cast<v2f *>(oc) = r0;
            *reinterpret_cast<v2f *>(oc + a.W) = r1;
          }
        }
    } else {
      float *o = a.dx + size_t(pn) * a.C * HW + prem;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int c = c0 + wm * (BM / 2) + i * 32 + 8 * (v >> 2) + 4 * lhalf + (v & 3);
          if (c < a.C) {
            float r = a.bias ? acc[i][v] + a.bias[c] : acc[i][v];
            if (a.accumulate) r += o[size_t(c) * HW];
            o[size_t(c) * HW] = r;
          }
        }
    }
  }
  }  // next segment (the last tap step ended with a barrier: the LDS buffers are free)
}

// Finishes the tiles that several workgroups shared: tile r of the shared region covers units
// [r * nchunks, (r + 1) * nchunks); the workgroups whose unit ranges meet it are visited in
// ascending order (= ascending chunk order) and their partial tiles summed, so the result does
// not depend on timing.  A tile that one workgroup computed alone was already stored by it.
// (I: the integer type of the unit arithmetic -- 32 bits wherever the products fit, which is every layer of the
// benchmark networks: without the 64-bit divisions of the owner search a launch on 128-row tiles takes 9.6
// instead of 11.3 us)
template <int BM, bool S2, class I>
__device__ __forceinline__ void dgrad3x3_fixup_body(const D3Args &a) {
  constexpr int NCLS = S2 ? 4 : 1;
  const int nchunks = a.KP / KC;
  const int r = blockIdx.x;
  const I x0 = I(r) * I(nchunks), x1 = x0 + I(nchunks) - 1;
  const I units = I(a.sk_units), wgs = I(a.sk_wgs);
  auto start = [&](I g) -> I { return g * units / wgs; };
  auto owner = [&](I x) -> int {
    I g = x * wgs / units;
    while (g + 1 < wgs && start(g + 1) <= x) ++g;
    while (g > 0 && start(g) > x) --g;
    return int(g);
  };
  const int g_lo = owner(x0), g_hi = owner(x1);
  if (g_lo == g_hi) return;
  const int tile = a.dp_tiles + r;
  const int c0 = (tile % a.ctiles) * BM, pix0 = (tile / a.ctiles) * BN;
  const int HW = a.H * a.W, PQ = a.P * a.Q;
  // a block covers 8 rows of the tile, a thread 4 consecutive pixels of one row
  typedef float v4f __attribute__((ext_vector_type(4)));
  typedef float v2f __attribute__((ext_vector_type(2)));
  const int m = blockIdx.y * 8 + (threadIdx.x >> 5), col = (threadIdx.x & 31) * 4;
  const int c = c0 + m;
  if (c >= a.C) return;
  v4f s[NCLS];
#pragma unroll
  for (int cl = 0; cl < NCLS; ++cl) s[cl] = v4f{0.f, 0.f, 0.f, 0.f};
  for (int g = g_lo; g <= g_hi; ++g) {
    const int slot = int(start(I(g)) / I(nchunks)) == r ? 0 : 1;
    const float *ps = a.partials + (size_t(g) * 2 + slot) * (NCLS * BM * BN) + m * BN + col;
#pragma unroll
    for (int cl = 0; cl < NCLS; ++cl) s[cl] += *reinterpret_cast<const v4f *>(ps + cl * BM * BN);
  }
  const float bb = a.bias ? a.bias[c] : 0.f;
  int pix = pix0 + col;
  int pn = pix / PQ, prem = pix - pn * PQ;
  if (!S2 && (PQ & 3) == 0 && pix + 3 < a.total_pix) {  // the four pixels lie in one image, 16-byte aligned
    v4f *o = reinterpret_cast<v4f *>(a.dx + (size_t(pn) * a.C + c) * HW + prem);
    *o = a.accumulate ? *o + (s[0] + bb) : s[0] + bb;
    return;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j, ++pix) {
    if (pix >= a.total_pix) break;
    if (S2) {
      const int i = prem / a.Q, jj = prem - i * a.Q;
      float *o = a.dx + (size_t(pn) * a.C + c) * HW + (2 * i) * a.W + 2 * jj;
      v2f r0 = v2f{s[0][j] + bb, s[NCLS > 1 ? 1 : 0][j] + bb};
      v2f r1 = v2f{s[NCLS > 2 ? 2 : 0][j] + bb, s[NCLS > 3 ? 3 : 0][j] + bb};
      if (a.accumulate) r0 += *reinterpret_cast<const v2f *>(o), r1 += *reinterpret_cast<const v2f *>(o + a.W);
      *reinterpret_cast<v2f *>(o) = r0;
      *reinterpret_cast<v2f *>(o + a.W) = r1;
    } else {
      float *o = a.dx + (size_t(pn) * a.C + c) * HW + prem;
      *o = a.accumulate ? *o + (s[0][j] + bb) : s[0][j] + bb;
    }
    if (++prem == PQ) prem = 0, ++pn;
  }
}

template <int BM, bool S2>
__global__ __launch_bounds__(256) void k_dgrad3x3_fixup(D3Args a) {
  if (a.sk_units * (a.sk_wgs + 1) < (long(1) << 31)) dgrad3x3_fixup_body<BM, S2, unsigned>(a);
  else dgrad3x3_fixup_body<BM, S2, long>(a);
}

struct D3Plan {
  bool ok, s2;
  int bm, logp, vr;
  int ctiles, tiles, dp_tiles, sk_wgs;  // whole-tile workgroups, then sk_wgs workgroups sharing the rest
  long sk_units;
  size_t lds;
};

inline D3Plan plan(const sgh_conv_geom *g) {
  D3Plan p{};
  p.ok = false;
  if (g->R != 3 || g->S != 3 || g->pad_h != 1 || g->pad_w != 1 || g->stride_h != g->stride_w) return p;
  p.s2 = g->stride_h == 2;
  if (g->stride_h != 1 && !p.s2) return p;
  if (p.s2 && (g->H != 2 * g->P || g->W != 2 * g->Q)) return p;  // even image: four residue classes of equal size
  if (g->C < 64 || g->C % 4 != 0 || g->K % KC != 0 || g->Q < 2) return p;
  if (sgh_env().dgrad3x3_off) return p;
  // slab columns: stride 1 has a halo column on both sides, stride 2 one zero column on the right
  const int cols = p.s2 ? g->Q + 1 : g->Q + 2;
  if (cols > 64) return p;
  p.logp = cols <= 8 ? 3 : (cols <= 16 ? 4 : (cols <= 32 ? 5 : 6));
  if (!p.s2 && p.logp < 4) p.logp = 4;
  // virtual rows a 128-pixel tile can touch: its pixel rows, the halo rows (stride 1: one each
  // side; stride 2: one below), and the zero rows of every image boundary it crosses
  const int rows = (BN + g->Q - 2) / g->Q + 1;
  const int crossings = (BN - 1) / (g->P * g->Q) + 1;
  const int need = p.s2 ? rows + 1 + crossings : rows + 2 + 2 * crossings;
  if (p.s2) {
    // instantiated: pitch 32 x 8 rows, pitch 16 x 16 rows, pitch 8 x 32 rows (256 floats per channel)
    if (p.logp == 6) return p;
    p.vr = 256 >> p.logp;
    p.bm = 64;  // four classes x 16 accumulators per 32-row tile: the 64-row tile keeps two workgroups per CU
  } else {
    if (p.logp == 6) p.vr = 8;
    else if (p.logp == 5) p.vr = 16;
    else p.vr = need <= 16 ? 16 : 32;
    p.bm = (g->C % 128 == 0 || g->C > 192) ? 128 : 64;
    if (sgh_env().dgrad3x3_bm) p.bm = sgh_env().dgrad3x3_bm;
  }
  if (need > p.vr) return p;
  const size_t chs = size_t(p.vr) * (1u << p.logp);
  p.lds = (size_t(2) * KC * (p.bm) + size_t(2) * KC * chs) * sizeof(float);
  if (p.lds > 160 * 1024) return p;
  const size_t lim = size_t(1) << 31;
  const size_t dx_elems = size_t(g->N) * g->C * g->H * g->W;
  if (size_t(g->N) * g->K * g->P * g->Q * 4 >= lim || dx_elems * 4 >= lim) return p;
  if (size_t(g->N) * (g->P + 2) + p.vr >= lim / 64) return p;
  // Work balance.  Whole multiples of the CU count of tiles run one tile per workgroup; the
  // remaining tiles (all of them when there are fewer tiles than CUs) are cut into (tile, chunk)
  // units and dealt evenly to one workgroup per CU (two per CU measured slower: twice the
  // partial tiles to write and sum), so that no CU is left with a whole extra tile while others idle.  Tiles shared between workgroups are finished by
  // k_dgrad3x3_fixup in a fixed order: results stay run-to-run identical.
  const int cus = sgh_num_cus();
  const int nchunks = (g->K + KC - 1) / KC;
  p.ctiles = (g->C + p.bm - 1) / p.bm;
  const long tiles = long(p.ctiles) * ((long(g->N) * g->P * g->Q + BN - 1) / BN);
  if (tiles >= (long(1) << 30)) return p;
  p.tiles = int(tiles);
  p.dp_tiles = int(tiles / cus * cus);
  p.sk_units = long(p.tiles - p.dp_tiles) * nchunks;
  p.sk_wgs = int(p.sk_units < cus ? p.sk_units : cus);
  p.ok = true;
  return p;
}

template <int BM, int LOGP, int VR, bool S2>
int launch(const D3Args &a, const D3Plan &p, dim3 grid, hipStream_t s) {
  auto kern = k_dgrad3x3<BM, LOGP, VR, S2>;
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

bool sgh_dgrad3x3_supported(const sgh_conv_geom *g) { return plan(g).ok; }

// Extra workspace (bytes, after the re-laid weights) for split-reduction partial images.
size_t sgh_dgrad3x3_partial_bytes(const sgh_conv_geom *g) {
  const D3Plan p = plan(g);
  if (!p.ok || p.sk_wgs == 0) return 0;
  return size_t(p.sk_wgs) * 2 * (p.s2 ? 4 : 1) * p.bm * BN * sizeof(float);
}

// `wt` holds the weights re-laid as [tap][KP][C] (KP = K rounded up to 16, zero rows beyond K);
// `partials` is sgh_dgrad3x3_partial_bytes(g) bytes of scratch (may be NULL when that is 0).
int sgh_dgrad3x3_run(const sgh_conv_geom *g, const float *dy, const float *wt, int KP, float *dx, float *partials,
                     hipStream_t s, const char *tag, const float *bias, bool accumulate) {
  const D3Plan p = plan(g);
  if (!p.ok) return SGH_EUNSUPPORTED;
  if (p.sk_wgs > 0 && !partials) return SGH_EWORKSPACE;
  D3Args a;
  a.dy = dy;
  a.wt = wt;
  a.bias = bias;
  a.accumulate = accumulate ? 1 : 0;
  a.dx = dx;
  a.N = g->N;
  a.C = g->C;
  a.H = g->H;
  a.W = g->W;
  a.K = g->K;
  a.KP = KP;
  a.P = g->P;
  a.Q = g->Q;
  a.total_pix = g->N * g->P * g->Q;
  a.ctiles = p.ctiles;
  a.xcd_runs = p.dp_tiles % 64 == 0 && !sgh_env().conv_xcd_off;
  a.dp_tiles = p.dp_tiles;
  a.sk_wgs = p.sk_wgs;
  a.sk_units = p.sk_units;
  a.partials = partials;
  a.dy_bytes = unsigned(size_t(g->N) * g->K * g->P * g->Q * 4);
  a.wt_bytes = unsigned(size_t(9) * KP * g->C * 4);
  dim3 grid(unsigned(p.dp_tiles + p.sk_wgs), 1, 1);
  int rc = SGH_EUNSUPPORTED;
  sgh_prof_kernel_begin(tag, 2.0 * g->N * g->K * g->P * g->Q * g->C * 9);
#define D3_CASE(BM_, LOGP_, VR_) \
  if (!p.s2 && p.bm == BM_ && p.logp == LOGP_ && p.vr == VR_) rc = launch<BM_, LOGP_, VR_, false>(a, p, grid, s);
#define D3_CASE_S2(LOGP_, VR_) \
  if (p.s2 && p.bm == 64 && p.logp == LOGP_ && p.vr == VR_) rc = launch<64, LOGP_, VR_, true>(a, p, grid, s);
  D3_CASE(128, 6, 8)
  D3_CASE(64, 6, 8)
  D3_CASE(128, 5, 16)
  D3_CASE(64, 5, 16)
  D3_CASE(128, 4, 16)
  D3_CASE(64, 4, 16)
  D3_CASE(128, 4, 32)
  D3_CASE(64, 4, 32)
  D3_CASE_S2(5, 8)
  D3_CASE_S2(4, 16)
  D3_CASE_S2(3, 32)
#undef D3_CASE
#undef D3_CASE_S2
  sgh_prof_kernel_end(s);
  if (rc != SGH_OK) return rc;
  if (p.sk_wgs > 0) {
    const int shared_tiles = p.tiles - p.dp_tiles;
    const dim3 fgrid(shared_tiles, p.bm / 8);
    if (p.s2) hipLaunchKernelGGL((k_dgrad3x3_fixup<64, true>), fgrid, dim3(256), 0, s, a);
    else if (p.bm == 64) hipLaunchKernelGGL((k_dgrad3x3_fixup<64, false>), fgrid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((k_dgrad3x3_fixup<128, false>), fgrid, dim3(256), 0, s, a);
    if (hipGetLastError() != hipSuccess) return SGH_EINVAL;
  }
  return SGH_OK;
}
