// Weight gradient of 3x3 stride-1 convolutions with an LDS input tile shared by all nine taps.
//
//   dW[k][c][r][s] = sum_{n,p,q} dy[n][k][p][q] * x[n][c][p - ph + r][q - pw + s]
//
// A workgroup owns BM output channels x BC input channels x 9 taps and walks "units" of the
// reduction: RU consecutive output rows of one image (<= 64 pixels).  Per unit it stages in LDS
//   dyS[pixel][m]            the BM x (RU*Q) slice of dy (MFMA A operand, k = pixel),
//   xS[c][row][col]          the BC x (RU+2) x (W+2) input slab, zero padding materialised,
// and every tap (r, s) reads its B operand from the SAME slab at offset r*pitch + s.  Each input
// element is therefore fetched once per unit instead of once per tap, the address arithmetic of an
// im2col gather disappears from the inner loop, and one operand fetch feeds nine MFMAs.
// The four wavefronts tile (BM/32) x (BC/32); each holds 9 accumulator tiles of 32x32
// (v_mfma_f32_32x32x2_f32: 144 accumulator registers).  The next unit's global loads are spread
// over the k-step groups of the current unit and land in the other LDS buffer.
//
// The reduction is split over workgroups (grid.z); partials are written as [split][tap][K][C] and
// summed in ascending split order by k_wgrad3x3_reduce: results are run-to-run identical.
#include <stdlib.h>

#include "common.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr int NT = 512;
constexpr int UPIXP = 64;        // padded pixels per unit (k dimension of one unit)
constexpr int kOOB = int(0x80000000u);

__device__ __forceinline__ rsrc_t make_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, bytes, 0x00020000);
}
__device__ __forceinline__ float buf_ld(rsrc_t r, int elem_off, int ok) {
  const int m = -ok;
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, ((elem_off << 2) & m) | (kOOB & ~m), 0, 0));
}

struct W3Args {
  const float *dy, *x;
  float *part;           // [splits][9][K][C]
  int N, C, H, W, K, P, Q, ph, pw;
  int RU;                // output rows per unit
  int units_per_image;   // ceil(P / RU)
  int total_units, units_per_split;
  unsigned dy_bytes, x_bytes;
};

// LOGP: log2 of the LDS row pitch (>= W + 2); ROWS = RU + 2 slab rows.
// 512 threads = 8 wavefronts: wavefronts 0-3 and 4-7 each tile the same (BM/32) x (BC/32) output
// block but take the first / second half of every unit's k-steps, and write separate partials
// (split index 2*z + half).  Two wavefronts per SIMD share one LDS tile, so one wavefront's
// address arithmetic and memory waits overlap the other's MFMAs (within a single wavefront
// VALU work does not overlap its own MFMAs).
template <int BM, int BC, int LOGP, int ROWS>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_wgrad3x3(W3Args a) {
  constexpr int PITCHP = 1 << LOGP;
  constexpr int PA = BM + 1;                         // dyS pitch: odd, so the pixel-major staging writes spread over banks
  constexpr int CHS = ROWS * PITCHP + 1;             // xS channel stride: odd -> lanes (channels) hit distinct banks
  constexpr int XBUF = BC * CHS;                     // one x buffer
  constexpr int ZPAD = 3 * PITCHP;                   // always-zero area read by the padded pixels of a short unit
  constexpr int WGC = BC / 32, WGM = 4 / WGC;
  static_assert(BM == WGM * 32, "four wavefronts of 32 rows x 32 channels per half");
  constexpr int DSLOTS = BM * UPIXP / NT;            // dy elements per thread per unit
  constexpr int XSLOTS = (BC * ROWS * PITCHP + NT - 1) / NT;
  constexpr int G = 2;                               // k-steps per software-pipeline group
  constexpr int NGMAX = UPIXP / 2 / 2 / G;           // groups per wavefront for a full unit
  constexpr int DPG = (DSLOTS + NGMAX - 1) / NGMAX + 1;
  constexpr int XPG = (XSLOTS + NGMAX - 1) / NGMAX + 1;

  extern __shared__ float smem[];
  float *dyS = smem;                                  // [2][UPIXP][PA]
  float *xS = smem + 2 * UPIXP * PA;                  // [2][BC][CHS], then ZPAD zeros, then 64 dummy words

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int half = wave >> 2, w4 = wave & 3;
  const int wm = w4 / WGC, wc = w4 % WGC;
  const int k0 = blockIdx.x * BM, c0 = blockIdx.y * BC;
  const int u_begin = blockIdx.z * a.units_per_split;
  const int u_end = min(u_begin + a.units_per_split, a.total_units);
  const rsrc_t rdy = make_rsrc(a.dy, a.dy_bytes), rx = make_rsrc(a.x, a.x_bytes);
  const int PQ = a.P * a.Q, HW = a.H * a.W;

  // the zero area is written once; the slabs (pad columns included) are fully rewritten per unit
  for (int i = t; i < 2 * XBUF + ZPAD; i += NT) xS[i] = 0.f;

  v16f acc[9];
#pragma unroll
  for (int i = 0; i < 9; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

  // ---- per-unit loaders -------------------------------------------------------------------
  auto unit_geom = [&](int u, int &n, int &p0, int &upix) {
    n = u / a.units_per_image;
    p0 = (u - n * a.units_per_image) * a.RU;
    const int rows = min(a.RU, a.P - p0);
    upix = rows * a.Q;
  };
  auto dy_get = [&](int e, int n, int p0, int upix) -> float {
    const int idx = e * NT + t, pix = idx & (UPIXP - 1), m = idx >> 6;
    const int ok = int(unsigned(e) < unsigned(DSLOTS)) & int(pix < upix) & int(k0 + m < a.K);
    return buf_ld(rdy, (n * a.K + k0 + m) * PQ + p0 * a.Q + pix, ok);
  };
  // The staging writes are branch-free: a slot outside the slab goes to a per-lane dummy word, so
  // that a k-step group stays one straight-line scheduling region.
  float *const dummy = xS + 2 * XBUF + ZPAD + lane;
  auto dy_put = [&](int e, float v, float *dst) {
    const int idx = e * NT + t, pix = idx & (UPIXP - 1), m = idx >> 6;
    float *p = unsigned(e) < unsigned(DSLOTS) ? dst + pix * PA + m : dummy;
    *p = v;
  };
  auto x_get = [&](int e, int n, int p0, int live) -> float {
    const int idx = e * NT + t, col = idx & (PITCHP - 1), rc = idx >> LOGP, c = rc / ROWS, row = rc - c * ROWS;
    const int h = p0 - a.ph + row, w = col - a.pw;
    const int ok = live & int(e >= 0) & int(c < BC) & int(c0 + c < a.C) & int(unsigned(h) < unsigned(a.H)) &
                   int(unsigned(w) < unsigned(a.W));
    return buf_ld(rx, (n * a.C + c0 + c) * HW + h * a.W + w, ok);
  };
  auto x_put = [&](int e, float v, float *dst) {
    const int idx = e * NT + t, col = idx & (PITCHP - 1), rc = idx >> LOGP, c = rc / ROWS, row = rc - c * ROWS;
    float *p = (e >= 0) & (c < BC) ? dst + c * CHS + row * PITCHP + col : dummy;
    *p = v;
  };

  if (u_begin < u_end) {
    int n, p0, upix;
    unit_geom(u_begin, n, p0, upix);
    __syncthreads();  // zero fill done before the first slab lands
    for (int e = 0; e < DSLOTS; ++e) dy_put(e, dy_get(e, n, p0, upix), dyS);
    for (int e = 0; e < XSLOTS; ++e) x_put(e, x_get(e, n, p0, 1), xS);
  }
  __syncthreads();

  int cur = 0;
  for (int u = u_begin; u < u_end; ++u) {
    int n, p0, upix;
    unit_geom(u, n, p0, upix);
    int nn, np0, nupix;
    const bool more = u + 1 < u_end;
    unit_geom(more ? u + 1 : u, nn, np0, nupix);
    if (!more) nupix = 0;

    const float *dcur = dyS + cur * (UPIXP * PA);
    const float *xcur = xS + cur * XBUF;
    float *dnxt = dyS + (cur ^ 1) * (UPIXP * PA);
    float *xnxt = xS + (cur ^ 1) * XBUF;

    // this wavefront's share of the unit's k-steps (two pixels each)
    const int ksteps = (upix + 1) >> 1;
    const int khalf = (ksteps + 1) >> 1;
    const int s_begin = half ? khalf : 0, s_end = half ? ksteps : khalf;
    const int nsteps = s_end - s_begin;
    const int ngroups = nsteps / G;

    // A operand: dyS[pix][m]; B operand: xS[c][pixoff(pix) + r*PITCHP + s]
    const float *ap = dcur + (lane >> 5) * PA + wm * 32 + (lane & 31);
    const float *bp = xcur + (wc * 32 + (lane & 31)) * CHS;
    const int zoff = int((xS + 2 * XBUF) - bp);  // this lane's offset of the zero area
    // running (column, LDS offset) of this lane's pixel: pix = 2*step + lane/32  (Q >= 2)
    const int pix0 = 2 * s_begin + (lane >> 5);
    const int row0 = pix0 / a.Q;
    int q = pix0 - row0 * a.Q, off = row0 * PITCHP + q;

    // Operand fragments of k-step s+1 are fetched while the MFMAs of k-step s run.
    float av[2], bv[2][9];
    auto fetch = [&](int step, int buf) {
      av[buf] = ap[(2 * step) * PA];
      // a pixel past the unit's end has a zero dy column; its x operand comes from the zero area
      // so that no stale LDS value can meet it
      const int o = (2 * step + (lane >> 5)) < upix ? off : zoff;
#pragma unroll
      for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int s = 0; s < 3; ++s) bv[buf][r * 3 + s] = bp[o + r * PITCHP + s];
      q += 2;
      off += 2;
      if (q >= a.Q) {
        q -= a.Q;
        off += PITCHP - a.Q;
      }
    };
    auto mfmas = [&](int buf) {
#pragma unroll
      for (int i = 0; i < 9; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[buf], bv[buf][i], acc[i], 0, 0, 0);
    };

    fetch(s_begin, 0);
    // Global loads issued in group g are written to LDS at the end of group g + 1.
    float pd[DPG], px[XPG];
#pragma unroll
    for (int j = 0; j < DPG; ++j) pd[j] = 0.f;
#pragma unroll
    for (int j = 0; j < XPG; ++j) px[j] = 0.f;
    for (int g = 0; g < ngroups; ++g) {
      float ld[DPG], lx[XPG];
#pragma unroll
      for (int j = 0; j < DPG; ++j) ld[j] = dy_get(g * DPG + j, nn, np0, nupix);
#pragma unroll
      for (int j = 0; j < XPG; ++j) lx[j] = x_get(g * XPG + j, nn, np0, int(more));
#pragma unroll
      for (int s2 = 0; s2 < G; ++s2) {
        fetch(s_begin + g * G + s2 + 1, (s2 + 1) & 1);
        mfmas(s2 & 1);
      }
      // previous group's loads (for g == 0 the slot index is negative: dummy word); written even
      // when no unit follows -- the other buffer is simply not read again
#pragma unroll
      for (int j = 0; j < DPG; ++j) dy_put((g - 1) * DPG + j, pd[j], dnxt);
#pragma unroll
      for (int j = 0; j < XPG; ++j) x_put((g - 1) * XPG + j, px[j], xnxt);
#pragma unroll
      for (int j = 0; j < DPG; ++j) pd[j] = ld[j];
#pragma unroll
      for (int j = 0; j < XPG; ++j) px[j] = lx[j];
    }
    if (ngroups > 0) {
#pragma unroll
      for (int j = 0; j < DPG; ++j) dy_put((ngroups - 1) * DPG + j, pd[j], dnxt);
#pragma unroll
      for (int j = 0; j < XPG; ++j) x_put((ngroups - 1) * XPG + j, px[j], xnxt);
    }
    for (int step = s_begin + ngroups * G; step < s_end; ++step) {
      // fragments sit in buffer 0 here (an even number of steps per group keeps the parity)
      mfmas(0);
      fetch(step + 1, 0);
    }
    // slots not reached by a short unit's groups
    if (more) {
      for (int e = ngroups * DPG; e < DSLOTS; ++e) dy_put(e, dy_get(e, nn, np0, nupix), dnxt);
      for (int e = ngroups * XPG; e < XSLOTS; ++e) x_put(e, x_get(e, nn, np0, 1), xnxt);
    }
    __syncthreads();
    cur ^= 1;
  }

  // partial[2*z + half][tap][k][c]
  float *pz = a.part + size_t(blockIdx.z * 2 + half) * 9 * a.K * a.C;
#pragma unroll
  for (int i = 0; i < 9; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = k0 + wm * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
      const int c = c0 + wc * 32 + (lane & 31);
      if (m < a.K && c < a.C) pz[(size_t(i) * a.K + m) * a.C + c] = acc[i][v];
    }
}

// dW[k][c][tap] = sum over splits of partial[z][tap][k][c], in a fixed order.
// A workgroup takes 64 consecutive (k, c) pairs.  Its 256 threads form 4 z-lanes x 64 pairs:
// lane zl sums the splits z = zl, zl + 4, ... (ascending) of all nine taps, the four lane sums are
// added in lane order, and the 576 results are transposed through LDS so that they leave as one
// contiguous run.  The summation order depends only on `splits`: results are run-to-run identical.
__global__ __launch_bounds__(256) void k_wgrad3x3_reduce(const float *__restrict__ part, float *__restrict__ dW, int K,
                                                        int C, int splits) {
  __shared__ float lanes[4][9][64];
  __shared__ float tile[64 * 9];
  const long KC = long(K) * C;
  const long kc0 = long(blockIdx.x) * 64;
  const int e = threadIdx.x & 63, zl = threadIdx.x >> 6;
  const long kc = kc0 + e;
  float s[9];
#pragma unroll
  for (int tap = 0; tap < 9; ++tap) s[tap] = 0.f;
  if (kc < KC) {
    for (int z = zl; z < splits; z += 4) {
      const float *pz = part + long(z) * 9 * KC + kc;
#pragma unroll
      for (int tap = 0; tap < 9; ++tap) s[tap] += pz[tap * KC];
    }
  }
#pragma unroll
  for (int tap = 0; tap < 9; ++tap) lanes[zl][tap][e] = s[tap];
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * 9; i += 256) {
    const int tap = i >> 6, ee = i & 63;
    tile[ee * 9 + tap] = ((lanes[0][tap][ee] + lanes[1][tap][ee]) + lanes[2][tap][ee]) + lanes[3][tap][ee];
  }
  __syncthreads();
  const long nvalid = (KC - kc0 < 64 ? KC - kc0 : 64) * 9;
  for (int i = threadIdx.x; i < nvalid; i += 256) dW[kc0 * 9 + i] = tile[i];
}

struct W3Plan {
  bool ok;
  int bm, bc, logp, rows, ru, splits, units_per_split, total_units, upi;
  size_t lds;
};

inline W3Plan plan(const sgh_conv_geom *g) {
  W3Plan p{};
  p.ok = false;
  if (g->R != 3 || g->S != 3 || g->stride_h != 1 || g->stride_w != 1) return p;
  if (g->pad_h > 2 || g->pad_w > 2) return p;
  if (g->W + 2 > 64 || g->Q < 2 || g->Q > 64 || g->C < 32 || g->K < 64) return p;
  if (getenv("SGH_WGRAD3X3_OFF")) return p;
  // instantiated slabs: pitch 64 x 3 rows (RU 1), pitch 32 x 4 rows (RU 2), pitch 16 x 6 rows (RU 4),
  // pitch 16 x 9 rows (RU 7: a whole 7x7 plane)
  p.logp = g->W + 2 <= 16 ? 4 : (g->W + 2 <= 32 ? 5 : 6);
  if (p.logp == 6) p.ru = 1;
  else if (p.logp == 5) p.ru = 2;
  else p.ru = (7 * g->Q <= UPIXP && g->P >= 7) ? 7 : 4;
  if (p.ru > g->P || p.ru * g->Q > UPIXP) return p;
  p.rows = p.ru + 2;
  p.bm = g->K >= 128 ? 128 : 64;
  p.bc = p.bm == 128 ? 32 : 64;
  if (p.bc == 64 && g->C < 64) return p;
  p.upi = (g->P + p.ru - 1) / p.ru;
  p.total_units = g->N * p.upi;
  const long tiles = long((g->K + p.bm - 1) / p.bm) * ((g->C + p.bc - 1) / p.bc);
  // the LDS footprint allows one workgroup per CU: aim at one full wave of workgroups
  long want = (long(sgh_num_cus()) + tiles - 1) / tiles;
  long max_splits = p.total_units / 2;
  if (max_splits < 1) max_splits = 1;
  long s = want < max_splits ? want : max_splits;
  if (s < 1) s = 1;
  p.units_per_split = int((p.total_units + s - 1) / s);
  p.splits = (p.total_units + p.units_per_split - 1) / p.units_per_split;
  const int pitchp = 1 << p.logp, chs = p.rows * pitchp + 1;
  p.lds = (size_t(2) * UPIXP * (p.bm + 1) + size_t(2) * p.bc * chs + 3 * pitchp + 64) * sizeof(float);
  if (p.lds > 160 * 1024) return p;
  if (size_t(g->N) * g->K * g->P * g->Q * 4 >= (size_t(1) << 31) || size_t(g->N) * g->C * g->H * g->W * 4 >= (size_t(1) << 31))
    return p;
  p.ok = true;
  return p;
}

template <int BM, int BC, int LOGP, int ROWS>
int launch(const W3Args &a, const W3Plan &p, dim3 grid, hipStream_t s) {
  auto kern = k_wgrad3x3<BM, BC, LOGP, ROWS>;
  static bool attr_set = false;  // one process, one GPU: set the LDS opt-in once per instantiation
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024) != hipSuccess)
      return SGH_EUNSUPPORTED;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, grid, dim3(NT), p.lds, s, a);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

}  // namespace

size_t sgh_wgrad3x3_workspace_bytes(const sgh_conv_geom *g) {
  const W3Plan p = plan(g);
  return p.ok ? size_t(2) * p.splits * 9 * g->K * g->C * sizeof(float) : 0;
}

// Returns SGH_EUNSUPPORTED when the geometry is not covered (the caller then uses the generic path).
int sgh_wgrad3x3_run(const sgh_conv_geom *g, const float *dy, const float *x, float *dW, void *workspace,
                     size_t ws_bytes, hipStream_t s) {
  const W3Plan p = plan(g);
  if (!p.ok) return SGH_EUNSUPPORTED;
  const size_t need = size_t(2) * p.splits * 9 * g->K * g->C * sizeof(float);
  if (!workspace || ws_bytes < need) return SGH_EWORKSPACE;
  W3Args a;
  a.dy = dy;
  a.x = x;
  a.part = static_cast<float *>(workspace);
  a.N = g->N;
  a.C = g->C;
  a.H = g->H;
  a.W = g->W;
  a.K = g->K;
  a.P = g->P;
  a.Q = g->Q;
  a.ph = g->pad_h;
  a.pw = g->pad_w;
  a.RU = p.ru;
  a.units_per_image = p.upi;
  a.total_units = p.total_units;
  a.units_per_split = p.units_per_split;
  a.dy_bytes = unsigned(size_t(g->N) * g->K * g->P * g->Q * 4);
  a.x_bytes = unsigned(size_t(g->N) * g->C * g->H * g->W * 4);
  dim3 grid((g->K + p.bm - 1) / p.bm, (g->C + p.bc - 1) / p.bc, p.splits);
  int rc = SGH_EUNSUPPORTED;
  sgh_prof_start("conv_wgrad", 2.0 * g->N * g->K * g->P * g->Q * g->C * 9, s);
#define W3_CASE(BM_, BC_, LOGP_, ROWS_) \
  if (p.bm == BM_ && p.bc == BC_ && p.logp == LOGP_ && p.rows == ROWS_) rc = launch<BM_, BC_, LOGP_, ROWS_>(a, p, grid, s);
  W3_CASE(128, 32, 6, 3)
  W3_CASE(64, 64, 6, 3)
  W3_CASE(128, 32, 5, 4)
  W3_CASE(64, 64, 5, 4)
  W3_CASE(128, 32, 4, 6)
  W3_CASE(64, 64, 4, 6)
  W3_CASE(128, 32, 4, 9)
  W3_CASE(64, 64, 4, 9)
#undef W3_CASE
  sgh_prof_stop(s);
  if (rc != SGH_OK) return rc;
  const long blocks = (long(g->K) * g->C + 63) / 64;
  hipLaunchKernelGGL(k_wgrad3x3_reduce, dim3(int(blocks)), dim3(256), 0, s, a.part, dW, g->K, g->C, 2 * p.splits);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}
