// Weight gradient of convolutions with few input channels and a large filter (the 7x7 stride-2
// stem: C*R*S = 147), with an LDS input slab shared by every filter tap.
//
//   dW[k][c][r][s] = sum_{n,p,q} dy[n][k][p][q] * x[n][c][p*stride - ph + r][q*stride - pw + s]
//
// GEMM view: M = K (64 per workgroup), N = C*R*S columns j = (c, r, s) (at most 160 = five 32-wide
// MFMA tiles, so 147 columns waste 8 % instead of the 43 % of a 256-wide tile), reduction =
// (n, p, q).  A workgroup walks "units" of one output row (n, p): it stages
//   dyS[q][k]           the 64 x Q slice of dy        (A operand, k-dimension = pixel q),
//   xS[c][r][col]       the R input rows the row's windows touch, zero padding materialised,
// and column j of pixel q is the slab element at  laneconst(j) + q*stride : the B operand needs no
// im2col, one v_add per unit and immediates after that.  512 threads = 8 wavefronts as 2 (32-row
// M tiles) x 4 (quarters of the unit's k-steps); each holds five 32x32 accumulator tiles
// (v_mfma_f32_32x32x2_f32).  The quarters are summed through LDS at the end; the reduction is split
// over workgroups and the partials [split][K][CRS] are summed in a fixed order: results are
// run-to-run identical.
//
// Staging uses 128-bit loads, so W and Q must be multiples of 4 (the caller falls back to the
// generic implicit GEMM otherwise).
#include <stdlib.h>

#include "common.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr int NT = 512;
constexpr int BM = 64;
constexpr int NTL = 5;             // 32-column tiles
constexpr int UPIXP = 128;         // padded pixels per unit
constexpr int PA = BM + 1;         // dyS pitch (odd: pixel-major staging writes spread over banks)
constexpr int DROWS = UPIXP + 8;   // dyS rows: pixels, 3 rows of operand look-ahead, 4 spare rows for unused slots
constexpr int COL0 = 4;            // slab column of input column 0 (keeps 128-bit LDS writes aligned)
constexpr int kOOB = int(0x80000000u);

__device__ __forceinline__ rsrc_t make_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, bytes, 0x00020000);
}

struct WFArgs {
  const float *dy, *x;
  float *part;            // [splits][K][CRS]
  int N, C, H, W, K, P, Q, R, S, ph, pw;
  int pitch;              // slab row pitch (multiple of 4)
  int total_units, units_per_split;
};

template <int STRIDE>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_wgrad_fewc(WFArgs a) {
  constexpr int DSLOTS = BM * UPIXP / 4 / NT;   // 128-bit dy loads per thread per unit (upper bound)
  constexpr int XSLOTS = 4;                     // 128-bit x loads per thread per unit (upper bound)
  constexpr int NSQ = UPIXP / 2 / 4;            // k-steps of one wavefront in a full unit
  constexpr int LAT = 3;

  extern __shared__ float smem[];
  const int CR = a.C * a.R, XBUF = CR * a.pitch;
  float *dyS = smem;                            // [2][DROWS][PA]
  float *xS = smem + 2 * DROWS * PA;            // [2][C*R][pitch]

  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = wave >> 2, wq = wave & 3;
  const int k0 = blockIdx.x * BM;
  const int u_begin = blockIdx.z * a.units_per_split;
  const int u_end = min(u_begin + a.units_per_split, a.total_units);
  const int PQ = a.P * a.Q, HW = a.H * a.W, RS = a.R * a.S, CRS = a.C * RS;
  const unsigned dy_img_bytes = unsigned(a.K) * PQ * 4u, x_img_bytes = unsigned(a.C) * HW * 4u;

  // slabs start as zeros: pad columns are never written, image columns are rewritten per unit
  for (int i = t; i < 2 * XBUF; i += NT) xS[i] = 0.f;
  for (int i = t; i < 2 * DROWS * PA; i += NT) dyS[i] = 0.f;

  v16f acc[NTL];
#pragma unroll
  for (int i = 0; i < NTL; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

  // ---- staging roles of this thread (unit independent) ---------------------------------------
  // dy: float4 index f = e*NT + t over [BM][Q/4]  -> channel m = f / (Q/4), pixels 4*(f % (Q/4)) ..
  // x : float4 index f = e*NT + t over [C*R][W/4] -> slab row cr = f / (W/4), columns 4*(f % (W/4)) ..
  const int Q4 = a.Q >> 2, W4 = a.W >> 2;
  int dg[DSLOTS], dl[DSLOTS];
#pragma unroll
  for (int e = 0; e < DSLOTS; ++e) {
    const int f = e * NT + t, m = f / Q4, p4 = f - m * Q4;
    const bool ok = m < BM;
    dg[e] = ok ? (m * PQ + p4 * 4) * 4 : kOOB;
    dl[e] = ok ? (p4 * 4) * PA + m : (UPIXP + 4) * PA;  // unused slots land in the spare rows
  }
  int xg[XSLOTS], xl[XSLOTS], xr[XSLOTS];
#pragma unroll
  for (int e = 0; e < XSLOTS; ++e) {
    const int f = e * NT + t, cr = f / W4, c4 = f - cr * W4;
    const bool ok = cr < CR;
    const int c = cr / a.R, r = cr - c * a.R;
    xg[e] = ok ? (c * HW + r * a.W + c4 * 4) * 4 : kOOB;
    xl[e] = ok ? cr * a.pitch + COL0 + c4 * 4 : 0;
    xr[e] = ok ? r : -0x10000;  // slab row's filter row (a huge negative makes the row test fail)
  }
  auto ldv = [&](rsrc_t r, int voff) -> v4f {
    return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
  };
  // x rows outside the image read as zero: offset forced out of range
  auto x_voff = [&](int e, int hbase) -> int {
    const int h = hbase + xr[e];
    return unsigned(h) < unsigned(a.H) ? xg[e] + hbase * a.W * 4 : kOOB;
  };
  auto dy_put = [&](float *buf, int e, v4f v) {
    float *d = buf + dl[e];
    d[0] = v[0];
    d[PA] = v[1];
    d[2 * PA] = v[2];
    d[3 * PA] = v[3];
  };
  auto x_put = [&](float *buf, int e, v4f v) {
    if (xr[e] >= 0) *reinterpret_cast<v4f *>(buf + xl[e]) = v;
  };

  // ---- B operand lane constants: column j = tile*32 + lane%32 -> (c, r, s) ---------------------
  int bconst[NTL];
#pragma unroll
  for (int ti = 0; ti < NTL; ++ti) {
    const int j = ti * 32 + (lane & 31);
    const int jj = j < CRS ? j : 0;  // columns past C*R*S compute garbage that is never stored
    const int c = jj / RS, rs = jj - c * RS, r = rs / a.S, s = rs - r * a.S;
    bconst[ti] = (c * a.R + r) * a.pitch + s + COL0 - a.pw + STRIDE * (lane >> 5);
  }

  const int ksteps = (a.Q + 1) >> 1;             // k-steps of a unit (two pixels each)
  const int nsq = (ksteps + 3) >> 2;             // per quarter
  const int s_begin = wq * nsq;
  const int nsteps = max(0, min(nsq, ksteps - s_begin));

  auto unit_geom = [&](int u, int &n, int &p) {
    n = u / a.P;
    p = u - n * a.P;
  };

  if (u_begin < u_end) {
    int n, p;
    unit_geom(u_begin, n, p);
    const rsrc_t rdy = make_rsrc(a.dy + size_t(n) * a.K * PQ, dy_img_bytes);
    const rsrc_t rx = make_rsrc(a.x + size_t(n) * a.C * HW, x_img_bytes);
    const int sd = (k0 * PQ + p * a.Q) * 4, hbase = p * STRIDE - a.ph;
    __syncthreads();  // zero fill done
#pragma unroll
    for (int e = 0; e < DSLOTS; ++e) dy_put(dyS, e, ldv(rdy, dg[e] + sd));
#pragma unroll
    for (int e = 0; e < XSLOTS; ++e) x_put(xS, e, ldv(rx, x_voff(e, hbase)));
  }
  __syncthreads();

  int cur = 0;
  for (int u = u_begin; u < u_end; ++u) {
    int nn, np;
    const bool more = u + 1 < u_end;
    unit_geom(more ? u + 1 : u, nn, np);
    // no next unit: an empty descriptor makes every staging load return zero
    const rsrc_t rdy = make_rsrc(a.dy + size_t(nn) * a.K * PQ, more ? dy_img_bytes : 0u);
    const rsrc_t rx = make_rsrc(a.x + size_t(nn) * a.C * HW, more ? x_img_bytes : 0u);
    const int sd = (k0 * PQ + np * a.Q) * 4, hbase = np * STRIDE - a.ph;

    const float *dcur = dyS + cur * (DROWS * PA);
    const float *xcur = xS + cur * XBUF;
    float *dnxt = dyS + (cur ^ 1) * (DROWS * PA);
    float *xnxt = xS + (cur ^ 1) * XBUF;

    const float *ap = dcur + (2 * s_begin + (lane >> 5)) * PA + wm * 32 + (lane & 31);
    const float *bp[NTL];
#pragma unroll
    for (int ti = 0; ti < NTL; ++ti) bp[ti] = xcur + bconst[ti] + 2 * STRIDE * s_begin;

    float av[2], bv[2][NTL];
    auto frag = [&](int i, int buf) {
      av[buf] = ap[2 * i * PA];
#pragma unroll
      for (int ti = 0; ti < NTL; ++ti) bv[buf][ti] = bp[ti][2 * STRIDE * i];
    };
    auto mfmas = [&](int buf) {
#pragma unroll
      for (int ti = 0; ti < NTL; ++ti)
        acc[ti] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[buf], bv[buf][ti], acc[ti], 0, 0, 0);
    };

    frag(0, 0);
    v4f st[LAT + 1];
#pragma unroll
    for (int i = 0; i < NSQ + LAT; ++i) {
      // one staging load per k-step: dy slots first, then x slots
      if (i < NSQ && i < nsteps) {
        if (i < DSLOTS) st[i % (LAT + 1)] = ldv(rdy, dg[i % DSLOTS] + sd);
        else if (i < DSLOTS + XSLOTS) st[i % (LAT + 1)] = ldv(rx, x_voff((i - DSLOTS) % XSLOTS, hbase));
        frag(i + 1, (i + 1) & 1);
        mfmas(i & 1);
      }
      if (i >= LAT && i - LAT < nsteps) {
        const int w = i - LAT;
        if (w < DSLOTS) dy_put(dnxt, w % DSLOTS, st[w % (LAT + 1)]);
        else if (w < DSLOTS + XSLOTS) x_put(xnxt, (w - DSLOTS) % XSLOTS, st[w % (LAT + 1)]);
      }
    }
    // slots not reached by a short unit's k-steps
    if (more) {
#pragma unroll
      for (int e = 0; e < DSLOTS + XSLOTS; ++e) {
        if (e < nsteps) continue;
        if (e < DSLOTS) dy_put(dnxt, e % DSLOTS, ldv(rdy, dg[e % DSLOTS] + sd));
        else x_put(xnxt, (e - DSLOTS) % XSLOTS, ldv(rx, x_voff((e - DSLOTS) % XSLOTS, hbase)));
      }
    }
    __syncthreads();
    cur ^= 1;
  }

  // ---- sum the four quarters through LDS (the staging buffers are free now) --------------------
  float *xch = smem + (wm * NTL * 16) * 64 + lane;
#pragma unroll 1
  for (int q = 1; q < 4; ++q) {
    if (wq == q) {
#pragma unroll
      for (int ti = 0; ti < NTL; ++ti)
#pragma unroll
        for (int v = 0; v < 16; ++v) xch[(ti * 16 + v) * 64] = acc[ti][v];
    }
    __syncthreads();
    if (wq == 0) {
#pragma unroll
      for (int ti = 0; ti < NTL; ++ti)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[ti][v] += xch[(ti * 16 + v) * 64];
    }
    __syncthreads();
  }
  if (wq == 0) {
    float *pz = a.part + size_t(blockIdx.z) * a.K * CRS;
#pragma unroll
    for (int ti = 0; ti < NTL; ++ti) {
      const int j = ti * 32 + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = k0 + wm * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (m < a.K && j < CRS) pz[size_t(m) * CRS + j] = acc[ti][v];
      }
    }
  }
}

// out[i] = sum over splits of part[z][i] in a fixed order: 16 z-lanes x 16 elements per workgroup,
// lane zl sums z = zl, zl + 16, ... (ascending), the lane sums are added in lane order.
__global__ __launch_bounds__(256) void k_wgrad_fewc_reduce(const float *__restrict__ part, float *__restrict__ out,
                                                          long n, int splits) {
  __shared__ float lanes[16][16];
  const int e = threadIdx.x & 15, zl = threadIdx.x >> 4;
  const long i = long(blockIdx.x) * 16 + e;
  float s = 0.f;
  if (i < n) {   // (four loads in flight, added in the same ascending order)
    int z = zl;
    for (; z + 48 < splits; z += 64) {
      float v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = part[long(z + 16 * u) * n + i];
#pragma unroll
      for (int u = 0; u < 4; ++u) s += v[u];
    }
    for (; z < splits; z += 16) s += part[long(z) * n + i];
  }
  lanes[zl][e] = s;
  __syncthreads();
  if (threadIdx.x < 16 && i < n) {
    float r = lanes[0][e];
#pragma unroll
    for (int l = 1; l < 16; ++l) r += lanes[l][e];
    out[i] = r;
  }
}

struct WFPlan {
  bool ok;
  int pitch, splits, units_per_split, total_units;
  size_t lds;
};

inline WFPlan plan(const sgh_conv_geom *g) {
  WFPlan p{};
  p.ok = false;
  if (sgh_env().wgrad_fewc_off) return p;
  if (g->stride_h != g->stride_w || (g->stride_h != 1 && g->stride_h != 2)) return p;
  const int CRS = g->C * g->R * g->S;
  if (CRS > NTL * 32 || CRS <= 64) return p;            // narrower problems fit the generic 64-wide tile
  if (g->W % 4 != 0 || g->Q % 4 != 0 || g->Q > UPIXP || g->Q < 8) return p;
  if (g->C * g->R * (g->W / 4) > 4 * NT) return p;      // x staging slots per thread
  if (g->pad_w > COL0) return p;
  // slab columns: COL0 + W image columns, and the windows of the (padded) pixels up to UPIXP/.. + S
  const int need = COL0 - g->pad_w + ((g->Q + 2) * g->stride_w) + g->S + 1;
  const int have = COL0 + g->W + g->pad_w + 1;
  p.pitch = ((need > have ? need : have) + 3) & ~3;
  p.lds = (size_t(2) * DROWS * PA + size_t(2) * g->C * g->R * p.pitch) * sizeof(float);
  if (p.lds > 160 * 1024 || p.lds < size_t(2) * NTL * 16 * 64 * sizeof(float)) return p;
  if (size_t(g->K) * g->P * g->Q * 4 >= (size_t(1) << 30) || size_t(g->C) * g->H * g->W * 4 >= (size_t(1) << 30)) return p;
  p.total_units = g->N * g->P;
  const long tiles = (g->K + BM - 1) / BM;
  long want = (long(sgh_num_cus()) + tiles - 1) / tiles;
  long max_splits = p.total_units / 2;
  if (max_splits < 1) max_splits = 1;
  long s = want < max_splits ? want : max_splits;
  if (s < 1) s = 1;
  p.units_per_split = int((p.total_units + s - 1) / s);
  p.splits = (p.total_units + p.units_per_split - 1) / p.units_per_split;
  p.ok = true;
  return p;
}

template <int STRIDE>
int launch(const WFArgs &a, const WFPlan &p, dim3 grid, hipStream_t s) {
  auto kern = k_wgrad_fewc<STRIDE>;
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

size_t sgh_wgrad_fewc_workspace_bytes(const sgh_conv_geom *g) {
  const WFPlan p = plan(g);
  return p.ok ? size_t(p.splits) * g->K * g->C * g->R * g->S * sizeof(float) : 0;
}

// Returns SGH_EUNSUPPORTED when the geometry is not covered (the caller then uses the generic path).
int sgh_wgrad_fewc_run(const sgh_conv_geom *g, const float *dy, const float *x, float *dW, void *workspace,
                       size_t ws_bytes, hipStream_t s) {
  const WFPlan p = plan(g);
  if (!p.ok) return SGH_EUNSUPPORTED;
  const size_t need = size_t(p.splits) * g->K * g->C * g->R * g->S * sizeof(float);
  if (!workspace || ws_bytes < need) return SGH_EWORKSPACE;
  WFArgs a;
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
  a.R = g->R;
  a.S = g->S;
  a.ph = g->pad_h;
  a.pw = g->pad_w;
  a.pitch = p.pitch;
  a.total_units = p.total_units;
  a.units_per_split = p.units_per_split;
  dim3 grid((g->K + BM - 1) / BM, 1, p.splits);
  sgh_prof_kernel_begin("conv_wgrad/k_wgrad_fewc", 2.0 * g->N * g->K * g->P * g->Q * g->C * g->R * g->S);
  const int rc = g->stride_h == 1 ? launch<1>(a, p, grid, s) : launch<2>(a, p, grid, s);
  sgh_prof_kernel_end(s);
  if (rc != SGH_OK) return rc;
  const long n = long(g->K) * g->C * g->R * g->S;
  hipLaunchKernelGGL(k_wgrad_fewc_reduce, dim3(int((n + 15) / 16)), dim3(256), 0, s, a.part, dW, n, p.splits);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}
