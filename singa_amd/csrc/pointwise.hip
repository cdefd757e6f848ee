// Data gradient of 1x1 convolutions without padding (fp32): dx[n][c][s*p][s*q] = sum_k W[k][c] * dy[n][k][p][q],
// the other positions of each s x s block zero -- the downsample convolutions of a residual network
// (reference call: GpuConvBackwardx, src/model/operation/convolution.cc:634-656).
//
// The reduction index k is the strided one in both operands while channels (W rows) and pixels (dy rows)
// are contiguous, which is exactly the operand shape of v_mfma_f32_32x32x2_f32: lane (i = lane % 32,
// h = lane / 32) supplies A[i][h] and B[h][i].  So a wavefront feeds its matrix instructions straight from
// global memory -- lane (i, h) loads W[2 j + h][c0 + i] and dy[..][2 j + h][col0 + i], 128 contiguous bytes per
// half wavefront -- with no LDS, no barrier and two adds of address arithmetic per step.  The generic
// implicit-GEMM kernel spent 23 vector and 13 scalar instructions per matrix instruction on these layers
// (staging arithmetic of its general loaders) and ran them at 27 TFLOP/s whatever their size; they are
// bandwidth kernels: 0.8 GFLOP against 13 - 77 MB of tensors.
//
// One wavefront owns (32 * TM) channels x 32 consecutive pixels of the flattened (n, p, q) index; the four
// wavefronts of a workgroup take the channel tiles of one pixel tile first (they read the same gradient
// pixels).  Every lane owns one pixel column for the whole kernel, so (n, p, q) is computed once.
#include "common.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int kOOB = int(0x80000000u);

__device__ __forceinline__ rsrc_t make_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, int(bytes), 0x00020000);
}

struct PwArgs {
  const float *W, *dy;
  float *dx;
  int N, C, K, H, Wd, P, Q, s;   // stride s in both directions
  int ncols, mtiles, ctiles;     // N * P * Q; channel tiles of 32 * TM; pixel tiles of 32 * TN
  unsigned w_bytes, dy_bytes;
};

template <int TM, int TN>
__global__ __launch_bounds__(256) void k_pw_dgrad(PwArgs a) {
  const int lane = threadIdx.x & 63, i32 = lane & 31, h = lane >> 5;
  const int wave = int(blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int ct = wave / a.mtiles, mt = wave - ct * a.mtiles;
  if (ct >= a.ctiles) return;
  const int PQ = a.P * a.Q;
  const int m0 = mt * (32 * TM);
  const rsrc_t rw = make_rsrc(a.W, a.w_bytes), rdy = make_rsrc(a.dy, a.dy_bytes);
  // byte offsets of this lane's first elements (k = h); a k step of 2 adds 2 * C / 2 * PQ elements
  int woff[TM], doff[TN], img[TN], rem[TN];
  bool col_ok[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) woff[i] = m0 + 32 * i + i32 < a.C ? (h * a.C + m0 + 32 * i + i32) * 4 : kOOB;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = (ct * TN + j) * 32 + i32;
    col_ok[j] = col < a.ncols;
    img[j] = col_ok[j] ? col / PQ : 0, rem[j] = col_ok[j] ? col - img[j] * PQ : 0;
    doff[j] = col_ok[j] ? ((img[j] * a.K + h) * PQ + rem[j]) * 4 : kOOB;
  }
  const int wstep = 2 * a.C * 4, dstep = 2 * PQ * 4;

  v16f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // Batches of U matrix steps; the loads of batch j + 2 are issued before the matrix instructions of batch j
  // (three register sets, the loop unrolled three times so that they are addressed statically): a batch holds
  // U * 64 cycles of matrix work, a load takes longer than that to come back from HBM.
  constexpr int U = 16 / (TM * TN > 2 ? 2 : 1), SETS = 3;   // (K is a multiple of 2 * U)
  float av[SETS][TM][U], bv[SETS][TN][U];
  auto load = [&](int set, int batch) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
        av[set][i][u] =
            __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rw, woff[i], (batch * U + u) * wstep, 0));
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bv[set][j][u] =
            __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rdy, doff[j], (batch * U + u) * dstep, 0));
    }
  };
  auto mma = [&](int set) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[set][i][u], bv[set][j][u], acc[i][j], 0, 0, 0);
  };
  const int nb = a.K / (2 * U);
  load(0, 0);
  if (nb > 1) load(1, 1);
  for (int b = 0; b < nb; b += SETS) {
#pragma unroll
    for (int i = 0; i < SETS; ++i) {
      if (b + i < nb) {
        if (b + i + 2 < nb) load((i + 2) % SETS, b + i + 2);
        mma(i);
      }
    }
  }

  const size_t plane = size_t(a.H) * a.Wd;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    if (!col_ok[j]) continue;
    const int p = rem[j] / a.Q, q = rem[j] - p * a.Q;
    float *base = a.dx + (size_t(img[j]) * a.C) * plane + size_t(a.s * p) * a.Wd + a.s * q;
    // the s x s block of this pixel: the value at its origin, zeros elsewhere; the last block of a row / column
    // also covers what lies beyond s * Q (s * P), and stops at the image border
    const int he = p == a.P - 1 ? a.H - p * a.s : a.s, we = q == a.Q - 1 ? a.Wd - q * a.s : a.s;
    const bool pair = a.s == 2 && he == 2 && we == 2 && (a.Wd & 1) == 0 && (reinterpret_cast<uintptr_t>(a.dx) & 7u) == 0;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + 32 * i + 8 * (v >> 2) + 4 * h + (v & 3);
        if (m >= a.C) continue;
        float *o = base + size_t(m) * plane;
        if (a.s == 1) {
          *o = acc[i][j][v];
        } else if (pair) {
          *reinterpret_cast<v2f *>(o) = v2f{acc[i][j][v], 0.f};
          *reinterpret_cast<v2f *>(o + a.Wd) = v2f{0.f, 0.f};
        } else {
          for (int r = 0; r < he; ++r)
            for (int c = 0; c < we; ++c) o[r * a.Wd + c] = (r == 0 && c == 0) ? acc[i][j][v] : 0.f;
        }
      }
  }
}

// ------------------------------------------------------------------------------------------------
// Weight gradient of the same layers: dW[k][c] = sum_{n,p,q} dy[n][k][p][q] * x[n][c][s*p][s*q].
//
// The reduction runs over pixels, which are contiguous in dy and every s-th element of every s-th row in x.
// A unit of the reduction is one output row (n, p): Q pixels.  Per unit a workgroup (4 wavefronts, tile
// 128 k x 64 c) stages dyS[k][q] and xS[c][q] in LDS -- every staging address is a thread constant plus a
// scalar term of the unit (no division and no predicate per element: what the generic implicit-GEMM loaders
// spend their time on for these layers) -- and multiplies with v_mfma_f32_32x32x2_f32, lane (i, h) reading
// element (row i, pixel 2 t + h) of each operand (row pitch odd: conflict-free).  The loads of the next unit
// are in flight while the current one is multiplied.  The units are split over workgroups; partial sums
// [split][K][C] are added in ascending split order by k_pw_wgrad_reduce (16 z-lanes in a fixed order), so the
// result is run-to-run identical.
struct PwWArgs {
  const float *dy, *x;
  float *part;
  int N, C, K, H, Wd, P, Q, s;
  int mtiles, ntiles, units, ups;   // units = N * P rows, `ups` of them per split
  unsigned dy_bytes, x_bytes;
};

template <int QC>   // the number of pixels per row Q, known at compile time (divisions by it become multiplications)
__global__ __launch_bounds__(256) void k_pw_wgrad(PwWArgs a) {
  constexpr int BM = 128, BN = 64, Q = QC, DS = (BM * Q + 255) / 256, XS = (BN * Q + 255) / 256;
  constexpr int QP = (Q + 1) | 1;               // odd, and a zero column behind an odd number of pixels
  constexpr int STEPS = (Q + 1) / 2;
  extern __shared__ float lds[];
  float *dyS0 = lds, *xS0 = lds + BM * QP, *dyS1 = lds + (BM + BN) * QP, *xS1 = dyS1 + BM * QP;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, i32 = lane & 31, h = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  const int tile = int(blockIdx.x) % (a.mtiles * a.ntiles), split = int(blockIdx.x) / (a.mtiles * a.ntiles);
  const int k0 = (tile / a.ntiles) * BM, c0 = (tile % a.ntiles) * BN;
  const int u0 = split * a.ups, u1 = min(u0 + a.ups, a.units);
  const int PQ = a.P * Q, HW = a.H * a.Wd;
  const rsrc_t rdy = make_rsrc(a.dy, a.dy_bytes), rx = make_rsrc(a.x, a.x_bytes);
  // the columns behind the pixels stay zero (nothing else is read before it is written)
  for (int i = t; i < 2 * (BM + BN); i += 256)
#pragma unroll
    for (int q = Q; q < QP; ++q) lds[i * QP + q] = 0.f;

  int dvo[DS], dlo[DS], xvo[XS], xlo[XS];
#pragma unroll
  for (int i = 0; i < DS; ++i) {
    const int e = i * 256 + t, k = e / Q, q = e - k * Q;
    const bool ok = k < BM && k0 + k < a.K;
    dvo[i] = ok ? ((k0 + k) * PQ + q) * 4 : kOOB;
    dlo[i] = k < BM ? k * QP + q : -1;
  }
#pragma unroll
  for (int i = 0; i < XS; ++i) {
    const int e = i * 256 + t, c = e / Q, q = e - c * Q;
    const bool ok = c < BN && c0 + c < a.C;
    xvo[i] = ok ? ((c0 + c) * HW + a.s * q) * 4 : kOOB;
    xlo[i] = c < BN ? c * QP + q : -1;
  }
  // two register sets: the loads of unit u + 2 are issued before unit u is multiplied
  float dr[2][DS], xr[2][XS];
  auto load = [&](int set, int u) {
    const bool live = u < u1;
    const int n = live ? u / a.P : 0, p = live ? u - n * a.P : 0;
    const int dso = (n * a.K * PQ + p * Q) * 4, xso = (n * a.C * HW + a.s * p * a.Wd) * 4;
#pragma unroll
    for (int i = 0; i < DS; ++i)
      dr[set][i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rdy, live ? dvo[i] : kOOB, dso, 0));
#pragma unroll
    for (int i = 0; i < XS; ++i)
      xr[set][i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rx, live ? xvo[i] : kOOB, xso, 0));
  };
  auto stage = [&](int set, float *dS, float *xS) {
#pragma unroll
    for (int i = 0; i < DS; ++i)
      if (dlo[i] >= 0) dS[dlo[i]] = dr[set][i];
#pragma unroll
    for (int i = 0; i < XS; ++i)
      if (xlo[i] >= 0) xS[xlo[i]] = xr[set][i];
  };
  v16f acc0, acc1;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc0[v] = 0.f, acc1[v] = 0.f;
  const int ao = (wm * 64 + i32) * QP + h, bo = (wn * 32 + i32) * QP + h;
  auto mma = [&](const float *dS, const float *xS) {
    float a0[STEPS], a1[STEPS], b[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS; ++st) a0[st] = dS[ao + 2 * st], a1[st] = dS[ao + 32 * QP + 2 * st], b[st] = xS[bo + 2 * st];
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[st], b[st], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[st], b[st], acc1, 0, 0, 0);
    }
  };
  load(0, u0);
  load(1, u0 + 1);
  __syncthreads();   // (the zero columns)
  for (int u = u0; u < u1; u += 2) {
    stage(0, dyS0, xS0);
    __syncthreads();
    load(0, u + 2);
    mma(dyS0, xS0);
    if (u + 1 >= u1) break;
    stage(1, dyS1, xS1);
    __syncthreads();
    load(1, u + 3);
    mma(dyS1, xS1);
  }
  float *out = a.part + size_t(split) * a.K * a.C;
  const int c = c0 + wn * 32 + i32;
  if (c < a.C) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = k0 + wm * 64 + 8 * (v >> 2) + 4 * h + (v & 3);
      if (m < a.K) out[size_t(m) * a.C + c] = acc0[v];
      if (m + 32 < a.K) out[size_t(m + 32) * a.C + c] = acc1[v];
    }
  }
}

// out[i] = sum over splits of part[z][i], z ascending within each of 16 z-lanes, the lanes added in lane order
__global__ __launch_bounds__(256) void k_pw_wgrad_reduce(const float *__restrict__ part, float *__restrict__ out, long n,
                                                        int splits) {
  __shared__ float lanes[16][17];
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

struct PwWPlan {
  bool ok;
  int mtiles, ntiles, units, ups, splits;
};

PwWPlan pw_wgrad_plan(const sgh_conv_geom *g) {
  PwWPlan p{};
  if (g->R != 1 || g->S != 1 || g->pad_h != 0 || g->pad_w != 0 || g->stride_h != g->stride_w || g->stride_h < 2) return p;
  if ((g->Q != 28 && g->Q != 14 && g->Q != 7) || g->K < 32 || g->C < 32) return p;   // (the rows of the residual networks)
  const size_t lim = size_t(1) << 29;   // byte offsets stay below 2^31
  if (size_t(g->N) * g->K * g->P * g->Q >= lim || size_t(g->N) * g->C * g->H * g->W >= lim) return p;
  p.mtiles = (g->K + 127) / 128, p.ntiles = (g->C + 63) / 64;
  p.units = g->N * g->P;
  // about two workgroups per CU; at least four rows per workgroup so that the pipeline has something to overlap
  int splits = 2 * sgh_num_cus() / (p.mtiles * p.ntiles);
  if (splits < 1) splits = 1;
  if (splits > p.units / 4) splits = p.units / 4 > 0 ? p.units / 4 : 1;
  p.ups = (p.units + splits - 1) / splits;
  p.splits = (p.units + p.ups - 1) / p.ups;
  p.ok = true;
  return p;
}

}  // namespace

bool sgh_pw_dgrad_supported(const sgh_conv_geom *g) {
  if (g->R != 1 || g->S != 1 || g->pad_h != 0 || g->pad_w != 0 || g->stride_h != g->stride_w) return false;
  if (g->K % 32 != 0 || g->C < 32) return false;
  const size_t lim = size_t(1) << 29;   // byte offsets stay below 2^31
  return size_t(g->N) * g->K * g->P * g->Q < lim && size_t(g->K) * g->C < lim;
}

int sgh_pw_dgrad_run(const sgh_conv_geom *g, const float *dy, const float *W, float *dx, hipStream_t s) {
  if (!sgh_pw_dgrad_supported(g)) return SGH_EUNSUPPORTED;
  PwArgs a{};
  a.W = W, a.dy = dy, a.dx = dx;
  a.N = g->N, a.C = g->C, a.K = g->K, a.H = g->H, a.Wd = g->W, a.P = g->P, a.Q = g->Q, a.s = g->stride_h;
  a.ncols = g->N * g->P * g->Q;
  a.w_bytes = unsigned(size_t(g->K) * g->C * 4), a.dy_bytes = unsigned(size_t(a.ncols) * g->K * 4);
  // wavefront tiles of 64 x 64 (half the operand loads per matrix instruction) while that still gives every
  // SIMD a wavefront, else 32 x 32
  const int force = sgh_env().pw_tile;
  const long waves64 = long((g->C + 63) / 64) * ((a.ncols + 63) / 64);
  const bool big = force > 0 ? force == 2 : (g->C >= 64 && waves64 >= 3L * sgh_num_cus());
  a.mtiles = big ? (g->C + 63) / 64 : (g->C + 31) / 32;
  a.ctiles = big ? (a.ncols + 63) / 64 : (a.ncols + 31) / 32;
  const long waves = long(a.mtiles) * a.ctiles;
  const unsigned blocks = unsigned((waves + 3) / 4);
  sgh_prof_kernel_begin("conv_dgrad/k_pw_dgrad", 2.0 * g->N * g->K * g->P * g->Q * g->C);
  if (big) SGH_LAUNCH_TIMED((k_pw_dgrad<2, 2>), dim3(blocks), dim3(256), 0, s, a);
  else SGH_LAUNCH_TIMED((k_pw_dgrad<1, 1>), dim3(blocks), dim3(256), 0, s, a);
  sgh_prof_kernel_end(s);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

size_t sgh_pw_wgrad_workspace_bytes(const sgh_conv_geom *g) {
  const PwWPlan p = pw_wgrad_plan(g);
  return p.ok ? size_t(p.splits) * g->K * g->C * sizeof(float) : 0;
}

int sgh_pw_wgrad_run(const sgh_conv_geom *g, const float *dy, const float *x, float *dW, void *workspace, size_t ws_bytes,
                     hipStream_t s) {
  const PwWPlan p = pw_wgrad_plan(g);
  if (!p.ok) return SGH_EUNSUPPORTED;
  if (!workspace || ws_bytes < sgh_pw_wgrad_workspace_bytes(g)) return SGH_EWORKSPACE;
  PwWArgs a{};
  a.dy = dy, a.x = x, a.part = static_cast<float *>(workspace);
  a.N = g->N, a.C = g->C, a.K = g->K, a.H = g->H, a.Wd = g->W, a.P = g->P, a.Q = g->Q, a.s = g->stride_h;
  a.mtiles = p.mtiles, a.ntiles = p.ntiles, a.units = p.units, a.ups = p.ups;
  a.dy_bytes = unsigned(size_t(g->N) * g->K * g->P * g->Q * 4), a.x_bytes = unsigned(size_t(g->N) * g->C * g->H * g->W * 4);
  const int QP = (g->Q + 1) | 1;
  const size_t lds = size_t(2) * (128 + 64) * QP * sizeof(float);
  const dim3 grid(unsigned(p.mtiles * p.ntiles * p.splits));
  sgh_prof_kernel_begin("conv_wgrad/k_pw_wgrad", 2.0 * g->N * g->K * g->P * g->Q * g->C);
  if (g->Q == 7) SGH_LAUNCH_TIMED(k_pw_wgrad<7>, grid, dim3(256), lds, s, a);
  else if (g->Q == 14) SGH_LAUNCH_TIMED(k_pw_wgrad<14>, grid, dim3(256), lds, s, a);
  else SGH_LAUNCH_TIMED(k_pw_wgrad<28>, grid, dim3(256), lds, s, a);
  sgh_prof_kernel_end(s);
  if (hipGetLastError() != hipSuccess) return SGH_EINVAL;
  const long n = long(g->K) * g->C;
  hipLaunchKernelGGL(k_pw_wgrad_reduce, dim3(unsigned((n + 15) / 16)), dim3(256), 0, s, a.part, dW, n, p.splits);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}
