// Forward convolution of the residual networks' stem in fp32: 7 x 7, stride 2, padding 3, up to three input
// channels, 64 filters (GpuConvForward, src/model/operation/convolution.cc:585-620, on the geometry of
// examples/cnn/model/resnet.py:133-135).  The layout of the work is that of the 16-bit kernel (fwd_fewc16.hip):
// pixels are the matrix rows, filters the columns, the reduction runs over the filter window -- C * 7 window rows
// padded to eight columns -- four indices per v_mfma_f32_16x16x4_f32:
//
//   * a workgroup (four wavefronts) takes four output rows of one image, a wavefront one of them, as Q / 16 blocks
//     of 16 pixels times four blocks of 16 filters, all accumulators in registers;
//   * the 2 * 4 + 5 input rows per channel sit in LDS as stored behind four zero columns, so that the window row
//     of pixel q starts at column 2 q; step j of the reduction reads column 2 q + 4 (j mod 2) + g of window row
//     j / 2 in lane group g: every LDS address is a per-lane base plus a constant of the unrolled step;
//   * the filters, re-laid [k][window row][8] with a zero first column by a small kernel beforehand, are copied
//     into LDS (row pitch 169 dwords: the 16 filters of a read fall into 16 banks);
//   * a lane ends up with four neighbouring pixels of one filter: one 16-byte store each.
//
// An element in front of a window (column 2 q - 4 of the image) meets a zero weight; it is replaced by zero before
// the multiplication so that an infinity next to a window does not turn into a NaN inside it.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kNT = 256, kRowsOut = 4, kFilters = 64, kR = 7, kChannels = 3;
constexpr int kSteps = kChannels * kR * 2;        // 42 steps of four reduction indices
constexpr int kWPitch = kSteps * 4 + 1;           // dwords per filter in LDS
constexpr int kRowsIn = 2 * kRowsOut + 5;

struct FwArgs {
  const float *x, *wp, *bias;
  float *y;
  int N, C, H, W, P, Q;
};

// W[k][c][r][s] -> wp[k * kWPitch + (c * 7 + r) * 8 + 1 + s], zero elsewhere
__global__ __launch_bounds__(256) void k_fwd_fewc_weights(const float *__restrict__ W, float *__restrict__ wp, int C) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= kFilters * kWPitch) return;
  const int k = idx / kWPitch, rem = idx - k * kWPitch, o = rem >> 3, s2 = rem & 7;
  float v = 0.f;
  if (rem < kSteps * 4 && o < C * kR && s2 >= 1) {
    const int c = o / kR, r = o - c * kR;
    v = W[((k * C + c) * kR + r) * kR + (s2 - 1)];
  }
  wp[idx] = v;
}

template <int NB>
__global__ __launch_bounds__(kNT) void k_fwd_fewc(FwArgs a) {
  extern __shared__ __align__(16) unsigned char lds[];
  constexpr int W = 32 * NB, XP = W + 8;
  constexpr int kWDwords = (kFilters * kWPitch + 3) & ~3;
  float *ws = reinterpret_cast<float *>(lds);            // [64][kWPitch]
  float *xs = ws + kWDwords;                             // [3][kRowsIn][XP], image column w at w + 4
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63, i = lane & 15, g = lane >> 4;
  const int n = blockIdx.y, p0 = blockIdx.x * kRowsOut;

  // filters: a straight copy (the workspace holds kWDwords)
  {
    const f32x4 *src = reinterpret_cast<const f32x4 *>(a.wp);
    f32x4 *dst = reinterpret_cast<f32x4 *>(ws);
    for (int v = t; v < kWDwords / 4; v += kNT) dst[v] = src[v];
  }
  // input rows 2 p0 - 3 .. 2 p0 + 2 * 4 + 1 of three channels; rows outside the image, channels the tensor does
  // not have and the columns around the image are zero
  {
    constexpr int VPR = W / 4;
    const int h0 = 2 * p0 - 3;
    for (int v = t; v < kChannels * kRowsIn * VPR; v += kNT) {
      const int cr = v / VPR, col = (v - cr * VPR) * 4;
      const int c = cr / kRowsIn, rr = cr - c * kRowsIn, h = h0 + rr;
      f32x4 d = {0.f, 0.f, 0.f, 0.f};
      if (c < a.C && h >= 0 && h < a.H)
        d = *reinterpret_cast<const f32x4 *>(a.x + ((size_t(n) * a.C + c) * a.H + h) * a.W + col);
      *reinterpret_cast<f32x4 *>(xs + cr * XP + 4 + col) = d;
    }
    for (int v = t; v < kChannels * kRowsIn * 2; v += kNT) {
      const int cr = v >> 1;
      *reinterpret_cast<f32x4 *>(xs + cr * XP + ((v & 1) ? W + 4 : 0)) = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }
  __syncthreads();

  f32x4 acc[NB][4];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int m = 0; m < 4; ++m) acc[b][m] = f32x4{0.f, 0.f, 0.f, 0.f};

  const float *ap = xs + (2 * wave) * XP + 2 * i + g;   // + (c * kRowsIn + r) * XP + 4 * (j & 1) + 32 * b
  const float *bp = ws + i * kWPitch + g;               // + 16 * m * kWPitch + 4 * j
#pragma unroll
  for (int j = 0; j < kSteps; ++j) {
    const int o = j >> 1, c = o / kR, r = o - c * kR;
    float bf[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) bf[m] = bp[16 * m * kWPitch + 4 * j];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      float af = ap[(c * kRowsIn + r) * XP + 4 * (j & 1) + 32 * b];
      if ((j & 1) == 0) af = g == 0 ? 0.f : af;
#pragma unroll
      for (int m = 0; m < 4; ++m) acc[b][m] = __builtin_amdgcn_mfma_f32_16x16x4f32(af, bf[m], acc[b][m], 0, 0, 0);
    }
  }

  // lane (i, g) holds pixels 16 b + 4 g .. + 3 of filter 16 m + i
  const int p = p0 + wave;
  if (p >= a.P) return;
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    const int k = 16 * m + i;
    const float bb = a.bias ? a.bias[k] : 0.f;
    float *row = a.y + ((size_t(n) * kFilters + k) * a.P + p) * a.Q + 4 * g;
#pragma unroll
    for (int b = 0; b < NB; ++b) *reinterpret_cast<f32x4 *>(row + 16 * b) = acc[b][m] + bb;
  }
}

template <int NB>
int launch(const FwArgs &a, hipStream_t s) {
  auto kern = k_fwd_fewc<NB>;
  const size_t lds = (size_t((kFilters * kWPitch + 3) & ~3) + size_t(kChannels) * kRowsIn * (32 * NB + 8)) * sizeof(float);
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)) !=
        hipSuccess)
      return SGH_EUNSUPPORTED;
    attr = true;
  }
  hipLaunchKernelGGL(kern, dim3(unsigned((a.P + kRowsOut - 1) / kRowsOut), unsigned(a.N)), dim3(kNT), lds, s, a);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

}  // namespace

bool sgh_fwd_fewc_supported(const sgh_conv_geom *g) {
  if (g->groups != 1 || g->R != kR || g->S != kR || g->stride_h != 2 || g->stride_w != 2 || g->pad_h != 3 || g->pad_w != 3)
    return false;
  if (g->C < 1 || g->C > kChannels || g->K != kFilters || g->H % 2 != 0 || g->W != 2 * g->Q || g->P % kRowsOut != 0)
    return false;
  const int nb = g->Q / 16;
  if (g->Q % 16 != 0 || !(nb == 1 || nb == 2 || nb == 4 || nb == 7)) return false;
  return g->N <= 65535;
}

size_t sgh_fwd_fewc_workspace_bytes(const sgh_conv_geom *g) {
  return sgh_fwd_fewc_supported(g) ? size_t((kFilters * kWPitch + 3) & ~3) * sizeof(float) : 0;
}

int sgh_fwd_fewc_run(const sgh_conv_geom *g, const float *x, const float *W, const float *bias, float *y, void *workspace,
                     size_t ws_bytes, hipStream_t s) {
  if (!sgh_fwd_fewc_supported(g)) return SGH_EUNSUPPORTED;
  if (!sgh_aligned16(x) || !sgh_aligned16(y) || !sgh_aligned16(workspace)) return SGH_EUNSUPPORTED;
  if (!workspace || ws_bytes < sgh_fwd_fewc_workspace_bytes(g)) return SGH_EWORKSPACE;
  float *wp = static_cast<float *>(workspace);
  hipLaunchKernelGGL(k_fwd_fewc_weights, dim3((kFilters * kWPitch + 255) / 256), dim3(256), 0, s, W, wp, g->C);
  SGH_LAUNCH_CHECK();
  const FwArgs a{x, wp, bias, y, g->N, g->C, g->H, g->W, g->P, g->Q};
  sgh_prof_scope prof("conv_fwd/k_fwd_fewc", 2.0 * g->N * g->K * g->P * g->Q * g->C * g->R * g->S, s);
  switch (g->Q / 16) {
    case 1: return launch<1>(a, s);
    case 2: return launch<2>(a, s);
    case 4: return launch<4>(a, s);
    case 7: return launch<7>(a, s);
  }
  return SGH_EUNSUPPORTED;
}
