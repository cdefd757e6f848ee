// Forward convolution of the residual networks' stem on 16-bit tensors: 7 x 7, stride 2, padding 3, up to three
// input channels, 64 filters (GpuConvForward, src/model/operation/convolution.cc:585-620, on the geometry of
// examples/cnn/model/resnet.py:133-135).  With so few input channels the reduction of the implicit GEMM is
// the filter window itself: C * 7 rows of the window, each padded to eight columns, are the "octets" of
// v_mfma_f32_16x16x32_{f16,bf16} (four octets per instruction).  Pixels are the matrix rows, filters the columns:
//
//   * a workgroup (four wavefronts) takes four output rows of one image, a wavefront one of them, as Q / 16 blocks
//     of 16 pixels times four blocks of 16 filters, all accumulators in registers;
//   * the input rows the four output rows touch (2 * 4 + 5 of them per channel) sit in LDS as stored, four zero
//     columns in front, so that the window row of pixel q starts at the even column 2 q: a lane reads the eight
//     elements of its octet as four dwords (the first element, column 2 q - 4 of the image, belongs to no
//     window and is masked out; the filter's padded column is zero as well);
//   * the filters, re-laid [k][octet][8] with that zero column by a small kernel beforehand, are copied into LDS
//     with 16-byte accesses; a lane's octet of its filter is one aligned 16-byte read;
//   * a lane ends up with four neighbouring pixels of one filter: one 8-byte store each.
//
// Sums are fp32 (the matrix instruction's accumulator), rounded once at the store; the bias is added in fp32.
#include <hip/hip_runtime.h>

#include "common.h"
#include "storage.h"

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kNT = 256, kRowsOut = 4, kFilters = 64, kR = 7;
constexpr int kOctets = 24;                       // 3 channels x 7 window rows, padded to whole instructions
constexpr int kWPitch = kOctets * 8 + 8;          // 16-bit elements per filter in LDS (the 8 keep 16-byte reads apart)
constexpr int kRowsIn = 2 * kRowsOut + 5;

struct FwArgs {
  const uint16_t *x, *wp, *bias;
  uint16_t *y;
  int N, C, H, W, P, Q;
};

// W[k][c][r][s] -> wp[k][c * 7 + r][1 + s], zero elsewhere (column 0 of an octet, octets beyond C * 7)
__global__ __launch_bounds__(256) void k_fwd_fewc16_weights(const uint16_t *__restrict__ W, uint16_t *__restrict__ wp, int C) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= kFilters * kWPitch) return;
  const int k = idx / kWPitch, rem = idx - k * kWPitch, o = rem >> 3, s2 = rem & 7;
  uint16_t v = 0;
  if (o < C * kR && s2 >= 1) {
    const int c = o / kR, r = o - c * kR;
    v = W[((k * C + c) * kR + r) * kR + (s2 - 1)];
  }
  wp[idx] = v;
}

template <int NB, bool BF16>
__global__ __launch_bounds__(kNT) void k_fwd_fewc16(FwArgs a) {
  extern __shared__ __align__(16) unsigned char lds[];
  uint16_t *ws = reinterpret_cast<uint16_t *>(lds);      // [64][kWPitch]
  uint16_t *xs = ws + kFilters * kWPitch;                // [C][kRowsIn][XP], image column w at w + 4
  constexpr int W = 32 * NB, XP = W + 8;
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63, i = lane & 15, g = lane >> 4;
  const int n = blockIdx.y, p0 = blockIdx.x * kRowsOut;

  // filters: a straight copy
  {
    const u32x4 *src = reinterpret_cast<const u32x4 *>(a.wp);
    u32x4 *dst = reinterpret_cast<u32x4 *>(ws);
    for (int v = t; v < kFilters * kWPitch / 8; v += kNT) dst[v] = src[v];
  }
  // input rows 2 p0 - 3 .. 2 p0 + 2 * 4 + 1 of every channel; rows outside the image and the columns around it are zero
  {
    constexpr int VPR = W / 8;
    const int h0 = 2 * p0 - 3;
    for (int v = t; v < a.C * kRowsIn * VPR; v += kNT) {
      const int cr = v / VPR, col = (v - cr * VPR) * 8;
      const int c = cr / kRowsIn, rr = cr - c * kRowsIn, h = h0 + rr;
      u32x4 d = {0u, 0u, 0u, 0u};
      if (h >= 0 && h < a.H)
        d = *reinterpret_cast<const u32x4 *>(a.x + ((size_t(n) * a.C + c) * a.H + h) * a.W + col);
      u32x2 *o = reinterpret_cast<u32x2 *>(xs + cr * XP + 4 + col);   // (8-byte aligned)
      o[0] = u32x2{d[0], d[1]};
      o[1] = u32x2{d[2], d[3]};
    }
    for (int v = t; v < a.C * kRowsIn * 2; v += kNT) {
      const int cr = v >> 1;
      *reinterpret_cast<u32x2 *>(xs + cr * XP + ((v & 1) ? W + 4 : 0)) = u32x2{0u, 0u};
    }
  }
  __syncthreads();

  f32x4 acc[NB][4];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int m = 0; m < 4; ++m) acc[b][m] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int noct = a.C * kR;
#pragma unroll
  for (int j = 0; j < kOctets / 4; ++j) {
    const int o = 4 * j + g;
    const bool live = o < noct;
    const int oc = live ? o : 0;
    const int c = oc / kR, r = oc - c * kR;
    // pixel q of output row p0 + wave: window row r starts at image row 2 (p0 + wave) - 3 + r = slab row 2 wave + r,
    // LDS column 2 q
    const unsigned *ap = reinterpret_cast<const unsigned *>(xs + (c * kRowsIn + 2 * wave + r) * XP + 2 * i);
    u32x4 bf[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) bf[m] = *reinterpret_cast<const u32x4 *>(ws + (16 * m + i) * kWPitch + o * 8);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      u32x4 af = {ap[16 * b] & 0xffff0000u, ap[16 * b + 1], ap[16 * b + 2], ap[16 * b + 3]};
      if (!live) af = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        if constexpr (BF16)
          acc[b][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af), __builtin_bit_cast(bf16x8, bf[m]),
                                                              acc[b][m], 0, 0, 0);
        else
          acc[b][m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af), __builtin_bit_cast(f16x8, bf[m]),
                                                             acc[b][m], 0, 0, 0);
      }
    }
  }

  // lane (i, g) holds pixels 16 b + 4 g .. + 3 of filter 16 m + i
  const int p = p0 + wave;
  if (p >= a.P) return;
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    const int k = 16 * m + i;
    float bb = 0.f;
    if (a.bias) bb = BF16 ? sgh_bf16_to_f32(a.bias[k]) : sgh_f16_to_f32(a.bias[k]);
    uint16_t *row = a.y + ((size_t(n) * kFilters + k) * a.P + p) * a.Q + 4 * g;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const f32x4 r = acc[b][m] + bb;
      *reinterpret_cast<u32x2 *>(row + 16 * b) = BF16 ? u32x2{sgh_pack2_bf16(r[0], r[1]), sgh_pack2_bf16(r[2], r[3])}
                                                      : u32x2{sgh_pack2_f16(r[0], r[1]), sgh_pack2_f16(r[2], r[3])};
    }
  }
}

template <int NB, bool BF16>
int launch(const FwArgs &a, hipStream_t s) {
  auto kern = k_fwd_fewc16<NB, BF16>;
  const size_t lds = (size_t(kFilters) * kWPitch + size_t(a.C) * kRowsIn * (32 * NB + 8)) * sizeof(uint16_t);
  static bool attr = false;
  if (!attr) {   // (once, for the largest case: three channels)
    const size_t lds_max = (size_t(kFilters) * kWPitch + size_t(3) * kRowsIn * (32 * NB + 8)) * sizeof(uint16_t);
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            int(lds_max)) != hipSuccess)
      return SGH_EUNSUPPORTED;
    attr = true;
  }
  hipLaunchKernelGGL(kern, dim3(unsigned((a.P + kRowsOut - 1) / kRowsOut), unsigned(a.N)), dim3(kNT), lds, s, a);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

template <bool BF16>
int launch_nb(const FwArgs &a, hipStream_t s) {
  switch (a.Q / 16) {
    case 1: return launch<1, BF16>(a, s);
    case 2: return launch<2, BF16>(a, s);
    case 4: return launch<4, BF16>(a, s);
    case 7: return launch<7, BF16>(a, s);
  }
  return SGH_EUNSUPPORTED;
}

}  // namespace

bool sgh_fwd_fewc16_supported(const sgh_conv_geom *g) {
  if (g->groups != 1 || g->R != kR || g->S != kR || g->stride_h != 2 || g->stride_w != 2 || g->pad_h != 3 || g->pad_w != 3)
    return false;
  if (g->C < 1 || g->C > 3 || g->K != kFilters || g->H % 2 != 0 || g->W != 2 * g->Q || g->P % kRowsOut != 0) return false;
  const int nb = g->Q / 16;
  if (g->Q % 16 != 0 || !(nb == 1 || nb == 2 || nb == 4 || nb == 7)) return false;
  if (g->N > 65535) return false;
  return size_t(g->N) * g->K * g->P * g->Q < (size_t(1) << 31);
}

size_t sgh_fwd_fewc16_workspace_bytes(const sgh_conv_geom *g) {
  return sgh_fwd_fewc16_supported(g) ? size_t(kFilters) * kWPitch * sizeof(uint16_t) : 0;
}

int sgh_fwd_fewc16_run(const sgh_conv_geom *g, const uint16_t *x, const uint16_t *W, const uint16_t *bias, uint16_t *y,
                       void *workspace, size_t ws_bytes, bool bf16, hipStream_t s) {
  if (!sgh_fwd_fewc16_supported(g)) return SGH_EUNSUPPORTED;
  if (!sgh_aligned16(x) || !sgh_aligned16(y) || !sgh_aligned16(workspace)) return SGH_EUNSUPPORTED;
  if (!workspace || ws_bytes < sgh_fwd_fewc16_workspace_bytes(g)) return SGH_EWORKSPACE;
  uint16_t *wp = static_cast<uint16_t *>(workspace);
  hipLaunchKernelGGL(k_fwd_fewc16_weights, dim3((kFilters * kWPitch + 255) / 256), dim3(256), 0, s, W, wp, g->C);
  SGH_LAUNCH_CHECK();
  const FwArgs a{x, wp, bias, y, g->N, g->C, g->H, g->W, g->P, g->Q};
  sgh_prof_scope prof("conv_fwd16/k_fwd_fewc16", 2.0 * g->N * g->K * g->P * g->Q * g->C * g->R * g->S, s);
  return bf16 ? launch_nb<true>(a, s) : launch_nb<false>(a, s);
}
