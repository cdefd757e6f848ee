// Spatial BatchNorm (NCHW fp32): forward-training (to produce the saved mean / inverse std the
// backward consumes) and backward.
//
// Layout: channel c of image n is HW contiguous floats at ((n * C + c) * HW).  A channel's
// reduction domain is therefore N runs of HW floats.  Both passes split every channel over
// `S` workgroups (S chosen so the grid fills the chip), each workgroup reducing a contiguous
// range of the channel's (n, hw) index space with 16-byte loads where HW % 4 == 0.
// Reductions are a fixed tree (lane partials -> wavefront shuffle -> LDS -> ordered sum over
// the S partials), so results are run-to-run identical.
#include <mutex>

#include "common.h"
#include "storage.h"

// Partial sums of sgh_bn_bwd_noalloc_f32: device memory the library owns from load time on, so the
// entry point has nothing to allocate.  In host code this name is only a handle for
// hipGetSymbolAddress; kernels receive the address looked up per device (noalloc_scratch_of).
constexpr int kNoAllocMaxPairs = 16384;  // (channel, split) pairs of two floats: 128 KiB per device
static __device__ __align__(256) float scratch[kNoAllocMaxPairs * 2];

namespace {

constexpr int kBlock = 256;

struct BnShape {
  int N, C, HW;
  int S;          // splits per channel
  int per_split;  // elements of the (n, hw) space per split (multiple of 4 when HW % 4 == 0)
  int stream;     // tensor too large to stay cache resident between kernels: non-temporal loads
};

// Visit elements [lo, hi) of channel c's (n, hw) index space.  S is the storage type (storage.h):
// the 16-byte path loads four vectors of x (and of dy when `dy` is not null) per thread before the
// first use, so that eight loads are in flight per thread, and tracks (image, offset) incrementally
// instead of dividing.  fv(offset, x[VEC], dy[VEC]) / f1(offset) do the arithmetic and any store.
template <int NT, bool STREAM, class S, class FV, class F1>
__device__ __forceinline__ void channel_range_impl(const BnShape s, int c, int lo, int hi,
                                                   const typename S::elem *__restrict__ x,
                                                   const typename S::elem *__restrict__ dy, FV fv, F1 f1) {
  constexpr int V = S::VEC;
  const int M = s.N * s.HW;
  if (hi > M) hi = M;
  if (s.HW % V == 0) {
    // lo and per_split are multiples of V and a vector never straddles an image boundary
    constexpr int U = 4;
    int i = lo + threadIdx.x * V;
    int n = i / s.HW, r = i - n * s.HW;
    for (; i + (U - 1) * NT * V < hi; i += U * NT * V) {
      size_t off[U];
      float xv[U][V], dv[U][V];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        off[u] = (size_t(n) * s.C + c) * s.HW + r;
        r += NT * V;
        while (r >= s.HW) {
          r -= s.HW;
          ++n;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        S::template load16<STREAM>(x + off[u], xv[u]);
        if (dy) S::template load16<STREAM>(dy + off[u], dv[u]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) fv(off[u], xv[u], dv[u]);
    }
    for (; i < hi; i += NT * V) {
      const size_t off = (size_t(n) * s.C + c) * s.HW + r;
      float xv[V], dv[V];
      S::template load16<false>(x + off, xv);
      if (dy) S::template load16<false>(dy + off, dv);
      fv(off, xv, dv);
      r += NT * V;
      while (r >= s.HW) {
        r -= s.HW;
        ++n;
      }
    }
  } else {
    for (int i = lo + threadIdx.x; i < hi; i += NT) {
      const int n = i / s.HW, r = i - n * s.HW;
      f1((size_t(n) * s.C + c) * s.HW + r);
    }
  }
}

template <int NT, class S, class FV, class F1>
__device__ __forceinline__ void channel_range(const BnShape s, int c, int lo, int hi, const typename S::elem *__restrict__ x,
                                              const typename S::elem *__restrict__ dy, FV fv, F1 f1) {
  if (s.stream) channel_range_impl<NT, true, S>(s, c, lo, hi, x, dy, fv, f1);
  else channel_range_impl<NT, false, S>(s, c, lo, hi, x, dy, fv, f1);
}

// y = gamma * xhat + beta, written so that forward and the fused ReLU backward (which recomputes y
// to find the elements the ReLU passed) round identically.
__device__ __forceinline__ float bn_out(float v, float mean, float invstd, float g, float be) {
  return __builtin_fmaf(g, (v - mean) * invstd, be);
}

// ---- forward, pass 1: per (c, split) partial sum and sum of squares about a pivot ---------
// The pivot (the channel's first element) keeps the single-pass variance well conditioned.
template <class S>
__global__ __launch_bounds__(kBlock) void k_bn_fwd_partial(const typename S::elem *__restrict__ x, float *__restrict__ part,
                                                          BnShape s) {
  __shared__ float red[16];
  const int c = blockIdx.x / s.S, sp = blockIdx.x % s.S;
  const float pivot = S::ld(x + size_t(c) * s.HW);
  float a = 0.f, b = 0.f;
  channel_range<kBlock, S>(
      s, c, sp * s.per_split, (sp + 1) * s.per_split, x, nullptr,
      [&](size_t, const float *v, const float *) {
#pragma unroll
        for (int q = 0; q < S::VEC; q += 4) {
          const float d0 = v[q] - pivot, d1 = v[q + 1] - pivot, d2 = v[q + 2] - pivot, d3 = v[q + 3] - pivot;
          a += (d0 + d1) + (d2 + d3);
          b += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
        }
      },
      [&](size_t off) {
        const float d = S::ld(x + off) - pivot;
        a += d;
        b += d * d;
      });
  a = sgh_block_sum(a, red);
  b = sgh_block_sum(b, red);
  if (threadIdx.x == 0) {
    part[(size_t(c) * s.S + sp) * 2 + 0] = a;
    part[(size_t(c) * s.S + sp) * 2 + 1] = b;
  }
}

// ---- forward, pass 2: finish statistics (every workgroup redoes the tiny S-sum), normalise --
template <class S>
__global__ __launch_bounds__(kBlock) void k_bn_fwd_apply(const typename S::elem *__restrict__ x,
                                                        const float *__restrict__ gamma, const float *__restrict__ beta,
                                                        const float *__restrict__ part, float *__restrict__ running_mean,
                                                        float *__restrict__ running_var, float factor, float eps,
                                                        typename S::elem *__restrict__ y, float *__restrict__ save_mean,
                                                        float *__restrict__ save_invstd, BnShape s) {
  const int c = blockIdx.x / s.S, sp = blockIdx.x % s.S;
  const double M = double(s.N) * s.HW;
  double a = 0, b = 0;
  for (int i = 0; i < s.S; ++i) {
    a += part[(size_t(c) * s.S + i) * 2 + 0];
    b += part[(size_t(c) * s.S + i) * 2 + 1];
  }
  const float pivot = S::ld(x + size_t(c) * s.HW);
  const double dm = a / M;
  double var = b / M - dm * dm;
  if (var < 0) var = 0;
  const float mean = float(double(pivot) + dm);
  const float invstd = float(1.0 / sqrt(var + double(eps)));
  if (sp == 0 && threadIdx.x == 0) {
    save_mean[c] = mean;
    save_invstd[c] = invstd;
    if (running_mean) running_mean[c] = (1.f - factor) * running_mean[c] + factor * mean;
    if (running_var) {
      const double unb = M > 1 ? var * M / (M - 1) : var;
      running_var[c] = (1.f - factor) * running_var[c] + factor * float(unb);
    }
  }
  const float g = gamma[c], be = beta[c];
  channel_range<kBlock, S>(
      s, c, sp * s.per_split, (sp + 1) * s.per_split, x, nullptr,
      [&](size_t off, const float *v, const float *) {
        float r[S::VEC];
#pragma unroll
        for (int q = 0; q < S::VEC; ++q) r[q] = bn_out(v[q], mean, invstd, g, be);
        S::store16(y + off, r);
      },
      [&](size_t off) { S::st(y + off, bn_out(S::ld(x + off), mean, invstd, g, be)); });
}

// ---- forward, inference: normalise with the running statistics ------------------------------
template <class S>
__global__ __launch_bounds__(kBlock) void k_bn_fwd_infer(const typename S::elem *__restrict__ x,
                                                        const float *__restrict__ gamma, const float *__restrict__ beta,
                                                        const float *__restrict__ running_mean,
                                                        const float *__restrict__ running_var, float eps,
                                                        typename S::elem *__restrict__ y, BnShape s) {
  const int c = blockIdx.x / s.S, sp = blockIdx.x % s.S;
  const float mean = running_mean[c];
  const float invstd = float(1.0 / sqrt(double(running_var[c]) + double(eps)));
  const float g = gamma[c], be = beta[c];
  channel_range<kBlock, S>(
      s, c, sp * s.per_split, (sp + 1) * s.per_split, x, nullptr,
      [&](size_t off, const float *v, const float *) {
        float r[S::VEC];
#pragma unroll
        for (int q = 0; q < S::VEC; ++q) r[q] = bn_out(v[q], mean, invstd, g, be);
        S::store16(y + off, r);
      },
      [&](size_t off) { S::st(y + off, bn_out(S::ld(x + off), mean, invstd, g, be)); });
}

// ---- backward, pass 1: partial sum(dy) and sum(dy * xhat) ---------------------------------
// RELU: dy is the gradient behind a ReLU that consumed this BatchNorm's output; the gradient that
// reaches the BatchNorm is dy where the recomputed output is > 0 and 0 elsewhere (ReLUBackward's
// rule), applied on the fly instead of by a kernel of its own.
template <class S, bool RELU>
__global__ __launch_bounds__(kBlock) void k_bn_bwd_partial(const typename S::elem *__restrict__ dy,
                                                          const typename S::elem *__restrict__ x,
                                                          const float *__restrict__ gamma, const float *__restrict__ beta,
                                                          const float *__restrict__ save_mean,
                                                          const float *__restrict__ save_invstd,
                                                          float *__restrict__ part, BnShape s) {
  __shared__ float red[16];
  const int c = blockIdx.x / s.S, sp = blockIdx.x % s.S;
  const float mean = save_mean[c], invstd = save_invstd[c];
  const float g = RELU ? gamma[c] : 0.f, be = RELU ? beta[c] : 0.f;
  auto gate = [&](float d, float v) { return !RELU || S::stored_positive(bn_out(v, mean, invstd, g, be)) ? d : 0.f; };
  // (the products are accumulated with explicit fused multiply-adds: the fused and the plain
  // instantiation then round identically whatever the compiler does around the gate)
  float a = 0.f, b = 0.f, b1 = 0.f;
  channel_range<kBlock, S>(
      s, c, sp * s.per_split, (sp + 1) * s.per_split, x, dy,
      [&](size_t, const float *v, const float *d) {
#pragma unroll
        for (int q = 0; q < S::VEC; q += 4) {
          const float d0 = gate(d[q], v[q]), d1 = gate(d[q + 1], v[q + 1]), d2 = gate(d[q + 2], v[q + 2]),
                      d3 = gate(d[q + 3], v[q + 3]);
          a += (d0 + d1) + (d2 + d3);
          b = __builtin_fmaf(d0, (v[q] - mean) * invstd, b);
          b1 = __builtin_fmaf(d1, (v[q + 1] - mean) * invstd, b1);
          b = __builtin_fmaf(d2, (v[q + 2] - mean) * invstd, b);
          b1 = __builtin_fmaf(d3, (v[q + 3] - mean) * invstd, b1);
        }
      },
      [&](size_t off) {
        const float v = S::ld(x + off), d = gate(S::ld(dy + off), v);
        a += d;
        b = __builtin_fmaf(d, (v - mean) * invstd, b);
      });
  b += b1;
  a = sgh_block_sum(a, red);
  b = sgh_block_sum(b, red);
  if (threadIdx.x == 0) {
    part[(size_t(c) * s.S + sp) * 2 + 0] = a;
    part[(size_t(c) * s.S + sp) * 2 + 1] = b;
  }
}

// ---- backward, pass 2: dx = k * (dy - (dbeta + xhat * dgamma) / M), k = gamma * invstd -----
template <class S, bool RELU>
__global__ __launch_bounds__(kBlock) void k_bn_bwd_apply(const typename S::elem *__restrict__ dy,
                                                        const typename S::elem *__restrict__ x,
                                                        const float *__restrict__ gamma, const float *__restrict__ beta,
                                                        const float *__restrict__ save_mean,
                                                        const float *__restrict__ save_invstd,
                                                        const float *__restrict__ part, typename S::elem *__restrict__ dx,
                                                        float *__restrict__ dgamma, float *__restrict__ dbeta,
                                                        BnShape s) {
  const int c = blockIdx.x / s.S, sp = blockIdx.x % s.S;
  double a = 0, b = 0;
  for (int i = 0; i < s.S; ++i) {
    a += part[(size_t(c) * s.S + i) * 2 + 0];
    b += part[(size_t(c) * s.S + i) * 2 + 1];
  }
  const float db = float(a), dg = float(b);
  if (sp == 0 && threadIdx.x == 0) {
    dbeta[c] = db;
    dgamma[c] = dg;
  }
  const float mean = save_mean[c], invstd = save_invstd[c];
  const float g = gamma[c], be = RELU ? beta[c] : 0.f;
  const float k = g * invstd;
  const float rM = float(1.0 / (double(s.N) * s.HW));
  const float c0 = db * rM, c1 = dg * rM;
  auto gate = [&](float d, float v) { return !RELU || S::stored_positive(bn_out(v, mean, invstd, g, be)) ? d : 0.f; };
  channel_range<kBlock, S>(
      s, c, sp * s.per_split, (sp + 1) * s.per_split, x, dy,
      [&](size_t off, const float *v, const float *d) {
        float r[S::VEC];
#pragma unroll
        for (int q = 0; q < S::VEC; ++q)
          r[q] = k * (gate(d[q], v[q]) - __builtin_fmaf((v[q] - mean) * invstd, c1, c0));
        S::store16(dx + off, r);
      },
      [&](size_t off) {
        const float v = S::ld(x + off);
        S::st(dx + off, k * (gate(S::ld(dy + off), v) - __builtin_fmaf((v - mean) * invstd, c1, c0)));
      });
}

// ---- backward in one pass for small channels: one workgroup per channel keeps the channel's x and
// dy (N * HW elements each, raw storage) in LDS between the reduction and the normalisation, so the
// tensors are read once instead of twice and the two launches become one.  Same arithmetic per
// element as the two-pass kernels; the reduction tree differs (one workgroup instead of S splits).
constexpr int kResNT = 1024;
constexpr size_t kResidentLdsMax = size_t(144) << 10;

template <int BYTES>
struct RawVec;
template <>
struct RawVec<16> {
  typedef sgh_v4u type;
};
template <>
struct RawVec<8> {
  typedef unsigned int type __attribute__((ext_vector_type(2)));
};

inline size_t resident_half_bytes(int N, int HW, size_t esize) { return (size_t(N) * HW * esize + 15) & ~size_t(15); }

template <class S, bool RELU>
__global__ __launch_bounds__(kResNT) void k_bn_bwd_resident(const typename S::elem *__restrict__ dy,
                                                           const typename S::elem *__restrict__ x,
                                                           const float *__restrict__ gamma, const float *__restrict__ beta,
                                                           const float *__restrict__ save_mean,
                                                           const float *__restrict__ save_invstd,
                                                           typename S::elem *__restrict__ dx, float *__restrict__ dgamma,
                                                           float *__restrict__ dbeta, BnShape s) {
  typedef typename S::elem elem;
  constexpr int V = S::VEC, NT = kResNT;
  typedef typename RawVec<V * sizeof(elem)>::type raw;
  extern __shared__ __align__(16) unsigned char resident[];
  __shared__ float red[16];
  const int c = blockIdx.x, M = s.N * s.HW, t = threadIdx.x;
  elem *xs = reinterpret_cast<elem *>(resident);
  elem *ds = reinterpret_cast<elem *>(resident + ((size_t(M) * sizeof(elem) + 15) & ~size_t(15)));
  const float mean = save_mean[c], invstd = save_invstd[c];
  const float g = gamma[c], be = RELU ? beta[c] : 0.f;
  auto gate = [&](float d, float v) { return !RELU || S::stored_positive(bn_out(v, mean, invstd, g, be)) ? d : 0.f; };
  const bool vec = s.HW % V == 0;
  const int PV = vec ? s.HW / V : s.HW, TV = s.N * PV;   // vectors (or elements) per plane / per channel
  // stage: four (eight) independent loads per tensor in flight per thread
  if (vec) {
    const raw *xg = reinterpret_cast<const raw *>(x), *dg_ = reinterpret_cast<const raw *>(dy);
    for (int base = 0; base < TV; base += 4 * NT) {
      raw xv[4], dv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int iv = base + u * NT + t;
        if (iv < TV) {
          const int n = iv / PV, r = iv - n * PV;
          const size_t off = (size_t(n) * s.C + c) * PV + r;
          xv[u] = xg[off], dv[u] = dg_[off];
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int iv = base + u * NT + t;
        if (iv < TV) reinterpret_cast<raw *>(xs)[iv] = xv[u], reinterpret_cast<raw *>(ds)[iv] = dv[u];
      }
    }
  } else {
    for (int base = 0; base < TV; base += 8 * NT) {
      elem xv[8], dv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = base + u * NT + t;
        if (i < TV) {
          const int n = i / PV, r = i - n * PV;
          const size_t off = (size_t(n) * s.C + c) * PV + r;
          xv[u] = x[off], dv[u] = dy[off];
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = base + u * NT + t;
        if (i < TV) xs[i] = xv[u], ds[i] = dv[u];
      }
    }
  }
  __syncthreads();
  // sum(dy) and sum(dy * xhat), products as explicit fused multiply-adds (as in the two-pass kernels)
  float a = 0.f, b = 0.f, b1 = 0.f;
  if (vec) {
    for (int iv = t; iv < TV; iv += NT) {
      float v[V], d[V];
      S::template load16<false>(xs + size_t(iv) * V, v);
      S::template load16<false>(ds + size_t(iv) * V, d);
#pragma unroll
      for (int q = 0; q < V; q += 4) {
        const float d0 = gate(d[q], v[q]), d1 = gate(d[q + 1], v[q + 1]), d2 = gate(d[q + 2], v[q + 2]),
                    d3 = gate(d[q + 3], v[q + 3]);
        a += (d0 + d1) + (d2 + d3);
        b = __builtin_fmaf(d0, (v[q] - mean) * invstd, b);
        b1 = __builtin_fmaf(d1, (v[q + 1] - mean) * invstd, b1);
        b = __builtin_fmaf(d2, (v[q + 2] - mean) * invstd, b);
        b1 = __builtin_fmaf(d3, (v[q + 3] - mean) * invstd, b1);
      }
    }
  } else {
    for (int i = t; i < TV; i += NT) {
      const float v = S::ld(xs + i), d = gate(S::ld(ds + i), v);
      a += d;
      b = __builtin_fmaf(d, (v - mean) * invstd, b);
    }
  }
  b += b1;
  const float db = sgh_block_sum(a, red), dg = sgh_block_sum(b, red);
  if (t == 0) {
    dbeta[c] = db;
    dgamma[c] = dg;
  }
  const float k = g * invstd;
  const float rM = float(1.0 / (double(s.N) * s.HW));
  const float c0 = db * rM, c1 = dg * rM;
  if (vec) {
    for (int iv = t; iv < TV; iv += NT) {
      const int n = iv / PV, r = iv - n * PV;
      float v[V], d[V], o[V];
      S::template load16<false>(xs + size_t(iv) * V, v);
      S::template load16<false>(ds + size_t(iv) * V, d);
#pragma unroll
      for (int q = 0; q < V; ++q) o[q] = k * (gate(d[q], v[q]) - __builtin_fmaf((v[q] - mean) * invstd, c1, c0));
      S::store16(dx + ((size_t(n) * s.C + c) * PV + r) * V, o);
    }
  } else {
    for (int i = t; i < TV; i += NT) {
      const int n = i / PV, r = i - n * PV;
      const float v = S::ld(xs + i);
      S::st(dx + (size_t(n) * s.C + c) * PV + r, k * (gate(S::ld(ds + i), v) - __builtin_fmaf((v - mean) * invstd, c1, c0)));
    }
  }
}

// the one-pass kernel pays when a channel fits in LDS and there is a workgroup for at least half the CUs
inline bool resident_ok(int N, int C, int HW, size_t esize) {
  return 2 * resident_half_bytes(N, HW, esize) <= kResidentLdsMax && C >= sgh_num_cus() / 2;
}

template <class S, bool RELU>
int launch_resident(const typename S::elem *dy, const typename S::elem *x, const float *gamma, const float *beta,
                    const float *save_mean, const float *save_invstd, typename S::elem *dx, float *dgamma, float *dbeta,
                    const BnShape &s, hipStream_t st) {
  auto kern = k_bn_bwd_resident<S, RELU>;
  static bool attr = false;
  if (!attr) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            int(kResidentLdsMax)) != hipSuccess)
      return SGH_EUNSUPPORTED;
    attr = true;
  }
  const size_t lds = 2 * resident_half_bytes(s.N, s.HW, sizeof(typename S::elem));
  hipLaunchKernelGGL(kern, dim3(s.C), dim3(kResNT), lds, st, dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta,
                     s);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

inline bool shape_ok(int N, int C, int HW) {
  return N > 0 && C > 0 && HW > 0 && size_t(N) * HW < 0x7fffffffu;
}

// `vec`: elements per 16-byte access of the storage type; `esize`: bytes per element
inline BnShape make_shape(int N, int C, int HW, int vec, int esize) {
  // (measured: non-temporal loads gain 20 % on the 205 MB stem tensors and lose a few per cent on
  // tensors the previous kernel left in the 256 MB Infinity Cache)
  BnShape s{N, C, HW, 1, 0, size_t(N) * C * HW * esize >= (size_t(96) << 20) ? 1 : 0};
  const long M = long(N) * HW;
  // aim at ~8 workgroups per CU in total, at least 2048 elements per workgroup
  long want = (long(sgh_num_cus()) * 8 + C - 1) / C;
  long max_by_work = (M + 2047) / 2048;
  long S = want < max_by_work ? want : max_by_work;
  if (S < 1) S = 1;
  if (S > 1024) S = 1024;
  long per = (M + S - 1) / S;
  per = (per + vec - 1) / vec * vec;
  S = (M + per - 1) / per;
  s.S = int(S);
  s.per_split = int(per);
  return s;
}

template <class S>
int bn_fwd_train(const typename S::elem *x, const float *gamma, const float *beta, float *running_mean,
                 float *running_var, float factor, float eps, typename S::elem *y, float *save_mean, float *save_invstd,
                 int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  if (!shape_ok(N, C, HW) || !x || !gamma || !beta || !y || !save_mean || !save_invstd) return SGH_EINVAL;
  const BnShape s = make_shape(N, C, HW, S::VEC, int(sizeof(typename S::elem)));
  if (!sgh_aligned16(x) || !sgh_aligned16(y)) return SGH_EINVAL;
  if (!workspace || ws_bytes < size_t(C) * s.S * 2 * sizeof(float)) return SGH_EWORKSPACE;
  float *scratch = static_cast<float *>(workspace);
  hipLaunchKernelGGL(k_bn_fwd_partial<S>, dim3(C * s.S), dim3(kBlock), 0, sgh_stream_of(stream), x, scratch, s);
  SGH_LAUNCH_CHECK();
  hipLaunchKernelGGL(k_bn_fwd_apply<S>, dim3(C * s.S), dim3(kBlock), 0, sgh_stream_of(stream), x, gamma, beta, scratch,
                     running_mean, running_var, factor, eps, y, save_mean, save_invstd, s);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

template <class S>
int bn_fwd_infer(const typename S::elem *x, const float *gamma, const float *beta, const float *running_mean,
                 const float *running_var, float eps, typename S::elem *y, int N, int C, int HW, void *stream) {
  if (!shape_ok(N, C, HW) || !x || !gamma || !beta || !running_mean || !running_var || !y) return SGH_EINVAL;
  if (!sgh_aligned16(x) || !sgh_aligned16(y)) return SGH_EINVAL;
  const BnShape s = make_shape(N, C, HW, S::VEC, int(sizeof(typename S::elem)));
  hipLaunchKernelGGL(k_bn_fwd_infer<S>, dim3(C * s.S), dim3(kBlock), 0, sgh_stream_of(stream), x, gamma, beta,
                     running_mean, running_var, eps, y, s);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

// beta != NULL selects the fused ReLU + BatchNorm backward
template <class S>
int bn_bwd(const typename S::elem *dy, const typename S::elem *x, const float *gamma, const float *beta,
           const float *save_mean, const float *save_invstd, typename S::elem *dx, float *dgamma, float *dbeta, int N,
           int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  if (!shape_ok(N, C, HW) || !dy || !x || !gamma || !save_mean || !save_invstd || !dx || !dgamma || !dbeta)
    return SGH_EINVAL;
  if (!sgh_aligned16(x) || !sgh_aligned16(dy) || !sgh_aligned16(dx)) return SGH_EINVAL;
  const BnShape s = make_shape(N, C, HW, S::VEC, int(sizeof(typename S::elem)));
  if (!workspace || ws_bytes < size_t(C) * s.S * 2 * sizeof(float)) return SGH_EWORKSPACE;
  float *part = static_cast<float *>(workspace);
  const dim3 grid(C * s.S), block(kBlock);
  hipStream_t st = sgh_stream_of(stream);
  // algorithmic bytes: x and dy in, dx out (the fused form covers the ReLU backward as well)
  sgh_prof_scope prof(beta ? "bn_relu_bwd/k_bn_bwd" : "bn_bwd/k_bn_bwd", 3.0 * N * C * HW * sizeof(typename S::elem), st);
  if (resident_ok(N, C, HW, sizeof(typename S::elem))) {
    const int rc = beta ? launch_resident<S, true>(dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, s, st)
                        : launch_resident<S, false>(dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, s, st);
    if (rc != SGH_EUNSUPPORTED) return rc;
  }
  if (beta) {
    hipLaunchKernelGGL((k_bn_bwd_partial<S, true>), grid, block, 0, st, dy, x, gamma, beta, save_mean, save_invstd, part, s);
    SGH_LAUNCH_CHECK();
    hipLaunchKernelGGL((k_bn_bwd_apply<S, true>), grid, block, 0, st, dy, x, gamma, beta, save_mean, save_invstd, part,
                       dx, dgamma, dbeta, s);
  } else {
    hipLaunchKernelGGL((k_bn_bwd_partial<S, false>), grid, block, 0, st, dy, x, gamma, beta, save_mean, save_invstd, part, s);
    SGH_LAUNCH_CHECK();
    hipLaunchKernelGGL((k_bn_bwd_apply<S, false>), grid, block, 0, st, dy, x, gamma, beta, save_mean, save_invstd, part,
                       dx, dgamma, dbeta, s);
  }
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

// ---- device address of `scratch`, looked up once per device with that device current
constexpr int kNoAllocMaxDevices = 64;
float *g_noalloc_ptr[kNoAllocMaxDevices];
std::mutex g_noalloc_mu;

int noalloc_scratch_of_current_device(float **out) {
  int dev = -1;
  SGH_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kNoAllocMaxDevices) return SGH_EUNSUPPORTED;
  std::lock_guard<std::mutex> lk(g_noalloc_mu);
  if (!g_noalloc_ptr[dev]) {
    void *p = nullptr;
    SGH_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return SGH_EUNSUPPORTED;
    g_noalloc_ptr[dev] = static_cast<float *>(p);
  }
  *out = g_noalloc_ptr[dev];
  return SGH_OK;
}

}  // namespace

int sgh_bn_noalloc_setup() {
  float *p = nullptr;
  return noalloc_scratch_of_current_device(&p);
}

extern "C" {

size_t sgh_bn_workspace_bytes(int N, int C, int HW) {
  if (!shape_ok(N, C, HW)) return 0;
  // one size for every storage type: the larger of the fp32 and the 16-bit split counts
  const int s4 = make_shape(N, C, HW, 4, 4).S, s8 = make_shape(N, C, HW, 8, 2).S, s4h = make_shape(N, C, HW, 4, 2).S;
  const int smax = s4 > s8 ? (s4 > s4h ? s4 : s4h) : (s8 > s4h ? s8 : s4h);
  return size_t(C) * smax * 2 * sizeof(float);
}

// 16-bit planes that are a multiple of 4 but not of 8 elements (14 x 14) use the 8-byte vector class
#define SGH_BN_DISPATCH16(fn, F16X8, F16X4, ...) \
  (HW % 8 != 0 && HW % 4 == 0 ? fn<F16X4>(__VA_ARGS__) : fn<F16X8>(__VA_ARGS__))

int sgh_bn_fwd_train_f32(const float *x, const float *gamma, const float *beta, float *running_mean,
                         float *running_var, float factor, float eps, float *y, float *save_mean, float *save_invstd,
                         int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  return bn_fwd_train<StF32>(x, gamma, beta, running_mean, running_var, factor, eps, y, save_mean, save_invstd, N, C, HW,
                             workspace, ws_bytes, stream);
}
int sgh_bn_fwd_train_f16(const uint16_t *x, const float *gamma, const float *beta, float *running_mean,
                         float *running_var, float factor, float eps, uint16_t *y, float *save_mean,
                         float *save_invstd, int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  return SGH_BN_DISPATCH16(bn_fwd_train, StF16, StF16x4, x, gamma, beta, running_mean, running_var, factor, eps, y,
                           save_mean, save_invstd, N, C, HW, workspace, ws_bytes, stream);
}
int sgh_bn_fwd_train_bf16(const uint16_t *x, const float *gamma, const float *beta, float *running_mean,
                          float *running_var, float factor, float eps, uint16_t *y, float *save_mean,
                          float *save_invstd, int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  return SGH_BN_DISPATCH16(bn_fwd_train, StBF16, StBF16x4, x, gamma, beta, running_mean, running_var, factor, eps, y,
                           save_mean, save_invstd, N, C, HW, workspace, ws_bytes, stream);
}

int sgh_bn_bwd_f32(const float *dy, const float *x, const float *gamma, const float *save_mean,
                   const float *save_invstd, float *dx, float *dgamma, float *dbeta, int N, int C, int HW,
                   void *workspace, size_t ws_bytes, void *stream) {
  return bn_bwd<StF32>(dy, x, gamma, nullptr, save_mean, save_invstd, dx, dgamma, dbeta, N, C, HW, workspace, ws_bytes,
                       stream);
}
int sgh_bn_bwd_noalloc_f32(const float *dy, const float *x, const float *gamma, const float *save_mean,
                           const float *save_invstd, float *dx, float *dgamma, float *dbeta, int N, int C, int HW,
                           void *stream) {
  if (!shape_ok(N, C, HW)) return SGH_EINVAL;
  const size_t pairs = size_t(C) * make_shape(N, C, HW, StF32::VEC, int(sizeof(float))).S;
  if (pairs > size_t(kNoAllocMaxPairs)) return SGH_ELIMIT;
  float *part = nullptr;  // (every slot the second kernel reads is written by the first: nothing to clear)
  const int rc = noalloc_scratch_of_current_device(&part);
  if (rc != SGH_OK) return rc;
  return bn_bwd<StF32>(dy, x, gamma, nullptr, save_mean, save_invstd, dx, dgamma, dbeta, N, C, HW, part,
                       pairs * 2 * sizeof(float), stream);
}
int sgh_bn_bwd_f16(const uint16_t *dy, const uint16_t *x, const float *gamma, const float *save_mean,
                   const float *save_invstd, uint16_t *dx, float *dgamma, float *dbeta, int N, int C, int HW,
                   void *workspace, size_t ws_bytes, void *stream) {
  return SGH_BN_DISPATCH16(bn_bwd, StF16, StF16x4, dy, x, gamma, nullptr, save_mean, save_invstd, dx, dgamma, dbeta, N,
                           C, HW, workspace, ws_bytes, stream);
}
int sgh_bn_bwd_bf16(const uint16_t *dy, const uint16_t *x, const float *gamma, const float *save_mean,
                    const float *save_invstd, uint16_t *dx, float *dgamma, float *dbeta, int N, int C, int HW,
                    void *workspace, size_t ws_bytes, void *stream) {
  return SGH_BN_DISPATCH16(bn_bwd, StBF16, StBF16x4, dy, x, gamma, nullptr, save_mean, save_invstd, dx, dgamma, dbeta, N,
                           C, HW, workspace, ws_bytes, stream);
}

int sgh_bn_fwd_infer_f32(const float *x, const float *gamma, const float *beta, const float *running_mean,
                         const float *running_var, float eps, float *y, int N, int C, int HW, void *stream) {
  return bn_fwd_infer<StF32>(x, gamma, beta, running_mean, running_var, eps, y, N, C, HW, stream);
}
int sgh_bn_fwd_infer_f16(const uint16_t *x, const float *gamma, const float *beta, const float *running_mean,
                         const float *running_var, float eps, uint16_t *y, int N, int C, int HW, void *stream) {
  return SGH_BN_DISPATCH16(bn_fwd_infer, StF16, StF16x4, x, gamma, beta, running_mean, running_var, eps, y, N, C, HW,
                           stream);
}
int sgh_bn_fwd_infer_bf16(const uint16_t *x, const float *gamma, const float *beta, const float *running_mean,
                          const float *running_var, float eps, uint16_t *y, int N, int C, int HW, void *stream) {
  return SGH_BN_DISPATCH16(bn_fwd_infer, StBF16, StBF16x4, x, gamma, beta, running_mean, running_var, eps, y, N, C, HW,
                           stream);
}

int sgh_bn_relu_bwd_f32(const float *dy, const float *x, const float *gamma, const float *beta, const float *save_mean,
                        const float *save_invstd, float *dx, float *dgamma, float *dbeta, int N, int C, int HW,
                        void *workspace, size_t ws_bytes, void *stream) {
  if (!beta) return SGH_EINVAL;
  return bn_bwd<StF32>(dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, N, C, HW, workspace, ws_bytes,
                       stream);
}
int sgh_bn_relu_bwd_f16(const uint16_t *dy, const uint16_t *x, const float *gamma, const float *beta,
                        const float *save_mean, const float *save_invstd, uint16_t *dx, float *dgamma, float *dbeta,
                        int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  if (!beta) return SGH_EINVAL;
  return SGH_BN_DISPATCH16(bn_bwd, StF16, StF16x4, dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, N, C,
                           HW, workspace, ws_bytes, stream);
}
int sgh_bn_relu_bwd_bf16(const uint16_t *dy, const uint16_t *x, const float *gamma, const float *beta,
                         const float *save_mean, const float *save_invstd, uint16_t *dx, float *dgamma, float *dbeta,
                         int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  if (!beta) return SGH_EINVAL;
  return SGH_BN_DISPATCH16(bn_bwd, StBF16, StBF16x4, dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, N, C,
                           HW, workspace, ws_bytes, stream);
}
#undef SGH_BN_DISPATCH16

}  // extern "C"
