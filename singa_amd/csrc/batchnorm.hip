// Spatial BatchNorm (NCHW fp32): forward-training (to produce the saved mean / inverse std the
// backward consumes) and backward.
//
// Layout: channel c of image n is HW contiguous floats at ((n * C + c) * HW).  A channel's
// reduction domain is therefore N runs of HW floats.  Both passes split every channel over
// `S` workgroups (S chosen so the grid fills the chip), each workgroup reducing a contiguous
// range of the channel's (n, hw) index space with 16-byte loads where HW % 4 == 0.
// Reductions are a fixed tree (lane partials -> wavefront shuffle -> LDS -> ordered sum over
// the S partials), so results are run-to-run identical.
#include <atomic>
#include <mutex>
#include <random>

#include "common.h"
#include "storage.h"

// Partial sums of sgh_bn_bwd_noalloc_f32: device memory the library owns from load time on, so the
// entry point has nothing to allocate.  In host code this name is only a handle for
// hipGetSymbolAddress; kernels receive the address looked up per device (noalloc_scratch_of).
constexpr int kNoAllocMaxPairs = 32768;  // partial sums: 256 KiB per device
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
// The same value as an fp32 number the compiler cannot look behind: a binary16 store right behind the fmaf
// otherwise becomes one instruction that rounds the exact product-sum to 16 bits once, and a store with
// anything in between (the ReLU selection) rounds twice -- one unit in the last place apart now and then.
__device__ __forceinline__ float bn_out_rounded(float v, float mean, float invstd, float g, float be) {
  float r = bn_out(v, mean, invstd, g, be);
  asm volatile("" : "+v"(r));
  return r;
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
// RELU: the ReLU that consumes this BatchNorm's output folded in -- what the two separate calls store, bit for bit
// (fp32: y >= 0 ? y : 0 as the ReLU kernel; 16-bit: the stored value where it is positive, else 0)
template <class S>
__device__ __forceinline__ float bn_relu_value(float y) {
  if constexpr (sizeof(typename S::elem) == 4) return y >= 0.f ? y : 0.f;
  else return S::stored_positive(y) ? y : 0.f;
}

// ACT: what is stored -- 0: y; 1: relu(y); 2: relu(y + z) for a second tensor z (the end of a residual block), with
// the roundings of the separate calls: y to the storage type, the sum to the storage type, then the selection
template <class S, int ACT>
__device__ __forceinline__ float bn_fwd_value(float y, float z) {
  if constexpr (ACT == 0) return y;
  else if constexpr (ACT == 1) return bn_relu_value<S>(y);
  else {
    const float sum = S::stored(S::stored(y) + z);
    if constexpr (sizeof(typename S::elem) == 4) return sum >= 0.f ? sum : 0.f;
    else return sum > 0.f ? sum : 0.f;
  }
}

template <class S, int ACT>
__global__ __launch_bounds__(kBlock) void k_bn_fwd_apply(const typename S::elem *__restrict__ x,
                                                        const typename S::elem *__restrict__ z,
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
      s, c, sp * s.per_split, (sp + 1) * s.per_split, x, ACT == 2 ? z : nullptr,
      [&](size_t off, const float *v, const float *zv) {
        float r[S::VEC];
#pragma unroll
        for (int q = 0; q < S::VEC; ++q)
          r[q] = bn_fwd_value<S, ACT>(bn_out_rounded(v[q], mean, invstd, g, be), ACT == 2 ? zv[q] : 0.f);
        S::store16(y + off, r);
      },
      [&](size_t off) {
        const float r = bn_out_rounded(S::ld(x + off), mean, invstd, g, be);
        S::st(y + off, bn_fwd_value<S, ACT>(r, ACT == 2 ? S::ld(z + off) : 0.f));
      });
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
        for (int q = 0; q < S::VEC; ++q) r[q] = bn_out_rounded(v[q], mean, invstd, g, be);
        S::store16(y + off, r);
      },
      [&](size_t off) { S::st(y + off, bn_out_rounded(S::ld(x + off), mean, invstd, g, be)); });
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
  // workgroup w runs on XCD w % 8: each XCD takes a run of consecutive channels, whose planes share cache
  // lines when a plane is not a whole number of lines (49 or 196 elements), so a line is fetched into one L2
  const int c = int(blockIdx.x & 7) * int(gridDim.x >> 3) + int(blockIdx.x >> 3), M = s.N * s.HW, t = threadIdx.x;
  if (c >= s.C) return;
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

// ---- backward in one pass for planes of whole vectors: a channel is cut into G consecutive slices, one
// workgroup per slice keeps its slice of x and dy IN REGISTERS (raw storage, up to chip_nv() vectors per
// tensor and thread) from the reduction to the normalisation.  The G workgroups of a channel exchange their
// partial sums through the workspace.  Each publishes (sum dy, sum dy * xhat) as two 64-bit words that carry
// their own validity: the float in the upper half, half of a 64-bit ticket -- a number unique to the call --
// in the lower half, written with relaxed device-scope atomic stores (no fence: a word is either the old
// one or the new one).  Each then polls the 2 G words of its channel until all carry the ticket and adds the
// G partials in slice order, so every workgroup of the channel obtains the same bits.  Having read them, a
// A launch carries two tickets.  A workgroup first looks at what its own words hold: if that is the first
// ticket it publishes under the second one, otherwise under the first -- so a recorded launch, which
// carries the same two tickets into every replay, alternates between them (all words of a channel are
// rewritten by every execution, so they agree on which one is next), and no word ever has to be cleared.
// Only the G workgroups of one channel have to be on the chip together (G <= kChipMaxG, far below the number
// of CUs); their ids are consecutive, workgroups are dispatched in id order, and a waiting workgroup waits
// only for its own channel's slices, so the oldest unfinished channel always has all its slices dispatched
// and finishes.  The wait is bounded all the same: after `spin_limit` polls a workgroup gives up and the
// channel's outputs become NaN.
// x and dy are read once and dx written once: 3 tensor passes instead of 5.
constexpr int kChipMaxG = 128, kChipSpinLimit = 1 << 20;
// workgroups that gave up waiting for the other slices of their channel since the counter was last read
// (sgh_bn_exchange_failures; sgh_device_sync reports it as SGH_EEXCHANGE)
__device__ int g_bn_gave_up = 0;
// the number of polls after which a workgroup gives up: kChipSpinLimit unless a test lowered it
std::atomic<int> g_spin_limit{kChipSpinLimit};
// set by every launch of a one-pass kernel whose channels have several slices: the counter is read back (a small
// blocking copy) only when one has run since the last look
std::atomic<bool> g_exchange_ran{false};
#ifndef BN_CHIP_NL_ON
#define BN_CHIP_NL_ON 1
#endif

// vectors per tensor and thread: 8 (64 registers of raw data), 5 for 16-byte vectors of 16-bit elements,
// whose eight conversions per vector need more registers beside the data
template <class S>
constexpr int chip_nv() { return (sizeof(typename S::elem) == 2 && S::VEC == 8) ? 5 : 8; }
// 16-byte vectors of 16-bit elements: four more vectors per tensor and thread wait in LDS, which the kernel does
// not use otherwise (2 tensors x 4 x 512 threads x 16 bytes = 64 KB: still two workgroups per CU).  They are
// loaded straight into LDS (buffer_load ... lds: no destination registers while in flight), every thread reads
// back only what it loaded itself.  What a CU streams is (bytes resident) / (lifetime of a workgroup): the five
// register vectors alone left these shapes at 3.2-4.0 TB/s against 4.3-4.7 for fp32 with its eight.
template <class S>
constexpr int chip_nl() { return BN_CHIP_NL_ON && sizeof(typename S::elem) == 2 && S::VEC == 8 ? 4 : 0; }

struct ChipSlot {   // one per (channel, slice): {bits(a) : ticket low half}, {bits(b) : ticket high half}
  unsigned long long wa, wb;
};
inline size_t chip_workspace_bytes(int C, int G) { return size_t(C) * size_t(G) * sizeof(ChipSlot); }

struct ChipPlan {
  bool ok;
  int G, vpg, nt;   // slices per channel, vectors per slice, threads per workgroup
  int nl;           // vectors per tensor and thread kept in LDS (0: registers only)
  bool ragged;      // planes that are not whole vectors (7 x 7): see RAGGED in k_bn_bwd_onchip
};

// The exchange only terminates if all G workgroups of the oldest unfinished channel are running together.  A
// 512-thread workgroup of these kernels fits twice on a CU (registers and LDS are budgeted for that), a
// 1024-thread one once; with a run of channels per XCD (`xcd_runs` in the launchers: G <= 16 and C >= 8) the G
// slices of a channel all land on one XCD, an eighth of the CUs.  A device with fewer CUs than that (a
// partition) gets the two-pass kernels instead.
inline bool chip_slices_fit(int G, int C, int nt) {
  const long slots = long(sgh_num_cus()) * (nt == 512 ? 2 : 1);
  const bool xcd_runs = G <= 16 && C >= 8;
  return xcd_runs ? long(G) <= slots / 8 : long(G) <= slots;
}

template <class S>
inline ChipPlan chip_plan(int N, int C, int HW) {
  ChipPlan p{false, 0, 0, 0, 0, false};
  p.ragged = HW % S::VEC != 0;
  if (p.ragged && (S::VEC * sizeof(typename S::elem) != 16 || HW < S::VEC || sgh_env().bn_ragged_off ||
                   size_t(N) * C * HW * sizeof(typename S::elem) >= (size_t(1) << 31)))
    return p;
  if (size_t(N) * C * HW * sizeof(typename S::elem) >= (size_t(1) << 32)) return p;   // (32-bit byte offsets)
  const long TV = long(N) * ((HW + S::VEC - 1) / S::VEC);        // vectors per channel
  // 512 threads (two workgroups per CU: one loads while the other waits or stores) unless that cuts the
  // channel into more slices than one wavefront can poll
  p.nt = 512;
  // (the vectors in LDS only with 512 threads, and only for tensors up to 128 MB: measured at N = 128, fused with
  // the ReLU gate, C64 56x56 47.5 -> 40.2 us, C128 28x28 23.9 -> 21.5, C512 28x28 83.9 -> 79.4, C128 56x56 83.7 ->
  // 80.0, but the 205 MB tensors C256 56x56 153.8 -> 166.1 and C64 112x112 168.6 -> 174.8, with or without the
  // non-temporal hint that the register loads carry)
  const bool lds_ok = chip_nl<S>() > 0 && !p.ragged && size_t(N) * C * HW * sizeof(typename S::elem) <= (size_t(128) << 20);
  int per_thread = chip_nv<S>() + (lds_ok ? chip_nl<S>() : 0);
  long G = (TV + long(p.nt) * per_thread - 1) / (long(p.nt) * per_thread);
  if (G > kChipMaxG) {
    p.nt = 1024;
    per_thread = chip_nv<S>();
    G = (TV + long(p.nt) * per_thread - 1) / (long(p.nt) * per_thread);
  }
  p.nl = p.nt == 512 && lds_ok ? chip_nl<S>() : 0;
  // a channel that two workgroups of 512 threads would share but one of 1024 threads holds alone, with a channel for
  // every CU: one workgroup per channel and nothing to exchange (16-bit 128 x 256 x 14 x 14: 3200 pieces per channel)
  // -- 16.0 -> 15.0 us, 128 x 1024 x 14 x 14 50.6 -> 48.0 us
  if (p.nt == 512 && G == 2 && p.nl == 0 && C >= sgh_num_cus() && TV <= 1024L * chip_nv<S>()) {
    p.nt = 1024;
    G = 1;
  }
  // few channels: thinner slices, so that there are two workgroups for every CU (at least one wavefront of vectors
  // each) -- unless a channel fits one workgroup and there is a channel for every CU: then nothing is exchanged
  const bool whole_channels = G == 1 && C >= sgh_num_cus();
  const long want = whole_channels ? 1 : (2L * sgh_num_cus() + C - 1) / C;
  if (G < want) G = want;
  // whole rounds: as many slices as still fit into the rounds of (2 workgroups x CUs) that this many need
  const long slots = 2L * sgh_num_cus(), rounds = (long(C) * G + slots - 1) / slots;
  long fill = rounds * slots / C;
  if (fill > kChipMaxG) fill = kChipMaxG;
  if (fill > G && !whole_channels) G = fill;
  while (G > 1 && (TV + G - 1) / G < 64) --G;
  if (G > kChipMaxG || G < 1) return p;
  p.vpg = int((TV + G - 1) / G);
  p.G = int((TV + p.vpg - 1) / p.vpg);
  p.ok = long(C) * p.G < 0x7fffffffL && chip_slices_fit(p.G, C, p.nt);
  return p;
}

// (image, piece within the plane) of a thread's vectors: vector j of a thread is number first + j * NT of the
// channel, so one division places the first and every later one is a step of NT / PV images and NT % PV pieces
// with at most one carry -- a division by a run-time value per vector costs about twenty vector instructions,
// a step four.
struct ChipWalk {
  int n, r;
  __device__ __forceinline__ void step(int dn, int dr, int PV) {
    n += dn;
    r += dr;
    if (r >= PV) r -= PV, ++n;
  }
};

// RAGGED: planes that are not whole vectors.  A plane of HW elements is covered by ceil(HW / V) pieces of 16 bytes
// at 2- or 4-byte alignment (buffer loads and stores take any); the last piece starts at HW - V, i.e. overlaps
// the one before it instead of running into the next plane: its first V - HW % V elements are left out of the
// sums, and its store rewrites them with the values the piece before it stores (same inputs, same expression).
template <class S, bool RELU, int NT, int NL = 0, bool RAGGED = false>
__global__ __launch_bounds__(NT, 4) void k_bn_bwd_onchip(const typename S::elem *__restrict__ dy,
                                                          const typename S::elem *__restrict__ x,
                                                          const float *__restrict__ gamma, const float *__restrict__ beta,
                                                          const float *__restrict__ save_mean,
                                                          const float *__restrict__ save_invstd,
                                                          typename S::elem *__restrict__ dx, float *__restrict__ dgamma,
                                                          float *__restrict__ dbeta, unsigned long long *__restrict__ ws,
                                                          BnShape s, int G, int vpg, unsigned long long ticket1,
                                                          unsigned long long ticket2, int spin_limit, int xcd_runs,
                                                          int dephase_ticks) {
  typedef typename S::elem elem;
  constexpr int V = S::VEC, NV = chip_nv<S>();
  typedef typename RawVec<V * sizeof(elem)>::type raw;
  __shared__ float red[16];
  __shared__ float part_a[kChipMaxG], part_b[kChipMaxG];
  __shared__ int gave_up;
  __shared__ unsigned long long ticket_s;
  // Channels of few slices: each XCD (workgroup w runs on XCD w % 8) takes a run of consecutive channels, see
  // k_bn_bwd_resident; gridDim.x is then 8 * (channels per XCD) * G.  The slices of a channel stay G
  // consecutive workgroups of their XCD, so the oldest unfinished channel of an XCD still completes.
  const int unit = xcd_runs ? int(blockIdx.x & 7) * int(gridDim.x >> 3) + int(blockIdx.x >> 3) : int(blockIdx.x);
  const int c = unit / G, g = unit - c * G, t = threadIdx.x;
  if (c >= s.C) return;
  // Launches of many rounds: all workgroups of the first round start together and stay in step -- everybody loads,
  // then everybody waits for the exchange, then everybody stores -- and the later rounds inherit the rhythm, so the
  // memory system idles through every exchange.  The odd channels of the first round start `dephase_ticks` (of the
  // 100 MHz wall clock) late; from then on one half of the chip loads while the other half exchanges and stores.
  if (dephase_ticks > 0 && int(blockIdx.x) < int(2 * 256) && (c & 1)) {
    if (t == 0) {
      const unsigned long long t0 = wall_clock64();
      while (wall_clock64() - t0 < (unsigned long long)(dephase_ticks)) __builtin_amdgcn_s_sleep(16);
    }
    __syncthreads();
  }
  unsigned long long *words = ws + size_t(c) * 2 * size_t(G);   // the channel's G slots
  if (G > 1 && t == 0) {
    const unsigned long long wa = __hip_atomic_load(words + 2 * g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long wb = __hip_atomic_load(words + 2 * g + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ticket_s = (unsigned(wa) == unsigned(ticket1) && unsigned(wb) == unsigned(ticket1 >> 32)) ? ticket2 : ticket1;
    gave_up = 0;
  }
  static_assert(!RAGGED || (NL == 0 && V * sizeof(elem) == 16), "ragged planes: 16-byte pieces in registers");
  const int PV = RAGGED ? (s.HW + V - 1) / V : s.HW / V, TV = s.N * PV;
  const int tail_skip = RAGGED && s.HW % V ? V - s.HW % V : 0;   // elements of a plane's last piece that are not its own
  const int lo = g * vpg, hi = min(lo + vpg, TV);
  const float mean = save_mean[c], invstd = save_invstd[c];
  const float gm = gamma[c], be = RELU ? beta[c] : 0.f;
  auto gate = [&](float d, float v) { return !RELU || S::stored_positive(bn_out(v, mean, invstd, gm, be)) ? d : 0.f; };
  // byte offsets within a tensor are 32 bits (the plan leaves larger tensors to the two-pass kernels): the
  // addresses are then a uniform base plus a per-lane offset, with no 64-bit arithmetic per vector
  const char *xb = reinterpret_cast<const char *>(x), *db_ = reinterpret_cast<const char *>(dy);
  const unsigned CPV = unsigned(s.C) * unsigned(PV), cPV = unsigned(c) * unsigned(PV);
  const int dn = NT / PV, dr = NT - dn * PV;
  ChipWalk first;
  first.n = (lo + t) / PV, first.r = (lo + t) - first.n * PV;
  auto vec_bytes = [&](const ChipWalk &w) { return (unsigned(w.n) * CPV + cPV + unsigned(w.r)) * unsigned(sizeof(raw)); };
  const int tensor_bytes = RAGGED ? int(size_t(s.N) * s.C * s.HW * sizeof(elem)) : 0;
  const __amdgpu_buffer_rsrc_t rxb = __builtin_amdgcn_make_buffer_rsrc(const_cast<elem *>(x), 0, tensor_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rdb = __builtin_amdgcn_make_buffer_rsrc(const_cast<elem *>(dy), 0, tensor_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rob = __builtin_amdgcn_make_buffer_rsrc(dx, 0, tensor_bytes, 0x00020000);
  // byte offset of piece r of plane (n, c)
  auto piece = [&](int n, int r) {
    return int(((unsigned(n) * unsigned(s.C) + unsigned(c)) * unsigned(s.HW) + unsigned(r == PV - 1 ? s.HW - V : r * V)) *
               unsigned(sizeof(elem)));
  };
  raw xv[NV], dv[NV];
  // vectors 0 .. NL-1 of a thread go to LDS: slot j of tensor z at ((z * NL + j) * NT + t) * 16 bytes.  A
  // wavefront's instruction writes 64 consecutive slots (LDS address = wavefront-uniform base + 16 * lane).
  extern __shared__ __align__(16) unsigned char chip_lds[];
  if constexpr (NL > 0) {
    typedef __amdgpu_buffer_rsrc_t rsrc_t;
    const unsigned bytes = unsigned(size_t(s.N) * s.C * s.HW * sizeof(elem));
    const rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<elem *>(x), 0, int(bytes), 0x00020000);
    const rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(const_cast<elem *>(dy), 0, int(bytes), 0x00020000);
    const int wbase = __builtin_amdgcn_readfirstlane(t & ~63);
    ChipWalk w = first;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      const int iv = lo + j * NT + t;
      int voff = int(0x80000000u);   // (beyond the buffer: the slot reads as zero and is never used)
      if (iv < hi) voff = int(vec_bytes(w));
      w.step(dn, dr, PV);
      typedef unsigned char __attribute__((address_space(3))) * lds_ptr;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr)(chip_lds + size_t((0 * NL + j) * NT + wbase) * 16), 16, voff, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rd, (lds_ptr)(chip_lds + size_t((1 * NL + j) * NT + wbase) * 16), 16, voff, 0, 0, 0);
    }
  }
  // every load of the slice is issued before the first value is used
  ChipWalk wreg = first;   // the walk at the first register vector
#pragma unroll
  for (int j = 0; j < NL; ++j) wreg.step(dn, dr, PV);
  {
    ChipWalk w = wreg;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int iv = lo + (NL + i) * NT + t;
      if (iv < hi) {
        if constexpr (RAGGED) {
          xv[i] = __builtin_bit_cast(raw, __builtin_amdgcn_raw_buffer_load_b128(rxb, piece(w.n, w.r), 0, 0));
          dv[i] = __builtin_bit_cast(raw, __builtin_amdgcn_raw_buffer_load_b128(rdb, piece(w.n, w.r), 0, 0));
        } else {
          const unsigned off = vec_bytes(w);
          xv[i] = __builtin_nontemporal_load(reinterpret_cast<const raw *>(xb + off));
          dv[i] = __builtin_nontemporal_load(reinterpret_cast<const raw *>(db_ + off));
        }
      }
      w.step(dn, dr, PV);
    }
  }
  float a = 0.f, b = 0.f, b1 = 0.f;
  // (a macro, not a lambda: with the vectors passed to a lambda the register arrays went to scratch memory)
#define BN_CHIP_ACCUMULATE(XR, DR, SKIP)                                                                      \
  {                                                                                                           \
    float v[V], d[V];                                                                                         \
    S::template load16<false>(reinterpret_cast<const elem *>(&(XR)), v);                                      \
    S::template load16<false>(reinterpret_cast<const elem *>(&(DR)), d);                                      \
    if constexpr (RELU) {   /* the gated gradient replaces the stored one (exactly: it is that value or zero), */ \
                            /* so the second pass does not evaluate the gate again */                         \
      _Pragma("unroll") for (int q = 0; q < V; ++q) d[q] = gate(d[q], v[q]);                                  \
      S::store16(reinterpret_cast<elem *>(&(DR)), d);                                                         \
    }                                                                                                         \
    if constexpr (RAGGED) {                                                                                   \
      _Pragma("unroll") for (int q = 0; q < V; ++q) d[q] = q < (SKIP) ? 0.f : d[q];                           \
    }                                                                                                         \
    _Pragma("unroll") for (int q = 0; q < V; q += 4) {                                                        \
      const float d0 = d[q], d1 = d[q + 1], d2 = d[q + 2], d3 = d[q + 3];                                     \
      a += (d0 + d1) + (d2 + d3);                                                                             \
      b = __builtin_fmaf(d0, (v[q] - mean) * invstd, b);                                                      \
      b1 = __builtin_fmaf(d1, (v[q + 1] - mean) * invstd, b1);                                                \
      b = __builtin_fmaf(d2, (v[q + 2] - mean) * invstd, b);                                                  \
      b1 = __builtin_fmaf(d3, (v[q + 3] - mean) * invstd, b1);                                                \
    }                                                                                                         \
  }
  if constexpr (NL > 0) {
    // the loads into LDS are the oldest: wait for everything (the compiler does not count them for LDS reads)
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("" ::: "memory");
#pragma unroll
    for (int j = 0; j < NL; ++j)
      if (lo + j * NT + t < hi) {
        const raw xl = *reinterpret_cast<const raw *>(chip_lds + size_t((0 * NL + j) * NT + t) * 16);
        raw dl = *reinterpret_cast<const raw *>(chip_lds + size_t((1 * NL + j) * NT + t) * 16);
        BN_CHIP_ACCUMULATE(xl, dl, 0)
        if constexpr (RELU) *reinterpret_cast<raw *>(chip_lds + size_t((1 * NL + j) * NT + t) * 16) = dl;
      }
  }
  {
    ChipWalk w = wreg;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int iv = lo + (NL + i) * NT + t;
      if (iv < hi) BN_CHIP_ACCUMULATE(xv[i], dv[i], (w.r == PV - 1 ? tail_skip : 0))
      if constexpr (RAGGED) w.step(dn, dr, PV);
    }
  }
#undef BN_CHIP_ACCUMULATE
  b += b1;
  float db = sgh_block_sum(a, red), dg = sgh_block_sum(b, red);
  if (G > 1) {
    // (the block sums above contain barriers: ticket_s and gave_up are visible to every thread)
    const unsigned long long ticket = ticket_s;
    const unsigned lo32 = unsigned(ticket), hi32 = unsigned(ticket >> 32);   // (both halves are nonzero)
    if (t == 0) {
      __hip_atomic_store(words + 2 * g, (static_cast<unsigned long long>(__float_as_uint(db)) << 32) | lo32,
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(words + 2 * g + 1, (static_cast<unsigned long long>(__float_as_uint(dg)) << 32) | hi32,
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (t < G) {   // one lane per slice of the channel polls that slice's words (the second one until it is
                   // there, then the first one: one load per poll)
      unsigned long long wa = 0, wb = 0;
      int spins = 0;
      bool have_b = false;
      for (;;) {
        if (!have_b) {
          wb = __hip_atomic_load(words + 2 * t + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          have_b = unsigned(wb) == hi32;
        }
        if (have_b) {
          wa = __hip_atomic_load(words + 2 * t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (unsigned(wa) == lo32) break;
        }
        if (++spins >= spin_limit) {
          gave_up = 1;
          break;
        }
        __builtin_amdgcn_s_sleep(4);
      }
      part_a[t] = __uint_as_float(unsigned(wa >> 32));
      part_b[t] = __uint_as_float(unsigned(wb >> 32));
    }
    __syncthreads();
    // the same G numbers in the same order in every workgroup of the channel
    db = 0.f, dg = 0.f;
    for (int i = 0; i < G; ++i) db += part_a[i], dg += part_b[i];
    if (gave_up) {
      db = dg = __builtin_nanf("");
      if (t == 0) atomicAdd(&g_bn_gave_up, 1);
    }
  }
  if (g == 0 && t == 0) {
    dbeta[c] = db;
    dgamma[c] = dg;
  }
  const float k = gm * invstd;
  const float rM = float(1.0 / (double(s.N) * s.HW));
  const float c0 = db * rM, c1 = dg * rM;
  char *ob = reinterpret_cast<char *>(dx);
#define BN_CHIP_FINISH(W, XR, DR)                                                                             \
  {                                                                                                           \
    float v[V], d[V], o[V];                                                                                \
    S::template load16<false>(reinterpret_cast<const elem *>(&(XR)), v);                                      \
    S::template load16<false>(reinterpret_cast<const elem *>(&(DR)), d);                                      \
    _Pragma("unroll") for (int q = 0; q < V; ++q)                                                             \
        o[q] = k * (d[q] - __builtin_fmaf((v[q] - mean) * invstd, c1, c0));   /* (d: gated in the first pass) */ \
    raw ov;                                                                                                   \
    S::store16(reinterpret_cast<elem *>(&ov), o);                                                             \
    if constexpr (RAGGED)                                                                                     \
      __builtin_amdgcn_raw_buffer_store_b128(ov, rob, piece((W).n, (W).r), 0, 0);                             \
    else   /* (non-temporal: 3-7 % on the 25-50 MB tensors, whose lines otherwise wait dirty in L2 for the end of the kernel) */ \
      __builtin_nontemporal_store(ov, reinterpret_cast<raw *>(ob + vec_bytes(W)));                            \
  }
  if constexpr (NL > 0) {
    ChipWalk w = first;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      const int iv = lo + j * NT + t;
      if (iv < hi) {
        const raw xl = *reinterpret_cast<const raw *>(chip_lds + size_t((0 * NL + j) * NT + t) * 16);
        const raw dl = *reinterpret_cast<const raw *>(chip_lds + size_t((1 * NL + j) * NT + t) * 16);
        BN_CHIP_FINISH(w, xl, dl)
      }
      w.step(dn, dr, PV);
    }
  }
  {
    ChipWalk w = wreg;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int iv = lo + (NL + i) * NT + t;
      if (iv < hi) BN_CHIP_FINISH(w, xv[i], dv[i])
      w.step(dn, dr, PV);
    }
  }
#undef BN_CHIP_FINISH
}

// ---- forward (training) in one pass, the same way: a slice of x stays in registers (more vectors than in the
// backward kernel, there is only one tensor) from the sums to the normalisation, the G workgroups of a channel
// exchange (sum (x - pivot), sum (x - pivot)^2) through the tagged words described above and finish the
// statistics in double precision in slice order, like k_bn_fwd_apply does over its splits.  x is read once and
// y written once: 2 tensor passes instead of 3.
// vectors per thread: what stays clear of register spills beside the double-precision statistics
// (with a second tensor -- `two`, ACT == 2 in the kernel -- as many vectors of z wait in registers from before the
// exchange, so fewer of each)
template <class S>
constexpr int chip_fwd_nv(bool two) {
  return two ? (sizeof(typename S::elem) == 4 ? 7 : (S::VEC == 8 ? 5 : 7)) : (sizeof(typename S::elem) == 4 ? 12 : (S::VEC == 8 ? 8 : 12));
}

template <class S>
inline ChipPlan chip_fwd_plan(int N, int C, int HW, bool two) {
  ChipPlan p{false, 0, 0, 512, 0, false};
  if (HW % S::VEC != 0 || size_t(N) * C * HW * sizeof(typename S::elem) >= (size_t(1) << 32)) return p;
  const long TV = long(N) * (HW / S::VEC);
  const long per_wg = 512L * chip_fwd_nv<S>(two);
  long G = (TV + per_wg - 1) / per_wg;
  const long want = (2L * sgh_num_cus() + C - 1) / C;   // few channels: thinner slices, two workgroups for every CU
  if (G < want) G = want;
  const long slots = 2L * sgh_num_cus(), rounds = (long(C) * G + slots - 1) / slots;
  long fill = rounds * slots / C;                       // whole rounds
  if (fill > kChipMaxG) fill = kChipMaxG;
  if (fill > G) G = fill;
  while (G > 1 && (TV + G - 1) / G < 64) --G;
  if (G > kChipMaxG || G < 1) return p;
  p.vpg = int((TV + G - 1) / G);
  p.G = int((TV + p.vpg - 1) / p.vpg);
  p.ok = long(C) * p.G < 0x7fffffffL && chip_slices_fit(p.G, C, 512);
  return p;
}

template <class S, int ACT>
__global__ __launch_bounds__(512, 4) void k_bn_fwd_onchip(const typename S::elem *__restrict__ x,
                                                           const typename S::elem *__restrict__ z,
                                                           const float *__restrict__ gamma, const float *__restrict__ beta,
                                                           float *__restrict__ running_mean, float *__restrict__ running_var,
                                                           float factor, float eps, typename S::elem *__restrict__ y,
                                                           float *__restrict__ save_mean, float *__restrict__ save_invstd,
                                                           unsigned long long *__restrict__ ws, BnShape s, int G, int vpg,
                                                           unsigned long long ticket1, unsigned long long ticket2,
                                                           int spin_limit, int xcd_runs) {
  typedef typename S::elem elem;
  constexpr int V = S::VEC, NV = chip_fwd_nv<S>(ACT == 2), NT = 512;
  typedef typename RawVec<V * sizeof(elem)>::type raw;
  __shared__ float red[16];
  __shared__ float part_a[kChipMaxG], part_b[kChipMaxG];
  __shared__ int gave_up;
  __shared__ unsigned long long ticket_s;
  const int unit = xcd_runs ? int(blockIdx.x & 7) * int(gridDim.x >> 3) + int(blockIdx.x >> 3) : int(blockIdx.x);
  const int c = unit / G, g = unit - c * G, t = threadIdx.x;
  if (c >= s.C) return;
  unsigned long long *words = ws + size_t(c) * 2 * size_t(G);   // the channel's G slots
  if (G > 1 && t == 0) {
    const unsigned long long wa = __hip_atomic_load(words + 2 * g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long wb = __hip_atomic_load(words + 2 * g + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ticket_s = (unsigned(wa) == unsigned(ticket1) && unsigned(wb) == unsigned(ticket1 >> 32)) ? ticket2 : ticket1;
    gave_up = 0;
  }
  const int PV = s.HW / V, TV = s.N * PV;
  const int lo = g * vpg, hi = min(lo + vpg, TV);
  const float pivot = S::ld(x + size_t(c) * s.HW);
  // the vectors of a thread are walked in steps of NT (ChipWalk), byte offsets are 32 bits from a uniform base
  const char *xb = reinterpret_cast<const char *>(x);
  const unsigned CPV = unsigned(s.C) * unsigned(PV), cPV = unsigned(c) * unsigned(PV);
  const int dn = NT / PV, dr = NT - dn * PV;
  ChipWalk first;
  first.n = (lo + t) / PV, first.r = (lo + t) - first.n * PV;
  auto vec_bytes = [&](const ChipWalk &w) { return (unsigned(w.n) * CPV + cPV + unsigned(w.r)) * unsigned(sizeof(raw)); };
  raw xv[NV];
  {
    ChipWalk w = first;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (lo + i * NT + t < hi) xv[i] = __builtin_nontemporal_load(reinterpret_cast<const raw *>(xb + vec_bytes(w)));
      w.step(dn, dr, PV);
    }
  }
  float a = 0.f, b = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i)
    if (lo + i * NT + t < hi) {
      float v[V];
      S::template load16<false>(reinterpret_cast<const elem *>(&xv[i]), v);
#pragma unroll
      for (int q = 0; q < V; q += 4) {
        const float d0 = v[q] - pivot, d1 = v[q + 1] - pivot, d2 = v[q + 2] - pivot, d3 = v[q + 3] - pivot;
        a += (d0 + d1) + (d2 + d3);
        b += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
      }
    }
  // the second tensor's slice is requested now and arrives during the block sums and the exchange
  raw zr[ACT == 2 ? NV : 1];
  if constexpr (ACT == 2) {
    const char *zb = reinterpret_cast<const char *>(z);
    ChipWalk w = first;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (lo + i * NT + t < hi) zr[i] = __builtin_nontemporal_load(reinterpret_cast<const raw *>(zb + vec_bytes(w)));
      w.step(dn, dr, PV);
    }
  }
  a = sgh_block_sum(a, red);
  b = sgh_block_sum(b, red);
  double A = a, B = b;
  if (G > 1) {
    // (the block sums above contain barriers: ticket_s and gave_up are visible to every thread)
    const unsigned long long ticket = ticket_s;
    const unsigned lo32 = unsigned(ticket), hi32 = unsigned(ticket >> 32);   // (both halves are nonzero)
    if (t == 0) {
      __hip_atomic_store(words + 2 * g, (static_cast<unsigned long long>(__float_as_uint(a)) << 32) | lo32,
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(words + 2 * g + 1, (static_cast<unsigned long long>(__float_as_uint(b)) << 32) | hi32,
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (t < G) {   // one lane per slice of the channel polls that slice's words
      unsigned long long wa = 0, wb = 0;
      int spins = 0;
      bool have_b = false;
      for (;;) {
        if (!have_b) {
          wb = __hip_atomic_load(words + 2 * t + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          have_b = unsigned(wb) == hi32;
        }
        if (have_b) {
          wa = __hip_atomic_load(words + 2 * t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (unsigned(wa) == lo32) break;
        }
        if (++spins >= spin_limit) {
          gave_up = 1;
          break;
        }
        __builtin_amdgcn_s_sleep(4);
      }
      part_a[t] = __uint_as_float(unsigned(wa >> 32));
      part_b[t] = __uint_as_float(unsigned(wb >> 32));
    }
    __syncthreads();
    A = 0, B = 0;
    for (int i = 0; i < G; ++i) A += part_a[i], B += part_b[i];   // the same numbers in the same order in every slice
  }
  const double M = double(s.N) * s.HW;
  const double dm = A / M;
  double var = B / M - dm * dm;
  if (var < 0) var = 0;
  float mean = float(double(pivot) + dm);
  const float invstd = float(1.0 / sqrt(var + double(eps)));
  if (G > 1 && gave_up) {
    mean = __builtin_nanf("");
    if (t == 0) atomicAdd(&g_bn_gave_up, 1);
  }
  if (g == 0 && t == 0) {
    save_mean[c] = mean;
    save_invstd[c] = invstd;
    if (running_mean) running_mean[c] = (1.f - factor) * running_mean[c] + factor * mean;
    if (running_var) {
      const double unb = M > 1 ? var * M / (M - 1) : var;
      running_var[c] = (1.f - factor) * running_var[c] + factor * float(unb);
    }
  }
  const float gm = gamma[c], be = beta[c];
  char *ob = reinterpret_cast<char *>(y);
  ChipWalk w = first;
#pragma unroll
  for (int i = 0; i < NV; ++i, w.step(dn, dr, PV)) {
    const int iv = lo + i * NT + t;
    if (iv < hi) {
      float v[V], o[V], zv[V];
      S::template load16<false>(reinterpret_cast<const elem *>(&xv[i]), v);
      if constexpr (ACT == 2) S::template load16<false>(reinterpret_cast<const elem *>(&zr[i]), zv);
#pragma unroll
      for (int q = 0; q < V; ++q)
        o[q] = bn_fwd_value<S, ACT>(bn_out_rounded(v[q], mean, invstd, gm, be), ACT == 2 ? zv[q] : 0.f);
      raw ov;
      S::store16(reinterpret_cast<elem *>(&ov), o);
      *reinterpret_cast<raw *>(ob + vec_bytes(w)) = ov;
    }
  }
}

// tickets: a random 64-bit start (so that whatever an uninitialised workspace holds is not the next
// ticket, up to a chance of 2^-64 per slot) and one step per call
inline unsigned long long next_ticket() {
  static std::atomic<unsigned long long> t{[] {
    std::random_device rd;
    return (static_cast<unsigned long long>(rd()) << 32) ^ rd() ^ 0x9e3779b97f4a7c15ull;
  }()};
  unsigned long long v;
  do v = t.fetch_add(0x9e3779b97f4a7c15ull | 1ull, std::memory_order_relaxed);
  while (unsigned(v) == 0 || unsigned(v >> 32) == 0);   // a zeroed word must never look valid
  return v;
}

template <class S, int ACT>
int launch_fwd_onchip(const typename S::elem *x, const typename S::elem *z, const float *gamma, const float *beta,
                      float *running_mean,
                      float *running_var, float factor, float eps, typename S::elem *y, float *save_mean,
                      float *save_invstd, void *workspace, const BnShape &s, const ChipPlan &p, hipStream_t st) {
  const int xcd_runs = p.G <= 16 && s.C >= 8 ? 1 : 0;
  const dim3 grid(xcd_runs ? unsigned((s.C + 7) / 8) * 8u * p.G : unsigned(s.C) * p.G);
  const unsigned long long t1 = next_ticket(), t2 = next_ticket();
  if (p.G > 1) g_exchange_ran.store(true, std::memory_order_relaxed);
  hipLaunchKernelGGL((k_bn_fwd_onchip<S, ACT>), grid, dim3(512), 0, st, x, z, gamma, beta, running_mean, running_var, factor,
                     eps, y, save_mean, save_invstd, static_cast<unsigned long long *>(workspace), s, p.G, p.vpg, t1, t2,
                     g_spin_limit.load(std::memory_order_relaxed), xcd_runs);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

template <class S, bool RELU>
int launch_onchip(const typename S::elem *dy, const typename S::elem *x, const float *gamma, const float *beta,
                  const float *save_mean, const float *save_invstd, typename S::elem *dx, float *dgamma, float *dbeta,
                  void *workspace, const BnShape &s, const ChipPlan &p, hipStream_t st) {
  unsigned long long *ws = static_cast<unsigned long long *>(workspace);
  // (a run of channels per XCD needs the G workgroups of a channel resident on one XCD's 32 CUs together)
  const int xcd_runs = p.G <= 16 && s.C >= 8 ? 1 : 0;
  const dim3 grid(xcd_runs ? unsigned((s.C + 7) / 8) * 8u * p.G : unsigned(s.C) * p.G);
  // from four rounds on, half of the first round starts 6 us late (fp32 64 x 64 x 112 x 112, seven rounds: 135 -> 128 us;
  // two-round launches lose: 64 x 64 x 56 x 56 36 -> 41 us); SGH_BN_DEPHASE_US overrides the delay (0: off)
  static const int dephase_env = getenv("SGH_BN_DEPHASE_US") ? atoi(getenv("SGH_BN_DEPHASE_US")) : 6;
  const long rounds = (long(s.C) * p.G + 2L * sgh_num_cus() - 1) / (2L * sgh_num_cus());
  // (fp32 only: the 16-bit launches of many rounds lose a little with it -- ResNet-50 in binary16, N = 128, BatchNorm
  // backward 2.29 -> 2.33 ms per step)
  const int dephase = p.G > 1 && rounds >= 4 && p.nt == 512 && sizeof(typename S::elem) == 4 ? dephase_env * 100 : 0;
  const unsigned long long t1 = next_ticket(), t2 = next_ticket();
  if (p.G > 1) g_exchange_ran.store(true, std::memory_order_relaxed);
  if constexpr (chip_nl<S>() > 0) {
    if (p.nl > 0) {
      constexpr int NL = chip_nl<S>();
      auto kern = k_bn_bwd_onchip<S, RELU, 512, NL>;
      constexpr int lds = 2 * NL * 512 * 16;
      static bool attr = false;
      if (!attr) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds) !=
            hipSuccess)
          return SGH_EUNSUPPORTED;
        attr = true;
      }
      SGH_LAUNCH_TIMED(kern, grid, dim3(512), lds, st, dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, ws,
                         s, p.G, p.vpg, t1, t2, g_spin_limit.load(std::memory_order_relaxed), xcd_runs, dephase);
      return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
    }
  }
  if constexpr (S::VEC * sizeof(typename S::elem) == 16) {
    if (p.ragged && p.nt == 1024) {
      SGH_LAUNCH_TIMED((k_bn_bwd_onchip<S, RELU, 1024, 0, true>), grid, dim3(1024), 0, st, dy, x, gamma, beta, save_mean,
                         save_invstd, dx, dgamma, dbeta, ws, s, p.G, p.vpg, t1, t2, g_spin_limit.load(std::memory_order_relaxed), xcd_runs, dephase);
      return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
    }
    if (p.ragged) {
      SGH_LAUNCH_TIMED((k_bn_bwd_onchip<S, RELU, 512, 0, true>), grid, dim3(512), 0, st, dy, x, gamma, beta, save_mean,
                         save_invstd, dx, dgamma, dbeta, ws, s, p.G, p.vpg, t1, t2, g_spin_limit.load(std::memory_order_relaxed), xcd_runs, dephase);
      return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
    }
  }
  if (p.ragged) return SGH_EUNSUPPORTED;
  if (p.nt == 512)
    SGH_LAUNCH_TIMED((k_bn_bwd_onchip<S, RELU, 512>), grid, dim3(512), 0, st, dy, x, gamma, beta, save_mean, save_invstd,
                       dx, dgamma, dbeta, ws, s, p.G, p.vpg, t1, t2, g_spin_limit.load(std::memory_order_relaxed), xcd_runs, dephase);
  else
    SGH_LAUNCH_TIMED((k_bn_bwd_onchip<S, RELU, 1024>), grid, dim3(1024), 0, st, dy, x, gamma, beta, save_mean,
                       save_invstd, dx, dgamma, dbeta, ws, s, p.G, p.vpg, t1, t2, g_spin_limit.load(std::memory_order_relaxed), xcd_runs, dephase);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
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
  SGH_LAUNCH_TIMED(kern, dim3((s.C + 7) / 8 * 8), dim3(kResNT), lds, st, dy, x, gamma, beta, save_mean, save_invstd, dx,
                   dgamma, dbeta, s);
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

// Layout of a BatchNorm workspace (sgh_bn_workspace_bytes), three parts, each a multiple of 256 bytes:
//   [0, twopass)            partial sums of the two-pass kernels, forward and backward, any storage type
//   [twopass, + bwd words)  exchange words of the one-pass backward kernel
//   [.., + fwd words)       exchange words of the one-pass forward kernel
// A recorded one-pass launch tells which of its two tickets is next from what its own words hold, so every word
// of a channel must be written by that kernel only between two replays: each one-pass kernel owns its part, and
// nothing else writes there (a two-pass forward on the same handle between two replays of a recorded backward
// used to overwrite the head of the backward words while they shared offset 0).
inline size_t round256(size_t v) { return (v + 255) & ~size_t(255); }

inline size_t twopass_workspace_bytes(int N, int C, int HW) {
  const int s4 = make_shape(N, C, HW, 4, 4).S, s8 = make_shape(N, C, HW, 8, 2).S, s4h = make_shape(N, C, HW, 4, 2).S;
  const int smax = s4 > s8 ? (s4 > s4h ? s4 : s4h) : (s8 > s4h ? s8 : s4h);
  return round256(size_t(C) * smax * 2 * sizeof(float));
}

template <class S>
inline size_t bwd_words_bytes_of(int N, int C, int HW) {
  const ChipPlan cp = chip_plan<S>(N, C, HW);
  return cp.ok ? chip_workspace_bytes(C, cp.G) : 0;
}

inline size_t bwd_words_bytes(int N, int C, int HW) {
  const size_t b[3] = {bwd_words_bytes_of<StF32>(N, C, HW), bwd_words_bytes_of<StF16>(N, C, HW),
                       bwd_words_bytes_of<StF16x4>(N, C, HW)};
  size_t need = 0;
  for (size_t v : b) need = v > need ? v : need;
  return round256(need);
}

// where the one-pass forward kernel's words start
inline size_t shared_workspace_bytes(int N, int C, int HW) {
  return twopass_workspace_bytes(N, C, HW) + bwd_words_bytes(N, C, HW);
}

// bytes of workspace the backward pass of storage class S needs: the partial sums of the two-pass kernels, and
// behind that part the words of the one-pass kernel where the shape takes it
template <class S>
inline size_t bwd_workspace_need(int N, int C, int HW) {
  const size_t two_pass = size_t(C) * make_shape(N, C, HW, S::VEC, int(sizeof(typename S::elem))).S * 2 * sizeof(float);
  const size_t words = bwd_words_bytes_of<S>(N, C, HW);
  const size_t chip = words ? twopass_workspace_bytes(N, C, HW) + words : 0;
  return two_pass > chip ? two_pass : chip;
}

// the same for a caller that keeps the words at the start of a buffer of its own (sgh_bn_bwd_noalloc_f32)
template <class S>
inline size_t bwd_workspace_need_flat(int N, int C, int HW) {
  const size_t two_pass = size_t(C) * make_shape(N, C, HW, S::VEC, int(sizeof(typename S::elem))).S * 2 * sizeof(float);
  const size_t words = bwd_words_bytes_of<S>(N, C, HW);
  return two_pass > words ? two_pass : words;
}

template <class S, int ACT>
int bn_fwd_train_act(const typename S::elem *x, const typename S::elem *z, const float *gamma, const float *beta,
                     float *running_mean, float *running_var, float factor, float eps, typename S::elem *y,
                     float *save_mean, float *save_invstd, int N, int C, int HW, void *workspace, size_t ws_bytes,
                     void *stream) {
  if (!shape_ok(N, C, HW) || !x || !gamma || !beta || !y || !save_mean || !save_invstd) return SGH_EINVAL;
  if (ACT == 2 && (!z || !sgh_aligned16(z))) return SGH_EINVAL;
  const BnShape s = make_shape(N, C, HW, S::VEC, int(sizeof(typename S::elem)));
  if (!sgh_aligned16(x) || !sgh_aligned16(y)) return SGH_EINVAL;
  if (!workspace || ws_bytes < size_t(C) * s.S * 2 * sizeof(float)) return SGH_EWORKSPACE;
  const ChipPlan fp = chip_fwd_plan<S>(N, C, HW, ACT == 2);
  // the one-pass kernel's words lie behind everything the backward pass and the two-pass kernels write: a
  // recorded launch tells which of its two tickets is next from what its own words hold, so no other kernel
  // may write some of a channel's words between two replays
  const size_t slots_at = shared_workspace_bytes(N, C, HW);
  if (fp.ok && !sgh_env().bn_onchip_off && !sgh_env().bn_fwd_onchip_off && sgh_aligned16(workspace) &&
      ws_bytes >= slots_at + chip_workspace_bytes(C, fp.G))
    return launch_fwd_onchip<S, ACT>(x, z, gamma, beta, running_mean, running_var, factor, eps, y, save_mean, save_invstd,
                                     static_cast<char *>(workspace) + slots_at, s, fp, sgh_stream_of(stream));
  float *scratch = static_cast<float *>(workspace);
  hipLaunchKernelGGL(k_bn_fwd_partial<S>, dim3(C * s.S), dim3(kBlock), 0, sgh_stream_of(stream), x, scratch, s);
  SGH_LAUNCH_CHECK();
  hipLaunchKernelGGL((k_bn_fwd_apply<S, ACT>), dim3(C * s.S), dim3(kBlock), 0, sgh_stream_of(stream), x, z, gamma, beta,
                     scratch, running_mean, running_var, factor, eps, y, save_mean, save_invstd, s);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

// (act: 0 = BatchNorm alone, 1 = + ReLU, 2 = + the second tensor z, then ReLU)
template <class S>
int bn_fwd_train(const typename S::elem *x, const float *gamma, const float *beta, float *running_mean,
                 float *running_var, float factor, float eps, typename S::elem *y, float *save_mean, float *save_invstd,
                 int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream, int act = 0,
                 const typename S::elem *z = nullptr) {
  switch (act) {
    case 0:
      return bn_fwd_train_act<S, 0>(x, nullptr, gamma, beta, running_mean, running_var, factor, eps, y, save_mean,
                                    save_invstd, N, C, HW, workspace, ws_bytes, stream);
    case 1:
      return bn_fwd_train_act<S, 1>(x, nullptr, gamma, beta, running_mean, running_var, factor, eps, y, save_mean,
                                    save_invstd, N, C, HW, workspace, ws_bytes, stream);
    default:
      return bn_fwd_train_act<S, 2>(x, z, gamma, beta, running_mean, running_var, factor, eps, y, save_mean, save_invstd,
                                    N, C, HW, workspace, ws_bytes, stream);
  }
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
           int C, int HW, void *workspace, size_t ws_bytes, void *stream, bool flat_workspace = false) {
  if (!shape_ok(N, C, HW) || !dy || !x || !gamma || !save_mean || !save_invstd || !dx || !dgamma || !dbeta)
    return SGH_EINVAL;
  if (!sgh_aligned16(x) || !sgh_aligned16(dy) || !sgh_aligned16(dx)) return SGH_EINVAL;
  const BnShape s = make_shape(N, C, HW, S::VEC, int(sizeof(typename S::elem)));
  if (!workspace || ws_bytes < (flat_workspace ? bwd_workspace_need_flat<S>(N, C, HW) : bwd_workspace_need<S>(N, C, HW)))
    return SGH_EWORKSPACE;
  // the one-pass kernel's words: a part of their own behind the two-pass partial sums (see the layout above);
  // `flat_workspace`: at the start of a buffer whose owner clears them before every call
  void *words = flat_workspace ? workspace : static_cast<char *>(workspace) + twopass_workspace_bytes(N, C, HW);
  float *part = static_cast<float *>(workspace);
  const dim3 grid(C * s.S), block(kBlock);
  hipStream_t st = sgh_stream_of(stream);
  // algorithmic bytes: x and dy in, dx out (the fused form covers the ReLU backward as well)
  sgh_prof_kernel_scope prof(beta ? "bn_relu_bwd/k_bn_bwd" : "bn_bwd/k_bn_bwd", 3.0 * N * C * HW * sizeof(typename S::elem), st);
  const ChipPlan cp = chip_plan<S>(N, C, HW);
  // (channels of at most 4096 vectors that fit in LDS are a little faster through the LDS-resident kernel below:
  // 13.4 against 14.9 us at 64 x 256 x 14 x 14 fp32)
  // (ragged planes of few elements -- 7 x 7 -- as well, unless the channels need more than two rounds of its
  // one workgroup per channel: f16 128 x 512 x 7 x 7 13.3 us there, 13.9 here, but 128 x 2048 x 7 x 7 42.6 against
  // 23.7 -- the LDS-resident kernel moves single elements)
  // (shapes that give every CU a whole channel -- no exchange, G = 1 -- run faster in registers: fp32 64 x 256 x 14 x 14
  // 11.5 -> 10.2 us, 64 x 512 x 7 x 7 10.2 -> 7.7 us, kernels alone on cold tensors; binary16 128 x 512 x 7 x 7 16.3 ->
  // 13.6 us between events)
  const bool small_resident = !(cp.ok && cp.G == 1) &&
                              resident_ok(N, C, HW, sizeof(typename S::elem)) &&
                              (cp.ragged ? HW <= 64 && C <= 2 * sgh_num_cus() : long(N) * (HW / S::VEC) <= 4096);
  if (cp.ok && !small_resident && !sgh_env().bn_onchip_off) {
    if (!sgh_aligned16(workspace)) return SGH_EINVAL;
    return beta ? launch_onchip<S, true>(dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, words, s, cp, st)
                : launch_onchip<S, false>(dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, words, s, cp, st);
  }
  if (resident_ok(N, C, HW, sizeof(typename S::elem))) {
    const int rc = beta ? launch_resident<S, true>(dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, s, st)
                        : launch_resident<S, false>(dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, s, st);
    if (rc != SGH_EUNSUPPORTED) return rc;
  }
  prof.span();   // two kernels
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

// the exchange words of the one-pass kernel in the shared buffer, zeroed (no ticket has a zero half)
__global__ __launch_bounds__(256) void k_bn_clear_words(unsigned long long *__restrict__ w, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) w[i] = 0ull;
}

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

// Reads and clears the give-up counter of the current device if a multi-slice one-pass kernel has been launched
// since the last look (so a caller that never runs one pays nothing); the stream(s) must be idle.
int sgh_bn_take_exchange_failures(int *count) {
  *count = 0;
  if (!g_exchange_ran.exchange(false, std::memory_order_relaxed)) return SGH_OK;
  int v = 0;
  SGH_HIP_TRY(hipMemcpyFromSymbol(&v, HIP_SYMBOL(g_bn_gave_up), sizeof(int), 0, hipMemcpyDeviceToHost));
  if (v != 0) {
    const int zero = 0;
    SGH_HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(g_bn_gave_up), &zero, sizeof(int), 0, hipMemcpyHostToDevice));
  }
  *count = v;
  return SGH_OK;
}

void sgh_bn_mark_exchange_ran() { g_exchange_ran.store(true, std::memory_order_relaxed); }

int sgh_bn_noalloc_setup() {
  float *p = nullptr;
  return noalloc_scratch_of_current_device(&p);
}

extern "C" {

int sgh_bn_exchange_failures(void *stream, int *count) {
  if (!count) return SGH_EINVAL;
  SGH_HIP_TRY(hipStreamSynchronize(sgh_stream_of(stream)));
  g_exchange_ran.store(true, std::memory_order_relaxed);   // (asked for explicitly: always look)
  return sgh_bn_take_exchange_failures(count);
}

void sgh_bn_exchange_spin_limit(int polls) {
  g_spin_limit.store(polls > 0 ? polls : kChipSpinLimit, std::memory_order_relaxed);
}

size_t sgh_bn_workspace_bytes(int N, int C, int HW) {
  if (!shape_ok(N, C, HW)) return 0;
  // the shared part, then the words of the one-pass forward kernel
  size_t fwd = 0;
  const ChipPlan f[6] = {chip_fwd_plan<StF32>(N, C, HW, false), chip_fwd_plan<StF16>(N, C, HW, false),
                         chip_fwd_plan<StF16x4>(N, C, HW, false), chip_fwd_plan<StF32>(N, C, HW, true),
                         chip_fwd_plan<StF16>(N, C, HW, true), chip_fwd_plan<StF16x4>(N, C, HW, true)};
  for (const ChipPlan &p : f)
    if (p.ok && chip_workspace_bytes(C, p.G) > fwd) fwd = chip_workspace_bytes(C, p.G);
  return shared_workspace_bytes(N, C, HW) + fwd;
}

// 16-bit planes that are a multiple of 4 but not of 8 elements (14 x 14) use the 8-byte vector class
#define SGH_BN_DISPATCH16(fn, F16X8, F16X4, ...) \
  (HW % 8 != 0 && HW % 4 == 0 ? fn<F16X4>(__VA_ARGS__) : fn<F16X8>(__VA_ARGS__))
// (the backward pass takes such planes in 16-byte pieces, the last one overlapping -- RAGGED in k_bn_bwd_onchip:
// 128 x 1024 x 14 x 14 47.4 -> 41.4 us, fused with the ReLU gate 52.2 -> 44.9)
#define SGH_BN_DISPATCH16_BWD(fn, F16X8, F16X4, ...) \
  (HW % 8 != 0 && HW % 4 == 0 && sgh_env().bn_ragged_off ? fn<F16X4>(__VA_ARGS__) : fn<F16X8>(__VA_ARGS__))

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

int sgh_bn_relu_fwd_train_f32(const float *x, const float *gamma, const float *beta, float *running_mean,
                              float *running_var, float factor, float eps, float *y, float *save_mean,
                              float *save_invstd, int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  return bn_fwd_train<StF32>(x, gamma, beta, running_mean, running_var, factor, eps, y, save_mean, save_invstd, N, C, HW,
                             workspace, ws_bytes, stream, 1);
}
int sgh_bn_relu_fwd_train_f16(const uint16_t *x, const float *gamma, const float *beta, float *running_mean,
                              float *running_var, float factor, float eps, uint16_t *y, float *save_mean,
                              float *save_invstd, int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  return SGH_BN_DISPATCH16(bn_fwd_train, StF16, StF16x4, x, gamma, beta, running_mean, running_var, factor, eps, y,
                           save_mean, save_invstd, N, C, HW, workspace, ws_bytes, stream, 1);
}
int sgh_bn_relu_fwd_train_bf16(const uint16_t *x, const float *gamma, const float *beta, float *running_mean,
                               float *running_var, float factor, float eps, uint16_t *y, float *save_mean,
                               float *save_invstd, int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  return SGH_BN_DISPATCH16(bn_fwd_train, StBF16, StBF16x4, x, gamma, beta, running_mean, running_var, factor, eps, y,
                           save_mean, save_invstd, N, C, HW, workspace, ws_bytes, stream, 1);
}
int sgh_bn_add_relu_fwd_train_f32(const float *x, const float *z, const float *gamma, const float *beta,
                                  float *running_mean, float *running_var, float factor, float eps, float *y,
                                  float *save_mean, float *save_invstd, int N, int C, int HW, void *workspace,
                                  size_t ws_bytes, void *stream) {
  return bn_fwd_train<StF32>(x, gamma, beta, running_mean, running_var, factor, eps, y, save_mean, save_invstd, N, C, HW,
                             workspace, ws_bytes, stream, 2, z);
}
int sgh_bn_add_relu_fwd_train_f16(const uint16_t *x, const uint16_t *z, const float *gamma, const float *beta,
                                  float *running_mean, float *running_var, float factor, float eps, uint16_t *y,
                                  float *save_mean, float *save_invstd, int N, int C, int HW, void *workspace,
                                  size_t ws_bytes, void *stream) {
  return SGH_BN_DISPATCH16(bn_fwd_train, StF16, StF16x4, x, gamma, beta, running_mean, running_var, factor, eps, y,
                           save_mean, save_invstd, N, C, HW, workspace, ws_bytes, stream, 2, z);
}
int sgh_bn_add_relu_fwd_train_bf16(const uint16_t *x, const uint16_t *z, const float *gamma, const float *beta,
                                   float *running_mean, float *running_var, float factor, float eps, uint16_t *y,
                                   float *save_mean, float *save_invstd, int N, int C, int HW, void *workspace,
                                   size_t ws_bytes, void *stream) {
  return SGH_BN_DISPATCH16(bn_fwd_train, StBF16, StBF16x4, x, gamma, beta, running_mean, running_var, factor, eps, y,
                           save_mean, save_invstd, N, C, HW, workspace, ws_bytes, stream, 2, z);
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
  if (!shape_ok(N, C, HW) || !dy || !x || !gamma || !save_mean || !save_invstd || !dx || !dgamma || !dbeta)
    return SGH_EINVAL;
  if (!sgh_aligned16(x) || !sgh_aligned16(dy) || !sgh_aligned16(dx)) return SGH_EINVAL;   // (before anything is launched)
  const size_t need = bwd_workspace_need_flat<StF32>(N, C, HW);
  if (need > sizeof(float) * 2 * size_t(kNoAllocMaxPairs)) return SGH_ELIMIT;
  float *part = nullptr;
  const int rc = noalloc_scratch_of_current_device(&part);
  if (rc != SGH_OK) return rc;
  // The two-pass kernels read only what the same call wrote.  The one-pass kernel tells from what its words
  // hold which of its two tickets a replay of a recorded launch publishes under, and that needs every word of a
  // channel in the same state: here calls of other shapes write the same buffer in between, some words of a
  // channel and not others, so its words are cleared first (by a kernel: a recorded call replays it too) and
  // every execution publishes under its first ticket.
  const ChipPlan cp = chip_plan<StF32>(N, C, HW);
  if (cp.ok && cp.G > 1) {
    const int words = int(chip_workspace_bytes(C, cp.G) / sizeof(unsigned long long));
    hipLaunchKernelGGL(k_bn_clear_words, dim3((words + 255) / 256), dim3(256), 0, sgh_stream_of(stream),
                       reinterpret_cast<unsigned long long *>(part), words);
    SGH_LAUNCH_CHECK();
  }
  return bn_bwd<StF32>(dy, x, gamma, nullptr, save_mean, save_invstd, dx, dgamma, dbeta, N, C, HW, part, need, stream, true);
}
int sgh_bn_bwd_f16(const uint16_t *dy, const uint16_t *x, const float *gamma, const float *save_mean,
                   const float *save_invstd, uint16_t *dx, float *dgamma, float *dbeta, int N, int C, int HW,
                   void *workspace, size_t ws_bytes, void *stream) {
  return SGH_BN_DISPATCH16_BWD(bn_bwd, StF16, StF16x4, dy, x, gamma, nullptr, save_mean, save_invstd, dx, dgamma, dbeta, N,
                           C, HW, workspace, ws_bytes, stream);
}
int sgh_bn_bwd_bf16(const uint16_t *dy, const uint16_t *x, const float *gamma, const float *save_mean,
                    const float *save_invstd, uint16_t *dx, float *dgamma, float *dbeta, int N, int C, int HW,
                    void *workspace, size_t ws_bytes, void *stream) {
  return SGH_BN_DISPATCH16_BWD(bn_bwd, StBF16, StBF16x4, dy, x, gamma, nullptr, save_mean, save_invstd, dx, dgamma, dbeta, N,
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
  return SGH_BN_DISPATCH16_BWD(bn_bwd, StF16, StF16x4, dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, N, C,
                           HW, workspace, ws_bytes, stream);
}
int sgh_bn_relu_bwd_bf16(const uint16_t *dy, const uint16_t *x, const float *gamma, const float *beta,
                         const float *save_mean, const float *save_invstd, uint16_t *dx, float *dgamma, float *dbeta,
                         int N, int C, int HW, void *workspace, size_t ws_bytes, void *stream) {
  if (!beta) return SGH_EINVAL;
  return SGH_BN_DISPATCH16_BWD(bn_bwd, StBF16, StBF16x4, dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, N, C,
                           HW, workspace, ws_bytes, stream);
}
#undef SGH_BN_DISPATCH16
#undef SGH_BN_DISPATCH16_BWD

}  // extern "C"
