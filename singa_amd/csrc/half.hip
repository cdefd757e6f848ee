// 16-bit storage variants of the bandwidth-bound backward ops: IEEE binary16 ("f16") and bfloat16
// ("bf16") tensors travel as uint16_t arrays; arithmetic is fp32 with ONE rounding (to nearest,
// ties to even) when a result is stored, which is what the reference's half kernels do through
// __half2float / __float2half (src/core/tensor/math_kernel.cu:111-117, :261-271, :353-375).
// ReLU backward keeps the CPU rule (gradient 0 at x == 0), not the CUDA half kernel's '>='.
//
// Each thread moves 16 bytes (8 elements) per access; a workgroup streams contiguous 16 KB
// chunks, as in the fp32 kernels.
#include <string.h>

#include "common.h"
#include "storage.h"
#include "sgd_math.h"

namespace {

constexpr int kBlock = 256;
constexpr int kUnroll = 4;

typedef unsigned short u16;
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

struct F16 {
  static __device__ __forceinline__ float load(u16 b) { return sgh_f16_to_f32(b); }
  static __device__ __forceinline__ u16 store(float f) { return sgh_f32_to_f16(f); }
  static __device__ __forceinline__ unsigned pack2(float lo, float hi) { return sgh_pack2_f16(lo, hi); }
};

struct BF16 {
  static __device__ __forceinline__ float load(u16 b) { return sgh_bf16_to_f32(b); }
  static __device__ __forceinline__ u16 store(float f) { return sgh_f32_to_bf16(f); }
  static __device__ __forceinline__ unsigned pack2(float lo, float hi) { return sgh_pack2_bf16(lo, hi); }
};

inline int grid_for(size_t nvec) {
  size_t per_block = size_t(kBlock) * kUnroll;
  size_t blocks = (nvec + per_block - 1) / per_block;
  const size_t cap = size_t(sgh_num_cus()) * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return int(blocks);
}

// out = f(a, b) over 16-bit tensors; vectors of 8 elements
template <class T, class F>
__global__ __launch_bounds__(kBlock) void k_map2_h(const u16 *a, const u16 *b, u16 *o, size_t n, F f, int vec) {
  if (vec) {
    const size_t nvec = n >> 3;
    const v4u *a4 = reinterpret_cast<const v4u *>(a);
    const v4u *b4 = reinterpret_cast<const v4u *>(b);
    v4u *o4 = reinterpret_cast<v4u *>(o);
    const size_t step = size_t(gridDim.x) * (kBlock * kUnroll);
    for (size_t base = size_t(blockIdx.x) * (kBlock * kUnroll); base < nvec; base += step) {
      v4u va[kUnroll], vb[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const size_t i = base + u * kBlock + threadIdx.x;
        if (i < nvec) {
          va[u] = a4[i];
          vb[u] = b4[i];
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const size_t i = base + u * kBlock + threadIdx.x;
        if (i < nvec) {
          v4u r;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float lo = f(T::load(u16(va[u][j] & 0xffffu)), T::load(u16(vb[u][j] & 0xffffu)));
            const float hi = f(T::load(u16(va[u][j] >> 16)), T::load(u16(vb[u][j] >> 16)));
            r[j] = T::pack2(lo, hi);
          }
          o4[i] = r;
        }
      }
    }
    if (blockIdx.x == 0) {
      const size_t t = (nvec << 3) + threadIdx.x;
      if (t < n) o[t] = T::store(f(T::load(a[t]), T::load(b[t])));
    }
  } else {
    const size_t stride = size_t(gridDim.x) * kBlock;
    for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride)
      o[i] = T::store(f(T::load(a[i]), T::load(b[i])));
  }
}

template <class T, class F>
int launch_map2_h(const uint16_t *a, const uint16_t *b, uint16_t *o, size_t n, F f, void *stream) {
  if (n == 0) return SGH_OK;
  if (!a || !b || !o) return SGH_EINVAL;
  const int vec = sgh_aligned16(a) && sgh_aligned16(b) && sgh_aligned16(o);
  SGH_LAUNCH_TIMED((k_map2_h<T, F>), dim3(grid_for(vec ? n >> 3 : n)), dim3(kBlock), 0, sgh_stream_of(stream), a, b, o,
                     n, f, vec);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

struct ReluBwd {
  __device__ __forceinline__ float operator()(float dy, float x) const { return x > 0.f ? dy : 0.f; }
};
struct ReluFwd {   // (math_kernel.cu:242-251: in > 0 ? in : 0)
  __device__ __forceinline__ float operator()(float x, float) const { return x > 0.f ? x : 0.f; }
};

// dx = x > 0 ? dy0 + dy1 : 0: ReLU backward on a gradient that arrives as two summands (the two
// branches of a residual block), so that the sum is never stored.  dx may alias dy0 or dy1.
template <class S>
__global__ __launch_bounds__(kBlock) void k_relu_bwd_add(const typename S::elem *dy0, const typename S::elem *dy1,
                                                         const typename S::elem *x, typename S::elem *dx, size_t n,
                                                         int vec) {
  constexpr int V = S::VEC;
  if (vec) {
    const size_t nvec = n / V;
    const size_t step = size_t(gridDim.x) * (kBlock * kUnroll);
    for (size_t base = size_t(blockIdx.x) * (kBlock * kUnroll); base < nvec; base += step) {
      float a[kUnroll][V], b[kUnroll][V], g[kUnroll][V];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const size_t i = base + u * kBlock + threadIdx.x;
        if (i < nvec) {
          S::template load16<true>(dy0 + i * V, a[u]);
          S::template load16<true>(dy1 + i * V, b[u]);
          S::template load16<true>(x + i * V, g[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const size_t i = base + u * kBlock + threadIdx.x;
        if (i < nvec) {
          float r[V];
#pragma unroll
          for (int j = 0; j < V; ++j) r[j] = g[u][j] > 0.f ? a[u][j] + b[u][j] : 0.f;
          S::store16(dx + i * V, r);
        }
      }
    }
    if (blockIdx.x == 0) {
      const size_t t = nvec * V + threadIdx.x;
      if (t < n) S::st(dx + t, S::ld(x + t) > 0.f ? S::ld(dy0 + t) + S::ld(dy1 + t) : 0.f);
    }
  } else {
    const size_t stride = size_t(gridDim.x) * kBlock;
    for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride)
      S::st(dx + i, S::ld(x + i) > 0.f ? S::ld(dy0 + i) + S::ld(dy1 + i) : 0.f);
  }
}

template <class S>
int launch_relu_bwd_add(const typename S::elem *dy0, const typename S::elem *dy1, const typename S::elem *x,
                        typename S::elem *dx, size_t n, void *stream) {
  if (n == 0) return SGH_OK;
  if (!dy0 || !dy1 || !x || !dx) return SGH_EINVAL;
  const int vec = sgh_aligned16(dy0) && sgh_aligned16(dy1) && sgh_aligned16(x) && sgh_aligned16(dx);
  SGH_LAUNCH_TIMED(k_relu_bwd_add<S>, dim3(grid_for(vec ? n / S::VEC : n)), dim3(kBlock), 0, sgh_stream_of(stream),
                     dy0, dy1, x, dx, n, vec);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}
struct AddOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
template <class T>
struct AddReluOp {  // the stored sum where it is positive, else 0: Add followed by the 16-bit ReLU
  __device__ __forceinline__ float operator()(float a, float b) const {
    const float s = T::load(T::store(a + b));
    return s > 0.f ? s : 0.f;
  }
};
struct MulOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a * b; }
};
struct AxpyOp {  // (x, y) -> y + alpha * x in fp32 (two fp32 roundings, then the storage rounding)
  float alpha;
  __device__ __forceinline__ float operator()(float x, float y) const {
#pragma clang fp contract(off)
    const float t = alpha * x;
    return y + t;
  }
};

// casts: fp32 <-> 16-bit, 8 elements per thread per access on the 16-bit side
template <class T>
__global__ __launch_bounds__(kBlock) void k_cast_to16(const float *__restrict__ src, u16 *__restrict__ dst, size_t n,
                                                     int vec) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  if (vec) {
    const size_t nvec = n >> 3;
    const float4 *s4 = reinterpret_cast<const float4 *>(src);
    v4u *d4 = reinterpret_cast<v4u *>(dst);
    for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < nvec; i += stride) {
      const float4 x0 = s4[2 * i], x1 = s4[2 * i + 1];
      v4u r;
      r[0] = T::pack2(x0.x, x0.y);
      r[1] = T::pack2(x0.z, x0.w);
      r[2] = T::pack2(x1.x, x1.y);
      r[3] = T::pack2(x1.z, x1.w);
      d4[i] = r;
    }
    if (blockIdx.x == 0) {
      const size_t t = (nvec << 3) + threadIdx.x;
      if (t < n) dst[t] = T::store(src[t]);
    }
  } else {
    for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) dst[i] = T::store(src[i]);
  }
}

template <class T>
__global__ __launch_bounds__(kBlock) void k_cast_from16(const u16 *__restrict__ src, float *__restrict__ dst, size_t n,
                                                       int vec) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  if (vec) {
    const size_t nvec = n >> 3;
    const v4u *s4 = reinterpret_cast<const v4u *>(src);
    float4 *d4 = reinterpret_cast<float4 *>(dst);
    for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < nvec; i += stride) {
      const v4u v = s4[i];
      d4[2 * i] = make_float4(T::load(u16(v[0] & 0xffffu)), T::load(u16(v[0] >> 16)), T::load(u16(v[1] & 0xffffu)),
                              T::load(u16(v[1] >> 16)));
      d4[2 * i + 1] = make_float4(T::load(u16(v[2] & 0xffffu)), T::load(u16(v[2] >> 16)), T::load(u16(v[3] & 0xffffu)),
                                  T::load(u16(v[3] >> 16)));
    }
    if (blockIdx.x == 0) {
      const size_t t = (nvec << 3) + threadIdx.x;
      if (t < n) dst[t] = T::load(src[t]);
    }
  } else {
    for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) dst[i] = T::load(src[i]);
  }
}

template <class T>
int cast_to16(const float *src, uint16_t *dst, size_t n, void *stream) {
  if (n == 0) return SGH_OK;
  if (!src || !dst) return SGH_EINVAL;
  const int vec = sgh_aligned16(src) && sgh_aligned16(dst);
  hipLaunchKernelGGL(k_cast_to16<T>, dim3(grid_for(vec ? n >> 3 : n)), dim3(kBlock), 0, sgh_stream_of(stream), src, dst, n,
                     vec);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

template <class T>
int cast_from16(const uint16_t *src, float *dst, size_t n, void *stream) {
  if (n == 0) return SGH_OK;
  if (!src || !dst) return SGH_EINVAL;
  const int vec = sgh_aligned16(src) && sgh_aligned16(dst);
  hipLaunchKernelGGL(k_cast_from16<T>, dim3(grid_for(vec ? n >> 3 : n)), dim3(kBlock), 0, sgh_stream_of(stream), src, dst,
                     n, vec);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

// Fused SGD-momentum on 16-bit gradients.
//   MASTER = false: p, g, v all 16-bit (opt.SGD constructed with dtype float16): fp32 arithmetic,
//                   p and v rounded once per step;
//   MASTER = true : fp32 master weights p32 and fp32 momentum v32 are updated from the 16-bit
//                   gradient and the 16-bit working copy p16 is refreshed from the master.
template <class T, bool MASTER>
__global__ __launch_bounds__(kBlock) void k_sgd_h(u16 *__restrict__ p16, const u16 *__restrict__ g16,
                                                 u16 *__restrict__ v16, float *__restrict__ p32,
                                                 float *__restrict__ v32, size_t n, SgdHyper h, int nesterov) {
  const bool has_v = h.mu != 0.f && (MASTER ? v32 != nullptr : v16 != nullptr);
  const size_t stride = size_t(gridDim.x) * kBlock;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
    float pp = MASTER ? p32[i] : T::load(p16[i]);
    float vv = has_v ? (MASTER ? v32[i] : T::load(v16[i])) : 0.f;
    sgd_one(pp, T::load(g16[i]), vv, h, nesterov, has_v);
    if (MASTER) {
      p32[i] = pp;
      if (has_v) v32[i] = vv;
    } else if (has_v) {
      v16[i] = T::store(vv);
    }
    p16[i] = T::store(pp);
  }
}

template <class T, bool MASTER>
int sgd_h(uint16_t *p16, const uint16_t *g16, uint16_t *v16, float *p32, float *v32, size_t n, float lr, float mu,
          float damp, float wd, int nesterov, void *stream) {
  if (n == 0) return SGH_OK;
  if (!p16 || !g16 || (MASTER && !p32)) return SGH_EINVAL;
  if (mu != 0.f && (MASTER ? !v32 : !v16)) return SGH_EINVAL;
  hipLaunchKernelGGL((k_sgd_h<T, MASTER>), dim3(grid_for(n)), dim3(kBlock), 0, sgh_stream_of(stream), p16, g16, v16, p32,
                     v32, n, SgdHyper{lr, mu, damp, wd}, nesterov);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

// All parameters of a mixed-precision network in one launch: fp32 items (p, g, v fp32) and master
// items (16-bit gradient, fp32 master p and momentum v, 16-bit working copy p16 refreshed) share a
// table; a block takes chunks of kMixChunk elements, the chunk -> item lookup goes through an LDS
// prefix table built once per block.  Per element the same sgd_one as the single-tensor kernels.
constexpr int kMixChunk = kBlock * 8;
constexpr int kMixTab = 2048;

template <class T>
__global__ __launch_bounds__(kBlock) void k_sgd_multi_mixed(const sgh_sgd_mixed_item *__restrict__ table, int count,
                                                           SgdHyper h, int nesterov) {
  __shared__ unsigned pre[kMixTab + 1];  // pre[i] = chunks of items 0 .. i-1
  for (int i = threadIdx.x; i < count; i += kBlock) pre[i + 1] = unsigned((table[i].n + kMixChunk - 1) / kMixChunk);
  if (threadIdx.x == 0) pre[0] = 0;
  __syncthreads();
  if (threadIdx.x < 64) {  // wavefront 0: inclusive scan in tiles of 64 with a running carry
    unsigned carry = 0;
    for (int base = 0; base < count; base += 64) {
      const int i = base + threadIdx.x;
      unsigned v = i < count ? pre[i + 1] : 0u;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const unsigned u = __shfl_up(v, o, 64);
        if (int(threadIdx.x) >= o) v += u;
      }
      v += carry;
      if (i < count) pre[i + 1] = v;
      carry = __shfl(v, 63, 64);
    }
  }
  __syncthreads();
  int it = 0;
  for (unsigned chunk = blockIdx.x; chunk < pre[count]; chunk += gridDim.x) {
    while (chunk >= pre[it + 1]) ++it;
    const sgh_sgd_mixed_item item = table[it];
    const bool has_v = h.mu != 0.f && item.v != nullptr;
    const size_t base = size_t(chunk - pre[it]) * kMixChunk;
    const size_t end = base + kMixChunk < item.n ? base + kMixChunk : size_t(item.n);
    const float *g32 = static_cast<const float *>(item.g);
    const u16 *g16 = static_cast<const u16 *>(item.g);
    for (size_t i = base + threadIdx.x; i < end; i += kBlock) {
      float pp = item.p[i];
      float vv = has_v ? item.v[i] : 0.f;
      sgd_one(pp, item.p16 ? T::load(g16[i]) : g32[i], vv, h, nesterov, has_v);
      item.p[i] = pp;
      if (has_v) item.v[i] = vv;
      if (item.p16) item.p16[i] = T::store(pp);
    }
  }
}

// Tensor::SetValue on a 16-bit tensor: the value rounded once, written as pairs where aligned
__global__ __launch_bounds__(kBlock) void k_fill16(u16 *dst, u16 bits, size_t n) {
  const size_t stride = size_t(gridDim.x) * kBlock, t = size_t(blockIdx.x) * kBlock + threadIdx.x;
  const size_t head = (reinterpret_cast<uintptr_t>(dst) & 2u) ? 1 : 0;   // elements before the first 4-byte boundary
  if (t == 0 && head && n) dst[0] = bits;
  if (n <= head) return;
  unsigned *d2 = reinterpret_cast<unsigned *>(dst + head);
  const size_t pairs = (n - head) >> 1;
  const unsigned two = unsigned(bits) | (unsigned(bits) << 16);
  for (size_t i = t; i < pairs; i += stride) d2[i] = two;
  if (t == 0 && ((n - head) & 1)) dst[n - 1] = bits;
}

int fill16(uint16_t *dst, uint16_t bits, size_t n, void *stream) {
  if (n == 0) return SGH_OK;
  if (!dst || (reinterpret_cast<uintptr_t>(dst) & 1u)) return SGH_EINVAL;
  hipLaunchKernelGGL(k_fill16, dim3(grid_for((n + 1) >> 1)), dim3(kBlock), 0, sgh_stream_of(stream), dst, bits, n);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

// host-side rounding to nearest even, the same results as the device conversions of storage.h
uint16_t host_f32_to_bf16(float f) {
  unsigned u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return uint16_t(u >> 16);
}
uint16_t host_f32_to_f16(float f) {
  unsigned u;
  memcpy(&u, &f, 4);
  const unsigned sign = (u >> 16) & 0x8000u;
  u &= 0x7fffffffu;
  if (u > 0x7f800000u) return uint16_t(sign | 0x7e00u);   // NaN
  if (u >= 0x38800000u) {                                  // normal in binary16 (or beyond its range)
    u += 0xfffu + ((u >> 13) & 1u);
    if (u >= 0x47800000u) return uint16_t(sign | 0x7c00u);  // rounds to infinity (|f| >= 65520)
    return uint16_t(sign | ((u - 0x38000000u) >> 13));
  }
  // subnormal result: adding 0.5 puts the unit in the last place at 2^-24, the FPU rounds to even
  float a;
  memcpy(&a, &u, 4);
  a += 0.5f;
  memcpy(&u, &a, 4);
  return uint16_t(sign | (u - 0x3f000000u));
}

}  // namespace

extern "C" {

int sgh_memset_f16(uint16_t *dst, float value, size_t n, void *stream) {
  sgh_weights_epoch_bump();
  return fill16(dst, host_f32_to_f16(value), n, stream);
}
int sgh_memset_bf16(uint16_t *dst, float value, size_t n, void *stream) {
  sgh_weights_epoch_bump();
  return fill16(dst, host_f32_to_bf16(value), n, stream);
}

int sgh_sgd_momentum_multi_mixed(const sgh_sgd_mixed_item *table_dev, int count, size_t total_n, int bf16, float lr,
                                 float mu, float damp, float wd, int nesterov, void *stream) {
  sgh_weights_epoch_bump();
  if (count == 0) return SGH_OK;
  if (!table_dev || count < 0 || count > kMixTab) return SGH_EINVAL;
  size_t chunks = total_n / kMixChunk + size_t(count);  // upper bound on the sum of per-item chunk counts
  const size_t cap = size_t(sgh_num_cus()) * 8;
  if (chunks > cap) chunks = cap;
  const SgdHyper h{lr, mu, damp, wd};
  // fp32 items: p, g, v in, p, v out; 16-bit items: p, v (4) + g (2) in, p, v (4) + p16 (2) out: 20 bytes either way
  sgh_prof_kernel_scope prof("sgd/k_sgd_multi_mixed", 20.0 * total_n, sgh_stream_of(stream));
  if (bf16) SGH_LAUNCH_TIMED(k_sgd_multi_mixed<BF16>, dim3(int(chunks)), dim3(kBlock), 0, sgh_stream_of(stream), table_dev, count, h, nesterov);
  else SGH_LAUNCH_TIMED(k_sgd_multi_mixed<F16>, dim3(int(chunks)), dim3(kBlock), 0, sgh_stream_of(stream), table_dev, count, h, nesterov);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_sgd_momentum_f16(uint16_t *p, const uint16_t *g, uint16_t *v, size_t n, float lr, float mu, float damp,
                         float wd, int nesterov, void *stream) {
  sgh_weights_epoch_bump();
  return sgd_h<F16, false>(p, g, v, nullptr, nullptr, n, lr, mu, damp, wd, nesterov, stream);
}
int sgh_sgd_momentum_bf16(uint16_t *p, const uint16_t *g, uint16_t *v, size_t n, float lr, float mu, float damp,
                          float wd, int nesterov, void *stream) {
  sgh_weights_epoch_bump();
  return sgd_h<BF16, false>(p, g, v, nullptr, nullptr, n, lr, mu, damp, wd, nesterov, stream);
}
int sgh_sgd_momentum_master_f16(float *p_master, const uint16_t *g, float *v, uint16_t *p_out, size_t n, float lr,
                                float mu, float damp, float wd, int nesterov, void *stream) {
  sgh_weights_epoch_bump();
  return sgd_h<F16, true>(p_out, g, nullptr, p_master, v, n, lr, mu, damp, wd, nesterov, stream);
}
int sgh_sgd_momentum_master_bf16(float *p_master, const uint16_t *g, float *v, uint16_t *p_out, size_t n, float lr,
                                 float mu, float damp, float wd, int nesterov, void *stream) {
  sgh_weights_epoch_bump();
  return sgd_h<BF16, true>(p_out, g, nullptr, p_master, v, n, lr, mu, damp, wd, nesterov, stream);
}


int sgh_cast_f32_to_f16(const float *src, uint16_t *dst, size_t n, void *stream) { sgh_note_write(dst, n * 2); return cast_to16<F16>(src, dst, n, stream); }
int sgh_cast_f16_to_f32(const uint16_t *src, float *dst, size_t n, void *stream) { sgh_note_write(dst, n * 4); return cast_from16<F16>(src, dst, n, stream); }
int sgh_cast_f32_to_bf16(const float *src, uint16_t *dst, size_t n, void *stream) { sgh_note_write(dst, n * 2); return cast_to16<BF16>(src, dst, n, stream); }
int sgh_cast_bf16_to_f32(const uint16_t *src, float *dst, size_t n, void *stream) { sgh_note_write(dst, n * 4); return cast_from16<BF16>(src, dst, n, stream); }

// (both operands are x: the stored value where it is positive, else +0 -- exact, nothing is rounded)
int sgh_relu_fwd_f16(const uint16_t *x, uint16_t *y, size_t n, void *stream) {
  return launch_map2_h<F16>(x, x, y, n, ReluFwd{}, stream);
}
int sgh_relu_fwd_bf16(const uint16_t *x, uint16_t *y, size_t n, void *stream) {
  return launch_map2_h<BF16>(x, x, y, n, ReluFwd{}, stream);
}
int sgh_relu_bwd_f16(const uint16_t *dy, const uint16_t *x, uint16_t *dx, size_t n, void *stream) {
  sgh_prof_kernel_scope prof("relu_bwd/k_map2_h<ReluBwd>", 3.0 * n * 2, sgh_stream_of(stream));
  return launch_map2_h<F16>(dy, x, dx, n, ReluBwd{}, stream);
}
int sgh_relu_bwd_bf16(const uint16_t *dy, const uint16_t *x, uint16_t *dx, size_t n, void *stream) {
  sgh_prof_kernel_scope prof("relu_bwd/k_map2_h<ReluBwd>", 3.0 * n * 2, sgh_stream_of(stream));
  return launch_map2_h<BF16>(dy, x, dx, n, ReluBwd{}, stream);
}
int sgh_relu_bwd_add_f32(const float *dy0, const float *dy1, const float *x, float *dx, size_t n, void *stream) {
  sgh_prof_kernel_scope prof("relu_bwd_add/k_relu_bwd_add", 4.0 * n * 4, sgh_stream_of(stream));
  return launch_relu_bwd_add<StF32>(dy0, dy1, x, dx, n, stream);
}
int sgh_relu_bwd_add_f16(const uint16_t *dy0, const uint16_t *dy1, const uint16_t *x, uint16_t *dx, size_t n,
                         void *stream) {
  sgh_prof_kernel_scope prof("relu_bwd_add/k_relu_bwd_add", 4.0 * n * 2, sgh_stream_of(stream));
  return launch_relu_bwd_add<StF16>(dy0, dy1, x, dx, n, stream);
}
int sgh_relu_bwd_add_bf16(const uint16_t *dy0, const uint16_t *dy1, const uint16_t *x, uint16_t *dx, size_t n,
                          void *stream) {
  sgh_prof_kernel_scope prof("relu_bwd_add/k_relu_bwd_add", 4.0 * n * 2, sgh_stream_of(stream));
  return launch_relu_bwd_add<StBF16>(dy0, dy1, x, dx, n, stream);
}
int sgh_add_f16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream) {
  sgh_note_write(out, n * 2);
  sgh_prof_kernel_scope prof("add/k_map2_h<AddOp>", 3.0 * n * 2, sgh_stream_of(stream));
  return launch_map2_h<F16>(a, b, out, n, AddOp{}, stream);
}
int sgh_add_bf16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream) {
  sgh_note_write(out, n * 2);
  sgh_prof_kernel_scope prof("add/k_map2_h<AddOp>", 3.0 * n * 2, sgh_stream_of(stream));
  return launch_map2_h<BF16>(a, b, out, n, AddOp{}, stream);
}
int sgh_add_relu_f16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream) {
  sgh_note_write(out, n * 2);
  return launch_map2_h<F16>(a, b, out, n, AddReluOp<F16>{}, stream);
}
int sgh_add_relu_bf16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream) {
  sgh_note_write(out, n * 2);
  return launch_map2_h<BF16>(a, b, out, n, AddReluOp<BF16>{}, stream);
}
int sgh_eltwise_mult_f16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream) {
  sgh_note_write(out, n * 2);
  return launch_map2_h<F16>(a, b, out, n, MulOp{}, stream);
}
int sgh_eltwise_mult_bf16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream) {
  sgh_note_write(out, n * 2);
  return launch_map2_h<BF16>(a, b, out, n, MulOp{}, stream);
}
int sgh_axpy_f16(float alpha, const uint16_t *x, uint16_t *y, size_t n, void *stream) {
  sgh_weights_epoch_bump();
  return launch_map2_h<F16>(x, y, y, n, AxpyOp{alpha}, stream);
}
int sgh_axpy_bf16(float alpha, const uint16_t *x, uint16_t *y, size_t n, void *stream) {
  sgh_weights_epoch_bump();
  return launch_map2_h<BF16>(x, y, y, n, AxpyOp{alpha}, stream);
}

}  // extern "C"
