// Bandwidth-bound tensor_math kernels of the backward path: ReLU backward, softmax-cross-entropy
// backward, Axpy, EltwiseMult, Add, the fused SGD-momentum update and small row reductions.
// Each moves its operands through HBM exactly once with 16-byte accesses; arithmetic keeps the
// rounding sequence of the CPU reference (separate multiply and add, no contraction) so that
// results are comparable bit for bit where the reference is elementwise.
#include "common.h"
#include "sgd_math.h"
#include "storage.h"

// contraction is disabled per function where the reference rounds after each op
#define SGH_NO_CONTRACT _Pragma("clang fp contract(off)")

namespace {

constexpr int kBlock = 256;
constexpr int kUnroll = 4;  // float4 vectors in flight per thread per operand
// Tensors of at least this many bytes are streamed with non-temporal loads and stores: they cannot
// stay resident in the 256 MB Infinity Cache between kernels anyway (measured: +15 % on the 205 MB
// stem tensors, a few per cent slower on cache-resident ones).
constexpr size_t kStreamBytes = size_t(96) << 20;

inline int grid_for(size_t nvec) {
  size_t per_block = size_t(kBlock) * kUnroll;
  size_t blocks = (nvec + per_block - 1) / per_block;
  const size_t cap = size_t(sgh_num_cus()) * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return int(blocks);
}

// ---------------------------------------------------------------------------------------
// Generic streaming kernels: NIN read-only float streams + NIO read-write streams.
// F::apply gets references to one element of each.
// The vector body covers n/4 float4s with a grid-stride loop unrolled kUnroll times; the
// scalar tail (n % 4) is done by the first threads of block 0.
// ---------------------------------------------------------------------------------------
template <class F, bool kNonTemporal>
__global__ __launch_bounds__(kBlock) void k_map2_1(const float *a, const float *b, float *o, size_t n, F f) {
  // no __restrict__: the in-place forms (y += alpha*x, a += b) alias an input with the output
  typedef float v4f_ __attribute__((ext_vector_type(4)));
  const size_t nvec = n >> 2;
  const v4f_ *a4 = reinterpret_cast<const v4f_ *>(a);
  const v4f_ *b4 = reinterpret_cast<const v4f_ *>(b);
  v4f_ *o4 = reinterpret_cast<v4f_ *>(o);
  // a workgroup takes kUnroll * kBlock consecutive vectors per pass (16 KB per stream), so that
  // neighbouring workgroups stream neighbouring DRAM pages
  const size_t step = size_t(gridDim.x) * (kBlock * kUnroll);
  size_t i = size_t(blockIdx.x) * (kBlock * kUnroll) + threadIdx.x;
  for (; i + (kUnroll - 1) * kBlock < nvec; i += step) {
    v4f_ va[kUnroll], vb[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      va[u] = kNonTemporal ? __builtin_nontemporal_load(a4 + i + u * kBlock) : a4[i + u * kBlock];
      vb[u] = kNonTemporal ? __builtin_nontemporal_load(b4 + i + u * kBlock) : b4[i + u * kBlock];
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      v4f_ r;
      r[0] = f(va[u][0], vb[u][0]);
      r[1] = f(va[u][1], vb[u][1]);
      r[2] = f(va[u][2], vb[u][2]);
      r[3] = f(va[u][3], vb[u][3]);
      if (kNonTemporal) __builtin_nontemporal_store(r, o4 + i + u * kBlock);
      else o4[i + u * kBlock] = r;
    }
  }
  // the last, partial pass of the workgroup that owns it
  for (; i < nvec; i += kBlock) {
    if (i / (kBlock * kUnroll) % gridDim.x != blockIdx.x) break;
    const v4f_ va = a4[i], vb = b4[i];
    v4f_ r;
    r[0] = f(va[0], vb[0]);
    r[1] = f(va[1], vb[1]);
    r[2] = f(va[2], vb[2]);
    r[3] = f(va[3], vb[3]);
    o4[i] = r;
  }
  if (blockIdx.x == 0) {
    const size_t t = (nvec << 2) + threadIdx.x;
    if (t < n) o[t] = f(a[t], b[t]);
  }
}

// scalar fallback for pointers that are not 16-byte aligned
template <class F>
__global__ __launch_bounds__(kBlock) void k_map2_1_scalar(const float *a, const float *b, float *o, size_t n, F f) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) o[i] = f(a[i], b[i]);
}

template <class F>
int launch_map2(const float *a, const float *b, float *o, size_t n, F f, void *stream) {
  if (n == 0) return SGH_OK;
  if (!a || !b || !o) return SGH_EINVAL;
  if (sgh_aligned16(a) && sgh_aligned16(b) && sgh_aligned16(o)) {
    if (n * sizeof(float) >= kStreamBytes)
      SGH_LAUNCH_TIMED((k_map2_1<F, true>), dim3(grid_for(n >> 2)), dim3(kBlock), 0, sgh_stream_of(stream), a, b, o, n,
                         f);
    else
      SGH_LAUNCH_TIMED((k_map2_1<F, false>), dim3(grid_for(n >> 2)), dim3(kBlock), 0, sgh_stream_of(stream), a, b, o,
                         n, f);
  } else {
    SGH_LAUNCH_TIMED(k_map2_1_scalar<F>, dim3(grid_for(n)), dim3(kBlock), 0, sgh_stream_of(stream), a, b, o, n, f);
  }
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

struct ReluBwd {
  __device__ __forceinline__ float operator()(float dy, float x) const { return x > 0.f ? dy : 0.f; }
};
struct ReluFwd {  // second operand unused
  __device__ __forceinline__ float operator()(float x, float) const { return x >= 0.f ? x : 0.f; }
};
struct AddOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct AddReluOp {  // ReluFwd of the sum
  __device__ __forceinline__ float operator()(float a, float b) const {
    const float s = a + b;
    return s >= 0.f ? s : 0.f;
  }
};
struct ClampOp {  // second operand unused; NaN passes through, as in the CPU function's two comparisons
  float lo, hi;
  __device__ __forceinline__ float operator()(float x, float) const { return x < lo ? lo : (x > hi ? hi : x); }
};
struct MulOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a * b; }
};
struct SubOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a - b; }
};
struct DivOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a / b; }
};
struct AddScalarOp {  // second operand unused
  float s;
  __device__ __forceinline__ float operator()(float a, float) const { return a + s; }
};
struct MulScalarOp {
  float s;
  __device__ __forceinline__ float operator()(float a, float) const { return a * s; }
};
struct AxpyOp {  // (x, y) -> y + alpha * x, two roundings
  float alpha;
  __device__ __forceinline__ float operator()(float x, float y) const {
    SGH_NO_CONTRACT
    float t = alpha * x;
    return y + t;
  }
};
struct AxpyDevOp {
  const float *alpha;
  __device__ __forceinline__ float operator()(float x, float y) const {
    SGH_NO_CONTRACT
    float t = __ldg(alpha) * x;
    return y + t;
  }
};
struct MulScalarDevOp {  // second stream is ignored (aliased to the first by the launcher)
  const float *s;
  __device__ __forceinline__ float operator()(float a, float) const { return a * __ldg(s); }
};

// ---------------------------------------------------------------------------------------
// unary (one read stream) variants for ReLU forward / scalar multiply / fill
// ---------------------------------------------------------------------------------------
template <class F>
__global__ __launch_bounds__(kBlock) void k_map1_1(const float *a, float *o, size_t n, F f, int vec) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x;
  if (vec) {
    const size_t nvec = n >> 2;
    const float4 *a4 = reinterpret_cast<const float4 *>(a);
    float4 *o4 = reinterpret_cast<float4 *>(o);
    for (; i < nvec; i += stride) {
      float4 v = a4[i], r;
      r.x = f(v.x, 0.f);
      r.y = f(v.y, 0.f);
      r.z = f(v.z, 0.f);
      r.w = f(v.w, 0.f);
      o4[i] = r;
    }
    if (blockIdx.x == 0) {
      const size_t t = (nvec << 2) + threadIdx.x;
      if (t < n) o[t] = f(a[t], 0.f);
    }
  } else {
    for (; i < n; i += stride) o[i] = f(a[i], 0.f);
  }
}

template <class F>
int launch_map1(const float *a, float *o, size_t n, F f, void *stream) {
  if (n == 0) return SGH_OK;
  if (!a || !o) return SGH_EINVAL;
  const int vec = sgh_aligned16(a) && sgh_aligned16(o);
  hipLaunchKernelGGL(k_map1_1<F>, dim3(grid_for(vec ? (n >> 2) : n)), dim3(kBlock), 0, sgh_stream_of(stream), a, o, n,
                     f, vec);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

__global__ __launch_bounds__(kBlock) void k_fill(float *o, float v, size_t n) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) o[i] = v;
}

// ---------------------------------------------------------------------------------------
// Fused SGD-momentum: streams p, g, v in; p, v out (5 * 4 bytes per parameter element).
// ---------------------------------------------------------------------------------------
template <bool DEV_HYPER>
__global__ __launch_bounds__(kBlock) void k_sgd(float *__restrict__ p, const float *__restrict__ g,
                                               float *__restrict__ v, size_t n, SgdHyper hh,
                                               const float *__restrict__ hyper_dev, int nesterov, int vec) {
  SgdHyper h = hh;
  if (DEV_HYPER) {
    h.lr = __ldg(hyper_dev + 0);
    h.mu = __ldg(hyper_dev + 1);
    h.damp = __ldg(hyper_dev + 2);
    h.wd = __ldg(hyper_dev + 3);
  }
  const bool has_v = (h.mu != 0.f) && v != nullptr;
  const size_t stride = size_t(gridDim.x) * kBlock;
  size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x;
  if (vec) {
    const size_t nvec = n >> 2;
    float4 *p4 = reinterpret_cast<float4 *>(p);
    const float4 *g4 = reinterpret_cast<const float4 *>(g);
    float4 *v4 = reinterpret_cast<float4 *>(v);
    for (; i < nvec; i += stride) {
      float4 pp = p4[i], gg = g4[i], vv = has_v ? v4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
      sgd_one(pp.x, gg.x, vv.x, h, nesterov, has_v);
      sgd_one(pp.y, gg.y, vv.y, h, nesterov, has_v);
      sgd_one(pp.z, gg.z, vv.z, h, nesterov, has_v);
      sgd_one(pp.w, gg.w, vv.w, h, nesterov, has_v);
      p4[i] = pp;
      if (has_v) v4[i] = vv;
    }
    if (blockIdx.x == 0) {
      const size_t t = (nvec << 2) + threadIdx.x;
      if (t < n) {
        float pp = p[t], vv = has_v ? v[t] : 0.f;
        sgd_one(pp, g[t], vv, h, nesterov, has_v);
        p[t] = pp;
        if (has_v) v[t] = vv;
      }
    }
  } else {
    for (; i < n; i += stride) {
      float pp = p[i], vv = has_v ? v[i] : 0.f;
      sgd_one(pp, g[i], vv, h, nesterov, has_v);
      p[i] = pp;
      if (has_v) v[i] = vv;
    }
  }
}

// Multi-tensor variant: block b walks the concatenation of all items in chunks of kChunk elements;
// a chunk never crosses an item boundary.  Each workgroup first builds the prefix sums of the
// items' chunk counts in LDS (one parallel pass over the table), then finds the owner of its
// chunks by walking that array forward (its chunk indices only grow), so the table costs one
// global read per item per workgroup instead of a dependent scan per chunk.  All of a thread's
// 16-byte loads of a chunk are issued before the first store.
constexpr int kSgdVec = 4;                        // float4 per thread per tensor per chunk
constexpr int kChunk = kBlock * 4 * kSgdVec;      // 4096 elements per block-iteration
constexpr int kSgdTab = 2048;                     // items whose prefix sums fit the LDS table

__global__ __launch_bounds__(kBlock) void k_sgd_multi(const sgh_sgd_item *__restrict__ table, int count, SgdHyper h,
                                                     int nesterov) {
  __shared__ unsigned pre[kSgdTab + 1];  // pre[i] = chunks of items 0 .. i-1
  const bool use_v = h.mu != 0.f;
  const bool lds_tab = count <= kSgdTab;
  if (lds_tab) {
    for (int i = threadIdx.x; i < count; i += kBlock) pre[i + 1] = unsigned((table[i].n + kChunk - 1) / kChunk);
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
  }
  // chunk index space: sum over items of ceil(n / kChunk)
  size_t chunk = blockIdx.x;
  int it = 0;
  size_t it_first = 0;  // first chunk of item `it` (linear-scan fallback only)
  for (;;) {
    // locate the item that owns this chunk
    size_t c;
    if (lds_tab) {
      if (chunk >= pre[count]) return;
      while (chunk >= pre[it + 1]) ++it;
      c = chunk - pre[it];
    } else {
      for (; it < count; ++it) {
        const size_t nc = (table[it].n + kChunk - 1) / kChunk;
        if (chunk - it_first < nc) break;
        it_first += nc;
      }
      if (it >= count) return;
      c = chunk - it_first;
    }
    float *p = table[it].p;
    const float *g = table[it].g;
    float *v = table[it].v;
    const size_t n = table[it].n;
    const bool has_v = use_v && v != nullptr;
    const size_t base = c * kChunk;
    const size_t end = base + kChunk < n ? base + kChunk : n;
    const bool vec = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) |
                       reinterpret_cast<uintptr_t>(has_v ? v : p)) & 15u) == 0;
    if (vec && base + kChunk <= n) {
      // a full chunk: kSgdVec float4 per thread per tensor, all loaded before the first store
      float4 pp[kSgdVec], gg[kSgdVec], vv[kSgdVec];
#pragma unroll
      for (int u = 0; u < kSgdVec; ++u) {
        const size_t e = base + (size_t(u) * kBlock + threadIdx.x) * 4;
        pp[u] = *reinterpret_cast<const float4 *>(p + e);
        gg[u] = *reinterpret_cast<const float4 *>(g + e);
        vv[u] = has_v ? *reinterpret_cast<const float4 *>(v + e) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < kSgdVec; ++u) {
        const size_t e = base + (size_t(u) * kBlock + threadIdx.x) * 4;
        sgd_one(pp[u].x, gg[u].x, vv[u].x, h, nesterov, has_v);
        sgd_one(pp[u].y, gg[u].y, vv[u].y, h, nesterov, has_v);
        sgd_one(pp[u].z, gg[u].z, vv[u].z, h, nesterov, has_v);
        sgd_one(pp[u].w, gg[u].w, vv[u].w, h, nesterov, has_v);
        *reinterpret_cast<float4 *>(p + e) = pp[u];
        if (has_v) *reinterpret_cast<float4 *>(v + e) = vv[u];
      }
    } else if (vec) {
      for (size_t e = base + size_t(threadIdx.x) * 4; e < end; e += size_t(kBlock) * 4) {
        if (e + 4 <= end) {
          float4 pp = *reinterpret_cast<float4 *>(p + e), gg = *reinterpret_cast<const float4 *>(g + e);
          float4 vv = has_v ? *reinterpret_cast<float4 *>(v + e) : make_float4(0.f, 0.f, 0.f, 0.f);
          sgd_one(pp.x, gg.x, vv.x, h, nesterov, has_v);
          sgd_one(pp.y, gg.y, vv.y, h, nesterov, has_v);
          sgd_one(pp.z, gg.z, vv.z, h, nesterov, has_v);
          sgd_one(pp.w, gg.w, vv.w, h, nesterov, has_v);
          *reinterpret_cast<float4 *>(p + e) = pp;
          if (has_v) *reinterpret_cast<float4 *>(v + e) = vv;
        } else {
          for (size_t t = e; t < end; ++t) {
            float pp = p[t], vv = has_v ? v[t] : 0.f;
            sgd_one(pp, g[t], vv, h, nesterov, has_v);
            p[t] = pp;
            if (has_v) v[t] = vv;
          }
        }
      }
    } else {
      for (size_t t = base + threadIdx.x; t < end; t += kBlock) {
        float pp = p[t], vv = has_v ? v[t] : 0.f;
        sgd_one(pp, g[t], vv, h, nesterov, has_v);
        p[t] = pp;
        if (has_v) v[t] = vv;
      }
    }
    chunk += gridDim.x;
  }
}

// ---------------------------------------------------------------------------------------
// Softmax cross-entropy: one 256-thread block per sample row.
// ---------------------------------------------------------------------------------------
__device__ int g_label_errors = 0;

// S: the storage type of p and grad (fp32, or 16-bit with fp32 arithmetic and one rounding at the store)
template <class S>
__global__ __launch_bounds__(kBlock) void k_softmax_ce_bwd(const typename S::elem *__restrict__ p,
                                                          const int32_t *__restrict__ t,
                                                          typename S::elem *__restrict__ grad, size_t dim, int int_target,
                                                          float scale) {
  __shared__ float red[16];
  const size_t row = blockIdx.x;
  const typename S::elem *pr = p + row * dim;
  typename S::elem *gr = grad + row * dim;
  if (int_target) {
    const int label = t[row];
    const bool ok = label >= 0 && size_t(label) < dim;
    if (!ok && threadIdx.x == 0) atomicAdd(&g_label_errors, 1);
    for (size_t j = threadIdx.x; j < dim; j += kBlock) {
      float v = S::ld(pr + j);
      if (ok && j == size_t(label)) v = v - 1.0f;
      S::st(gr + j, v * scale);
    }
  } else {
    const int32_t *tr = t + row * dim;
    float s = 0.f;
    for (size_t j = threadIdx.x; j < dim; j += kBlock) s += float(tr[j]);
    s = sgh_block_sum(s, red);
    for (size_t j = threadIdx.x; j < dim; j += kBlock) {
      float v = S::ld(pr + j) - float(tr[j]) / s;
      S::st(gr + j, v * scale);
    }
  }
}

// Row softmax with the numerically safe max subtraction (row max, not the CPU path's
// zero-seeded max: the two agree whenever a row has a non-negative entry and differ only by
// rounding otherwise).
__global__ __launch_bounds__(kBlock) void k_softmax_fwd(const float *__restrict__ x, float *__restrict__ p, size_t dim) {
  __shared__ float red[16];
  const size_t row = blockIdx.x;
  const float *xr = x + row * dim;
  float *pr = p + row * dim;
  float m = -3.402823466e38f;
  for (size_t j = threadIdx.x; j < dim; j += kBlock) m = fmaxf(m, xr[j]);
  m = sgh_wave_max(m);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  m = red[0];
  for (int i = 1; i < kBlock / 64; ++i) m = fmaxf(m, red[i]);
  float s = 0.f;
  for (size_t j = threadIdx.x; j < dim; j += kBlock) {
    float e = expf(xr[j] - m);
    pr[j] = e;
    s += e;
  }
  s = sgh_block_sum(s, red);
  for (size_t j = threadIdx.x; j < dim; j += kBlock) pr[j] = pr[j] / s;
}

__global__ __launch_bounds__(kBlock) void k_ce_fwd(const float *__restrict__ p, const int32_t *__restrict__ t,
                                                  float *__restrict__ loss, size_t dim, int int_target) {
  __shared__ float red[16];
  const size_t row = blockIdx.x;
  const float *pr = p + row * dim;
  if (int_target) {
    if (threadIdx.x == 0) {
      const int label = t[row];
      if (label >= 0 && size_t(label) < dim) {
        loss[row] = -logf(fmaxf(pr[label], 1.17549435e-38f));
      } else {
        atomicAdd(&g_label_errors, 1);
        loss[row] = 0.f;
      }
    }
  } else {
    const int32_t *tr = t + row * dim;
    float s = 0.f;
    for (size_t j = threadIdx.x; j < dim; j += kBlock) s += float(tr[j]);
    s = sgh_block_sum(s, red);
    float l = 0.f;
    for (size_t j = threadIdx.x; j < dim; j += kBlock)
      l -= float(tr[j]) / s * logf(fmaxf(pr[j], 1.17549435e-38f));
    l = sgh_block_sum(l, red);
    if (threadIdx.x == 0) loss[row] = l;
  }
}

// ---------------------------------------------------------------------------------------
// Row reductions for Linear's bias:  out[j] = sum_i m[i][j]   and   m[i][j] += v[j]
// ---------------------------------------------------------------------------------------
// One thread per column, rows summed in ascending order (the order of the reference GEMV).
__global__ __launch_bounds__(kBlock) void k_sum_rows(const float *__restrict__ m, float *__restrict__ out, int rows,
                                                    int cols) {
  const int j = blockIdx.x * kBlock + threadIdx.x;
  if (j >= cols) return;
  // (32 loads in flight per thread; the additions stay in row order.  The loop of one load per addition waited
  // for each load in turn: 31 us for 128 x 1000)
  constexpr int U = 32;
  float s = 0.f;
  int i = 0;
  for (; i + U <= rows; i += U) {
    float v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = m[size_t(i + u) * cols + j];
#pragma unroll
    for (int u = 0; u < U; ++u) s += v[u];
  }
  for (; i < rows; ++i) s += m[size_t(i) * cols + j];
  out[j] = s;
}

__global__ __launch_bounds__(kBlock) void k_add_row(const float *__restrict__ v, float *__restrict__ m, size_t total,
                                                   int cols) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < total; i += stride) m[i] += v[i % cols];
}

template <class S>
int softmax_ce_bwd(const typename S::elem *p, const int32_t *t, typename S::elem *grad, size_t batch, size_t dim,
                          int int_target, float scale, void *stream) {
  if (batch == 0 || dim == 0) return SGH_OK;
  if (!p || !t || !grad) return SGH_EINVAL;
  if (batch > 0x7fffffffu) return SGH_EINVAL;
  hipLaunchKernelGGL(k_softmax_ce_bwd<S>, dim3((unsigned)batch), dim3(kBlock), 0, sgh_stream_of(stream), p, t, grad, dim,
                     int_target, scale);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

// CastCopy between float and int tensors: (int)x truncates toward zero (v_cvt_i32_f32 saturates out-of-range
// values and turns NaN into 0), (float)i rounds to nearest even
__global__ __launch_bounds__(kBlock) void k_cast_f32_i32(const float *__restrict__ src, int32_t *__restrict__ dst, size_t n) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) dst[i] = int32_t(src[i]);
}
__global__ __launch_bounds__(kBlock) void k_cast_i32_f32(const int32_t *__restrict__ src, float *__restrict__ dst, size_t n) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) dst[i] = float(src[i]);
}
inline int cast_grid(size_t n) {
  size_t blocks = (n + kBlock - 1) / kBlock;
  const size_t cap = size_t(sgh_num_cus()) * 16;
  return int(blocks > cap ? cap : (blocks < 1 ? 1 : blocks));
}

}  // namespace

extern "C" {

int sgh_relu_bwd_f32(const float *dy, const float *x, float *dx, size_t n, void *stream) {
  sgh_prof_kernel_scope prof("relu_bwd/k_map2_1<ReluBwd>", 3.0 * n * sizeof(float), sgh_stream_of(stream));
  return launch_map2(dy, x, dx, n, ReluBwd{}, stream);
}

int sgh_relu_fwd_f32(const float *x, float *y, size_t n, void *stream) {
  return launch_map1(x, y, n, ReluFwd{}, stream);
}

int sgh_cast_f32_to_i32(const float *src, int32_t *dst, size_t n, void *stream) {
  if (n == 0) return SGH_OK;
  if (!src || !dst) return SGH_EINVAL;
  hipLaunchKernelGGL(k_cast_f32_i32, dim3(cast_grid(n)), dim3(kBlock), 0, sgh_stream_of(stream), src, dst, n);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_cast_i32_to_f32(const int32_t *src, float *dst, size_t n, void *stream) {
  if (n == 0) return SGH_OK;
  if (!src || !dst) return SGH_EINVAL;
  hipLaunchKernelGGL(k_cast_i32_f32, dim3(cast_grid(n)), dim3(kBlock), 0, sgh_stream_of(stream), src, dst, n);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_clamp_f32(float low, float high, const float *x, float *out, size_t n, void *stream) {
  sgh_note_write(out, n * sizeof(float));
  return launch_map1(x, out, n, ClampOp{low, high}, stream);
}

int sgh_add_f32(const float *a, const float *b, float *out, size_t n, void *stream) {
  sgh_note_write(out, n * sizeof(float));
  sgh_prof_kernel_scope prof("add/k_map2_1<AddOp>", 3.0 * n * sizeof(float), sgh_stream_of(stream));
  return launch_map2(a, b, out, n, AddOp{}, stream);
}

int sgh_add_relu_f32(const float *a, const float *b, float *out, size_t n, void *stream) {
  sgh_note_write(out, n * sizeof(float));
  return launch_map2(a, b, out, n, AddReluOp{}, stream);
}

int sgh_sub_f32(const float *a, const float *b, float *out, size_t n, void *stream) {
  sgh_note_write(out, n * sizeof(float));
  return launch_map2(a, b, out, n, SubOp{}, stream);
}

int sgh_div_f32(const float *a, const float *b, float *out, size_t n, void *stream) {
  sgh_note_write(out, n * sizeof(float));
  return launch_map2(a, b, out, n, DivOp{}, stream);
}

int sgh_add_scalar_f32(const float *a, float x, float *out, size_t n, void *stream) {
  sgh_note_write(out, n * sizeof(float));
  return launch_map1(a, out, n, AddScalarOp{x}, stream);
}

int sgh_mult_scalar_f32(const float *a, float x, float *out, size_t n, void *stream) {
  sgh_note_write(out, n * sizeof(float));
  return launch_map1(a, out, n, MulScalarOp{x}, stream);
}

int sgh_eltwise_mult_f32(const float *a, const float *b, int b_is_scalar, float *out, size_t n, void *stream) {
  sgh_note_write(out, n * sizeof(float));
  if (n == 0) return SGH_OK;
  if (!a || !b || !out) return SGH_EINVAL;
  if (b_is_scalar) return launch_map1(a, out, n, MulScalarDevOp{b}, stream);
  return launch_map2(a, b, out, n, MulOp{}, stream);
}

int sgh_axpy_f32(float alpha, const float *x, float *y, size_t n, void *stream) {
  sgh_weights_epoch_bump();
  return launch_map2(x, y, y, n, AxpyOp{alpha}, stream);
}

int sgh_axpy_devalpha_f32(const float *alpha_dev, const float *x, float *y, size_t n, void *stream) {
  sgh_weights_epoch_bump();
  if (n != 0 && !alpha_dev) return SGH_EINVAL;
  return launch_map2(x, y, y, n, AxpyDevOp{alpha_dev}, stream);
}

int sgh_memset_f32(float *dst, float value, size_t n, void *stream) {
  sgh_weights_epoch_bump();
  if (n == 0) return SGH_OK;
  if (!dst) return SGH_EINVAL;
  hipLaunchKernelGGL(k_fill, dim3(grid_for(n)), dim3(kBlock), 0, sgh_stream_of(stream), dst, value, n);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

static int sgd_launch(float *p, const float *g, float *v, size_t n, SgdHyper h, const float *hyper_dev, int nesterov,
                      bool host_mu_nonzero_needs_v, void *stream) {
  if (n == 0) return SGH_OK;
  if (!p || !g) return SGH_EINVAL;
  if (host_mu_nonzero_needs_v && !v) return SGH_EINVAL;
  const int vec = sgh_aligned16(p) && sgh_aligned16(g) && (v == nullptr || sgh_aligned16(v));
  const int grid = grid_for(vec ? (n >> 2) : n);
  if (hyper_dev)
    hipLaunchKernelGGL(k_sgd<true>, dim3(grid), dim3(kBlock), 0, sgh_stream_of(stream), p, g, v, n, h, hyper_dev,
                       nesterov, vec);
  else
    hipLaunchKernelGGL(k_sgd<false>, dim3(grid), dim3(kBlock), 0, sgh_stream_of(stream), p, g, v, n, h, hyper_dev,
                       nesterov, vec);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_sgd_momentum_f32(float *p, const float *g, float *v, size_t n, float lr, float mu, float damp, float wd,
                         int nesterov, void *stream) {
  sgh_weights_epoch_bump();
  return sgd_launch(p, g, v, n, SgdHyper{lr, mu, damp, wd}, nullptr, nesterov, mu != 0.f, stream);
}

int sgh_sgd_momentum_devhyper_f32(float *p, const float *g, float *v, size_t n, const float *hyper_dev, int nesterov,
                                  void *stream) {
  sgh_weights_epoch_bump();
  if (!hyper_dev) return SGH_EINVAL;
  // mu lives on the device: a NULL v is only legal if mu turns out to be 0, which the kernel checks
  return sgd_launch(p, g, v, n, SgdHyper{0, 0, 0, 0}, hyper_dev, nesterov, false, stream);
}

int sgh_sgd_momentum_multi_f32(const sgh_sgd_item *table_dev, int count, size_t total_n, float lr, float mu, float damp,
                               float wd, int nesterov, void *stream) {
  sgh_weights_epoch_bump();
  if (count == 0 || total_n == 0) return SGH_OK;
  if (!table_dev || count < 0) return SGH_EINVAL;
  size_t chunks = total_n / kChunk + size_t(count);  // upper bound on sum of per-item chunk counts
  const size_t cap = size_t(sgh_num_cus()) * 8;
  if (chunks > cap) chunks = cap;
  sgh_prof_kernel_scope prof("sgd/k_sgd_multi", 20.0 * total_n, sgh_stream_of(stream));   // p, g, v in; p, v out
  SGH_LAUNCH_TIMED(k_sgd_multi, dim3(int(chunks)), dim3(kBlock), 0, sgh_stream_of(stream), table_dev, count,
                     SgdHyper{lr, mu, damp, wd}, nesterov);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_softmax_ce_bwd_f32(const float *p, const int32_t *t, float *grad, size_t batch, size_t dim, int int_target,
                           float scale, void *stream) {
  return softmax_ce_bwd<StF32>(p, t, grad, batch, dim, int_target, scale, stream);
}
int sgh_softmax_ce_bwd_f16(const uint16_t *p, const int32_t *t, uint16_t *grad, size_t batch, size_t dim, int int_target,
                           float scale, void *stream) {
  return softmax_ce_bwd<StF16>(p, t, grad, batch, dim, int_target, scale, stream);
}
int sgh_softmax_ce_bwd_bf16(const uint16_t *p, const int32_t *t, uint16_t *grad, size_t batch, size_t dim, int int_target,
                            float scale, void *stream) {
  return softmax_ce_bwd<StBF16>(p, t, grad, batch, dim, int_target, scale, stream);
}

int sgh_softmax_ce_label_errors(void *stream, int *count) {
  if (!count) return SGH_EINVAL;
  SGH_HIP_TRY(hipStreamSynchronize(sgh_stream_of(stream)));
  int v = 0;
  SGH_HIP_TRY(hipMemcpyFromSymbol(&v, HIP_SYMBOL(g_label_errors), sizeof(int), 0, hipMemcpyDeviceToHost));
  const int zero = 0;
  SGH_HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(g_label_errors), &zero, sizeof(int), 0, hipMemcpyHostToDevice));
  *count = v;
  return SGH_OK;
}

int sgh_softmax_fwd_f32(const float *x, float *p, size_t batch, size_t dim, void *stream) {
  if (batch == 0 || dim == 0) return SGH_OK;
  if (!x || !p || batch > 0x7fffffffu) return SGH_EINVAL;
  hipLaunchKernelGGL(k_softmax_fwd, dim3((unsigned)batch), dim3(kBlock), 0, sgh_stream_of(stream), x, p, dim);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_cross_entropy_fwd_f32(const float *p, const int32_t *t, float *loss, size_t batch, size_t dim, int int_target,
                              void *stream) {
  if (batch == 0 || dim == 0) return SGH_OK;
  if (!p || !t || !loss || batch > 0x7fffffffu) return SGH_EINVAL;
  hipLaunchKernelGGL(k_ce_fwd, dim3((unsigned)batch), dim3(kBlock), 0, sgh_stream_of(stream), p, t, loss, dim,
                     int_target);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_sum_rows_f32(const float *m, float *out, int rows, int cols, void *stream) {
  if (rows < 0 || cols < 0) return SGH_EINVAL;
  if (cols == 0) return SGH_OK;
  if (!out || (rows > 0 && !m)) return SGH_EINVAL;
  hipLaunchKernelGGL(k_sum_rows, dim3((cols + kBlock - 1) / kBlock), dim3(kBlock), 0, sgh_stream_of(stream), m, out,
                     rows, cols);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_add_row_f32(const float *v, float *m, int rows, int cols, void *stream) {
  if (rows < 0 || cols < 0) return SGH_EINVAL;
  const size_t total = size_t(rows) * cols;
  if (total == 0) return SGH_OK;
  if (!v || !m) return SGH_EINVAL;
  hipLaunchKernelGGL(k_add_row, dim3(grid_for(total)), dim3(kBlock), 0, sgh_stream_of(stream), v, m, total, cols);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

}  // extern "C"
