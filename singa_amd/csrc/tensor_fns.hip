// The remaining Tensor functions that python/singa/autograd.py and opt.py touch on the benchmark
// models: Transform (strided / broadcast / transposed view -> dense), RowMax, Dot, Sum over all
// elements, Uniform and Gaussian fills.  References: src/core/tensor/tensor_math_cpp.h:126-138
// (next_offset: how a strided view is walked), :655-663 (Sum), :685-700 (Transform), :712-740
// (Gaussian / Uniform), :827-849 (Dot), :1122-1140 (RowMax); CUDA twins tensor_math_cuda.h:284-300,
// :950-1000, :1075-1092, :1493-1520.
#include "common.h"

namespace {

constexpr int kBlock = 256;

struct View {   // a view of up to SGH_MAX_DIMS dimensions, innermost last
  int ndim;
  unsigned shape[SGH_MAX_DIMS];
  long stride[SGH_MAX_DIMS];   // in elements; 0 = broadcast
};

// out[i] = in[offset of the i-th element of the view in row-major order of its shape]
__global__ __launch_bounds__(kBlock) void k_transform(const float *__restrict__ in, float *__restrict__ out, size_t n,
                                                     View v) {
  const size_t step = size_t(gridDim.x) * kBlock;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += step) {
    size_t rem = i;
    long off = 0;
#pragma unroll
    for (int d = SGH_MAX_DIMS - 1; d >= 0; --d) {
      if (d < v.ndim) {
        const size_t q = rem / v.shape[d];
        off += long(rem - q * v.shape[d]) * v.stride[d];
        rem = q;
      }
    }
    out[i] = in[off];
  }
}

// out[r] = max_c in[r][c], seeded with the row's first element like the reference's accelerator kernel
// (src/core/tensor/math_kernel.cu:488-499); ZERO_SEEDED: max(0, ...), the reference's CPU function
// (tensor_math_cpp.h:1132)
template <bool ZERO_SEEDED>
__global__ __launch_bounds__(kBlock) void k_row_max(const float *__restrict__ in, float *__restrict__ out, int ncol) {
  __shared__ float red[4];
  const float *row = in + size_t(blockIdx.x) * ncol;
  float m = ZERO_SEEDED ? 0.f : row[0];
  for (int c = threadIdx.x; c < ncol; c += kBlock) m = fmaxf(m, row[c]);
  m = sgh_wave_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// Sum of a[i] * b[i] (b null: of a[i]) in a fixed order: workgroup w sums elements w * per .. (w + 1) * per
// with a fixed tree, the second kernel adds the workgroups' sums in ascending order.
constexpr int kReduceBlocks = 1024;

__global__ __launch_bounds__(kBlock) void k_dot_partial(const float *__restrict__ a, const float *__restrict__ b, size_t n,
                                                       size_t per, float *__restrict__ part) {
  __shared__ float red[16];
  const size_t lo = size_t(blockIdx.x) * per, hi = lo + per < n ? lo + per : n;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  size_t i = lo + threadIdx.x;
  for (; i + 3 * kBlock < hi; i += 4 * kBlock) {
    s0 += b ? a[i] * b[i] : a[i];
    s1 += b ? a[i + kBlock] * b[i + kBlock] : a[i + kBlock];
    s2 += b ? a[i + 2 * kBlock] * b[i + 2 * kBlock] : a[i + 2 * kBlock];
    s3 += b ? a[i + 3 * kBlock] * b[i + 3 * kBlock] : a[i + 3 * kBlock];
  }
  for (; i < hi; i += kBlock) s0 += b ? a[i] * b[i] : a[i];
  const float s = sgh_block_sum((s0 + s1) + (s2 + s3), red);
  if (threadIdx.x == 0) part[blockIdx.x] = s;
}

__global__ __launch_bounds__(kBlock) void k_dot_finish(const float *__restrict__ part, int blocks, float *__restrict__ out) {
  __shared__ float red[16];
  float s = 0.f;
  for (int i = threadIdx.x; i < blocks; i += kBlock) s += part[i];
  s = sgh_block_sum(s, red);
  if (threadIdx.x == 0) *out = s;
}

// ---- counter-based random numbers: element i of a fill is a pure function of (seed, offset + i).
// The k-th output of splitmix64 seeded with `seed` is mix(seed + (k + 1) * golden): no state to carry.
__device__ __forceinline__ unsigned long long splitmix64_at(unsigned long long seed, unsigned long long k) {
  unsigned long long z = seed + (k + 1ull) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
__device__ __forceinline__ double unit_double(unsigned long long r) { return double(r >> 11) * 0x1.0p-53; }   // [0, 1)

__global__ __launch_bounds__(kBlock) void k_uniform(float *out, size_t n, unsigned long long seed, unsigned long long offset,
                                                   double low, double high) {
  const size_t step = size_t(gridDim.x) * kBlock;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += step)
    out[i] = float(low + unit_double(splitmix64_at(seed, offset + i)) * (high - low));
}

// Box-Muller on two consecutive outputs per element, in double: z = sqrt(-2 ln(1 - u1)) cos(2 pi u2)
__global__ __launch_bounds__(kBlock) void k_gaussian(float *out, size_t n, unsigned long long seed, unsigned long long offset,
                                                    double mean, double std) {
  const size_t step = size_t(gridDim.x) * kBlock;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += step) {
    const double u1 = unit_double(splitmix64_at(seed, offset + 2 * i));
    const double u2 = unit_double(splitmix64_at(seed, offset + 2 * i + 1));
    const double z = sqrt(-2.0 * log(1.0 - u1)) * cos(6.283185307179586476925286766559 * u2);
    out[i] = float(mean + std * z);
  }
}

inline int grid_for(size_t n) {
  size_t b = (n + kBlock - 1) / kBlock;
  const size_t cap = size_t(sgh_num_cus()) * 16;
  return int(b < 1 ? 1 : (b > cap ? cap : b));
}

int reduce_all(const float *a, const float *b, size_t n, float *out, void *workspace, size_t ws_bytes, void *stream) {
  if (!out) return SGH_EINVAL;
  if (n > 0 && !a) return SGH_EINVAL;
  if (!workspace || ws_bytes < sgh_reduce_workspace_bytes()) return SGH_EWORKSPACE;
  float *part = static_cast<float *>(workspace);
  // at least 4096 elements per workgroup; the split depends on n only
  size_t blocks = (n + 4095) / 4096;
  if (blocks > size_t(kReduceBlocks)) blocks = kReduceBlocks;
  if (blocks < 1) blocks = 1;
  const size_t per = (n + blocks - 1) / blocks;
  hipStream_t s = sgh_stream_of(stream);
  hipLaunchKernelGGL(k_dot_partial, dim3(unsigned(blocks)), dim3(kBlock), 0, s, a, b, n, per, part);
  SGH_LAUNCH_CHECK();
  hipLaunchKernelGGL(k_dot_finish, dim3(1), dim3(kBlock), 0, s, part, int(blocks), out);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

}  // namespace

extern "C" {

int sgh_transform_f32(const float *in, float *out, int ndim, const size_t *shape, const int64_t *strides, void *stream) {
  if (ndim < 0 || ndim > SGH_MAX_DIMS || (ndim > 0 && (!shape || !strides))) return SGH_EINVAL;
  View v{};
  v.ndim = ndim;
  size_t n = 1;
  for (int d = 0; d < ndim; ++d) {
    if (shape[d] > 0xffffffffull || strides[d] < 0) return SGH_EINVAL;   // (views that run backwards do not occur)
    v.shape[d] = unsigned(shape[d]);
    v.stride[d] = strides[d];
    n *= shape[d];
  }
  if (n == 0) return SGH_OK;
  if (!in || !out) return SGH_EINVAL;
  hipLaunchKernelGGL(k_transform, dim3(grid_for(n)), dim3(kBlock), 0, sgh_stream_of(stream), in, out, n, v);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_row_max_f32(const float *in, float *out, size_t nrow, size_t ncol, void *stream) {
  if (nrow == 0) return SGH_OK;
  if (!in || !out || ncol == 0 || nrow > 0x7fffffffull || ncol > 0x7fffffffull) return SGH_EINVAL;
  hipLaunchKernelGGL(k_row_max<false>, dim3(unsigned(nrow)), dim3(kBlock), 0, sgh_stream_of(stream), in, out, int(ncol));
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_row_max_zero_seeded_f32(const float *in, float *out, size_t nrow, size_t ncol, void *stream) {
  if (nrow == 0) return SGH_OK;
  if (!in || !out || ncol == 0 || nrow > 0x7fffffffull || ncol > 0x7fffffffull) return SGH_EINVAL;
  hipLaunchKernelGGL(k_row_max<true>, dim3(unsigned(nrow)), dim3(kBlock), 0, sgh_stream_of(stream), in, out, int(ncol));
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

size_t sgh_reduce_workspace_bytes(void) { return size_t(kReduceBlocks) * sizeof(float); }

int sgh_dot_f32(const float *a, const float *b, size_t n, float *out, void *workspace, size_t ws_bytes, void *stream) {
  if (n > 0 && !b) return SGH_EINVAL;
  return reduce_all(a, b, n, out, workspace, ws_bytes, stream);
}

int sgh_sum_all_f32(const float *a, size_t n, float *out, void *workspace, size_t ws_bytes, void *stream) {
  return reduce_all(a, nullptr, n, out, workspace, ws_bytes, stream);
}

int sgh_uniform_f32(float low, float high, float *out, size_t n, uint64_t seed, uint64_t offset, void *stream) {
  if (n == 0) return SGH_OK;
  if (!out) return SGH_EINVAL;
  sgh_weights_epoch_bump();   // (weights are initialised this way)
  hipLaunchKernelGGL(k_uniform, dim3(grid_for(n)), dim3(kBlock), 0, sgh_stream_of(stream), out, n,
                     static_cast<unsigned long long>(seed), static_cast<unsigned long long>(offset), double(low),
                     double(high));
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

int sgh_gaussian_f32(float mean, float std, float *out, size_t n, uint64_t seed, uint64_t offset, void *stream) {
  if (n == 0) return SGH_OK;
  if (!out) return SGH_EINVAL;
  sgh_weights_epoch_bump();
  hipLaunchKernelGGL(k_gaussian, dim3(grid_for(n)), dim3(kBlock), 0, sgh_stream_of(stream), out, n,
                     static_cast<unsigned long long>(seed), static_cast<unsigned long long>(offset), double(mean),
                     double(std));
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

}  // extern "C"
