// tensor_math specialisations for lang::Hip.  Lands in a SINGA tree as
// src/core/tensor/tensor_math_hip.h and is included by src/core/tensor/tensor.cc beside
// tensor_math_cuda.h; TYPE_LANG_SWITCH / TYPE_TYPE_LANG_SWITCH get kHip cases
// (glue/apply_to_tree.py makes both edits).
//
// Each function has the signature of its primary template in src/core/tensor/tensor_math.h and
// makes one call into singa_hip.h on ctx->hip_stream.  They run on the host thread inside the
// Exec lambda and only enqueue work.  Operands that are not dense (transposed or broadcast views)
// are first copied to a dense temporary with Transform, which is what the reference's CUDA
// functions do (src/core/tensor/tensor_math_cuda.h:300-362).
#ifndef SINGA_CORE_TENSOR_TENSOR_MATH_HIP_H_
#define SINGA_CORE_TENSOR_TENSOR_MATH_HIP_H_

#include "singa/singa_config.h"
#ifdef USE_HIP

#include <cstdint>
#include <vector>

#include "./tensor_math.h"
#include "singa/core/common.h"
#include "singa/core/hip_gpu.h"
#include "singa/core/tensor.h"
#include "singa_hip.h"

namespace singa {
namespace hipglue {

typedef half_float::half half_t;

inline void *stream_of(Context *ctx) { return ctx->hip_stream; }

template <typename T>
inline const T *in_ptr(const Tensor &t) {
  return static_cast<const T *>(t.block()->data());
}
template <typename T>
inline T *out_ptr(Tensor *t) {
  return static_cast<T *>(t->block()->mutable_data());
}
// half tensors cross the ABI as their raw 16-bit words
inline const uint16_t *in_h(const Tensor &t) { return static_cast<const uint16_t *>(t.block()->data()); }
inline uint16_t *out_h(Tensor *t) { return static_cast<uint16_t *>(t->block()->mutable_data()); }

// Dense copy of a strided view (Tensor::stride() holds element strides, 0 for a broadcast
// dimension: src/core/tensor/tensor.cc:481-503).
inline void transform_f32(const Tensor &in, Tensor *out, Context *ctx) {
  const size_t nd = in.nDim();
  CHECK_LE(nd, static_cast<size_t>(SGH_MAX_DIMS)) << "Transform: at most " << SGH_MAX_DIMS << " dimensions";
  size_t shape[SGH_MAX_DIMS];
  int64_t strides[SGH_MAX_DIMS];
  for (size_t d = 0; d < nd; ++d) {
    shape[d] = in.shape(d);
    strides[d] = in.stride().at(d);
  }
  HIP_ABI_CHECK(sgh_transform_f32(in_ptr<float>(in), out_ptr<float>(out), static_cast<int>(nd), shape, strides,
                                  stream_of(ctx)));
}

// A dense fp32 view of `t`: the tensor itself when it is contiguous, otherwise a temporary
// filled by Transform (kept alive by this object until the caller's launch is enqueued; the
// pool recycles it in stream order).
class DenseF32 {
 public:
  DenseF32(const Tensor &t, Context *ctx) {
    if (t.is_contiguous()) {
      ptr_ = in_ptr<float>(t);
    } else {
      tmp_ = Tensor(t.shape(), t.device(), t.data_type());
      transform_f32(t, &tmp_, ctx);
      ptr_ = in_ptr<float>(tmp_);
    }
  }
  const float *get() const { return ptr_; }

 private:
  Tensor tmp_;
  const float *ptr_ = nullptr;
};

// a stride-0 view of a 1-element tensor, e.g. `buf *= mom_value` (python/singa/opt.py:299-300)
inline bool is_scalar_view(const Tensor &t) { return t.broadcasted() && t.block()->size() == sizeof(float); }

}  // namespace hipglue

// ---- fp32 elementwise ----------------------------------------------------------------------
template <>
void Set<float, lang::Hip>(const float x, Tensor *out, Context *ctx) {
  HIP_ABI_CHECK(sgh_memset_f32(hipglue::out_ptr<float>(out), x, out->Size(), hipglue::stream_of(ctx)));
}

template <>
void Transform<float, lang::Hip>(const Tensor &in, Tensor *out, Context *ctx) {
  hipglue::transform_f32(in, out, ctx);
}

template <>
void ReLU<float, lang::Hip>(const Tensor &in, Tensor *out, Context *ctx) {
  hipglue::DenseF32 x(in, ctx);
  HIP_ABI_CHECK(sgh_relu_fwd_f32(x.get(), hipglue::out_ptr<float>(out), out->Size(), hipglue::stream_of(ctx)));
}

/// out = in2 > 0 ? in1 : 0 (in1 = dy, in2 = the ReLU's input)
template <>
void ReLUBackward<float, lang::Hip>(const Tensor &in1, const Tensor &in2, Tensor *out, Context *ctx) {
  hipglue::DenseF32 dy(in1, ctx), x(in2, ctx);
  HIP_ABI_CHECK(sgh_relu_bwd_f32(dy.get(), x.get(), hipglue::out_ptr<float>(out), out->Size(), hipglue::stream_of(ctx)));
}

template <>
void Add<float, lang::Hip>(const Tensor &in1, const Tensor &in2, Tensor *out, Context *ctx) {
  hipglue::DenseF32 a(in1, ctx), b(in2, ctx);
  HIP_ABI_CHECK(sgh_add_f32(a.get(), b.get(), hipglue::out_ptr<float>(out), out->Size(), hipglue::stream_of(ctx)));
}

template <>
void Add<float, lang::Hip>(const Tensor &in, const float x, Tensor *out, Context *ctx) {
  hipglue::DenseF32 a(in, ctx);
  HIP_ABI_CHECK(sgh_add_scalar_f32(a.get(), x, hipglue::out_ptr<float>(out), out->Size(), hipglue::stream_of(ctx)));
}

template <>
void Sub<float, lang::Hip>(const Tensor &in1, const Tensor &in2, Tensor *out, Context *ctx) {
  hipglue::DenseF32 a(in1, ctx), b(in2, ctx);
  HIP_ABI_CHECK(sgh_sub_f32(a.get(), b.get(), hipglue::out_ptr<float>(out), out->Size(), hipglue::stream_of(ctx)));
}

template <>
void Div<float, lang::Hip>(const Tensor &in1, const Tensor &in2, Tensor *out, Context *ctx) {
  hipglue::DenseF32 a(in1, ctx), b(in2, ctx);
  HIP_ABI_CHECK(sgh_div_f32(a.get(), b.get(), hipglue::out_ptr<float>(out), out->Size(), hipglue::stream_of(ctx)));
}

template <>
void EltwiseMult<float, lang::Hip>(const Tensor &in, const float x, Tensor *out, Context *ctx) {
  hipglue::DenseF32 a(in, ctx);
  HIP_ABI_CHECK(sgh_mult_scalar_f32(a.get(), x, hipglue::out_ptr<float>(out), out->Size(), hipglue::stream_of(ctx)));
}

/// out = in1 * in2; a stride-0 view of a 1-element tensor on the right is read in place
/// instead of being materialised.
template <>
void EltwiseMult<float, lang::Hip>(const Tensor &in1, const Tensor &in2, Tensor *out, Context *ctx) {
  hipglue::DenseF32 a(in1, ctx);
  if (hipglue::is_scalar_view(in2)) {
    HIP_ABI_CHECK(sgh_eltwise_mult_f32(a.get(), hipglue::in_ptr<float>(in2), 1, hipglue::out_ptr<float>(out),
                                       out->Size(), hipglue::stream_of(ctx)));
    return;
  }
  hipglue::DenseF32 b(in2, ctx);
  HIP_ABI_CHECK(sgh_eltwise_mult_f32(a.get(), b.get(), 0, hipglue::out_ptr<float>(out), out->Size(),
                                     hipglue::stream_of(ctx)));
}

template <>
void Clamp<float, lang::Hip>(const float low, const float high, const Tensor &in, Tensor *out, Context *ctx) {
  hipglue::DenseF32 a(in, ctx);
  HIP_ABI_CHECK(sgh_clamp_f32(low, high, a.get(), hipglue::out_ptr<float>(out), out->Size(), hipglue::stream_of(ctx)));
}

// ---- random fills: element i = f(seed, offset + i); the Context keeps (seed, offset) -------
template <>
void Uniform<float, lang::Hip>(const float low, const float high, Tensor *out, Context *ctx) {
  const size_t n = out->Size();
  HIP_ABI_CHECK(sgh_uniform_f32(low, high, hipglue::out_ptr<float>(out), n, ctx->hip_rng_seed, ctx->hip_rng_offset,
                                hipglue::stream_of(ctx)));
  ctx->hip_rng_offset += n;
}

template <>
void Gaussian<float, lang::Hip>(const float mean, const float std, Tensor *out, Context *ctx) {
  const size_t n = out->Size();
  HIP_ABI_CHECK(sgh_gaussian_f32(mean, std, hipglue::out_ptr<float>(out), n, ctx->hip_rng_seed, ctx->hip_rng_offset,
                                 hipglue::stream_of(ctx)));
  ctx->hip_rng_offset += 2 * n;
}

// ---- BLAS-like -----------------------------------------------------------------------------
template <>
void Axpy<float, lang::Hip>(const float alpha, const Tensor &in, Tensor *out, Context *ctx) {
  HIP_ABI_CHECK(sgh_axpy_f32(alpha, hipglue::in_ptr<float>(in), hipglue::out_ptr<float>(out), in.Size(),
                             hipglue::stream_of(ctx)));
}

/// alpha is a 1-element tensor on the device (the optimizer's lr / momentum tensors)
template <>
void Axpy<float, lang::Hip>(const Tensor &alpha, const Tensor &in, Tensor *out, Context *ctx) {
  HIP_ABI_CHECK(sgh_axpy_devalpha_f32(hipglue::in_ptr<float>(alpha), hipglue::in_ptr<float>(in),
                                      hipglue::out_ptr<float>(out), in.Size(), hipglue::stream_of(ctx)));
}

template <>
void Scale<float, lang::Hip>(const float x, Tensor *out, Context *ctx) {
  float *p = hipglue::out_ptr<float>(out);
  HIP_ABI_CHECK(sgh_mult_scalar_f32(p, x, p, out->Size(), hipglue::stream_of(ctx)));
}

/// the result lands in a 1-element tensor on the device
template <>
void Dot<float, lang::Hip>(const Tensor &in1, const Tensor &in2, Tensor *out, Context *ctx) {
  HIP_ABI_CHECK(sgh_dot_f32(hipglue::in_ptr<float>(in1), hipglue::in_ptr<float>(in2), in1.Size(),
                            hipglue::out_ptr<float>(out), ctx->hip_reduce_ws, ctx->hip_reduce_ws_bytes,
                            hipglue::stream_of(ctx)));
}

/// host result: the value is computed into the head of the device's reduction scratch and copied
/// back with a blocking copy
template <>
void Dot<float, lang::Hip>(const Tensor &in1, const Tensor &in2, float *out, Context *ctx) {
  float *result = static_cast<float *>(ctx->hip_reduce_result);
  HIP_ABI_CHECK(sgh_dot_f32(hipglue::in_ptr<float>(in1), hipglue::in_ptr<float>(in2), in1.Size(), result,
                            ctx->hip_reduce_ws, ctx->hip_reduce_ws_bytes, hipglue::stream_of(ctx)));
  HIP_ABI_CHECK(sgh_memcpy(ctx->hip_device, out, result, sizeof(float), 2));
}

template <>
void Sum<float, lang::Hip>(const Tensor &in, float *out, Context *ctx) {
  float *result = static_cast<float *>(ctx->hip_reduce_result);
  HIP_ABI_CHECK(sgh_sum_all_f32(hipglue::in_ptr<float>(in), in.Size(), result, ctx->hip_reduce_ws,
                                ctx->hip_reduce_ws_bytes, hipglue::stream_of(ctx)));
  HIP_ABI_CHECK(sgh_memcpy(ctx->hip_device, out, result, sizeof(float), 2));
}

/// C = alpha * A * B + beta * C.  A transposed view (Tensor::T()) keeps its block and swaps its
/// strides; shape() is the logical one, so the stored matrix of a transposed A is [K][M].
template <>
void GEMM<float, lang::Hip>(const float alpha, const Tensor &A, const Tensor &B, const float beta, Tensor *C,
                            Context *ctx) {
  const bool ta = A.transpose(), tb = B.transpose();
  const int M = static_cast<int>(A.shape(0)), K = static_cast<int>(A.shape(1)), N = static_cast<int>(B.shape(1));
  HIP_ABI_CHECK(sgh_gemm_f32(ta, tb, M, N, K, alpha, hipglue::in_ptr<float>(A), ta ? M : K, hipglue::in_ptr<float>(B),
                             tb ? K : N, beta, hipglue::out_ptr<float>(C), N, hipglue::stream_of(ctx)));
}

/// out = alpha * A * v + beta * out: the GEMM above with a single column.  Sum(dy, 0), the bias
/// gradient of a Linear layer, arrives here as A = dy^T, v = ones (src/core/tensor/tensor.cc:1523-1538).
template <>
void GEMV<float, lang::Hip>(const float alpha, const Tensor &A, const Tensor &v, const float beta, Tensor *out,
                            Context *ctx) {
  const bool ta = A.transpose();
  const int M = static_cast<int>(A.shape(0)), K = static_cast<int>(A.shape(1));
  HIP_ABI_CHECK(sgh_gemm_f32(ta, 0, M, 1, K, alpha, hipglue::in_ptr<float>(A), ta ? M : K, hipglue::in_ptr<float>(v), 1,
                             beta, hipglue::out_ptr<float>(out), 1, hipglue::stream_of(ctx)));
}

// ---- softmax / cross entropy ---------------------------------------------------------------
/// rows of a [batch, dim] matrix (a 1-D tensor is one row)
template <>
void SoftMax<float, lang::Hip>(const Tensor &in, Tensor *out, Context *ctx) {
  hipglue::DenseF32 x(in, ctx);
  const size_t dim = in.shape(in.nDim() - 1), batch = in.Size() / dim;
  HIP_ABI_CHECK(sgh_softmax_fwd_f32(x.get(), hipglue::out_ptr<float>(out), batch, dim, hipglue::stream_of(ctx)));
}

/// RowMax of the reference's accelerator path: the true maximum of each row
/// (src/core/tensor/math_kernel.cu:488-499).
template <>
void RowMax<float, lang::Hip>(const Tensor &in, Tensor *out, Context *ctx) {
  hipglue::DenseF32 x(in, ctx);
  HIP_ABI_CHECK(sgh_row_max_f32(x.get(), hipglue::out_ptr<float>(out), in.shape(0), in.shape(1), hipglue::stream_of(ctx)));
}

/// `t` holds int32 class indices (int_target) or an int32 [batch, dim] array, whatever the
/// tensor's declared type: the reference reads it as `const int*` on every backend.
template <>
void ComputeCrossEntropy<float, lang::Hip>(bool int_target, const size_t batchsize, const size_t dim, const Tensor &p,
                                           const Tensor &t, Tensor *loss, Context *ctx) {
  HIP_ABI_CHECK(sgh_cross_entropy_fwd_f32(hipglue::in_ptr<float>(p), hipglue::in_ptr<int32_t>(t),
                                          hipglue::out_ptr<float>(loss), batchsize, dim, int_target,
                                          hipglue::stream_of(ctx)));
}

/// in place on a clone of p (src/core/tensor/tensor.cc:1741-1758)
template <>
void SoftmaxCrossEntropyBwd<float, lang::Hip>(bool int_target, const size_t batchsize, const size_t dim, const Tensor &p,
                                              const Tensor &t, Tensor *grad, Context *ctx) {
  CHECK_EQ(p.block(), grad->block()) << "Use the same pointer to optimize performance";
  HIP_ABI_CHECK(sgh_softmax_ce_bwd_f32(hipglue::in_ptr<float>(p), hipglue::in_ptr<int32_t>(t),
                                       hipglue::out_ptr<float>(grad), batchsize, dim, int_target, 1.0f,
                                       hipglue::stream_of(ctx)));
}

// ---- casts (Tensor::AsType) ----------------------------------------------------------------
template <>
void CastCopy<float, hipglue::half_t, lang::Hip>(const Tensor *src, Tensor *dst, Context *ctx) {
  HIP_ABI_CHECK(sgh_cast_f32_to_f16(hipglue::in_ptr<float>(*src), hipglue::out_h(dst), dst->Size(), hipglue::stream_of(ctx)));
}
template <>
void CastCopy<hipglue::half_t, float, lang::Hip>(const Tensor *src, Tensor *dst, Context *ctx) {
  HIP_ABI_CHECK(sgh_cast_f16_to_f32(hipglue::in_h(*src), hipglue::out_ptr<float>(dst), dst->Size(), hipglue::stream_of(ctx)));
}
template <>
void CastCopy<float, int, lang::Hip>(const Tensor *src, Tensor *dst, Context *ctx) {
  HIP_ABI_CHECK(sgh_cast_f32_to_i32(hipglue::in_ptr<float>(*src), hipglue::out_ptr<int32_t>(dst), dst->Size(),
                                    hipglue::stream_of(ctx)));
}
template <>
void CastCopy<int, float, lang::Hip>(const Tensor *src, Tensor *dst, Context *ctx) {
  HIP_ABI_CHECK(sgh_cast_i32_to_f32(hipglue::in_ptr<int32_t>(*src), hipglue::out_ptr<float>(dst), dst->Size(),
                                    hipglue::stream_of(ctx)));
}

// ---- half tensors: raw 16-bit words through the *_f16 entry points (fp32 arithmetic, one
// rounding at the store).  Dense operands only, as the layers of a half model produce them. ----
template <>
void Set<hipglue::half_t, lang::Hip>(const hipglue::half_t x, Tensor *out, Context *ctx) {
  HIP_ABI_CHECK(sgh_memset_f16(hipglue::out_h(out), static_cast<float>(x), out->Size(), hipglue::stream_of(ctx)));
}

template <>
void ReLU<hipglue::half_t, lang::Hip>(const Tensor &in, Tensor *out, Context *ctx) {
  CHECK(in.is_contiguous());
  HIP_ABI_CHECK(sgh_relu_fwd_f16(hipglue::in_h(in), hipglue::out_h(out), out->Size(), hipglue::stream_of(ctx)));
}

template <>
void ReLUBackward<hipglue::half_t, lang::Hip>(const Tensor &in1, const Tensor &in2, Tensor *out, Context *ctx) {
  CHECK(in1.is_contiguous() && in2.is_contiguous());
  HIP_ABI_CHECK(sgh_relu_bwd_f16(hipglue::in_h(in1), hipglue::in_h(in2), hipglue::out_h(out), out->Size(),
                                 hipglue::stream_of(ctx)));
}

template <>
void Add<hipglue::half_t, lang::Hip>(const Tensor &in1, const Tensor &in2, Tensor *out, Context *ctx) {
  CHECK(in1.is_contiguous() && in2.is_contiguous());
  HIP_ABI_CHECK(sgh_add_f16(hipglue::in_h(in1), hipglue::in_h(in2), hipglue::out_h(out), out->Size(), hipglue::stream_of(ctx)));
}

template <>
void EltwiseMult<hipglue::half_t, lang::Hip>(const Tensor &in1, const Tensor &in2, Tensor *out, Context *ctx) {
  CHECK(in1.is_contiguous() && in2.is_contiguous());
  HIP_ABI_CHECK(sgh_eltwise_mult_f16(hipglue::in_h(in1), hipglue::in_h(in2), hipglue::out_h(out), out->Size(),
                                     hipglue::stream_of(ctx)));
}

template <>
void Axpy<hipglue::half_t, lang::Hip>(const hipglue::half_t alpha, const Tensor &in, Tensor *out, Context *ctx) {
  HIP_ABI_CHECK(sgh_axpy_f16(static_cast<float>(alpha), hipglue::in_h(in), hipglue::out_h(out), in.Size(),
                             hipglue::stream_of(ctx)));
}

/// Linear layers of a half model: 16-bit operands on the 16-bit matrix instructions, fp32
/// accumulation, one rounding (the reference calls cublasHgemm, tensor_math_cuda.h:1163-1187).
template <>
void GEMM<hipglue::half_t, lang::Hip>(const hipglue::half_t alpha, const Tensor &A, const Tensor &B,
                                      const hipglue::half_t beta, Tensor *C, Context *ctx) {
  const bool ta = A.transpose(), tb = B.transpose();
  const int M = static_cast<int>(A.shape(0)), K = static_cast<int>(A.shape(1)), N = static_cast<int>(B.shape(1));
  HIP_ABI_CHECK(sgh_gemm_f16(ta, tb, M, N, K, static_cast<float>(alpha), hipglue::in_h(A), ta ? M : K, hipglue::in_h(B),
                             tb ? K : N, static_cast<float>(beta), hipglue::out_h(C), N, hipglue::stream_of(ctx)));
}

template <>
void SoftmaxCrossEntropyBwd<hipglue::half_t, lang::Hip>(bool int_target, const size_t batchsize, const size_t dim,
                                                        const Tensor &p, const Tensor &t, Tensor *grad, Context *ctx) {
  CHECK_EQ(p.block(), grad->block()) << "Use the same pointer to optimize performance";
  HIP_ABI_CHECK(sgh_softmax_ce_bwd_f16(hipglue::in_h(p), hipglue::in_ptr<int32_t>(t), hipglue::out_h(grad), batchsize, dim,
                                       int_target, 1.0f, hipglue::stream_of(ctx)));
}

}  // namespace singa

#endif  // USE_HIP
#endif  // SINGA_CORE_TENSOR_TENSOR_MATH_HIP_H_
