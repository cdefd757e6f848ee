// Bodies of the handles and Gpu* operation functions declared in operation_hip.h.  Lands in a
// SINGA tree as src/model/operation/operation_hip.cc.
//
// Pattern of every function (that of the reference's cuDNN bodies,
// src/model/operation/convolution.cc:585-702, batchnorm.cc:287-404, pooling.cc:187-226): check
// devices and shapes on the host, allocate the results, submit ONE lambda through Device::Exec
// with the blocks it reads and writes; the lambda makes one singa_hip.h call on the device's
// stream.  Tensors are captured by value (reference counted), handles by reference: they belong
// to the Python layer and outlive the graph.
#include "./operation_hip.h"

#ifdef USE_HIP

#include "singa/core/hip_gpu.h"

namespace singa {

namespace {

const float kBnEpsilon = 1e-5f;   // CUDNN_BN_MIN_EPSILON, what the reference passes (batchnorm.cc:313)

inline bool is_half(const Tensor &t) { return t.data_type() == kFloat16; }
inline const float *f32(const Tensor &t) { return static_cast<const float *>(t.block()->data()); }
inline float *f32_out(const Tensor &t) { return static_cast<float *>(t.block()->mutable_data()); }
inline const uint16_t *f16(const Tensor &t) { return static_cast<const uint16_t *>(t.block()->data()); }
inline uint16_t *f16_out(const Tensor &t) { return static_cast<uint16_t *>(t.block()->mutable_data()); }

inline void check_on_hip(const Tensor &t) { CHECK_EQ(t.device()->lang(), kHip); }

inline void check_conv_dy(const Tensor &dy, const CudnnConvHandle &cch) {
  CHECK(dy.nDim() == 4u && dy.shape(0) == cch.batchsize && dy.shape(1) == cch.num_filters &&
        dy.shape(2) == cch.conv_height && dy.shape(3) == cch.conv_width)
      << "dy shape does not match the handle";
}

// a float tensor of at least `bytes` bytes on `dev`, the handle's scratch
inline Tensor scratch_tensor(size_t bytes, std::shared_ptr<Device> dev) {
  const size_t n = bytes / sizeof(float) + 1;
  return Tensor(Shape{n}, dev, kFloat32);
}

}  // namespace

// =================================== convolution ===========================================
CudnnConvHandle::CudnnConvHandle(const Tensor &input, const std::vector<size_t> &kernel_size,
                                 const std::vector<size_t> &stride, const std::vector<size_t> &padding,
                                 const size_t in_channels, const size_t out_channels, const bool bias,
                                 const size_t groups, const size_t workspace_byte_limit, const std::string &)
    : ConvHandle(input, kernel_size, stride, padding, in_channels, out_channels, bias, groups) {
  check_on_hip(input);
  CHECK_EQ(input.nDim(), 4u);
  dtype = input.data_type();
  CHECK(dtype == kFloat32 || dtype == kFloat16) << "convolution on the HIP device: float or half tensors";
  HIP_ABI_CHECK(sgh_conv_geom_init_grouped(&geom, static_cast<int>(batchsize), static_cast<int>(channels),
                                           static_cast<int>(height), static_cast<int>(width),
                                           static_cast<int>(num_filters), static_cast<int>(kernel_h),
                                           static_cast<int>(kernel_w), static_cast<int>(stride_h),
                                           static_cast<int>(stride_w), static_cast<int>(pad_h), static_cast<int>(pad_w),
                                           static_cast<int>(groups)));
  CHECK_EQ(static_cast<size_t>(geom.P), conv_height);
  CHECK_EQ(static_cast<size_t>(geom.Q), conv_width);
  channels_per_filter = channels / groups;
  size_t need = 0;
  for (int which : {SGH_CONV_FWD, SGH_CONV_DGRAD, SGH_CONV_WGRAD}) {
    const size_t b = dtype == kFloat32 ? sgh_conv_workspace_bytes(&geom, which) : sgh_conv_workspace_bytes_h(&geom, which);
    if (b > need) need = b;
  }
  CHECK_LE(need, workspace_byte_limit) << "convolution workspace exceeds the handle's limit";
  workspace = scratch_tensor(need, input.device());
  workspace_count = workspace.Size();
}

Tensor GpuConvForward(const Tensor &x, const Tensor &W, const Tensor &b, const CudnnConvHandle &cch) {
  check_on_hip(x);
  CHECK(x.shape(1) == cch.channels && x.shape(2) == cch.height && x.shape(3) == cch.width)
      << "input sample shape should not change";
  CHECK(W.shape(0) == cch.num_filters && W.shape(1) == cch.channels_per_filter && W.shape(2) == cch.kernel_h &&
        W.shape(3) == cch.kernel_w)
      << "weights shape should not change";
  Tensor y(Shape{cch.batchsize, cch.num_filters, cch.conv_height, cch.conv_width}, x.device(), x.data_type());
  const bool with_bias = cch.bias_term;
  std::vector<Block *> reads{x.block(), W.block()};
  if (with_bias) reads.push_back(b.block());
  y.device()->Exec(
      [y, x, W, b, with_bias, &cch](Context *ctx) mutable {
        void *ws = cch.workspace.block()->mutable_data();
        const size_t ws_bytes = cch.workspace.MemSize();
        if (is_half(x))
          HIP_ABI_CHECK(sgh_conv_fwd_f16(&cch.geom, f16(x), f16(W), with_bias ? f16(b) : nullptr, f16_out(y), ws,
                                         ws_bytes, ctx->hip_stream));
        else
          HIP_ABI_CHECK(sgh_conv_fwd_f32(&cch.geom, f32(x), f32(W), with_bias ? f32(b) : nullptr, f32_out(y), ws,
                                         ws_bytes, ctx->hip_stream));
      },
      reads, {y.block(), cch.workspace.block()}, "GpuConvForward");
  return y;
}

Tensor GpuConvBackwardx(const Tensor &dy, const Tensor &W, const Tensor &x, const CudnnConvHandle &cch) {
  check_on_hip(dy);
  check_conv_dy(dy, cch);
  Tensor dx;
  dx.ResetLike(x);
  dy.device()->Exec(
      [dx, dy, W, &cch](Context *ctx) mutable {
        void *ws = cch.workspace.block()->mutable_data();
        const size_t ws_bytes = cch.workspace.MemSize();
        if (is_half(dy))
          HIP_ABI_CHECK(sgh_conv_dgrad_f16(&cch.geom, f16(dy), f16(W), f16_out(dx), ws, ws_bytes, ctx->hip_stream));
        else
          HIP_ABI_CHECK(sgh_conv_dgrad_f32(&cch.geom, f32(dy), f32(W), f32_out(dx), ws, ws_bytes, ctx->hip_stream));
      },
      {dy.block(), W.block()}, {dx.block(), cch.workspace.block()}, "GpuConvBackwardx");
  return dx;
}

Tensor GpuConvBackwardW(const Tensor &dy, const Tensor &x, const Tensor &W, const CudnnConvHandle &cch) {
  check_on_hip(dy);
  check_conv_dy(dy, cch);
  Tensor dW;
  dW.ResetLike(W);
  dy.device()->Exec(
      [dW, dy, x, &cch](Context *ctx) mutable {
        void *ws = cch.workspace.block()->mutable_data();
        const size_t ws_bytes = cch.workspace.MemSize();
        if (is_half(dy))
          HIP_ABI_CHECK(sgh_conv_wgrad_f16(&cch.geom, f16(dy), f16(x), f16_out(dW), ws, ws_bytes, ctx->hip_stream));
        else
          HIP_ABI_CHECK(sgh_conv_wgrad_f32(&cch.geom, f32(dy), f32(x), f32_out(dW), ws, ws_bytes, ctx->hip_stream));
      },
      {dy.block(), x.block()}, {dW.block(), cch.workspace.block()}, "GpuConvBackwardW");
  return dW;
}

// (b only gives the result its shape, as in the reference)
Tensor GpuConvBackwardb(const Tensor &dy, const Tensor &b, const CudnnConvHandle &cch) {
  check_on_hip(dy);
  check_conv_dy(dy, cch);
  Tensor db;
  db.ResetLike(b);
  dy.device()->Exec(
      [dy, db, &cch](Context *ctx) mutable {
        if (is_half(dy))
          HIP_ABI_CHECK(sgh_conv_bgrad_f16(&cch.geom, f16(dy), f16_out(db), ctx->hip_stream));
        else
          HIP_ABI_CHECK(sgh_conv_bgrad_f32(&cch.geom, f32(dy), f32_out(db), ctx->hip_stream));
      },
      {dy.block()}, {db.block()}, "GpuConvBackwardb");
  return db;
}

void GpuConvBackwardxAccumulate(const Tensor &dy, const Tensor &W, const Tensor &x, const CudnnConvHandle &cch,
                                Tensor *dx_sum) {
  check_on_hip(dy);
  check_conv_dy(dy, cch);
  CHECK(dx_sum != nullptr && dx_sum->shape() == x.shape());
  // which geometries the accumulating kernels cover is a property of the handle
  const bool fused = !is_half(dy) && sgh_conv_dgrad_acc_supported(&cch.geom) != 0;
  if (!fused) {
    *dx_sum += GpuConvBackwardx(dy, W, x, cch);
    return;
  }
  Tensor acc(*dx_sum);
  dy.device()->Exec(
      [acc, dy, W, &cch](Context *ctx) mutable {
        HIP_ABI_CHECK(sgh_conv_dgrad_acc_f32(&cch.geom, f32(dy), f32(W), f32_out(acc),
                                             cch.workspace.block()->mutable_data(), cch.workspace.MemSize(),
                                             ctx->hip_stream));
      },
      {dy.block(), W.block(), acc.block()}, {acc.block(), cch.workspace.block()}, "GpuConvBackwardxAccumulate");
}

// =================================== batch normalisation ===================================
CudnnBatchNormHandle::CudnnBatchNormHandle(const float momentum, const Tensor &input)
    : BatchNormHandle(momentum, input) {
  check_on_hip(input);
  const size_t bytes = sgh_bn_workspace_bytes(static_cast<int>(batchsize), static_cast<int>(channels),
                                              static_cast<int>(height * width));
  workspace = scratch_tensor(bytes, input.device());
}

namespace {

// act: 0 BatchNorm alone, 1 + ReLU, 2 + z, then ReLU.  A 2-D input [N, C] is the spatial case with
// planes of one element (cuDNN's per-activation mode, batchnorm.cc:264-266).
std::vector<Tensor> bn_forward_training(const CudnnBatchNormHandle &cbnh, const Tensor &x, const Tensor *z,
                                        const Tensor &bnScale, const Tensor &bnBias, Tensor &running_mean,
                                        Tensor &running_var, int act, const char *name) {
  check_on_hip(x);
  check_on_hip(bnScale);
  check_on_hip(bnBias);
  check_on_hip(running_mean);
  check_on_hip(running_var);
  Tensor mean, var, y;
  mean.ResetLike(running_mean);
  var.ResetLike(running_var);
  y.ResetLike(x);
  Tensor zz = z ? *z : Tensor();
  const int N = static_cast<int>(cbnh.batchsize), C = static_cast<int>(cbnh.channels),
            HW = static_cast<int>(cbnh.height * cbnh.width);
  const float factor = cbnh.factor;
  std::vector<Block *> reads{x.block(), bnScale.block(), bnBias.block(), running_mean.block(), running_var.block()};
  if (z) reads.push_back(z->block());
  y.device()->Exec(
      [=, &cbnh](Context *ctx) mutable {
        void *ws = cbnh.workspace.block()->mutable_data();
        const size_t wsb = cbnh.workspace.MemSize();
        float *rm = f32_out(running_mean), *rv = f32_out(running_var), *sm = f32_out(mean), *sv = f32_out(var);
        const float *g = f32(bnScale), *be = f32(bnBias);
        void *st = ctx->hip_stream;
        if (is_half(x)) {
          if (act == 0)
            HIP_ABI_CHECK(sgh_bn_fwd_train_f16(f16(x), g, be, rm, rv, factor, kBnEpsilon, f16_out(y), sm, sv, N, C, HW, ws, wsb, st));
          else if (act == 1)
            HIP_ABI_CHECK(sgh_bn_relu_fwd_train_f16(f16(x), g, be, rm, rv, factor, kBnEpsilon, f16_out(y), sm, sv, N, C, HW, ws, wsb, st));
          else
            HIP_ABI_CHECK(sgh_bn_add_relu_fwd_train_f16(f16(x), f16(zz), g, be, rm, rv, factor, kBnEpsilon, f16_out(y), sm, sv, N, C, HW, ws, wsb, st));
        } else {
          if (act == 0)
            HIP_ABI_CHECK(sgh_bn_fwd_train_f32(f32(x), g, be, rm, rv, factor, kBnEpsilon, f32_out(y), sm, sv, N, C, HW, ws, wsb, st));
          else if (act == 1)
            HIP_ABI_CHECK(sgh_bn_relu_fwd_train_f32(f32(x), g, be, rm, rv, factor, kBnEpsilon, f32_out(y), sm, sv, N, C, HW, ws, wsb, st));
          else
            HIP_ABI_CHECK(sgh_bn_add_relu_fwd_train_f32(f32(x), f32(zz), g, be, rm, rv, factor, kBnEpsilon, f32_out(y), sm, sv, N, C, HW, ws, wsb, st));
        }
      },
      reads, {y.block(), running_mean.block(), running_var.block(), mean.block(), var.block(), cbnh.workspace.block()},
      name);
  return {y, mean, var};
}

std::vector<Tensor> bn_backward(const CudnnBatchNormHandle &cbnh, const Tensor &dy, const Tensor &x,
                                const Tensor &bnScale, const Tensor *bnBias, const Tensor &mean, const Tensor &var,
                                const char *name) {
  check_on_hip(dy);
  check_on_hip(x);
  check_on_hip(bnScale);
  check_on_hip(mean);
  check_on_hip(var);
  CHECK(dy.shape() == x.shape()) << "dy and x differ in shape";
  Tensor dx, dscale, dbias;
  dx.ResetLike(dy);
  dscale.ResetLike(bnScale);
  dbias.ResetLike(bnScale);
  Tensor bias = bnBias ? *bnBias : Tensor();
  const bool fused = bnBias != nullptr;
  const int N = static_cast<int>(cbnh.batchsize), C = static_cast<int>(cbnh.channels),
            HW = static_cast<int>(cbnh.height * cbnh.width);
  std::vector<Block *> reads{x.block(), dy.block(), bnScale.block(), mean.block(), var.block()};
  if (fused) reads.push_back(bias.block());
  dx.device()->Exec(
      [=, &cbnh](Context *ctx) mutable {
        void *ws = cbnh.workspace.block()->mutable_data();
        const size_t wsb = cbnh.workspace.MemSize();
        const float *g = f32(bnScale), *m = f32(mean), *iv = f32(var);
        float *dg = f32_out(dscale), *db = f32_out(dbias);
        void *st = ctx->hip_stream;
        if (is_half(dy)) {
          if (fused)
            HIP_ABI_CHECK(sgh_bn_relu_bwd_f16(f16(dy), f16(x), g, f32(bias), m, iv, f16_out(dx), dg, db, N, C, HW, ws, wsb, st));
          else
            HIP_ABI_CHECK(sgh_bn_bwd_f16(f16(dy), f16(x), g, m, iv, f16_out(dx), dg, db, N, C, HW, ws, wsb, st));
        } else {
          if (fused)
            HIP_ABI_CHECK(sgh_bn_relu_bwd_f32(f32(dy), f32(x), g, f32(bias), m, iv, f32_out(dx), dg, db, N, C, HW, ws, wsb, st));
          else
            HIP_ABI_CHECK(sgh_bn_bwd_f32(f32(dy), f32(x), g, m, iv, f32_out(dx), dg, db, N, C, HW, ws, wsb, st));
        }
      },
      reads, {dx.block(), dscale.block(), dbias.block(), cbnh.workspace.block()}, name);
  return {dx, dscale, dbias};
}

}  // namespace

/// Returns {y, mean, var}; `var` holds the saved INVERSE standard deviation, which is what
/// GpuBatchNormBackward reads back (cuDNN's convention, python/singa/autograd.py:1777-1781).
const std::vector<Tensor> GpuBatchNormForwardTraining(const CudnnBatchNormHandle &cbnh, const Tensor &x,
                                                      const Tensor &bnScale, const Tensor &bnBias,
                                                      Tensor &running_mean, Tensor &running_var) {
  return bn_forward_training(cbnh, x, nullptr, bnScale, bnBias, running_mean, running_var, 0,
                             "GpuBatchNormForwardTraining");
}

const std::vector<Tensor> GpuBatchNormReLUForwardTraining(const CudnnBatchNormHandle &cbnh, const Tensor &x,
                                                          const Tensor &bnScale, const Tensor &bnBias,
                                                          Tensor &running_mean, Tensor &running_var) {
  return bn_forward_training(cbnh, x, nullptr, bnScale, bnBias, running_mean, running_var, 1,
                             "GpuBatchNormReLUForwardTraining");
}

const std::vector<Tensor> GpuBatchNormAddReLUForwardTraining(const CudnnBatchNormHandle &cbnh, const Tensor &x,
                                                             const Tensor &z, const Tensor &bnScale,
                                                             const Tensor &bnBias, Tensor &running_mean,
                                                             Tensor &running_var) {
  CHECK(z.shape() == x.shape() && z.data_type() == x.data_type());
  return bn_forward_training(cbnh, x, &z, bnScale, bnBias, running_mean, running_var, 2,
                             "GpuBatchNormAddReLUForwardTraining");
}

Tensor GpuBatchNormForwardInference(const CudnnBatchNormHandle &cbnh, const Tensor &x, const Tensor &bnScale,
                                    const Tensor &bnBias, const Tensor &running_mean, const Tensor &running_var) {
  check_on_hip(x);
  check_on_hip(bnScale);
  check_on_hip(bnBias);
  check_on_hip(running_mean);
  check_on_hip(running_var);
  Tensor y;
  y.ResetLike(x);
  const int N = static_cast<int>(cbnh.batchsize), C = static_cast<int>(cbnh.channels),
            HW = static_cast<int>(cbnh.height * cbnh.width);
  y.device()->Exec(
      [=](Context *ctx) mutable {
        if (is_half(x))
          HIP_ABI_CHECK(sgh_bn_fwd_infer_f16(f16(x), f32(bnScale), f32(bnBias), f32(running_mean), f32(running_var),
                                             kBnEpsilon, f16_out(y), N, C, HW, ctx->hip_stream));
        else
          HIP_ABI_CHECK(sgh_bn_fwd_infer_f32(f32(x), f32(bnScale), f32(bnBias), f32(running_mean), f32(running_var),
                                             kBnEpsilon, f32_out(y), N, C, HW, ctx->hip_stream));
      },
      {x.block(), bnScale.block(), bnBias.block(), running_mean.block(), running_var.block()}, {y.block()},
      "GpuBatchNormForwardInference");
  return y;
}

const std::vector<Tensor> GpuBatchNormBackward(const CudnnBatchNormHandle &cbnh, const Tensor &dy, const Tensor &x,
                                               const Tensor &bnScale, const Tensor &mean, const Tensor &var) {
  return bn_backward(cbnh, dy, x, bnScale, nullptr, mean, var, "GpuBatchNormBackward");
}

const std::vector<Tensor> GpuBatchNormReLUBackward(const CudnnBatchNormHandle &cbnh, const Tensor &dy, const Tensor &x,
                                                   const Tensor &bnScale, const Tensor &bnBias, const Tensor &mean,
                                                   const Tensor &var) {
  check_on_hip(bnBias);
  return bn_backward(cbnh, dy, x, bnScale, &bnBias, mean, var, "GpuBatchNormReLUBackward");
}

// =================================== pooling ===============================================
CudnnPoolingHandle::CudnnPoolingHandle(const Tensor &input, const std::vector<int> &kernel_size,
                                       const std::vector<int> &stride, const std::vector<int> &padding,
                                       const bool is_max)
    : PoolingHandle(input, kernel_size, stride, padding, is_max) {
  check_on_hip(input);
  HIP_ABI_CHECK(sgh_pool_geom_init(&geom, batchsize, channels, height, width, kernel_h, kernel_w, stride_h, stride_w,
                                   pad_h, pad_w, is_max ? 1 : 0));
  CHECK_EQ(geom.P, pooled_height);
  CHECK_EQ(geom.Q, pooled_width);
}

Tensor GpuPoolingForward(const CudnnPoolingHandle &cph, const Tensor &x) {
  check_on_hip(x);
  CHECK_EQ(x.nDim(), 4u);
  Tensor y(Shape{static_cast<size_t>(cph.batchsize), static_cast<size_t>(cph.channels),
                 static_cast<size_t>(cph.pooled_height), static_cast<size_t>(cph.pooled_width)},
           x.device(), x.data_type());
  y.device()->Exec(
      [y, x, &cph](Context *ctx) mutable {
        if (is_half(x))
          HIP_ABI_CHECK(sgh_pool_fwd_f16(&cph.geom, f16(x), f16_out(y), ctx->hip_stream));
        else
          HIP_ABI_CHECK(sgh_pool_fwd_f32(&cph.geom, f32(x), f32_out(y), ctx->hip_stream));
      },
      {x.block()}, {y.block()}, "GpuPoolingForward");
  return y;
}

Tensor GpuPoolingBackward(const CudnnPoolingHandle &cph, const Tensor &dy, const Tensor &x, const Tensor &y) {
  check_on_hip(dy);
  check_on_hip(x);
  check_on_hip(y);
  CHECK_EQ(dy.nDim(), 4u);
  CHECK(dy.data_type() == x.data_type());
  Tensor dx;
  dx.ResetLike(x);
  dx.device()->Exec(
      [dx, dy, x, y, &cph](Context *ctx) mutable {
        if (is_half(x))
          HIP_ABI_CHECK(sgh_pool_bwd_f16(&cph.geom, f16(dy), f16(x), f16(y), f16_out(dx), ctx->hip_stream));
        else
          HIP_ABI_CHECK(sgh_pool_bwd_f32(&cph.geom, f32(dy), f32(x), f32(y), f32_out(dx), ctx->hip_stream));
      },
      {dy.block(), x.block(), y.block()}, {dx.block()}, "GpuPoolingBackward");
  return dx;
}

// =================================== elementwise fusions ===================================
Tensor ReLUBackwardSum(const Tensor &dy0, const Tensor &dy1, const Tensor &x) {
  check_on_hip(x);
  CHECK(dy0.shape() == x.shape() && dy1.shape() == x.shape());
  CHECK(dy0.data_type() == x.data_type() && dy1.data_type() == x.data_type());
  Tensor dx;
  dx.ResetLike(x);
  const size_t n = x.Size();
  dx.device()->Exec(
      [dx, dy0, dy1, x, n](Context *ctx) mutable {
        if (is_half(x))
          HIP_ABI_CHECK(sgh_relu_bwd_add_f16(f16(dy0), f16(dy1), f16(x), f16_out(dx), n, ctx->hip_stream));
        else
          HIP_ABI_CHECK(sgh_relu_bwd_add_f32(f32(dy0), f32(dy1), f32(x), f32_out(dx), n, ctx->hip_stream));
      },
      {dy0.block(), dy1.block(), x.block()}, {dx.block()}, "ReLUBackwardSum");
  return dx;
}

void SgdMomentum(Tensor *param, const Tensor &grad, Tensor *moment, const Tensor &hyper, bool nesterov) {
  CHECK(param != nullptr && moment != nullptr);
  check_on_hip(*param);
  CHECK_EQ(param->data_type(), kFloat32);
  CHECK_EQ(grad.Size(), param->Size());
  CHECK_EQ(moment->Size(), param->Size());
  CHECK_GE(hyper.Size(), 4u);
  Tensor p(*param), v(*moment);
  const size_t n = p.Size();
  p.device()->Exec(
      [p, grad, v, hyper, n, nesterov](Context *ctx) mutable {
        HIP_ABI_CHECK(sgh_sgd_momentum_devhyper_f32(f32_out(p), f32(grad), f32_out(v), n, f32(hyper), nesterov ? 1 : 0,
                                                    ctx->hip_stream));
      },
      {p.block(), grad.block(), v.block(), hyper.block()}, {p.block(), v.block()}, "SgdMomentum");
}

}  // namespace singa

#endif  // USE_HIP
