// Handles and Gpu* operation functions of src/model/operation/{convolution,batchnorm,pooling}.h
// for a SINGA tree built with USE_HIP.  Lands as src/model/operation/operation_hip.h beside the
// three operation headers, which stay as they are: they declare the cuDNN classes only under
// USE_CUDNN, which a HIP build does not define, so the names are free.  src/api/model_operation.i
// includes this header under USE_HIP.
//
// The class and function names are the reference's (src/api/model_operation.i:121-191 exposes
// them to Python, and python/singa/autograd.py picks the Gpu* functions for any device that is
// not the host), so autograd.py runs unchanged.  Handles hold an sgh_conv_geom / sgh_pool_geom
// where the reference's hold cuDNN descriptors.
#ifndef SINGA_MODEL_OPERATION_OPERATION_HIP_H_
#define SINGA_MODEL_OPERATION_OPERATION_HIP_H_

#include "singa/singa_config.h"
#ifdef USE_HIP

#include <string>
#include <vector>

#include "./batchnorm.h"
#include "./convolution.h"
#include "./pooling.h"
#include "singa/core/tensor.h"
#include "singa_hip.h"

namespace singa {

// ---- convolution (src/model/operation/convolution.h:105-141) -------------------------------
class CudnnConvHandle : public ConvHandle {
 public:
  CudnnConvHandle(const Tensor &input, const std::vector<size_t> &kernel_size, const std::vector<size_t> &stride,
                  const std::vector<size_t> &padding, const size_t in_channels, const size_t out_channels,
                  const bool bias, const size_t groups = 1, const size_t workspace_byte_limit = 1024 * 1024 * 1024,
                  const std::string &prefer = "fastest");

  // (the library keeps a note of prepared weights inside the geometry: entry points take it non-const)
  mutable sgh_conv_geom geom;
  DataType dtype;              // a handle built from a half input runs every pass on half tensors
  size_t workspace_count;      // in elements of 4 bytes
  Tensor workspace;
  size_t channels_per_filter;
};

Tensor GpuConvForward(const Tensor &x, const Tensor &W, const Tensor &b, const CudnnConvHandle &cch);
Tensor GpuConvBackwardx(const Tensor &dy, const Tensor &W, const Tensor &x, const CudnnConvHandle &cch);
Tensor GpuConvBackwardW(const Tensor &dy, const Tensor &x, const Tensor &W, const CudnnConvHandle &cch);
Tensor GpuConvBackwardb(const Tensor &dy, const Tensor &b, const CudnnConvHandle &cch);

// ---- batch normalisation (src/model/operation/batchnorm.h:92-115) --------------------------
class CudnnBatchNormHandle : public BatchNormHandle {
 public:
  CudnnBatchNormHandle(const float momentum, const Tensor &input);
  Tensor workspace;            // per-channel partial sums of both passes
};

const std::vector<Tensor> GpuBatchNormForwardTraining(const CudnnBatchNormHandle &cbnh, const Tensor &x,
                                                      const Tensor &bnScale, const Tensor &bnBias,
                                                      Tensor &running_mean, Tensor &running_var);
Tensor GpuBatchNormForwardInference(const CudnnBatchNormHandle &cbnh, const Tensor &x, const Tensor &bnScale,
                                    const Tensor &bnBias, const Tensor &running_mean, const Tensor &running_var);
const std::vector<Tensor> GpuBatchNormBackward(const CudnnBatchNormHandle &cbnh, const Tensor &dy, const Tensor &x,
                                               const Tensor &bnScale, const Tensor &mean, const Tensor &var);

// ---- pooling (src/model/operation/pooling.h:80-96) -----------------------------------------
class CudnnPoolingHandle : public PoolingHandle {
 public:
  CudnnPoolingHandle(const Tensor &input, const std::vector<int> &kernel_size, const std::vector<int> &stride,
                     const std::vector<int> &padding, const bool is_max = true);
  sgh_pool_geom geom;
};

Tensor GpuPoolingForward(const CudnnPoolingHandle &cph, const Tensor &x);
Tensor GpuPoolingBackward(const CudnnPoolingHandle &cph, const Tensor &dy, const Tensor &x, const Tensor &y);

// ---- cross-op fusions the tape of a residual network permits (no counterpart in the
// reference; each returns the bits of the separate calls it replaces) -------------------------
/// ReLU.backward then _BatchNorm2d.backward of conv -> BatchNorm -> ReLU in one pass: `dy` is the
/// gradient behind the ReLU, the BatchNorm output is recomputed from x.  {dx, dscale, dbias}.
const std::vector<Tensor> GpuBatchNormReLUBackward(const CudnnBatchNormHandle &cbnh, const Tensor &dy, const Tensor &x,
                                                   const Tensor &bnScale, const Tensor &bnBias, const Tensor &mean,
                                                   const Tensor &var);
/// `*dx_sum += GpuConvBackwardx(dy, W, x, cch)` (the gradient fan-in of python/singa/autograd.py:204)
/// inside the data gradient's store where the kernel supports it, else the two separate steps.
void GpuConvBackwardxAccumulate(const Tensor &dy, const Tensor &W, const Tensor &x, const CudnnConvHandle &cch,
                                Tensor *dx_sum);
/// dx = x > 0 ? dy0 + dy1 : 0: `dy0 += dy1` followed by ReLU.backward without storing the sum.
Tensor ReLUBackwardSum(const Tensor &dy0, const Tensor &dy1, const Tensor &x);
/// {relu(BatchNorm(x)), mean, var} and {relu(BatchNorm(x) + z), mean, var}
const std::vector<Tensor> GpuBatchNormReLUForwardTraining(const CudnnBatchNormHandle &cbnh, const Tensor &x,
                                                          const Tensor &bnScale, const Tensor &bnBias,
                                                          Tensor &running_mean, Tensor &running_var);
const std::vector<Tensor> GpuBatchNormAddReLUForwardTraining(const CudnnBatchNormHandle &cbnh, const Tensor &x,
                                                             const Tensor &z, const Tensor &bnScale,
                                                             const Tensor &bnBias, Tensor &running_mean,
                                                             Tensor &running_var);
/// opt.SGD.apply (python/singa/opt.py:269-310) as one kernel; lr, momentum, dampening and weight
/// decay in `hyper`, four consecutive floats on the device.
void SgdMomentum(Tensor *param, const Tensor &grad, Tensor *moment, const Tensor &hyper, bool nesterov);

}  // namespace singa

#endif  // USE_HIP
#endif  // SINGA_MODEL_OPERATION_OPERATION_HIP_H_
