// The SGD-momentum update of one element: the four tensor ops of SGD.apply
// (python/singa/opt.py:269-310) in their order, each product and sum rounded to fp32 separately
// (no contraction), so that the fused kernels reproduce the unfused fp32 sequence bit for bit.
#ifndef SINGA_AMD_CSRC_SGD_MATH_H_
#define SINGA_AMD_CSRC_SGD_MATH_H_

#include <hip/hip_runtime.h>

#ifndef SGH_NO_CONTRACT
#define SGH_NO_CONTRACT _Pragma("clang fp contract(off)")
#endif

struct SgdHyper {
  float lr, mu, damp, wd;
};

__device__ __forceinline__ void sgd_one(float &p, float g, float &v, const SgdHyper h, int nesterov, bool has_v) {
  SGH_NO_CONTRACT
  const float one_minus_damp = 1.0f - h.damp;
  const float minus_lr = 0.0f - h.lr;
  if (h.wd != 0.f) {
    float t = h.wd * p;
    g = g + t;
  }
  if (has_v) {
    float vi = v * h.mu;
    float t = one_minus_damp * g;
    vi = vi + t;
    v = vi;
    if (nesterov) {
      float t2 = h.mu * vi;
      g = g + t2;
    } else {
      g = vi;
    }
  }
  float t = minus_lr * g;
  p = p + t;
}

#endif  // SINGA_AMD_CSRC_SGD_MATH_H_
