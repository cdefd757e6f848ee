// Shared host/device helpers for the gfx950 kernels of the SINGA backward engine.
#ifndef SINGA_AMD_CSRC_COMMON_H_
#define SINGA_AMD_CSRC_COMMON_H_

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stddef.h>
#include <stdint.h>

#include "singa_hip.h"

#define SGH_WAVE 64

// Host-side: turn a hipError_t into the ABI's positive error code and leave the function.
#define SGH_HIP_TRY(expr)                      \
  do {                                         \
    hipError_t sgh_e_ = (expr);                \
    if (sgh_e_ != hipSuccess) return (int)sgh_e_; \
  } while (0)

// After a kernel launch: report launch-configuration errors without synchronising.
#define SGH_LAUNCH_CHECK()                     \
  do {                                         \
    hipError_t sgh_e_ = hipGetLastError();     \
    if (sgh_e_ != hipSuccess) return (int)sgh_e_; \
  } while (0)

static inline hipStream_t sgh_stream_of(void *s) { return reinterpret_cast<hipStream_t>(s); }

static inline bool sgh_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The library's environment switches (A/B measurements; none is needed in normal use), read ONCE,
// when the first entry point asks: changing the environment later has no effect, so a geometry's
// workspace size and kernel choice cannot change between two calls.
struct sgh_env_switches {
  bool dgrad3x3_off, wgrad3x3_off, dgrad_fewc_off, wgrad_fewc_off, dgrad_pointwise_off, conv16_off, bn_onchip_off, pw_dgrad_off, pw_wgrad_off, dgrad_fewc16_off, slab16_off, bn_ragged_off, fwd_fewc_off, bn_fwd_onchip_off;
  int dgrad_tile, wgrad_tile, pw_tile;   // -1: chosen from the geometry
  int dgrad3x3_bm;              // 0: chosen from the geometry, else 64 or 128
  bool conv_xcd_off;            // tiles dealt to workgroups in launch order instead of per XCD
};
const sgh_env_switches &sgh_env();

// Number of compute units of the current device (cached per process; one GPU per process).
int sgh_num_cus();

// True when `s` is the auxiliary stream of an open device (sgh_device_aux_stream): work launched there runs
// beside the main stream's kernels and shares the chip with them.
bool sgh_stream_is_aux(hipStream_t s);

// Looks up, for the current device, the address of the library-owned partial-sum buffer of
// sgh_bn_bwd_noalloc_f32 (batchnorm.hip).  sgh_device_open calls it so that the entry point's first
// call on a device finds the address ready; the entry point repeats the lookup if it was not.
int sgh_bn_noalloc_setup();
// batchnorm.hip: reads and clears the count of workgroups that gave up in a one-pass kernel's exchange (current
// device, idle streams); and the note that such a kernel may have run without its launch being seen (a graph replay)
int sgh_bn_take_exchange_failures(int *count);
void sgh_bn_mark_exchange_ran();

// Weight epoch: a host-side counter that every entry point which may change a weight tensor advances
// (optimizer updates, Axpy, fills, casts, copies to the device, sgh_conv_weights_changed).  The note that
// sgh_conv_dgrad_prepare_multi leaves in a geometry is honoured only within the epoch it was written in.
unsigned long long sgh_weights_epoch();
void sgh_weights_epoch_bump();
// a weight tensor whose re-laid copy waits in a workspace / an elementwise entry point is about to write `bytes`
// at `out`: advances the epoch if that is inside such a weight tensor
void sgh_prepared_weights_add(const void *W, size_t bytes);
void sgh_note_write(const void *out, size_t bytes);
// True when the note in `g` covers a data gradient of storage type `dtype` (0 fp32, 1 binary16, 2 bfloat16)
// reading weights `W` with workspace `workspace` now.
bool sgh_prelaid_valid(const sgh_conv_geom *g, int dtype, const void *W, const void *workspace);
void sgh_prelaid_clear(sgh_conv_geom *g);
// Removes the note if [workspace, workspace + ws_bytes) overlaps the prepared workspace (a pass that writes there).
void sgh_prelaid_clear_if_overlap(sgh_conv_geom *g, const void *workspace, size_t ws_bytes);

// Kernel-level profiling hooks (no-ops unless sgh_prof_enable(1) was called).
bool sgh_prof_on();
void sgh_prof_start(const char *tag, double work, hipStream_t s);
void sgh_prof_stop(hipStream_t s);
// Record for the enclosing scope: `tag` is "class" or "class/kernel", `work` the algorithmic FLOPs or bytes.
struct sgh_prof_scope {
  hipStream_t s;
  bool on;
  sgh_prof_scope(const char *tag, double work, hipStream_t s_) : s(s_), on(sgh_prof_on()) {
    if (on) sgh_prof_start(tag, work, s);
  }
  ~sgh_prof_scope() {
    if (on) sgh_prof_stop(s);
  }
  sgh_prof_scope(const sgh_prof_scope &) = delete;
  sgh_prof_scope &operator=(const sgh_prof_scope &) = delete;
};

// Record for a scope that encloses ONE kernel launch made through SGH_LAUNCH_TIMED: the record's two events
// are handed to that dispatch (hipExtLaunchKernelGGL), so they carry the kernel's own start and end rather
// than two markers queued around it (which add a few microseconds to a short kernel).  A path with more
// than one launch calls span() first and is then timed by markers like sgh_prof_scope; a scope that
// launched nothing leaves a zero-length record.
void sgh_prof_kernel_begin(const char *tag, double work);
bool sgh_prof_kernel_take(hipEvent_t *start, hipEvent_t *stop);   // true once, for the launch after _begin
void sgh_prof_kernel_span(hipStream_t s);
void sgh_prof_kernel_end(hipStream_t s);
struct sgh_prof_kernel_scope {
  hipStream_t s;
  bool on;
  sgh_prof_kernel_scope(const char *tag, double work, hipStream_t s_) : s(s_), on(sgh_prof_on()) {
    if (on) sgh_prof_kernel_begin(tag, work);
  }
  void span() {
    if (on) sgh_prof_kernel_span(s);
  }
  ~sgh_prof_kernel_scope() {
    if (on) sgh_prof_kernel_end(s);
  }
  sgh_prof_kernel_scope(const sgh_prof_kernel_scope &) = delete;
  sgh_prof_kernel_scope &operator=(const sgh_prof_kernel_scope &) = delete;
};
#define SGH_LAUNCH_TIMED(kern, grid, block, lds, stream, ...)                                                    \
  do {                                                                                                           \
    hipEvent_t sgh_ev_a_, sgh_ev_b_;                                                                             \
    if (sgh_prof_on() && sgh_prof_kernel_take(&sgh_ev_a_, &sgh_ev_b_))                                           \
      hipExtLaunchKernelGGL(kern, grid, block, lds, stream, sgh_ev_a_, sgh_ev_b_, 0, __VA_ARGS__);               \
    else                                                                                                         \
      hipLaunchKernelGGL(kern, grid, block, lds, stream, __VA_ARGS__);                                           \
  } while (0)

// 3x3 (stride 1 or 2) weight gradient with a shared LDS input tile (wgrad3x3.hip).  *_run returns
// SGH_EUNSUPPORTED for geometries it does not cover; *_workspace_bytes is 0 for those.
size_t sgh_wgrad3x3_workspace_bytes(const sgh_conv_geom *g);
int sgh_wgrad3x3_run(const sgh_conv_geom *g, const float *dy, const float *x, float *dW, void *workspace,
                     size_t ws_bytes, hipStream_t s);

// Weight gradient for few input channels and a large filter (C*R*S in 65..160: the 7x7 stem),
// wgrad_fewc.hip.  Same conventions as the 3x3 kernel above.
size_t sgh_wgrad_fewc_workspace_bytes(const sgh_conv_geom *g);
int sgh_wgrad_fewc_run(const sgh_conv_geom *g, const float *dy, const float *x, float *dW, void *workspace,
                       size_t ws_bytes, hipStream_t s);

// 3x3 stride-1 pad-1 data gradient with a shared LDS gradient tile (dgrad3x3.hip).
// `wt` = weights re-laid as [tap][KP][C], KP = K rounded up to 16.
bool sgh_dgrad3x3_supported(const sgh_conv_geom *g);
size_t sgh_dgrad3x3_partial_bytes(const sgh_conv_geom *g);  // scratch for split-reduction partial images
// `tag` names the profiling record; `bias` (may be NULL) is added per output channel -- the forward
// convolution runs through this kernel as the data gradient of the channel-swapped problem.
// `accumulate`: dx += result (the sum in the fixed order result-then-add of the separate "+=").
int sgh_dgrad3x3_run(const sgh_conv_geom *g, const float *dy, const float *wt, int KP, float *dx, float *partials,
                     hipStream_t s, const char *tag, const float *bias, bool accumulate);

// Stride-2 data gradient for at most four input channels and a large filter (the 7x7 stem),
// dgrad_fewc.hip: direct 16-row MFMA kernel, W in its native [K][C][R][S] layout.
bool sgh_dgrad_fewc_supported(const sgh_conv_geom *g);
size_t sgh_dgrad_fewc_workspace_bytes(const sgh_conv_geom *g);
int sgh_dgrad_fewc_run(const sgh_conv_geom *g, const float *dy, const float *W, float *dx, void *workspace,
                       size_t ws_bytes, hipStream_t s);
// the same kernel reading a 16-bit dy and writing a 16-bit dx (fp32 weights, slab and arithmetic)
int sgh_dgrad_fewc_run16(const sgh_conv_geom *g, const uint16_t *dy, const float *W, uint16_t *dx, void *workspace,
                         size_t ws_bytes, bool bf16, hipStream_t s);

// Data gradient of 1x1 convolutions without padding, fed from global memory without LDS (pointwise.hip):
// K a multiple of 32, at least 32 input channels, equal strides.
size_t sgh_pw_wgrad_workspace_bytes(const sgh_conv_geom *g);   // 0: not a layer of the pointwise weight-gradient kernel
int sgh_pw_wgrad_run(const sgh_conv_geom *g, const float *dy, const float *x, float *dW, void *workspace, size_t ws_bytes,
                     hipStream_t s);
bool sgh_pw_dgrad_supported(const sgh_conv_geom *g);
int sgh_pw_dgrad_run(const sgh_conv_geom *g, const float *dy, const float *W, float *dx, hipStream_t s);

// Convolution gradients on 16-bit tensors with the 16-bit matrix instructions (conv16.hip).
// *_workspace_bytes is 0 and the run functions return SGH_EUNSUPPORTED for geometries they do not
// cover (strides above 2, K not a multiple of 8 for the data gradient, tensors of 2^31 elements).
size_t sgh_conv16_workspace_bytes(const sgh_conv_geom *g, int which);
int sgh_conv16_wgrad(const sgh_conv_geom *g, const uint16_t *dy, const uint16_t *x, uint16_t *dW, void *workspace,
                     size_t ws_bytes, bool bf16, hipStream_t s);
int sgh_conv16_dgrad(const sgh_conv_geom *g, const uint16_t *dy, const uint16_t *W, uint16_t *dx, void *workspace,
                     size_t ws_bytes, bool bf16, hipStream_t s, bool prelaid);
// Data-gradient weight re-layout of conv16.hip as a batch item: false when the geometry is not covered;
// otherwise the destination layout [tap][CP][KP] (sgh_conv16_dgrad skips its re-layout when told that the
// workspace already holds it).
bool sgh_conv16_dgrad_relayout_dims(const sgh_conv_geom *g, int *CP, int *KP);
// The stem's forward convolution in fp32 (7 x 7, stride 2, padding 3, up to 3 input channels, 64 filters):
// fwd_fewc.hip.  SGH_EUNSUPPORTED for every other geometry.
bool sgh_fwd_fewc_supported(const sgh_conv_geom *g);
size_t sgh_fwd_fewc_workspace_bytes(const sgh_conv_geom *g);
int sgh_fwd_fewc_run(const sgh_conv_geom *g, const float *x, const float *W, const float *bias, float *y, void *workspace,
                     size_t ws_bytes, hipStream_t s);
// The stem's forward convolution on 16-bit tensors (7 x 7, stride 2, padding 3, up to 3 input channels, 64 filters):
// fwd_fewc16.hip.  SGH_EUNSUPPORTED for every other geometry.
bool sgh_fwd_fewc16_supported(const sgh_conv_geom *g);
size_t sgh_fwd_fewc16_workspace_bytes(const sgh_conv_geom *g);
int sgh_fwd_fewc16_run(const sgh_conv_geom *g, const uint16_t *x, const uint16_t *W, const uint16_t *bias, uint16_t *y,
                       void *workspace, size_t ws_bytes, bool bf16, hipStream_t s);
int sgh_conv16_fwd(const sgh_conv_geom *g, const uint16_t *x, const uint16_t *W, const uint16_t *bias, uint16_t *y,
                   void *workspace, size_t ws_bytes, bool bf16, hipStream_t s);

// Sum across the 64 lanes of a wavefront; every lane gets the total.
__device__ __forceinline__ float sgh_wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

__device__ __forceinline__ float sgh_wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Block-wide sum for blocks of up to 1024 threads; result valid in every thread.
// `smem` must hold at least 16 floats.
__device__ __forceinline__ float sgh_block_sum(float v, float *smem) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = sgh_wave_sum(v);
  __syncthreads();
  if (lane == 0) smem[wid] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += smem[i];
  return t;
}

#endif  // SINGA_AMD_CSRC_COMMON_H_
