/*
 * singa_hip.h — C ABI of the MI355X (gfx950) backward-pass + SGD-update engine for Apache SINGA.
 *
 * Every entry point is what a HIP `Device` / `tensor_math` specialisation / operation function in
 * a SINGA tree would bind for the backward path.  Conventions:
 *   - plain pointers and sizes only; all data pointers are DEVICE pointers unless named host_*;
 *   - tensors are dense, row-major / NCHW, fp32 unless the suffix says otherwise;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); work is only enqueued,
 *     never synchronised, except where stated;
 *   - the return value is 0 on success, a positive hipError_t value when the HIP runtime failed,
 *     or a negative SGH_E* code when the arguments were rejected on the host.  Nothing throws or
 *     aborts: SINGA's glue wraps each call in CHECK_EQ(rc, 0) to keep its own abort-on-error
 *     convention (reference: src/utils/logging.cc:105-110, include/singa/utils/cuda_utils.h:96-117);
 *   - the library allocates device memory only inside sgh_malloc (the pool); kernels that need
 *     scratch take an explicit workspace whose size sgh_*_workspace_bytes reports.
 *
 * Reference paths below are relative to the apache/singa source tree.
 */
#ifndef SINGA_HIP_H_
#define SINGA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SGH_API __attribute__((visibility("default")))

/* ---- error codes (negative: rejected on the host before any launch) */
#define SGH_OK 0
#define SGH_EINVAL (-1)     /* bad argument (null pointer, negative size, bad geometry) */
#define SGH_EWORKSPACE (-2) /* workspace missing or too small */
#define SGH_EUNSUPPORTED (-3)
#define SGH_ELABEL (-4)     /* a class label was out of range (checked variant only) */
#define SGH_ENOMEM (-5)
#define SGH_ELIMIT (-6)     /* size beyond the fixed scratch of a non-allocating entry point */
#define SGH_EEXCHANGE (-7)  /* a one-pass BatchNorm kernel's workgroups gave up waiting for each other (see
                               sgh_bn_exchange_failures); returned by sgh_device_sync */

/* Human-readable text for a return code (static storage). */
SGH_API const char *sgh_error_string(int rc);
/* Library version and the GPU architecture the code objects were built for ("gfx950"). */
SGH_API const char *sgh_version(void);
SGH_API const char *sgh_arch(void);

/* =====================================================================================
 * Device runtime.  Replaces what CudaGPU provides to SINGA:
 *   include/singa/core/device.h:57-174 (Device), src/core/device/cuda_gpu.cc:56-209
 *   (Setup, DoExec's stream, CopyToFrom, Malloc/Free, Sync, TimeProfilingDoExec) and the
 *   DeviceMemPool of include/singa/core/memory.h:37-54 / src/core/memory/memory.cc.
 * One sgh_device owns one HIP stream (default priority) and one caching memory pool on
 * hipMalloc.  All pool blocks are recycled in submission order on that single stream, which
 * is the invariant SINGA's Graph relies on when it frees blocks right after enqueueing their
 * last consumer (src/core/scheduler/scheduler.cc:349-354).
 * ===================================================================================== */
typedef struct sgh_device sgh_device;

SGH_API int sgh_device_count(int *count);
/* Platform::CreateCudaGPUsOn analogue (src/core/device/platform.cc:137-160). */
SGH_API int sgh_device_open(int gpu_id, sgh_device **out);
SGH_API int sgh_device_close(sgh_device *dev);
/* The stream behind Device::Exec for this device (hipStream_t as void*). */
SGH_API void *sgh_device_stream(sgh_device *dev);
/* A second compute stream of the device (default priority, created on first use; NULL on failure),
 * for work that is independent of what the main stream runs next -- a layer's weight gradient
 * beside its data gradient.  No counterpart in the reference (CudaGPU has one stream).
 *   sgh_device_fork   work enqueued on the auxiliary stream after this call starts once everything
 *                     enqueued on the main stream so far has finished; returns the stream.
 *   sgh_device_join   work enqueued on the main stream after this call starts once everything
 *                     enqueued on the auxiliary stream so far has finished.
 *   sgh_block_used_on tells the pool that work on `stream` reads or writes the pool block `ptr`
 *                     (a pointer sgh_malloc returned).  The pool recycles freed blocks in the
 *                     submission order of the MAIN stream; a block marked as used on the auxiliary
 *                     stream may be freed at any time (SINGA's Graph frees a block right after it
 *                     enqueued the last consumer, src/core/scheduler/scheduler.cc:349-354) and is
 *                     handed out again only after the next sgh_device_join / sgh_device_sync.
 *                     A no-op for the main stream; SGH_EINVAL for a foreign stream or pointer.
 * Memory that did not come from sgh_malloc is the caller's to keep alive until the join. */
SGH_API void *sgh_device_aux_stream(sgh_device *dev);
SGH_API int sgh_device_fork(sgh_device *dev, void **aux_stream);
SGH_API int sgh_device_join(sgh_device *dev);
SGH_API int sgh_block_used_on(sgh_device *dev, void *ptr, void *stream);
/* Device::Sync (src/core/device/cuda_gpu.cc:206-209): blocks until the device's streams are idle.
 * Returns SGH_EEXCHANGE (once) if a one-pass BatchNorm kernel that ran since the last look could not
 * complete its exchange -- the outputs of that call are NaN; see sgh_bn_exchange_failures. */
SGH_API int sgh_device_sync(sgh_device *dev);

/* DeviceMemPool::Malloc / Free (include/singa/core/memory.h:41-45).  Size-bucketed cache:
 * a freed block goes back to its bucket and is handed out again without touching the driver.
 * Like CudaGPU::Malloc the memory is NOT zero-filled (src/core/device/cuda_gpu.cc:187-197). */
SGH_API int sgh_malloc(sgh_device *dev, void **ptr, size_t bytes);
SGH_API int sgh_free(sgh_device *dev, void *ptr);
/* DeviceMemPool::GetMemUsage: bytes handed out, bytes cached in the pool, driver calls made. */
SGH_API int sgh_pool_stats(sgh_device *dev, size_t *in_use, size_t *cached, size_t *driver_allocs);

/* Record-and-replay of everything enqueued on the device's stream, the counterpart of the
 * reference's graph mode (Device::EnableGraph / RunGraph / ResetGraph, include/singa/core/device.h
 * :69-98, src/core/device/device.cc:55-82: operations are buffered instead of executed while the
 * graph is enabled, then replayed every iteration).  Between sgh_graph_begin and sgh_graph_end the
 * entry points record into a HIP graph instead of running; sgh_graph_launch replays the recording
 * on the same stream.  While recording, nothing executes: sgh_device_sync and device-to-host copies
 * return SGH_EUNSUPPORTED, host-to-device copies are performed immediately (outside the graph), and
 * blocks freed to the pool stay reserved for the graph until sgh_graph_destroy.  The recording
 * holds raw pointers: tensors that exist before sgh_graph_begin and are used inside must outlive
 * the graph. */
typedef struct sgh_graph sgh_graph;
SGH_API int sgh_graph_begin(sgh_device *dev);
SGH_API int sgh_graph_end(sgh_device *dev, sgh_graph **out);
SGH_API int sgh_graph_launch(sgh_graph *g);
SGH_API int sgh_graph_destroy(sgh_graph *g);
/* Return every cached block to the driver. */
SGH_API int sgh_pool_trim(sgh_device *dev);

/* Device::CopyToFrom (src/core/device/cuda_gpu.cc:171-175).  kind: 0 H2H, 1 H2D, 2 D2H, 3 D2D
 * (= core.proto CopyDirection, src/proto/core.proto:43-48).  D2H and H2D block until the
 * copy has completed so the host may touch the buffer when the call returns. */
SGH_API int sgh_memcpy(sgh_device *dev, void *dst, const void *src, size_t bytes, int kind);
/* Host-to-device copy that does not wait (no counterpart in the reference, whose CopyDataFromHostPtr
 * blocks): `src` is copied to pinned staging memory before the call returns, so the caller may reuse
 * it at once; the copy to `dst` is enqueued on the device's stream in order with the kernels there.
 * For the small tables a step uploads (pointer tables of the multi-tensor update) -- a blocking copy
 * would drain the stream once per step.  Up to 64 KiB; larger copies and copies while the stream is
 * being recorded behave like sgh_memcpy(kind 1). */
SGH_API int sgh_upload_async(sgh_device *dev, void *dst, const void *src, size_t bytes);
/* Tensor::SetValue (src/core/tensor/tensor.cc:849-865, Set<DType, Lang>): every element = value.
 * The 16-bit variants round `value` once to the storage type (nearest, ties to even) and write
 * 2-byte elements; n counts elements. */
SGH_API int sgh_memset_f32(float *dst, float value, size_t n, void *stream);
SGH_API int sgh_memset_f16(uint16_t *dst, float value, size_t n, void *stream);
SGH_API int sgh_memset_bf16(uint16_t *dst, float value, size_t n, void *stream);

/* Per-op timing for Graph profiling (TimeProfilingDoExec / EvaluateTimeElapsed,
 * src/core/device/cuda_gpu.cc:117-169): event pairs on the device stream. */
typedef struct sgh_event sgh_event;
SGH_API int sgh_event_create(sgh_event **ev);
SGH_API int sgh_event_destroy(sgh_event *ev);
SGH_API int sgh_event_record(sgh_event *ev, void *stream);
/* Work enqueued on `stream` after this call starts only when what `ev` recorded has finished. */
SGH_API int sgh_stream_wait_event(void *stream, sgh_event *ev);
/* Blocks on `stop`, then returns stop - start in milliseconds. */
SGH_API int sgh_event_elapsed_ms(sgh_event *start, sgh_event *stop, float *ms);

/* Kernel-level profiling: the per-node timing of SINGA's Graph (Device::SetVerbosity,
 * TimeProfilingDoExec, Graph::PrintTimeProfiling: src/core/scheduler/scheduler.cc:240-295) at
 * kernel granularity.  While enabled, every GEMM / implicit-GEMM launch of this library is
 * timed by two events on its own stream and tagged with its algorithmic FLOP count:
 * "conv_wgrad" / "conv_dgrad" / "conv_fwd" cover the MFMA kernel alone, "conv_*_op" the whole
 * entry point (weight re-layout, split-K reduction and column-gather kernels included), "gemm"
 * a dense GEMM; the bandwidth-bound entry points ("bn_bwd", "bn_relu_bwd", "relu_bwd", "add",
 * "pool_bwd", "sgd" ...) are tagged with their algorithmic bytes.  A record of a single kernel
 * hands its events to the dispatch itself (hipExtLaunchKernelGGL), so they carry the kernel's
 * own start and end; a record over several kernels is a pair of markers around them, which adds
 * a few microseconds of queue time.  Records nest.  No record is taken while a device records a
 * graph (sgh_graph_begin .. sgh_graph_end): events inside a recording have no times.  The records
 * belong to one host thread at a time.  sgh_prof_enable(1) clears old records.
 * sgh_prof_get waits for record i to finish and returns its tag, duration and work. */
SGH_API int sgh_prof_enable(int on);
/* Drops the records taken so far and destroys their events (sgh_prof_enable(1) does the same before it starts;
 * this is for a caller that has read what it wanted and does not profile again).  Profiling must be off. */
SGH_API int sgh_prof_clear(void);
SGH_API int sgh_prof_count(int *n);
SGH_API int sgh_prof_get(int i, char *tag, size_t tag_len, float *ms, double *work);

/* =====================================================================================
 * tensor_math backward ops (HIP specialisations of src/core/tensor/tensor_math.h)
 * ===================================================================================== */

/* ReLUBackward<float, Lang>: tensor_math.h:175-179; CPU tensor_math_cpp.h:446-451;
 * CUDA math_kernel.cu:253-261.  dx[i] = x[i] > 0 ? dy[i] : 0 (x = the ReLU input). */
SGH_API int sgh_relu_bwd_f32(const float *dy, const float *x, float *dx, size_t n, void *stream);
/* ReLU<float, Lang>: tensor_math_cpp.h:585-589 (needed to produce the backward's inputs); on half
 * tensors ReLU<half, Lang>, src/core/tensor/math_kernel.cu:242-251 (16-bit variants: y = x > 0 ? x : 0
 * on the stored values, exact). */
SGH_API int sgh_relu_fwd_f32(const float *x, float *y, size_t n, void *stream);
SGH_API int sgh_relu_fwd_f16(const uint16_t *x, uint16_t *y, size_t n, void *stream);
SGH_API int sgh_relu_fwd_bf16(const uint16_t *x, uint16_t *y, size_t n, void *stream);

/* SoftmaxCrossEntropyBwd<float, Lang>: tensor_math.h:475-480; CPU tensor_math_cpp.h:1090-1119;
 * CUDA math_kernel.cu:564-611; host wrapper src/core/tensor/tensor.cc:1717-1758.
 * grad = (p - onehot(t)) * scale  (int_target = 1, t is int32 [batch]) or
 * grad = (p - t / rowsum(t)) * scale (int_target = 0, t is int32 [batch, dim]).
 * grad may alias p (the reference works in place on a clone of p).  scale = 1 reproduces the
 * reference op; scale = 1/batch additionally fuses the "dx /= N" that follows it in
 * python/singa/autograd.py:1319-1322.  Labels are trusted like on the reference GPU path;
 * a label outside [0, dim) leaves its row as p * scale and raises the device-side error
 * flag readable with sgh_softmax_ce_label_errors (the CPU reference aborts on negatives). */
SGH_API int sgh_softmax_ce_bwd_f32(const float *p, const int32_t *t, float *grad, size_t batch,
                                   size_t dim, int int_target, float scale, void *stream);
/* SoftmaxCrossEntropyBwd<half, Lang> (src/core/tensor/math_kernel.cu:588-611; a layer of a half
 * model casts its inputs to the layer's type, python/singa/layer.py:171-185, so the loss of a pure
 * half model arrives here).  p and grad are 16-bit, t stays int32; the subtraction (and the row sum
 * of an array target, the division, the scale) are fp32 on the widened values, one rounding at the
 * store.  Label handling and the error flag are those of the fp32 entry point. */
SGH_API int sgh_softmax_ce_bwd_f16(const uint16_t *p, const int32_t *t, uint16_t *grad, size_t batch,
                                   size_t dim, int int_target, float scale, void *stream);
SGH_API int sgh_softmax_ce_bwd_bf16(const uint16_t *p, const int32_t *t, uint16_t *grad, size_t batch,
                                    size_t dim, int int_target, float scale, void *stream);
/* Number of out-of-range labels seen since the last call (synchronises the stream). */
SGH_API int sgh_softmax_ce_label_errors(void *stream, int *count);
/* SoftMax<float, Lang> (rows) and ComputeCrossEntropy<float, Lang>: forward helpers,
 * tensor_math_cpp.h:361-379, :1058-1088; CUDA tensor_math_cuda.h:1274-1339. */
SGH_API int sgh_softmax_fwd_f32(const float *x, float *p, size_t batch, size_t dim, void *stream);
SGH_API int sgh_cross_entropy_fwd_f32(const float *p, const int32_t *t, float *loss, size_t batch,
                                      size_t dim, int int_target, void *stream);

/* Transform<float, Lang> (src/core/tensor/tensor_math_cpp.h:685-689, CUDA tensor_math_cuda.h:284-300):
 * the dense row-major copy of a strided view -- transposed, sliced or broadcast (stride 0, as
 * Tensor::Broadcast makes them, src/core/tensor/tensor.cc:481-503).  Element i of `out`, in
 * row-major order of `shape`, is in[sum_d index_d * strides[d]] (strides in elements, innermost
 * dimension last, at most SGH_MAX_DIMS dimensions) -- the walk of next_offset,
 * tensor_math_cpp.h:126-138.  What the reference's CUDA EltwiseMult / Add do first with an operand
 * that is not dense (tensor_math_cuda.h:300-362). */
#define SGH_MAX_DIMS 8
SGH_API int sgh_transform_f32(const float *in, float *out, int ndim, const size_t *shape,
                              const int64_t *strides, void *stream);
/* RowMax<float, Lang> for a dense nrow x ncol matrix.  The reference's two backends differ on rows
 * without a positive element: its accelerator kernel seeds the maximum with the row's first element
 * and returns the true maximum (src/core/tensor/math_kernel.cu:488-499, called from
 * tensor_math_cuda.h:1493-1507), its CPU function seeds it with 0 (tensor_math_cpp.h:1122-1140).
 *   sgh_row_max_f32             out[r] = max_c in[r][c]            (the accelerator rule: this
 *                                library replaces that path)
 *   sgh_row_max_zero_seeded_f32 out[r] = max(0, max_c in[r][c])    (the CPU rule, for comparisons
 *                                with the CPU path bit for bit) */
SGH_API int sgh_row_max_f32(const float *in, float *out, size_t nrow, size_t ncol, void *stream);
SGH_API int sgh_row_max_zero_seeded_f32(const float *in, float *out, size_t nrow, size_t ncol, void *stream);
/* Dot<float, Lang> with a Tensor result (tensor_math_cpp.h:839-849, cublasSdot in device pointer
 * mode tensor_math_cuda.h:1084-1092) and Sum<float, Lang> over all elements (tensor_math_cpp.h:
 * 655-663): *out = sum a[i] * b[i] / sum a[i], `out` in device memory.  Summed in an order that
 * depends on n only: run-to-run identical.  workspace: sgh_reduce_workspace_bytes() bytes. */
SGH_API size_t sgh_reduce_workspace_bytes(void);
SGH_API int sgh_dot_f32(const float *a, const float *b, size_t n, float *out, void *workspace,
                        size_t ws_bytes, void *stream);
SGH_API int sgh_sum_all_f32(const float *a, size_t n, float *out, void *workspace, size_t ws_bytes,
                            void *stream);
/* Uniform<float, Lang> / Gaussian<float, Lang> (tensor_math_cpp.h:712-740; cuRAND in
 * tensor_math_cuda.h:950-1000).  The reference draws from the device's generator state
 * (Device::SetRandSeed); here element i of a fill is a pure function of (seed, offset + i): the
 * (offset + i)-th output of splitmix64 seeded with `seed` gives a double in [0, 1), a Gaussian
 * takes two of them (offset + 2i, offset + 2i + 1) through Box-Muller in double precision.  The
 * caller advances `offset` by n (2n) per fill to continue the stream.  The reference's streams
 * (std::mt19937, cuRAND) are not reproduced: no test of the reference depends on their values. */
SGH_API int sgh_uniform_f32(float low, float high, float *out, size_t n, uint64_t seed,
                            uint64_t offset, void *stream);
SGH_API int sgh_gaussian_f32(float mean, float std, float *out, size_t n, uint64_t seed,
                             uint64_t offset, void *stream);

/* Clamp<float, Lang> (src/core/tensor/tensor_math_cpp.h:398-410; autograd.clip): out = min(max(x, low), high).
 * With the two casts above it is the single-GPU part of DistOpt.backward_and_update_half
 * (python/singa/opt.py:867-920): gradients optionally clipped, then sent through half precision. */
SGH_API int sgh_clamp_f32(float low, float high, const float *x, float *out, size_t n, void *stream);

/* Axpy<float, Lang>, scalar and Tensor-alpha overloads: tensor_math.h:393-402;
 * CPU tensor_math_cpp.h:788-823; CUDA tensor_math_cuda.h:1031-1072 (device pointer mode).
 * y += alpha * x. */
SGH_API int sgh_axpy_f32(float alpha, const float *x, float *y, size_t n, void *stream);
SGH_API int sgh_axpy_devalpha_f32(const float *alpha_dev, const float *x, float *y, size_t n,
                                  void *stream);

/* EltwiseMult<float, Lang>: tensor_math.h:162-172; CPU tensor_math_cpp.h:432-444; CUDA
 * tensor_math_cuda.h:300-362.  out = a * b; b_is_scalar = 1 reads b[0] for every element,
 * which is the stride-0 broadcast view of "buf *= mom_value" (python/singa/opt.py:299-300)
 * without materialising it.  out may alias a. */
SGH_API int sgh_eltwise_mult_f32(const float *a, const float *b, int b_is_scalar, float *out,
                                 size_t n, void *stream);
/* Add<float, Lang> (Tensor::operator+=, src/core/tensor/tensor.cc:579-586): gradient fan-in
 * of python/singa/autograd.py:204.  out may alias a or b. */
SGH_API int sgh_add_f32(const float *a, const float *b, float *out, size_t n, void *stream);
/* Add followed by ReLU in one pass: the forward of a residual block's end, relu(out + identity)
 * (examples/cnn/model/resnet.py:74-77, :112-115; python/singa/autograd.py add :1026-1040 then ReLU :421-430).
 * Stores what the two calls store (the sum rounded to the storage type, then the selection); the ReLU's
 * backward may gate on this output instead of the sum: both are positive at the same elements.
 * out may alias a or b. */
SGH_API int sgh_add_relu_f32(const float *a, const float *b, float *out, size_t n, void *stream);
SGH_API int sgh_add_relu_f16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream);
SGH_API int sgh_add_relu_bf16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream);
/* The other elementwise tensor functions the autograd ops of these models call around the
 * backward path (src/core/tensor/tensor_math_cpp.h): Sub :645-650, Div (tensor / tensor) :423-430,
 * Add(tensor, scalar) :383-388, EltwiseMult(tensor, scalar) :432-437.  Div(tensor, scalar) is
 * EltwiseMult by the fp32 reciprocal in the reference (tensor_math.h:149-153): callers pass 1/x to
 * sgh_mult_scalar_f32.  out may alias an input. */
SGH_API int sgh_sub_f32(const float *a, const float *b, float *out, size_t n, void *stream);
SGH_API int sgh_div_f32(const float *a, const float *b, float *out, size_t n, void *stream);
SGH_API int sgh_add_scalar_f32(const float *a, float x, float *out, size_t n, void *stream);
SGH_API int sgh_mult_scalar_f32(const float *a, float x, float *out, size_t n, void *stream);

/* -------------------------------------------------------------------------------------
 * 16-bit storage variants: IEEE binary16 ("f16", the reference's half_float::half / __half
 * tensors) and bfloat16 ("bf16") travel as uint16_t arrays.  Arithmetic is fp32 with one
 * rounding to nearest-even on store, like the reference's half kernels
 * (__half2float / __float2half in src/core/tensor/math_kernel.cu).
 * ------------------------------------------------------------------------------------- */
/* CastCopy<float, half, Lang> / CastCopy<half, float, Lang> (Tensor::AsType):
 * src/core/tensor/tensor_math_cuda.h:193-208, math_kernel.cu float2half / half2float. */
SGH_API int sgh_cast_f32_to_f16(const float *src, uint16_t *dst, size_t n, void *stream);
SGH_API int sgh_cast_f16_to_f32(const uint16_t *src, float *dst, size_t n, void *stream);
SGH_API int sgh_cast_f32_to_bf16(const float *src, uint16_t *dst, size_t n, void *stream);
SGH_API int sgh_cast_bf16_to_f32(const uint16_t *src, float *dst, size_t n, void *stream);
/* CastCopy<float, int, Lang> / CastCopy<int, float, Lang> (tensor_math_cuda.h:177-191,
 * src/core/tensor/math_kernel.cu:280-292: `(int)src[i]` and `(float)src[i]`).  float -> int truncates
 * toward zero; values outside the int32 range saturate to INT32_MIN / INT32_MAX and NaN gives 0 (what
 * the conversion instruction does; C leaves both undefined).  int -> float rounds to nearest even. */
SGH_API int sgh_cast_f32_to_i32(const float *src, int32_t *dst, size_t n, void *stream);
SGH_API int sgh_cast_i32_to_f32(const int32_t *src, float *dst, size_t n, void *stream);
/* ReLUBackward<half, Lang>: tensor_math_cuda.h:665-674, math_kernel.cu:261-271.  Follows the
 * CPU rule dx = x > 0 ? dy : 0 (the CUDA half kernel alone passes the gradient at x == 0). */
SGH_API int sgh_relu_bwd_f16(const uint16_t *dy, const uint16_t *x, uint16_t *dx, size_t n, void *stream);
SGH_API int sgh_relu_bwd_bf16(const uint16_t *dy, const uint16_t *x, uint16_t *dx, size_t n, void *stream);
/* ReLU backward on a gradient that arrives as two summands: dx[i] = x[i] > 0 ? dy0[i] + dy1[i] : 0,
 * the sum in fp32 and one rounding at the store -- bit-identical to the reference's two steps, the
 * gradient fan-in `dy0 += dy1` of a residual connection (python/singa/autograd.py:204) followed by
 * ReLUBackward (tensor_math.h:175-179), without storing the sum.  dx may alias dy0 or dy1. */
SGH_API int sgh_relu_bwd_add_f32(const float *dy0, const float *dy1, const float *x, float *dx, size_t n,
                                 void *stream);
SGH_API int sgh_relu_bwd_add_f16(const uint16_t *dy0, const uint16_t *dy1, const uint16_t *x,
                                 uint16_t *dx, size_t n, void *stream);
SGH_API int sgh_relu_bwd_add_bf16(const uint16_t *dy0, const uint16_t *dy1, const uint16_t *x,
                                  uint16_t *dx, size_t n, void *stream);
/* Add / EltwiseMult<half, Lang>: tensor_math_cuda.h:345-362, math_kernel.cu:111-117, :353-359.
 * out may alias an input. */
SGH_API int sgh_add_f16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream);
SGH_API int sgh_add_bf16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream);
SGH_API int sgh_eltwise_mult_f16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream);
SGH_API int sgh_eltwise_mult_bf16(const uint16_t *a, const uint16_t *b, uint16_t *out, size_t n, void *stream);
/* Axpy<half, Lang> (scalar alpha): tensor_math_cuda.h:1064-1072 (cublasAxpyEx, fp32 compute). */
SGH_API int sgh_axpy_f16(float alpha, const uint16_t *x, uint16_t *y, size_t n, void *stream);
SGH_API int sgh_axpy_bf16(float alpha, const uint16_t *x, uint16_t *y, size_t n, void *stream);

/* Fused SGD-momentum update = the four tensor ops of SGD.apply, python/singa/opt.py:269-310,
 * in one pass:  [g += wd*p];  v = mu*v + (1-damp)*g;  g' = nesterov ? g + mu*v : v;
 * p -= lr*g'.  wd == 0 and mu == 0 skip their terms exactly like the Python `if`s; with
 * mu == 0, v may be NULL.  g is not written.
 * hyper_dev (device variant) points at {lr, mu, damp, wd} as four consecutive device floats,
 * the 1-element device tensors the reference keeps (opt.py:222-259). */
SGH_API int sgh_sgd_momentum_f32(float *p, const float *g, float *v, size_t n, float lr, float mu,
                                 float damp, float wd, int nesterov, void *stream);
SGH_API int sgh_sgd_momentum_devhyper_f32(float *p, const float *g, float *v, size_t n,
                                          const float *hyper_dev, int nesterov, void *stream);
/* The same update for many parameter tensors in ONE launch (the per-parameter loop of
 * Optimizer.call, python/singa/opt.py:107-111).  table_dev is a device array of `count`
 * sgh_sgd_item; max_n is the largest item. */
typedef struct sgh_sgd_item {
  float *p;
  const float *g;
  float *v;
  uint64_t n;
} sgh_sgd_item;
SGH_API int sgh_sgd_momentum_multi_f32(const sgh_sgd_item *table_dev, int count, size_t total_n,
                                       float lr, float mu, float damp, float wd, int nesterov,
                                       void *stream);
/* The same update on 16-bit gradients.
 * sgh_sgd_momentum_f16 / _bf16: p, g, v all 16-bit, as opt.SGD(dtype=float16) keeps them
 *   (python/singa/opt.py:283-284); fp32 arithmetic, p and v rounded once per step (the
 *   reference's four unfused half ops round after each op: parity at the 16-bit tolerance).
 * sgh_sgd_momentum_master_f16 / _bf16: mixed precision -- fp32 master weights and fp32 momentum
 *   are updated from the 16-bit gradient, and p_out receives the master rounded to 16 bits
 *   (the working copy the next forward pass reads).  No counterpart in the reference's opt.py. */
/* sgh_sgd_momentum_multi_mixed: every parameter of a mixed-precision network in one launch (the
 *   loop of Optimizer.call, python/singa/opt.py:107-111, over fp32 parameters and 16-bit parameters
 *   with fp32 master copies alike).  An item with p16 == NULL is an fp32 parameter (g is float);
 *   otherwise p is the fp32 master, g the 16-bit gradient (binary16, or bfloat16 when `bf16` is
 *   set) and p16 the working copy that receives the updated master rounded once.  At most 2048
 *   items.  Per element identical to the single-tensor entry points. */
typedef struct sgh_sgd_mixed_item {
  float *p;
  const void *g;
  float *v;
  uint16_t *p16;
  uint64_t n;
} sgh_sgd_mixed_item;
SGH_API int sgh_sgd_momentum_multi_mixed(const sgh_sgd_mixed_item *table_dev, int count,
                                         size_t total_n, int bf16, float lr, float mu, float damp,
                                         float wd, int nesterov, void *stream);
SGH_API int sgh_sgd_momentum_f16(uint16_t *p, const uint16_t *g, uint16_t *v, size_t n, float lr,
                                 float mu, float damp, float wd, int nesterov, void *stream);
SGH_API int sgh_sgd_momentum_bf16(uint16_t *p, const uint16_t *g, uint16_t *v, size_t n, float lr,
                                  float mu, float damp, float wd, int nesterov, void *stream);
SGH_API int sgh_sgd_momentum_master_f16(float *p_master, const uint16_t *g, float *v,
                                        uint16_t *p_out, size_t n, float lr, float mu, float damp,
                                        float wd, int nesterov, void *stream);
SGH_API int sgh_sgd_momentum_master_bf16(float *p_master, const uint16_t *g, float *v,
                                         uint16_t *p_out, size_t n, float lr, float mu, float damp,
                                         float wd, int nesterov, void *stream);

/* GEMM<float, Lang>: tensor_math.h:444-448; CPU tensor_math_cpp.h:877-899 (cblas_sgemm,
 * row-major).  C[M,N] = alpha * op(A) * op(B) + beta * C; lda/ldb/ldc are row pitches of the
 * stored matrices.  Used by Linear backward: Mult(dy, W^T), Mult(x^T, dy)
 * (python/singa/autograd.py:613-623). */
SGH_API int sgh_gemm_f32(int transA, int transB, int M, int N, int K, float alpha, const float *A,
                         int lda, const float *B, int ldb, float beta, float *C, int ldc,
                         void *stream);
/* GEMM<half, Lang> (cublasHgemm in the reference, src/core/tensor/tensor_math_cuda.h:1163-1187): the
 * Linear layers of a half model.  A, B, C are binary16 (bfloat16); products of the stored values are
 * accumulated in fp32 on the 16-bit matrix instructions (v_mfma_f32_32x32x16), alpha and beta apply in
 * fp32, C is rounded once.  Same argument meaning as sgh_gemm_f32.  Run-to-run identical. */
SGH_API int sgh_gemm_f16(int transA, int transB, int M, int N, int K, float alpha, const uint16_t *A,
                         int lda, const uint16_t *B, int ldb, float beta, uint16_t *C, int ldc,
                         void *stream);
SGH_API int sgh_gemm_bf16(int transA, int transB, int M, int N, int K, float alpha, const uint16_t *A,
                          int lda, const uint16_t *B, int ldb, float beta, uint16_t *C, int ldc,
                          void *stream);
/* SumRows<float, Lang> (Sum(dy, 0), src/core/tensor/tensor.cc:1523-1538): out[j] = sum_i m[i][j].
 * Bias gradient of AddBias.backward (python/singa/autograd.py:696-709). */
SGH_API int sgh_sum_rows_f32(const float *m, float *out, int rows, int cols, void *stream);
/* AddRow (bias add of Linear forward, src/core/tensor/tensor.cc:1294-1316): m[i][j] += v[j]. */
SGH_API int sgh_add_row_f32(const float *v, float *m, int rows, int cols, void *stream);

/* =====================================================================================
 * Operation entry points (the Gpu* functions of src/model/operation/{convolution,batchnorm,pooling}.cc)
 * ===================================================================================== */

/* Geometry of a ConvHandle (src/model/operation/convolution.h:43-90; ctor
 * src/model/operation/convolution.cc:29-66).  P, Q are derived with the reference's integer
 * division; sgh_conv_geom_init fills them and validates the rest. */
typedef struct sgh_conv_geom {
  int N, C, H, W;       /* input  [N, C, H, W]                    */
  int K, R, S;          /* weight [K, C, R, S]                    */
  int stride_h, stride_w, pad_h, pad_w;
  int P, Q;             /* output [N, K, P, Q]                    */
  int groups;           /* 1, or the group count: weight [K, C / groups, R, S] (sgh_conv_geom_init_grouped) */
  /* Owned by the library (sgh_conv_geom_init zeroes them, callers never write them): the note
   * sgh_conv_dgrad_prepare_multi leaves for this layer's next data gradient -- which weight
   * tensor was re-laid, into which workspace, and the library's weight epoch at that moment. */
  int prelaid_dtype;
  const void *prelaid_W;
  const void *prelaid_ws;
  size_t prelaid_ws_bytes;
  unsigned long long prelaid_epoch;
} sgh_conv_geom;
SGH_API int sgh_conv_geom_init(sgh_conv_geom *g, int N, int C, int H, int W, int K, int R, int S,
                               int stride_h, int stride_w, int pad_h, int pad_w);
/* The handle of a grouped convolution (CudnnConvHandle's `groups` argument,
 * src/model/operation/convolution.cc:446-461 and :486-495: cudnnSetConvolutionGroupCount, filter descriptor
 * [K, C / groups, R, S]; python/singa/layer.py:668-718 and the depthwise layer of SeparableConv2d, :780-795).
 * C and K must be multiples of `groups`.  Group i convolves input channels [i C/groups, (i+1) C/groups) with
 * filters [i K/groups, (i+1) K/groups).  Every convolution entry point below takes such a geometry: each group
 * runs as a dense convolution on slices gathered in the workspace (sgh_conv_workspace_bytes[_h] account for
 * them); sgh_conv_dgrad_acc_f32 returns SGH_EUNSUPPORTED and sgh_conv_dgrad_prepare_multi skips it. */
SGH_API int sgh_conv_geom_init_grouped(sgh_conv_geom *g, int N, int C, int H, int W, int K, int R, int S,
                                       int stride_h, int stride_w, int pad_h, int pad_w, int groups);

#define SGH_CONV_FWD 0
#define SGH_CONV_DGRAD 1
#define SGH_CONV_WGRAD 2
/* Scratch bytes the given pass needs for this geometry (CudnnConvHandle::workspace_count,
 * src/model/operation/convolution.cc:560-571). */
SGH_API size_t sgh_conv_workspace_bytes(const sgh_conv_geom *g, int which);

/* GpuConvBackwardx (src/model/operation/convolution.cc:634-656; native algorithm
 * src/model/layer/convolution.cc:178-182 + Col2im :224-248):
 * dx[n,c,h,w] = sum_{k,r,s} dy[n,k,p,q] * W[k,c,r,s], h = p*stride - pad + r. */
SGH_API int sgh_conv_dgrad_f32(sgh_conv_geom *g, const float *dy, const float *W, float *dx,
                               void *workspace, size_t ws_bytes, void *stream);
/* dx += the data gradient: cudnnConvolutionBackwardData's beta = 1 (the reference passes beta = 0,
 * convolution.cc:649-654, and sums gradients that fan in with a separate `+=`,
 * python/singa/autograd.py:204).  Each element is computed exactly as above and then added to the
 * value already in dx, so the result equals the separate call followed by `dx_old += result`.
 * Covered by the shared-tile kernels (3x3, pad 1, stride 1, or stride 2 on even images, C >= 64,
 * K a multiple of 16); SGH_EUNSUPPORTED otherwise, with dx untouched. */
SGH_API int sgh_conv_dgrad_acc_f32(sgh_conv_geom *g, const float *dy, const float *W,
                                   float *dx, void *workspace, size_t ws_bytes, void *stream);
/* 1 if sgh_conv_dgrad_acc_f32 covers this geometry, else 0: a caller that has to schedule the
 * fallback (data gradient + Add) itself asks before it submits anything. */
SGH_API int sgh_conv_dgrad_acc_supported(const sgh_conv_geom *g);
/* The data gradient re-lays the weight tensor in its workspace before the matrix kernel runs:
 * a launch of a few microseconds per layer.  A caller that runs many data gradients while the
 * weights do not change (a backward pass) can have all of them re-laid by ONE launch up front:
 * sgh_conv_dgrad_prepare_multi writes each listed layer's workspace (fp32: dtype 0, binary16: 1,
 * bfloat16: 2) and leaves a note in the layer's geometry, for the layers whose kernel takes such
 * weights.  The layer's next data gradient (sgh_conv_dgrad_*, sgh_conv_dgrad_acc_f32) skips its
 * own re-layout if, and only if, the note still holds: same W pointer, same workspace, and no
 * call since the prepare that may have changed a weight tensor -- every sgh_sgd_momentum_*,
 * sgh_axpy_*, sgh_memset_*, random fill, host-to-device / device-to-device sgh_memcpy,
 * sgh_upload_async and sgh_graph_launch call (a recording may hold an update) advances the
 * library's weight epoch; the elementwise entry points with an output tensor (sgh_add_*,
 * sgh_sub_f32, sgh_div_f32, sgh_eltwise_mult_*, the scalar forms, sgh_clamp_f32, the casts)
 * advance it when their output lies inside a prepared weight tensor (Tensor `*=` / `+=` on a
 * weight); and so does sgh_conv_weights_changed(), which a caller that writes weights by other
 * means (its own kernels) calls.  Otherwise the data gradient re-lays the weights
 * itself, as without a prepare.  A note is used once: the data gradient that reads it, and any
 * forward pass or weight gradient of the same geometry whose workspace overlaps the prepared one,
 * removes it.  The workspaces listed must be private to their layer from the prepare call to the
 * layer's data gradient (a workspace shared between layers cannot hold two layers' weights).
 * Results are bit-identical with and without.  No counterpart in the reference (cuDNN keeps its
 * filter transforms to itself). */
typedef struct sgh_conv_prepare_item {
  sgh_conv_geom *g;
  const void *W;
  void *workspace;
  size_t ws_bytes;
} sgh_conv_prepare_item;
SGH_API int sgh_conv_dgrad_prepare_multi(const sgh_conv_prepare_item *items, int count, int dtype,
                                         void *stream);
SGH_API void sgh_conv_weights_changed(void);
/* GpuConvBackwardW (src/model/operation/convolution.cc:658-681; native algorithm
 * src/model/layer/convolution.cc:166-177 + Im2col :197-222):
 * dW[k,c,r,s] = sum_{n,p,q} dy[n,k,p,q] * x[n,c,p*stride-pad+r,q*stride-pad+s].
 * The split reduction is summed in a fixed order: results are run-to-run identical. */
SGH_API int sgh_conv_wgrad_f32(sgh_conv_geom *g, const float *dy, const float *x, float *dW,
                               void *workspace, size_t ws_bytes, void *stream);
/* GpuConvBackwardW and GpuConvBackwardb of one layer in one call (the reference makes two cuDNN
 * calls, src/model/operation/convolution.cc:658-702, both reading dy).  Where the generic
 * implicit-GEMM kernel runs the weight gradient and its last column tile has a spare column
 * (C*R*S not a multiple of the tile width), db is computed by the same matrix instructions as one
 * more column of the x operand -- a column of ones -- so dy is read once; other geometries run
 * the reduction of sgh_conv_bgrad_f32 behind the weight gradient.  Either way db agrees with
 * sgh_conv_bgrad_f32 to rounding (different summation order).  Workspace as for the weight
 * gradient. */
SGH_API int sgh_conv_wgrad_bias_f32(sgh_conv_geom *g, const float *dy, const float *x, float *dW,
                                    float *db, void *workspace, size_t ws_bytes, void *stream);
/* GpuConvBackwardb (src/model/operation/convolution.cc:684-702; native CPU :425-440):
 * db[k] = sum_{n,p,q} dy[n,k,p,q]. */
SGH_API int sgh_conv_bgrad_f32(const sgh_conv_geom *g, const float *dy, float *db, void *stream);
/* GpuConvForward (src/model/operation/convolution.cc:585-632); bias may be NULL. */
SGH_API int sgh_conv_fwd_f32(sgh_conv_geom *g, const float *x, const float *W,
                             const float *bias, float *y, void *workspace, size_t ws_bytes,
                             void *stream);

/* The three convolution passes on 16-bit tensors (x, W, y and their gradients all binary16 or
 * all bfloat16, as a reference handle built from a half input runs them:
 * src/model/operation/convolution.cc:444-572).  Arithmetic: fp32 accumulation of exact 16-bit
 * products, the result rounded once.  All three passes run on the 16-bit matrix instructions for
 * stride 1 or 2 (data gradient: K a multiple of 8, C >= 16, Q >= 2; forward: C a multiple of 8,
 * K >= 16, W >= 2), the stem's data gradient on the fp32 kernel reading and writing 16-bit
 * tensors; other geometries widen the operands to fp32 in the workspace and use the fp32 kernels.
 * Workspace: sgh_conv_workspace_bytes_h(g, which) bytes. */
SGH_API size_t sgh_conv_workspace_bytes_h(const sgh_conv_geom *g, int which);
SGH_API int sgh_conv_dgrad_f16(sgh_conv_geom *g, const uint16_t *dy, const uint16_t *W,
                               uint16_t *dx, void *workspace, size_t ws_bytes, void *stream);
SGH_API int sgh_conv_dgrad_bf16(sgh_conv_geom *g, const uint16_t *dy, const uint16_t *W,
                                uint16_t *dx, void *workspace, size_t ws_bytes, void *stream);
SGH_API int sgh_conv_wgrad_f16(sgh_conv_geom *g, const uint16_t *dy, const uint16_t *x,
                               uint16_t *dW, void *workspace, size_t ws_bytes, void *stream);
SGH_API int sgh_conv_wgrad_bf16(sgh_conv_geom *g, const uint16_t *dy, const uint16_t *x,
                                uint16_t *dW, void *workspace, size_t ws_bytes, void *stream);
/* How sgh_conv_wgrad_{f16,bf16} split their reduction.  -1 (the default): by the stream of the call -- on a
 * device's auxiliary stream (sgh_device_aux_stream) the launch shares the chip with the main stream's kernels
 * and the split is planned for one workgroup per CU (half the fp32 partials to write and sum), elsewhere for
 * two; 1: always the shared-chip plan, 0: never.  The plans sum the fp32 partials in different orders, so
 * results of different plans differ in the last place of the 16-bit result; each plan is run-to-run
 * identical.  Process-wide; meant for measurements and for comparing a two-stream tape bit by bit with a
 * one-stream one.  No counterpart in the reference (cuDNN chooses its algorithms by itself). */
SGH_API void sgh_conv_wgrad16_split_mode(int mode);
SGH_API int sgh_conv_bgrad_f16(const sgh_conv_geom *g, const uint16_t *dy, uint16_t *db, void *stream);
SGH_API int sgh_conv_bgrad_bf16(const sgh_conv_geom *g, const uint16_t *dy, uint16_t *db, void *stream);
SGH_API int sgh_conv_fwd_f16(sgh_conv_geom *g, const uint16_t *x, const uint16_t *W,
                             const uint16_t *bias, uint16_t *y, void *workspace, size_t ws_bytes,
                             void *stream);
SGH_API int sgh_conv_fwd_bf16(sgh_conv_geom *g, const uint16_t *x, const uint16_t *W,
                              const uint16_t *bias, uint16_t *y, void *workspace, size_t ws_bytes,
                              void *stream);

/* GpuBatchNormForwardTraining (src/model/operation/batchnorm.cc:287-329), spatial mode:
 * per-channel batch mean / biased variance over N*HW, y = gamma*(x-mean)*invstd + beta,
 * running = (1-factor)*running + factor*batch (unbiased variance), saves (mean, invstd) with
 * invstd = 1/sqrt(var + eps) in the slots Python calls (mean, var)
 * (python/singa/autograd.py:1777-1781).  running_* may be NULL.
 * workspace (both passes): sgh_bn_workspace_bytes(N, C, HW) bytes of per-channel partial sums; the
 * one-pass forward kernels keep their exchange words in a part of it that no other kernel writes, so
 * recorded forward and backward launches that share a workspace replay in any order. */
SGH_API size_t sgh_bn_workspace_bytes(int N, int C, int HW);
SGH_API int sgh_bn_fwd_train_f32(const float *x, const float *gamma, const float *beta,
                                 float *running_mean, float *running_var, float factor, float eps,
                                 float *y, float *save_mean, float *save_invstd, int N, int C,
                                 int HW, void *workspace, size_t ws_bytes, void *stream);
/* GpuBatchNormForwardTraining followed by ReLU in one call (conv -> BatchNorm -> ReLU,
 * examples/cnn/model/resnet.py:54-60; batchnorm.cc:287-329 then tensor_math_cpp.h:585-589): same statistics,
 * y holds relu(BatchNorm(x)) -- the bits the two calls store -- so the ReLU's pass over y disappears.
 * sgh_bn_relu_bwd_* is its backward (it recomputes the gate from x).  *_f16 / *_bf16 below likewise. */
SGH_API int sgh_bn_relu_fwd_train_f32(const float *x, const float *gamma, const float *beta,
                                      float *running_mean, float *running_var, float factor, float eps,
                                      float *y, float *save_mean, float *save_invstd, int N, int C,
                                      int HW, void *workspace, size_t ws_bytes, void *stream);
SGH_API int sgh_bn_relu_fwd_train_f16(const uint16_t *x, const float *gamma, const float *beta,
                                      float *running_mean, float *running_var, float factor, float eps,
                                      uint16_t *y, float *save_mean, float *save_invstd, int N, int C,
                                      int HW, void *workspace, size_t ws_bytes, void *stream);
SGH_API int sgh_bn_relu_fwd_train_bf16(const uint16_t *x, const float *gamma, const float *beta,
                                       float *running_mean, float *running_var, float factor, float eps,
                                       uint16_t *y, float *save_mean, float *save_invstd, int N, int C,
                                       int HW, void *workspace, size_t ws_bytes, void *stream);
/* The same with the sum that ends a residual block in between: y = relu(BatchNorm(x) + z), the forward of
 * relu(bn(conv(..)) + identity) (examples/cnn/model/resnet.py:70-77, :108-115) in one call -- the bits that
 * GpuBatchNormForwardTraining, the tensor addition (autograd.py add) and ReLU store one after the other (BatchNorm
 * output and sum each rounded to the storage type).  The BatchNorm's own output is not kept: its backward needs
 * x only, the ReLU's backward gates on y.  z has the shape and type of x. */
SGH_API int sgh_bn_add_relu_fwd_train_f32(const float *x, const float *z, const float *gamma, const float *beta,
                                          float *running_mean, float *running_var, float factor, float eps,
                                          float *y, float *save_mean, float *save_invstd, int N, int C,
                                          int HW, void *workspace, size_t ws_bytes, void *stream);
SGH_API int sgh_bn_add_relu_fwd_train_f16(const uint16_t *x, const uint16_t *z, const float *gamma, const float *beta,
                                          float *running_mean, float *running_var, float factor, float eps,
                                          uint16_t *y, float *save_mean, float *save_invstd, int N, int C,
                                          int HW, void *workspace, size_t ws_bytes, void *stream);
SGH_API int sgh_bn_add_relu_fwd_train_bf16(const uint16_t *x, const uint16_t *z, const float *gamma, const float *beta,
                                           float *running_mean, float *running_var, float factor, float eps,
                                           uint16_t *y, float *save_mean, float *save_invstd, int N, int C,
                                           int HW, void *workspace, size_t ws_bytes, void *stream);
/* GpuBatchNormForwardInference (src/model/operation/batchnorm.cc:331-366):
 * y = gamma * (x - running_mean) / sqrt(running_var + eps) + beta. */
SGH_API int sgh_bn_fwd_infer_f32(const float *x, const float *gamma, const float *beta,
                                 const float *running_mean, const float *running_var, float eps,
                                 float *y, int N, int C, int HW, void *stream);
/* GpuBatchNormBackward (src/model/operation/batchnorm.cc:368-404):
 * dbeta = sum dy, dgamma = sum dy*xhat, dx = gamma*invstd/M * (M*dy - dbeta - xhat*dgamma).
 * dbeta = sum dy etc. are summed in a fixed order: results are run-to-run identical. */
SGH_API int sgh_bn_bwd_f32(const float *dy, const float *x, const float *gamma,
                           const float *save_mean, const float *save_invstd, float *dx,
                           float *dgamma, float *dbeta, int N, int C, int HW, void *workspace,
                           size_t ws_bytes, void *stream);
/* The one-pass BatchNorm kernels (forward and backward; they read x, or x and dy, once) cut a channel
 * into slices, one workgroup per slice, and the workgroups of a channel exchange their partial sums
 * through the workspace while all of them are resident on the GPU.  That needs every slice of the oldest
 * unfinished channel to be running: the plan only uses these kernels when that many workgroups fit the
 * device at once (otherwise the two-pass kernels run), and workgroups are dispatched in index order.  The
 * wait is bounded all the same: a workgroup that has polled `polls` times gives up, the channel's outputs
 * become NaN, every kernel still ends normally, and a device-side counter records it.
 *   sgh_bn_exchange_failures    waits for `stream`, returns the number of workgroups that gave up since
 *                               the last look and clears it (sgh_device_sync looks too and returns
 *                               SGH_EEXCHANGE).  0 in normal operation.
 *   sgh_bn_exchange_spin_limit  sets `polls` for later launches (process-wide; <= 0 restores the default
 *                               of 2^20).  For tests of the failure path: with a limit of 1 the first
 *                               slices of a many-slice channel give up.
 * No counterpart in the reference (cuDNN's kernels are closed). */
SGH_API int sgh_bn_exchange_failures(void *stream, int *count);
SGH_API void sgh_bn_exchange_spin_limit(int polls);
/* sgh_bn_bwd_f32 for callers that cannot allocate device memory and have no workspace to pass
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same kernels, same results bit for bit; the per-channel partial
 * sums live in a buffer that is part of the library's code object (256 KiB on every GPU the
 * library runs on, held until the process ends) instead of a workspace.  Limit: the partial sums
 * of the shape must fit in those 256 KiB -- sgh_bn_workspace_bytes(N, C, HW) <= 262144 is
 * sufficient (8 bytes per channel and split of the two-pass kernels, 16 per channel and slice of
 * the one-pass kernel; every ResNet layer up to batch 128 fits) -- else SGH_ELIMIT is returned
 * and nothing is launched.  Calls no hipMalloc / hipFree.
 * All calls on one GPU share the buffer: calls that overlap on one GPU (two streams, two threads)
 * race; calls on one stream are ordered and safe, recorded calls of several shapes replayed in a
 * graph included.  The caller clears nothing: what a call reads it has written itself (the one-pass
 * kernel's exchange words are zeroed by a small kernel of the same call). */
SGH_API int sgh_bn_bwd_noalloc_f32(const float *dy, const float *x, const float *gamma,
                                   const float *save_mean, const float *save_invstd, float *dx,
                                   float *dgamma, float *dbeta, int N, int C, int HW,
                                   void *stream);
/* ReLUBackward followed by GpuBatchNormBackward in one pass, for a ReLU whose input is this
 * BatchNorm's output (python/singa/autograd.py:432-439 then batchnorm.cc:368-404; the tape of
 * conv -> BatchNorm -> ReLU, examples/cnn/model/resnet.py:54-60).  `dy` is the gradient behind the
 * ReLU; the BatchNorm output y = gamma*xhat + beta is recomputed from x exactly as the forward
 * kernel stored it, and the gradient entering the BatchNorm is dy where y > 0, else 0.  Same
 * outputs as the two separate calls, three tensor passes less.  *_f16 / *_bf16 below likewise. */
SGH_API int sgh_bn_relu_bwd_f32(const float *dy, const float *x, const float *gamma,
                                const float *beta, const float *save_mean,
                                const float *save_invstd, float *dx, float *dgamma, float *dbeta,
                                int N, int C, int HW, void *workspace, size_t ws_bytes,
                                void *stream);
/* The same two operations on 16-bit activations (x, y, dy, dx binary16 or bfloat16) with fp32
 * gamma / beta / statistics / parameter gradients -- cuDNN's convention for half tensors, which
 * the reference's handle selects from the input's data type (batchnorm.cc:261-285). */
SGH_API int sgh_bn_fwd_train_f16(const uint16_t *x, const float *gamma, const float *beta,
                                 float *running_mean, float *running_var, float factor, float eps,
                                 uint16_t *y, float *save_mean, float *save_invstd, int N, int C,
                                 int HW, void *workspace, size_t ws_bytes, void *stream);
SGH_API int sgh_bn_fwd_train_bf16(const uint16_t *x, const float *gamma, const float *beta,
                                  float *running_mean, float *running_var, float factor, float eps,
                                  uint16_t *y, float *save_mean, float *save_invstd, int N, int C,
                                  int HW, void *workspace, size_t ws_bytes, void *stream);
SGH_API int sgh_bn_fwd_infer_f16(const uint16_t *x, const float *gamma, const float *beta,
                                 const float *running_mean, const float *running_var, float eps,
                                 uint16_t *y, int N, int C, int HW, void *stream);
SGH_API int sgh_bn_fwd_infer_bf16(const uint16_t *x, const float *gamma, const float *beta,
                                  const float *running_mean, const float *running_var, float eps,
                                  uint16_t *y, int N, int C, int HW, void *stream);
SGH_API int sgh_bn_bwd_f16(const uint16_t *dy, const uint16_t *x, const float *gamma,
                           const float *save_mean, const float *save_invstd, uint16_t *dx,
                           float *dgamma, float *dbeta, int N, int C, int HW, void *workspace,
                           size_t ws_bytes, void *stream);
SGH_API int sgh_bn_bwd_bf16(const uint16_t *dy, const uint16_t *x, const float *gamma,
                            const float *save_mean, const float *save_invstd, uint16_t *dx,
                            float *dgamma, float *dbeta, int N, int C, int HW, void *workspace,
                            size_t ws_bytes, void *stream);
SGH_API int sgh_bn_relu_bwd_f16(const uint16_t *dy, const uint16_t *x, const float *gamma,
                                const float *beta, const float *save_mean,
                                const float *save_invstd, uint16_t *dx, float *dgamma,
                                float *dbeta, int N, int C, int HW, void *workspace,
                                size_t ws_bytes, void *stream);
SGH_API int sgh_bn_relu_bwd_bf16(const uint16_t *dy, const uint16_t *x, const float *gamma,
                                 const float *beta, const float *save_mean,
                                 const float *save_invstd, uint16_t *dx, float *dgamma,
                                 float *dbeta, int N, int C, int HW, void *workspace,
                                 size_t ws_bytes, void *stream);

/* Geometry of a PoolingHandle (src/model/operation/pooling.h:40-71; ctor pooling.cc:27-52). */
typedef struct sgh_pool_geom {
  int N, C, H, W;
  int kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w;
  int P, Q;
  int is_max;
} sgh_pool_geom;
SGH_API int sgh_pool_geom_init(sgh_pool_geom *g, int N, int C, int H, int W, int kernel_h,
                               int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
                               int is_max);
/* GpuPoolingForward (src/model/operation/pooling.cc:187-205).  Max: first maximum in
 * row-major window order wins (src/model/layer/pooling.cc:189-196); avg: count-exclude-padding
 * (pooling.cc:70-72, :172). */
SGH_API int sgh_pool_fwd_f32(const sgh_pool_geom *g, const float *x, float *y, void *stream);
/* GpuPoolingBackward (src/model/operation/pooling.cc:207-226), same (dy, x, y) arguments.
 * Max: dy[n,c,p,q] is routed to the first-maximum position of its window (recomputed from x;
 * y is accepted for signature parity and may be NULL), contributions of overlapping windows
 * are added in ascending (p, q) order — the order of src/model/layer/pooling.cc:208-233 — so
 * the result is bit-identical to the CPU loop.  Avg: dy / |clipped window| spread over the window. */
SGH_API int sgh_pool_bwd_f32(const sgh_pool_geom *g, const float *dy, const float *x,
                             const float *y, float *dx, void *stream);
/* Pooling on 16-bit tensors: comparisons and sums in fp32 (conversion keeps order, so the routing
 * of the max gradient is that of the stored values), one rounding on store. */
SGH_API int sgh_pool_fwd_f16(const sgh_pool_geom *g, const uint16_t *x, uint16_t *y, void *stream);
SGH_API int sgh_pool_fwd_bf16(const sgh_pool_geom *g, const uint16_t *x, uint16_t *y, void *stream);
SGH_API int sgh_pool_bwd_f16(const sgh_pool_geom *g, const uint16_t *dy, const uint16_t *x,
                             const uint16_t *y, uint16_t *dx, void *stream);
SGH_API int sgh_pool_bwd_bf16(const sgh_pool_geom *g, const uint16_t *dy, const uint16_t *x,
                              const uint16_t *y, uint16_t *dx, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SINGA_HIP_H_ */
