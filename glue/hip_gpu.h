// HipGPU: the SINGA Device that runs tensor operations on an MI355X through libsinga_hip.so.
// Lands in a SINGA tree as include/singa/core/hip_gpu.h (glue/apply_to_tree.py copies it and adds
// the include to include/singa/core/device.h under USE_HIP).
//
// Counterpart of CudaGPU (include/singa/core/device.h:207-240, src/core/device/cuda_gpu.cc:56-209):
// one stream behind Device::Exec, a caching pool behind Malloc / Free, blocking host copies, event
// pairs for the Graph's per-node timing.  Everything device-side goes through the C ABI of
// singa_hip.h; this class holds no HIP type.
#ifndef SINGA_CORE_HIP_GPU_H_
#define SINGA_CORE_HIP_GPU_H_

#include "singa/singa_config.h"
#ifdef USE_HIP

#include <memory>
#include <utility>
#include <vector>

#include "singa/core/device.h"
#include "singa/core/memory.h"
#include "singa_hip.h"

namespace singa {

/// rc != 0 aborts with the library's text, SINGA's convention for device-API failures
/// (CUDA_CHECK, include/singa/utils/cuda_utils.h:96-117).
#define HIP_ABI_CHECK(expr)                                                   \
  do {                                                                        \
    const int sgh_rc_ = (expr);                                               \
    CHECK_EQ(sgh_rc_, 0) << "singa_hip: " << sgh_error_string(sgh_rc_) << " in " #expr; \
  } while (0)

/// DeviceMemPool (include/singa/core/memory.h:37-54) over the pool of one sgh_device.  A HipGPU
/// owns one; it is a class of its own so that code written against DeviceMemPool (GetMemUsage)
/// keeps working.
class HipMemPool : public DeviceMemPool {
 public:
  explicit HipMemPool(sgh_device *dev) : dev_(dev) {}
  void Malloc(void **ptr, const size_t size) override;
  void Free(void *ptr) override;
  /// <free (cached, ready for reuse), total (handed out + cached)> in bytes
  std::pair<size_t, size_t> GetMemUsage() override;
  std::pair<size_t, size_t> GetMemUsage(int) override { return GetMemUsage(); }

 private:
  sgh_device *dev_;
};

class HipGPU : public Device {
 public:
  explicit HipGPU(int id = 0);
  ~HipGPU() override;

  /// Uniform / Gaussian fills are a pure function of (seed, offset): SetRandSeed stores the seed
  /// and rewinds the offset; every fill advances it.
  void SetRandSeed(unsigned seed) override;
  size_t GetAllocatedMem() override;
  void Sync() override;

  sgh_device *handle() const { return dev_; }

  /// The second compute stream (sgh_device_fork / sgh_device_join): a training loop that updates
  /// after the whole backward pass runs each weight gradient there.
  void *Fork();
  void Join();
  void UsedOnAux(Block *block);

  /// Graph mode on the device: EnableGraph(true) ... EnableGraph(false) of the reference buffer
  /// operations in singa::Graph; these record the stream into a HIP graph instead.
  void BeginRecord();
  void EndRecord();
  void Replay();
  void DropRecord();

 protected:
  void DoExec(function<void(Context *)> &&fn, int executor) override;
  void TimeProfilingDoExec(function<void(Context *)> &&fn, int executor, Node *node) override;
  void EvaluateTimeElapsed(Node *node) override;
  void CopyToFrom(void *dst, const void *src, size_t nBytes, CopyDirection direction,
                  Context *ctx) override;
  void *Malloc(int size) override;
  void Free(void *ptr) override;

 private:
  sgh_device *dev_ = nullptr;
  sgh_graph *recorded_ = nullptr;
  std::shared_ptr<HipMemPool> pool_;
};

/// Platform::CreateCudaGPUsOn's counterpart (src/core/device/platform.cc:137-160): one HipGPU per
/// listed id, created once per process and Reset() when asked for again.
int GetNumHipGPUs();
std::vector<std::shared_ptr<Device>> CreateHipGPUsOn(const std::vector<int> &devices);
std::shared_ptr<Device> CreateHipGPU();

}  // namespace singa

#endif  // USE_HIP
#endif  // SINGA_CORE_HIP_GPU_H_
