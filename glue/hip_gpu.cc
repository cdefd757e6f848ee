// HipGPU / HipMemPool / device factory.  Lands in a SINGA tree as src/core/device/hip_gpu.cc.
// Modelled on what CudaGPU provides (src/core/device/cuda_gpu.cc:56-209); every device call is an
// entry point of singa_hip.h.
#include "singa/core/hip_gpu.h"

#ifdef USE_HIP

#include <chrono>
#include <mutex>

namespace singa {

// ---- pool ----------------------------------------------------------------------------------
void HipMemPool::Malloc(void **ptr, const size_t size) { HIP_ABI_CHECK(sgh_malloc(dev_, ptr, size)); }

void HipMemPool::Free(void *ptr) { HIP_ABI_CHECK(sgh_free(dev_, ptr)); }

std::pair<size_t, size_t> HipMemPool::GetMemUsage() {
  size_t in_use = 0, cached = 0, driver_calls = 0;
  HIP_ABI_CHECK(sgh_pool_stats(dev_, &in_use, &cached, &driver_calls));
  return std::make_pair(cached, in_use + cached);
}

// ---- device --------------------------------------------------------------------------------
HipGPU::HipGPU(int id) : Device(id, 1) {
  lang_ = kHip;
  HIP_ABI_CHECK(sgh_device_open(id, &dev_));
  pool_ = std::make_shared<HipMemPool>(dev_);
  ctx_.hip_device = dev_;
  ctx_.hip_stream = sgh_device_stream(dev_);
  // scratch of Dot / Sum (a few KiB) and, behind it, the device word their host-result forms
  // copy back; owned by the device for its lifetime
  ctx_.hip_reduce_ws_bytes = sgh_reduce_workspace_bytes();
  pool_->Malloc(&ctx_.hip_reduce_ws, ctx_.hip_reduce_ws_bytes + 256);
  ctx_.hip_reduce_result = static_cast<char *>(ctx_.hip_reduce_ws) + ctx_.hip_reduce_ws_bytes;
  SetRandSeed(static_cast<unsigned>(std::chrono::system_clock::now().time_since_epoch().count()));
}

HipGPU::~HipGPU() {
  if (recorded_) sgh_graph_destroy(recorded_);
  if (dev_) {
    sgh_device_sync(dev_);
    if (ctx_.hip_reduce_ws) sgh_free(dev_, ctx_.hip_reduce_ws);
    sgh_device_close(dev_);
  }
}

void HipGPU::SetRandSeed(unsigned seed) {
  seed_ = seed;
  ctx_.hip_rng_seed = seed;
  ctx_.hip_rng_offset = 0;
}

size_t HipGPU::GetAllocatedMem() {
  const auto usage = pool_->GetMemUsage();
  return usage.second - usage.first;
}

// (cuda_gpu.cc:206-209: the wait is itself an operation, so that it is ordered with buffered ones)
void HipGPU::Sync() {
  Exec([this](Context *) { HIP_ABI_CHECK(sgh_device_sync(dev_)); }, {}, {}, "Waiting");
}

void HipGPU::DoExec(function<void(Context *)> &&fn, int) { fn(&ctx_); }

// Graph profiling keeps two events per Node (Node::hip_start_ / hip_end_, added to
// include/singa/core/scheduler.h beside the cudaEvent_t pair).
void HipGPU::TimeProfilingDoExec(function<void(Context *)> &&fn, int, Node *node) {
  HIP_ABI_CHECK(sgh_event_create(&node->hip_start_));
  HIP_ABI_CHECK(sgh_event_create(&node->hip_end_));
  HIP_ABI_CHECK(sgh_event_record(node->hip_start_, ctx_.hip_stream));
  fn(&ctx_);
  HIP_ABI_CHECK(sgh_event_record(node->hip_end_, ctx_.hip_stream));
}

void HipGPU::EvaluateTimeElapsed(Node *node) {
  float ms = 0.f;
  HIP_ABI_CHECK(sgh_event_elapsed_ms(node->hip_start_, node->hip_end_, &ms));
  HIP_ABI_CHECK(sgh_event_destroy(node->hip_start_));
  HIP_ABI_CHECK(sgh_event_destroy(node->hip_end_));
  node->hip_start_ = node->hip_end_ = nullptr;
  node->time_elapsed_inc(ms * 0.001f);
}

// Host copies block until done: Tensor::data<>() / GetValue read the host buffer right after the
// call (the CUDA device gets the same effect from cudaMemcpyAsync on pageable memory,
// cuda_gpu.cc:171-175).  CopyDirection's values are the ABI's `kind`.
void HipGPU::CopyToFrom(void *dst, const void *src, size_t nBytes, CopyDirection direction, Context *) {
  HIP_ABI_CHECK(sgh_memcpy(dev_, dst, src, nBytes, static_cast<int>(direction)));
}

// Like CudaGPU::Malloc the block is not zero-filled (cuda_gpu.cc:187-197).
void *HipGPU::Malloc(int size) {
  void *ptr = nullptr;
  if (size > 0) pool_->Malloc(&ptr, static_cast<size_t>(size));
  return ptr;
}

void HipGPU::Free(void *ptr) {
  if (ptr != nullptr) pool_->Free(ptr);
}

void *HipGPU::Fork() {
  void *aux = nullptr;
  HIP_ABI_CHECK(sgh_device_fork(dev_, &aux));
  return aux;
}

void HipGPU::Join() { HIP_ABI_CHECK(sgh_device_join(dev_)); }

void HipGPU::UsedOnAux(Block *block) {
  if (block != nullptr && block->initialized())
    HIP_ABI_CHECK(sgh_block_used_on(dev_, block->mutable_data(), sgh_device_aux_stream(dev_)));
}

void HipGPU::BeginRecord() {
  DropRecord();
  HIP_ABI_CHECK(sgh_graph_begin(dev_));
}

void HipGPU::EndRecord() { HIP_ABI_CHECK(sgh_graph_end(dev_, &recorded_)); }

void HipGPU::Replay() {
  CHECK(recorded_ != nullptr) << "no recorded graph on device " << id_;
  HIP_ABI_CHECK(sgh_graph_launch(recorded_));
}

void HipGPU::DropRecord() {
  if (recorded_) HIP_ABI_CHECK(sgh_graph_destroy(recorded_));
  recorded_ = nullptr;
}

// ---- factory -------------------------------------------------------------------------------
int GetNumHipGPUs() {
  int count = 0;
  HIP_ABI_CHECK(sgh_device_count(&count));
  return count;
}

std::vector<std::shared_ptr<Device>> CreateHipGPUsOn(const std::vector<int> &devices) {
  static std::mutex mu;
  static std::vector<std::shared_ptr<Device>> opened;
  std::lock_guard<std::mutex> lock(mu);
  if (opened.empty()) opened.resize(static_cast<size_t>(GetNumHipGPUs()));
  std::vector<std::shared_ptr<Device>> ret;
  for (int id : devices) {
    CHECK_GE(id, 0);
    CHECK_LT(static_cast<size_t>(id), opened.size()) << "no such GPU";
    if (opened[id] == nullptr)
      opened[id] = std::make_shared<HipGPU>(id);
    else
      opened[id]->Reset();
    ret.push_back(opened[id]);
  }
  return ret;
}

std::shared_ptr<Device> CreateHipGPU() { return CreateHipGPUsOn({0}).at(0); }

}  // namespace singa

#endif  // USE_HIP
