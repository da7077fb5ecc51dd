// Contexts, device memory helpers and error plumbing of the host layer.
// Interface after the reference's src/context.cc:21-156 (see include/arraydiff/context.hh).
#include "arraydiff/context.hh"

#include <hip/hip_runtime_api.h>

#include "adh_capi.h"
#include "arraydiff/array_gpu.hh"
#include "arraydiff/spatial.hh"

namespace arraydiff {

AdhError::AdhError(int c, const std::string &what) : std::runtime_error(what), code(c) {}

void adh_check(int code, const char *what) {
  if (code != ADH_OK) throw AdhError(code, std::string(what) + ": " + adh_error_string(code));
}

void hip_check(hipError_t e, const char *what) {
  if (e != hipSuccess) throw AdhError((int)e, std::string(what) + ": " + hipGetErrorString(e));
}

void *gpu_alloc_bytes(size_t bytes) {
  void *p = nullptr;
  hip_check(hipMalloc(&p, bytes), "hipMalloc");
  return p;
}
void gpu_free_bytes(void *p) {
  if (p) (void)hipFree(p);
}
void gpu_copy_h2d(void *dst, const void *src, size_t bytes, hipStream_t s) {
  hip_check(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s), "hipMemcpyAsync h2d");
}
void gpu_copy_d2h(void *dst, const void *src, size_t bytes, hipStream_t s) {
  hip_check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s), "hipMemcpyAsync d2h");
}
void gpu_copy_d2d(void *dst, const void *src, size_t bytes, hipStream_t s) {
  hip_check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s), "hipMemcpyAsync d2d");
}

void GPUConn::sync() { hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize"); }

shared_ptr<GPUContext> GPUContext::Make(int device) { return std::make_shared<GPUContext>(device); }
shared_ptr<GPUContext> GPUContext::MakeShared(int device, hipStream_t stream) {
  return std::make_shared<GPUContext>(device, stream);
}

GPUContext::GPUContext(int device) : device_(device), stream_(nullptr), owns_stream_(true), scratch_size_(0) {
  hip_check(hipSetDevice(device_), "hipSetDevice");
  hip_check(hipStreamCreate(&stream_), "hipStreamCreate");  // default priority
}

GPUContext::GPUContext(int device, hipStream_t shared_stream)
    : device_(device), stream_(shared_stream), owns_stream_(false), scratch_size_(0) {}

GPUContext::~GPUContext() {
  if (owns_stream_ && stream_) (void)hipStreamDestroy(stream_);
}

void GPUContext::sync() { hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize"); }

shared_ptr<GPUMemory<uint8_t>> GPUContext::get_scratch() {
  if (!scratch_) {
    const size_t rounded = (scratch_size_ + 4095) / 4096 * 4096;
    scratch_size_ = rounded;
    scratch_ = std::make_shared<GPUMemory<uint8_t>>(rounded, this);
  }
  return scratch_;
}

void GPUContext::reserve_scratch(size_t min_scratch_size) {
  if (min_scratch_size <= scratch_size_) return;
  // growing the scratch synchronises and reallocates, neither of which a stream that is being recorded
  // into a graph allows: say so instead of invalidating the recording with an opaque error
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream_, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone)
    throw std::logic_error("GPUContext::reserve_scratch: the scratch would grow while the stream is being recorded; "
                           "run one step eagerly first");
  scratch_size_ = (min_scratch_size + 4095) / 4096 * 4096;
  if (scratch_) {
    sync();  // work queued on the old scratch must finish before it is released
    scratch_->reallocate(scratch_size_, this);
  }
}

shared_ptr<MultiGPUContext> MultiGPUContext::Make(size_t num_ranks, int device) {
  return std::make_shared<MultiGPUContext>(num_ranks, device);
}

MultiGPUContext::MultiGPUContext(size_t num_ranks, int device) : device_(device), stream_(nullptr), spatial_comms_(nullptr) {
  if (num_ranks == 0 || num_ranks > ARRAYDIFF_MAX_PEERS) throw std::invalid_argument("MultiGPUContext: 1..16 ranks");
  hip_check(hipSetDevice(device_), "hipSetDevice");
  hip_check(hipStreamCreate(&stream_), "hipStreamCreate");
  for (size_t r = 0; r < num_ranks; ++r) dev_ctxs_.push_back(GPUContext::MakeShared(device_, stream_));
  spatial_comms_ = new Spatial2DComm[num_ranks];
  // rows only, like the reference (src/context.cc:134: InitAll(comms, 1, num_ranks))
  adh_check(Spatial2DComm::InitAll(spatial_comms_, 1, (uint32_t)num_ranks), "Spatial2DComm::InitAll");
}

MultiGPUContext::~MultiGPUContext() {
  delete[] spatial_comms_;
  dev_ctxs_.clear();
  if (stream_) (void)hipStreamDestroy(stream_);
}

void MultiGPUContext::sync() { hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize"); }
void MultiGPUContext::sync_rank(size_t rank) { dev_ctxs_.at(rank)->sync(); }
shared_ptr<GPUContext> MultiGPUContext::device_context(size_t rank) { return dev_ctxs_.at(rank); }
Spatial2DComm *MultiGPUContext::spatial_comm(size_t rank) {
  if (rank >= dev_ctxs_.size()) throw std::out_of_range("spatial_comm rank");
  return spatial_comms_ + rank;
}

StreamCapture::~StreamCapture() {
  abort();
  if (exec_) (void)hipGraphExecDestroy(exec_);
  if (graph_) (void)hipGraphDestroy(graph_);
}
// Ends a recording that is still open (an exception between begin() and end()) and drops what it held, so that
// the stream is usable again.
void StreamCapture::abort() {
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream_, &capturing) != hipSuccess || capturing == hipStreamCaptureStatusNone) return;
  hipGraph_t partial = nullptr;
  (void)hipStreamEndCapture(stream_, &partial);
  if (partial) (void)hipGraphDestroy(partial);
  (void)hipGetLastError();
}
void StreamCapture::begin() {
  if (graph_ || exec_) throw std::logic_error("StreamCapture: already recorded");
  hip_check(hipStreamBeginCapture(stream_, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
}
void StreamCapture::end() {
  hip_check(hipStreamEndCapture(stream_, &graph_), "hipStreamEndCapture");
  hip_check(hipGraphGetNodes(graph_, nullptr, &num_nodes_), "hipGraphGetNodes");
  hip_check(hipGraphInstantiate(&exec_, graph_, nullptr, nullptr, 0), "hipGraphInstantiate");
}
void StreamCapture::replay() {
  if (!exec_) throw std::logic_error("StreamCapture: nothing recorded");
  hip_check(hipGraphLaunch(exec_, stream_), "hipGraphLaunch");
}

}  // namespace arraydiff
