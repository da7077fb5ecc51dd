// Device context of the one-GPU spatial path.
//
// Mirrors the interface of the reference's Context / GPUConn / GPUContext / MultiGPUContext
// (include/arraydiff/context.hh:23-104, src/context.cc:21-156) with one change of substance:
// the reference's "ranks" are GPUs, here they are row-tiles of one activation held in ONE
// device's HBM.  MultiGPUContext therefore owns K rank contexts that all share one device and
// one in-order stream, so a halo exchange needs no host synchronisation around it: stream
// order is the barrier.
#ifndef ARRAYDIFF_CONTEXT_HH
#define ARRAYDIFF_CONTEXT_HH

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace arraydiff {

using std::shared_ptr;
using std::vector;

// The reference aborts on any runtime error (CUDA_CHECK -> assert, cuda_common.hh:6-9); the
// host classes here throw instead, the C ABI below them returns codes.
class AdhError : public std::runtime_error {
public:
  AdhError(int code, const std::string &what);
  int code;
};
void adh_check(int code, const char *what);
void hip_check(hipError_t e, const char *what);

template <typename T>
class GPUMemory;
class Spatial2DComm;

class Context {
public:
  virtual ~Context() {}
  virtual void sync() = 0;
};

// A (device, stream) handle handed to launchers, as in the reference; no cuBLAS / cuDNN
// handles because nothing on this path needs a library.
class GPUConn {
public:
  GPUConn(int device, hipStream_t stream) : device_(device), stream_(stream) {}
  int device() const { return device_; }
  hipStream_t stream() { return stream_; }
  void sync();

private:
  int device_;
  hipStream_t stream_;
};

class GPUContext : public virtual Context {
public:
  static shared_ptr<GPUContext> Make(int device);
  // a rank context that shares another context's stream (tiles of one GPU)
  static shared_ptr<GPUContext> MakeShared(int device, hipStream_t stream);

  explicit GPUContext(int device);
  GPUContext(int device, hipStream_t shared_stream);
  virtual ~GPUContext();

  virtual void sync();
  GPUConn conn() { return GPUConn(device_, stream_); }

  // growable scratch, 4 KiB granularity (GPUContext::get_scratch / reserve_scratch,
  // src/context.cc:68-100); used as the conv backward-filter workspace
  shared_ptr<GPUMemory<uint8_t>> get_scratch();
  void reserve_scratch(size_t min_scratch_size);

private:
  int device_;
  hipStream_t stream_;
  bool owns_stream_;
  size_t scratch_size_;
  shared_ptr<GPUMemory<uint8_t>> scratch_;
};

class MultiGPUContext : public virtual Context {
public:
  // the reference enumerates all visible GPUs (src/context.cc:116-124); here the number of
  // row-tiles is the caller's choice
  static shared_ptr<MultiGPUContext> Make(size_t num_ranks, int device = 0);

  MultiGPUContext(size_t num_ranks, int device);
  virtual ~MultiGPUContext();

  virtual void sync();
  void sync_rank(size_t rank);
  size_t num_ranks() const { return dev_ctxs_.size(); }
  shared_ptr<GPUContext> device_context(size_t rank);
  Spatial2DComm *spatial_comm(size_t rank);
  hipStream_t stream() { return stream_; }

private:
  int device_;
  hipStream_t stream_;
  vector<shared_ptr<GPUContext>> dev_ctxs_;
  Spatial2DComm *spatial_comms_;
};

// Everything enqueued on a stream between begin() and end(), recorded once as a HIP graph and replayed with
// one launch: for loops that are bound by the host's launch rate (a training step at a small batch is a
// thousand kernels of a few microseconds).  Not in the reference.  The host ops and the C ABI under them only
// enqueue kernels and device-to-device copies, so a whole forward + backward + optimizer step can be recorded
// once its buffers exist (run it eagerly first); host-to-device loads, read-backs and anything that
// synchronises stay outside.  A replay repeats the recorded launches with the recorded arguments: values that
// live in device memory (parameters, momentum, inputs copied into the same buffers) evolve, values that were
// kernel arguments (this iteration's step size) do not.
class StreamCapture {
public:
  explicit StreamCapture(hipStream_t stream) : stream_(stream), graph_(nullptr), exec_(nullptr) {}
  ~StreamCapture();
  StreamCapture(const StreamCapture &) = delete;
  StreamCapture &operator=(const StreamCapture &) = delete;
  void begin();
  void end();
  void replay();
  // ends a recording left open (the destructor calls it: an exception between begin() and end() leaves
  // the stream usable)
  void abort();
  size_t num_nodes() const { return num_nodes_; }

private:
  hipStream_t stream_;
  hipGraph_t graph_;
  hipGraphExec_t exec_;
  size_t num_nodes_ = 0;
};

}  // namespace arraydiff

#endif
