// C++17 convenience layer over the C ABI of et.h (header-only): status codes become exceptions, the handle and the
// device buffers follow RAII, and `et::Encoder` strings Input -> L x Layer -> Output together the way the reference's
// Python glue does (python/effective_transformer/__init__.py:40-84) for a host that is C++ -- the shape a TensorFlow
// OpKernel, a Triton backend or a plain server loop would give it.  Needs the HIP runtime headers for hipMalloc.
#ifndef ET_HPP_
#define ET_HPP_

#include <hip/hip_runtime.h>

#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "et.h"

namespace et {

class Error : public std::runtime_error {
 public:
  Error(et_status s, const std::string& what) : std::runtime_error(what), status(s) {}
  et_status status;
};

inline void check(et_status s, et_handle h) {
  if (s != ET_OK) throw Error(s, et_last_error(h));
}
inline void check_hip(hipError_t e, const char* what) {
  if (e != hipSuccess) throw Error(ET_RUNTIME_ERROR, std::string(what) + ": " + hipGetErrorString(e));
}

class Handle {
 public:
  explicit Handle(int device = 0) { check(et_create(&h_, device), nullptr); }
  ~Handle() { et_destroy(h_); }
  Handle(const Handle&) = delete;
  Handle& operator=(const Handle&) = delete;
  et_handle get() const { return h_; }

 private:
  et_handle h_ = nullptr;
};

// Device memory that grows on demand and is freed with its owner.
class DeviceBuffer {
 public:
  DeviceBuffer() = default;
  ~DeviceBuffer() { if (p_) (void)hipFree(p_); }
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  void* reserve(size_t bytes) {
    if (bytes > cap_) {
      if (p_) check_hip(hipFree(p_), "hipFree");
      p_ = nullptr;
      cap_ = 0;
      check_hip(hipMalloc(&p_, bytes), "hipMalloc");
      cap_ = bytes;
    }
    return p_;
  }
  void* get() const { return p_; }
  size_t capacity() const { return cap_; }

 private:
  void* p_ = nullptr;
  size_t cap_ = 0;
};

// Input -> L x Layer -> Output.  The weights are device pointers owned by the caller (one et_layer_weights per layer, the
// reference's 16 tensors); activations, masks and the result are device pointers owned by the caller as well.  The
// object owns only its scratch: packed activations, index arrays, workspaces.  Not thread-safe; one object per stream.
class Encoder {
 public:
  // prepare: the weights stay as they are for the life of this object, so the k-contiguous copies of the dense kernels
  // that the large-M fp16 GEMMs want are made here once (on the device's default stream, waited for) instead of in
  // every layer call.
  Encoder(int device, et_dtype dtype, int head_num, int size_per_head, std::vector<et_layer_weights> layers,
          bool prepare = true)
      : handle_(device), dtype_(dtype), heads_(head_num), d_(size_per_head), layers_(std::move(layers)) {
    prepared_.assign(layers_.size(),
                     et_layer_prepared{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0});
    // (the k-contiguous kernels take hidden sizes in multiples of 64; others run on the weights as they are)
    if (!prepare || dtype != ET_FP16 || ((size_t)head_num * size_per_head) % 64 != 0) return;
    check_hip(hipSetDevice(device), "hipSetDevice");
    const size_t H = (size_t)head_num * size_per_head;
    char* dst = (char*)wt_.reserve(layers_.size() * 12 * H * H * 2);
    auto transposed = [&](const void* src, int k, int n) {
      void* out = dst;
      check(et_transpose_weight(handle_.get(), ET_FP16, src, out, k, n, nullptr), handle_.get());
      dst += (size_t)k * n * 2;
      return (const void*)out;
    };
    for (size_t l = 0; l < layers_.size(); ++l) {
      const et_layer_weights& w = layers_[l];
      et_layer_prepared& p = prepared_[l];
      p.attr_kernel_Q_t = transposed(w.attr_kernel_Q, (int)H, (int)H);
      p.attr_kernel_K_t = transposed(w.attr_kernel_K, (int)H, (int)H);
      p.attr_kernel_V_t = transposed(w.attr_kernel_V, (int)H, (int)H);
      p.attr_output_kernel_t = transposed(w.attr_output_kernel, (int)H, (int)H);
      p.inter_kernel_t = transposed(w.inter_kernel, (int)H, (int)(4 * H));
      p.output_kernel_t = transposed(w.output_kernel, (int)(4 * H), (int)H);
    }
    // a layer's last kernel requests the next layer's Q/K/V and attention output copies (consecutive in wt_), which
    // would otherwise be read cold
    for (size_t l = 0; l + 1 < layers_.size(); ++l) {
      prepared_[l].warm = prepared_[l + 1].attr_kernel_Q_t;
      prepared_[l].warm_bytes = 4 * H * H * 2;
    }
    check_hip(hipStreamSynchronize(nullptr), "hipStreamSynchronize");
  }

  ~Encoder() {
    if (host_count_) (void)hipHostFree(host_count_);
    if (copied_) (void)hipEventDestroy(copied_);
  }
  Encoder(const Encoder&) = delete;
  Encoder& operator=(const Encoder&) = delete;

  // from_tensor [B,S,H], mask int32 [B,S], attr_mask [B,S,S] in dtype -> out [B,S,H] (zeros at padding).
  // sync_count: read the valid-token count back once per batch, so that the launches of layers 2 .. L are sized
  // exactly (the reference reads it back in every layer), or leave it on the device (launches sized for B*S rows).
  // The copy is asynchronous and the host waits for it behind the launches of the first layer, which is sized for
  // B*S rows and bounded on the device, so the GPU never idles for the read-back.
  // Returns the valid-token count, or -1 when it was not read back.
  int forward(const void* from_tensor, const int32_t* mask, const void* attr_mask, void* out, int batch, int seq_len,
              hipStream_t stream, bool sync_count = true) {
    const size_t e = dtype_ == ET_FP32 ? 4 : 2;
    const size_t H = (size_t)heads_ * d_, rows = (size_t)batch * seq_len;
    char* act = (char*)act_.reserve(3 * rows * H * e);                 // packed input + two layer outputs
    // batch_idx, word_idx, the count, then the sequence table (2 B + 1 words)
    int32_t* idx = (int32_t*)idx_.reserve((2 * rows + 1) * sizeof(int32_t) + et_seq_workspace_bytes(batch));
    int32_t *batch_idx = idx, *word_idx = idx + rows, *count = idx + 2 * rows, *starts = idx + 2 * rows + 1;
    const size_t in_ws = et_input_workspace_bytes(batch, seq_len);
    const size_t layer_ws = et_layer_workspace_bytes(dtype_, batch, seq_len, heads_, d_);
    void* ws = ws_.reserve(in_ws > layer_ws ? in_ws : layer_ws);
    int32_t host_count = -1;
    check(et_input(handle_.get(), dtype_, from_tensor, mask, act, count, batch_idx, word_idx, batch, seq_len, heads_, d_, ws,
                   ws_.capacity(), stream, nullptr),
          handle_.get());
    bool pending = false;
    if (sync_count) {
      if (!host_count_) check_hip(hipHostMalloc((void**)&host_count_, sizeof(int32_t), hipHostMallocDefault), "hipHostMalloc");
      if (!copied_) check_hip(hipEventCreateWithFlags(&copied_, hipEventDisableTiming), "hipEventCreate");
      check_hip(hipMemcpyAsync(host_count_, count, sizeof(int32_t), hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
      check_hip(hipEventRecord(copied_, stream), "hipEventRecord");
      pending = true;
    }
    // one sequence start table serves every layer of the batch
    check(et_sequence_starts(handle_.get(), batch_idx, count, batch, seq_len, starts, et_seq_workspace_bytes(batch), stream),
          handle_.get());
    const char* x = act;
    for (size_t l = 0; l < layers_.size(); ++l) {
      if (l == 1 && pending) {       // the first layer is in the queue: waiting here leaves the GPU with work
        check_hip(hipEventSynchronize(copied_), "hipEventSynchronize");
        host_count = *host_count_;
        pending = false;
      }
      char* y = act + (1 + (l & 1)) * rows * H * e;
      et_layer_prepared prep = prepared_[l];
      prep.seq_start = starts;
      prep.seq_start_bytes = et_seq_workspace_bytes(batch);
      check(et_layer_with_prepared(handle_.get(), dtype_, &layers_[l], &prep, x, x, attr_mask, count, batch_idx, word_idx, y,
                                   batch, seq_len, seq_len, heads_, d_, host_count, ws, ws_.capacity(), stream),
            handle_.get());
      x = y;
    }
    check(et_output(handle_.get(), dtype_, x, count, batch_idx, word_idx, out, batch, seq_len, heads_, d_, stream),
          handle_.get());
    if (pending) {                   // a single layer: nothing needed the count, the caller still gets it
      check_hip(hipEventSynchronize(copied_), "hipEventSynchronize");
      host_count = *host_count_;
    }
    return host_count;
  }

 private:
  Handle handle_;
  et_dtype dtype_;
  int heads_, d_;
  std::vector<et_layer_weights> layers_;
  std::vector<et_layer_prepared> prepared_;
  DeviceBuffer act_, idx_, ws_, wt_;
  int32_t* host_count_ = nullptr;      // pinned
  hipEvent_t copied_ = nullptr;
};

}  // namespace et

#endif  // ET_HPP_
