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
  Encoder(int device, et_dtype dtype, int head_num, int size_per_head, std::vector<et_layer_weights> layers)
      : handle_(device), dtype_(dtype), heads_(head_num), d_(size_per_head), layers_(std::move(layers)) {}

  // from_tensor [B,S,H], mask int32 [B,S], attr_mask [B,S,S] in dtype -> out [B,S,H] (zeros at padding).
  // sync_count: read the valid-token count back once (exact launch sizes, one stream synchronisation, as the reference
  // does in every layer) or leave it on the device (no synchronisation, launches sized for B*S rows).
  // Returns the valid-token count, or -1 when it was not read back.
  int forward(const void* from_tensor, const int32_t* mask, const void* attr_mask, void* out, int batch, int seq_len,
              hipStream_t stream, bool sync_count = true) {
    const size_t e = dtype_ == ET_FP32 ? 4 : 2;
    const size_t H = (size_t)heads_ * d_, rows = (size_t)batch * seq_len;
    char* act = (char*)act_.reserve(3 * rows * H * e);                 // packed input + two layer outputs
    int32_t* idx = (int32_t*)idx_.reserve((2 * rows + 1) * sizeof(int32_t));
    int32_t *batch_idx = idx, *word_idx = idx + rows, *count = idx + 2 * rows;
    const size_t in_ws = et_input_workspace_bytes(batch, seq_len);
    const size_t layer_ws = et_layer_workspace_bytes(dtype_, batch, seq_len, heads_, d_);
    void* ws = ws_.reserve(in_ws > layer_ws ? in_ws : layer_ws);
    int32_t host_count = -1;
    check(et_input(handle_.get(), dtype_, from_tensor, mask, act, count, batch_idx, word_idx, batch, seq_len, heads_, d_, ws,
                   ws_.capacity(), stream, sync_count ? &host_count : nullptr),
          handle_.get());
    const char* x = act;
    for (size_t l = 0; l < layers_.size(); ++l) {
      char* y = act + (1 + (l & 1)) * rows * H * e;
      check(et_layer(handle_.get(), dtype_, &layers_[l], x, x, attr_mask, count, batch_idx, word_idx, y, batch, seq_len,
                     seq_len, heads_, d_, sync_count ? host_count : -1, ws, ws_.capacity(), stream),
            handle_.get());
      x = y;
    }
    check(et_output(handle_.get(), dtype_, x, count, batch_idx, word_idx, out, batch, seq_len, heads_, d_, stream),
          handle_.get());
    return host_count;
  }

 private:
  Handle handle_;
  et_dtype dtype_;
  int heads_, d_;
  std::vector<et_layer_weights> layers_;
  DeviceBuffer act_, idx_, ws_;
};

}  // namespace et

#endif  // ET_HPP_
