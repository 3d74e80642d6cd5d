// C ABI of libet_hip.so: argument validation, workspace carve-up and launch order of the three
// ops (reference host side: tf_op/bert_transformer_op.cu.cc:33-373) plus the kernel-level entry
// points.  No call allocates device memory; a handle serialises its calls with a mutex like the
// reference's layer op does (tf_op/bert_transformer_op.cc:213).
#include "../../include/et.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "kernels.hpp"

namespace et {

namespace {
// A launcher cannot return a status; a failed attribute call is kept here until the entry point checks its launches.
thread_local hipError_t tls_attr_error = hipSuccess;
}  // namespace

void allow_dynamic_lds(const void* kernel, int bytes) {
  static std::mutex mu;
  static std::vector<std::pair<const void*, int>> done;      // (kernel, device) pairs already raised
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = -1;
  std::lock_guard<std::mutex> lock(mu);
  for (const auto& e : done)
    if (e.first == kernel && e.second == dev) return;
  const hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (err != hipSuccess) {
    tls_attr_error = err;          // reported as ET_RUNTIME_ERROR by the entry point; tried again on the next call
    return;
  }
  if (dev >= 0) done.emplace_back(kernel, dev);
}

hipError_t take_attribute_error() {
  const hipError_t e = tls_attr_error;
  tls_attr_error = hipSuccess;
  return e;
}

}  // namespace et

namespace {

// The persistent GEMM stores C with plain stores while the matrices of a layer (resp. A and C of a stand-alone call)
// are small enough to be found in the 256 MB last-level cache by the kernels that read them next, and with non-temporal
// stores beyond.  12-layer BERT-base, fp16: plain stores -6 % at 4000 tokens, -2.4 % at 15900, +-0.5 % at 20000,
// +2 % at 30000 and 40000; 24-layer BERT-large at 13100 tokens: -0.4 %.
constexpr double kCachedLayerBytes = 320.0 * 1048576.0;
constexpr double kCachedCallBytes = 96.0 * 1048576.0;
// While the layer's matrices stay below this, weights requested ahead of FFN-up survive until FFN-down reads them.
constexpr double kWarmLayerBytes = 256.0 * 1048576.0;

// Scratch of et_input_static: the tile totals of the mask scan (one int32 per tile of 1024 positions) for up to
// kStaticMaxPositions positions, in kStaticSlots independent slots.  A handle takes a free slot of its device when it
// is created and gives it back when it is destroyed, so that two handles never share tile totals; the handles beyond
// kStaticSlots per device have none.  Every GPU the library runs on holds its own copy of the array until the
// process ends.  In host code the array's name is only a handle for hipGetSymbolAddress: the address a kernel may use
// is looked up once per device (et_create) and kept in static_scratch_ptr.
constexpr int kStaticSlotWords = 1024;
constexpr int kStaticSlots = 8;
constexpr int kStaticMaxPositions = 1024 * 1024;
static __device__ __align__(256) int32_t scratch[kStaticSlots * kStaticSlotWords];

constexpr int kMaxDevices = 64;
std::mutex static_scratch_mu;
int32_t* static_scratch_ptr[kMaxDevices] = {};
unsigned static_slots_taken[kMaxDevices] = {};       // bit s: slot s of the device belongs to a live handle

// Looks up this device's copy of `scratch` (the device must be current).  Called by et_create.
hipError_t resolve_static_scratch(int device) {
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(static_scratch_mu);
  if (static_scratch_ptr[device]) return hipSuccess;
  void* p = nullptr;
  const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess) return e;
  static_scratch_ptr[device] = static_cast<int32_t*>(p);
  return hipSuccess;
}

// A free slot of the device for a new handle, -1 when all are taken.
int take_static_slot(int device) {
  std::lock_guard<std::mutex> lock(static_scratch_mu);
  for (int s = 0; s < kStaticSlots; ++s)
    if (!(static_slots_taken[device] & (1u << s))) {
      static_slots_taken[device] |= 1u << s;
      return s;
    }
  return -1;
}

void release_static_slot(int device, int slot) {
  if (slot < 0 || device < 0 || device >= kMaxDevices) return;
  std::lock_guard<std::mutex> lock(static_scratch_mu);
  static_slots_taken[device] &= ~(1u << slot);
}

}  // namespace

struct et_context {
  int device = 0;
  std::mutex mu;                   // serialises the calls on this handle
  std::mutex err_mu;               // guards last_error alone: a failure may be recorded before `mu` is taken
  std::string last_error;          // the last failure on this handle by any thread
  // et_input_static: the handle's slot of the device's static scratch (-1: none), and the stream its calls are bound to
  int static_slot = -1;
  bool static_stream_set = false;
  hipStream_t static_stream = nullptr;
};

namespace {

// The calling thread's last failure and the handle it happened on (null: without a handle).  et_last_error prefers it,
// so a thread reads its own message whatever other threads do on the same handle in the meantime.
thread_local std::string tls_error;
thread_local et_handle tls_error_handle = nullptr;
thread_local std::string tls_error_copy;      // et_last_error's copy of another thread's message

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

et_status fail(et_handle h, et_status s, const std::string& msg) {
  std::string full = std::string("[ET][ERROR] ") + et_status_string(s) + ": " + msg;
  if (h) {
    std::lock_guard<std::mutex> lock(h->err_mu);
    h->last_error = full;
  }
  tls_error = std::move(full);
  tls_error_handle = h;
  return s;
}

et_status check_hip(et_handle h, hipError_t e, const char* what, const char* file, int line) {
  if (e == hipSuccess) return ET_OK;
  return fail(h, ET_RUNTIME_ERROR,
              std::string(what) + ": " + hipGetErrorString(e) + " " + file + ":" + std::to_string(line));
}

et_status check_launch(et_handle h, const char* what) {
  const hipError_t attr = et::take_attribute_error();
  if (attr != hipSuccess) {
    (void)hipGetLastError();
    return fail(h, ET_RUNTIME_ERROR, std::string(what) + ": raising the kernel's LDS limit failed: " + hipGetErrorString(attr));
  }
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return ET_OK;
  return fail(h, ET_LAUNCH_FAILURE, std::string(what) + ": " + hipGetErrorString(e));
}

#define ET_HIP(h, call)                                                        \
  do {                                                                         \
    et_status _s = check_hip((h), (call), #call, __FILE__, __LINE__);          \
    if (_s != ET_OK) return _s;                                                \
  } while (0)

#define ET_REQUIRE(h, cond, msg)                                               \
  do {                                                                         \
    if (!(cond)) return fail((h), ET_INVALID_ARGUMENT, (msg));                 \
  } while (0)

bool dtype_ok(et_dtype d) { return d == ET_FP32 || d == ET_FP16; }
et::DType to_dt(et_dtype d) { return d == ET_FP32 ? et::DType::F32 : et::DType::F16; }

struct LayerWs {
  size_t qkv, ctx, attn, inter, seq, wt, total;
};

LayerWs layer_ws(et_dtype dtype, int B, int S, int heads, int d) {
  const size_t e = dtype == ET_FP32 ? 4 : 2;
  const size_t rows = (size_t)B * S, H = (size_t)heads * d;
  LayerWs w;
  size_t off = 0;
  w.qkv = off;   off += align_up(rows * 3 * H * e, 256);
  w.ctx = off;   off += align_up(rows * H * e, 256);
  w.attn = off;  off += align_up(rows * H * e, 256);
  // whole tiles of 256 rows: the FFN's intermediate may be handed over in blocks of [256 rows][64 columns]
  w.inter = off; off += align_up(align_up(rows, 256) * 4 * H * e, 256);
  w.seq = off;   off += align_up(et::seq_table_words(B) * sizeof(int32_t), 256);
  // fp16: k-contiguous copies of the six dense kernels (3 H^2 + H^2 + 4 H^2 + 4 H^2 elements) for the large-M GEMM
  w.wt = off;    off += dtype == ET_FP16 ? align_up(12 * H * H * e, 256) : 0;
  w.total = off;
  return w;
}

// First statement of every entry point that takes a handle: rejects a null handle, takes the handle's lock (calls on
// one handle are serialised, and the handle's message slot is only written under it) and makes the handle's device
// current for the calling thread.
struct Entry {
  std::unique_lock<std::mutex> lock;
  et_status status = ET_OK;
  explicit Entry(et_handle h) {
    if (!h) {
      status = fail(nullptr, ET_INVALID_ARGUMENT, "null handle");
      return;
    }
    lock = std::unique_lock<std::mutex>(h->mu);
    status = check_hip(h, hipSetDevice(h->device), "hipSetDevice", __FILE__, __LINE__);
  }
};

et_status dims_ok(et_handle h, int B, int S, int heads, int d) {
  ET_REQUIRE(h, B >= 1 && S >= 1 && heads >= 1 && d >= 1, "batch_size, seq_len, head_num, size_per_head must be >= 1");
  ET_REQUIRE(h, (long)B * S < (1L << 30), "batch_size * seq_len too large");
  // row widths and their multiples (3 H, 4 H, bytes per row) are held in 32-bit integers throughout
  ET_REQUIRE(h, (long)heads * d <= (1L << 20), "head_num * size_per_head above 1048576");
  return ET_OK;
}

// the attention kernels put the sequence on a grid dimension that holds 65535 entries
et_status batch_fits_grid(et_handle h, int B) {
  if (B > 65535) return fail(h, ET_UNSUPPORTED, "batch_size above 65535 is not supported by the attention kernels");
  return ET_OK;
}

float softmax_scaler(et_dtype dtype, int d) {
  float s = 1.0f / sqrtf((float)d);
  if (dtype == ET_FP16) s = (float)(_Float16)s;   // the reference holds the scaler in the element type
  return s;
}

}  // namespace

extern "C" {

const char* et_status_string(et_status s) {
  switch (s) {
    case ET_OK: return "ET_OK";
    case ET_INVALID_ARGUMENT: return "ET_INVALID_ARGUMENT";
    case ET_WORKSPACE_TOO_SMALL: return "ET_WORKSPACE_TOO_SMALL";
    case ET_UNSUPPORTED: return "ET_UNSUPPORTED";
    case ET_LAUNCH_FAILURE: return "ET_LAUNCH_FAILURE";
    case ET_RUNTIME_ERROR: return "ET_RUNTIME_ERROR";
  }
  return "<unknown>";
}

int et_device_ok(int device) {
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess) return 0;
  return std::strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
}

et_status et_create(et_handle* out, int device) {
  if (!out) return fail(nullptr, ET_INVALID_ARGUMENT, "null output handle");
  *out = nullptr;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess) return fail(nullptr, ET_RUNTIME_ERROR, std::string("hipGetDeviceCount: ") + hipGetErrorString(e));
  if (device < 0 || device >= count) return fail(nullptr, ET_INVALID_ARGUMENT, "no such device");
  if (!et_device_ok(device)) return fail(nullptr, ET_UNSUPPORTED, "device is not gfx950; the kernels are built for MI355X only");
  {
    // the address of the static scratch array on this device (et_input_static), looked up with the device current
    int prev = 0;
    e = hipGetDevice(&prev);
    if (e == hipSuccess) e = hipSetDevice(device);
    if (e == hipSuccess) {
      e = resolve_static_scratch(device);
      (void)hipSetDevice(prev);
    }
    if (e != hipSuccess)
      return fail(nullptr, ET_RUNTIME_ERROR, std::string("static scratch lookup: ") + hipGetErrorString(e));
  }
  et_context* c = new (std::nothrow) et_context();
  if (!c) return fail(nullptr, ET_RUNTIME_ERROR, "out of host memory");
  c->device = device;
  c->static_slot = device < kMaxDevices ? take_static_slot(device) : -1;
  *out = c;
  return ET_OK;
}

et_status et_destroy(et_handle h) {
  if (!h) return ET_OK;
  release_static_slot(h->device, h->static_slot);
  if (tls_error_handle == h) tls_error_handle = nullptr;
  delete h;
  return ET_OK;
}

const char* et_last_error(et_handle h) {
  if (tls_error_handle == h) return tls_error.c_str();       // this thread's own last failure (on h, or without a handle)
  if (!h) return "";
  std::lock_guard<std::mutex> lock(h->err_mu);
  tls_error_copy = h->last_error;
  return tls_error_copy.c_str();
}

size_t et_input_workspace_bytes(int batch_size, int seq_len) {
  if (batch_size < 1 || seq_len < 1) return 0;
  return align_up((et::scan_scratch_words(batch_size * seq_len) + 1) * sizeof(int32_t), 256);
}

size_t et_layer_workspace_bytes(et_dtype dtype, int batch_size, int seq_len, int head_num, int size_per_head) {
  if (batch_size < 1 || seq_len < 1 || head_num < 1 || size_per_head < 1 || !dtype_ok(dtype)) return 0;
  return layer_ws(dtype, batch_size, seq_len, head_num, size_per_head).total;
}

size_t et_seq_workspace_bytes(int batch_size) {
  if (batch_size < 1) return 0;
  return align_up(et::seq_table_words(batch_size) * sizeof(int32_t), 256);
}

et_status et_input(et_handle h, et_dtype dtype, const void* from_tensor, const int32_t* mask, void* to_tensor,
                   int32_t* valid_word_num_dev, int32_t* batch_idx, int32_t* word_idx, int batch_size, int seq_len,
                   int head_num, int size_per_head, void* workspace, size_t workspace_bytes, void* stream,
                   int32_t* valid_word_num_host) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, seq_len, head_num, size_per_head)) != ET_OK) return s;
  ET_REQUIRE(h, from_tensor && mask && to_tensor && valid_word_num_dev && batch_idx && word_idx, "null tensor pointer");
  ET_REQUIRE(h, workspace != nullptr, "null workspace");
  if (workspace_bytes < et_input_workspace_bytes(batch_size, seq_len))
    return fail(h, ET_WORKSPACE_TOO_SMALL, "et_input needs et_input_workspace_bytes(batch_size, seq_len)");
  const size_t row_bytes = (size_t)head_num * size_per_head * et::elem_size(to_dt(dtype));
  if (et::move_chunks(batch_size * seq_len, (int)row_bytes) >= (1ull << 31))
    return fail(h, ET_UNSUPPORTED, "tensor too large for one launch");
  hipStream_t st = (hipStream_t)stream;
  et::launch_scan_index(mask, batch_size * seq_len, nullptr, batch_idx, word_idx, valid_word_num_dev, seq_len,
                        (int32_t*)workspace, st);
  if ((s = check_launch(h, "mask scan")) != ET_OK) return s;
  et::launch_compress_rows(from_tensor, to_tensor, batch_idx, word_idx, valid_word_num_dev, nullptr, nullptr,
                           batch_size, seq_len, (int)row_bytes, st);
  if ((s = check_launch(h, "compress")) != ET_OK) return s;
  if (valid_word_num_host) {
    ET_HIP(h, hipMemcpyAsync(valid_word_num_host, valid_word_num_dev, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    ET_HIP(h, hipStreamSynchronize(st));
  }
  return ET_OK;
}

et_status et_input_static(et_handle h, et_dtype dtype, const void* from_tensor, const int32_t* mask, void* to_tensor,
                          int32_t* valid_word_num_dev, int32_t* batch_idx, int32_t* word_idx, int batch_size,
                          int seq_len, int head_num, int size_per_head, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, seq_len, head_num, size_per_head)) != ET_OK) return s;
  ET_REQUIRE(h, from_tensor && mask && to_tensor && valid_word_num_dev && batch_idx && word_idx, "null tensor pointer");
  if ((long)batch_size * seq_len > kStaticMaxPositions ||
      et::scan_scratch_words(batch_size * seq_len) > (size_t)kStaticSlotWords)
    return fail(h, ET_UNSUPPORTED,
                "et_input_static holds scratch for batch_size * seq_len <= 1048576 positions; larger batches go "
                "through et_input with a caller workspace");
  if (h->static_slot < 0)
    return fail(h, ET_UNSUPPORTED,
                "this handle holds no slot of the static scratch (at most 8 live handles per GPU do); use et_input");
  const size_t row_bytes = (size_t)head_num * size_per_head * et::elem_size(to_dt(dtype));
  if (et::move_chunks(batch_size * seq_len, (int)row_bytes) >= (1ull << 31))
    return fail(h, ET_UNSUPPORTED, "tensor too large for one launch");
  int32_t* scratch_dev = h->device < kMaxDevices ? static_scratch_ptr[h->device] : nullptr;
  if (!scratch_dev) return fail(h, ET_RUNTIME_ERROR, "no static scratch on this device");
  scratch_dev += (size_t)h->static_slot * kStaticSlotWords;
  // Calls that share a slot must not overlap on the GPU.  Calls queued on one stream cannot; a call on another stream
  // is accepted only once everything queued on the previous one has finished.
  hipStream_t st = (hipStream_t)stream;
  if (h->static_stream_set && h->static_stream != st) {
    // (any other answer than "not ready", e.g. for a stream that no longer exists, lets the call through)
    const hipError_t q = hipStreamQuery(h->static_stream);
    if (q != hipSuccess) (void)hipGetLastError();
    if (q == hipErrorNotReady) {
      return fail(h, ET_INVALID_ARGUMENT,
                  "et_input_static: the stream of this handle's previous call still has work in flight, and calls on "
                  "two streams would share the handle's scratch slot; wait for that stream or use a second handle");
    }
  }
  h->static_stream_set = true;
  h->static_stream = st;
  // the scan writes every tile total it later reads, so nothing of the previous call's contents has to be cleared
  et::launch_scan_index(mask, batch_size * seq_len, nullptr, batch_idx, word_idx, valid_word_num_dev, seq_len,
                        scratch_dev, st);
  if ((s = check_launch(h, "mask scan")) != ET_OK) return s;
  et::launch_compress_rows(from_tensor, to_tensor, batch_idx, word_idx, valid_word_num_dev, nullptr, nullptr,
                           batch_size, seq_len, (int)row_bytes, st);
  return check_launch(h, "compress");
}

et_status et_embedding_input(et_handle h, et_dtype dtype, const et_embedding_weights* emb, const int32_t* input_ids,
                             const int32_t* token_type_ids, const int32_t* mask, void* to_tensor,
                             int32_t* valid_word_num_dev, int32_t* batch_idx, int32_t* word_idx, int batch_size,
                             int seq_len, int head_num, int size_per_head, void* workspace, size_t workspace_bytes,
                             void* stream, int32_t* valid_word_num_host) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, seq_len, head_num, size_per_head)) != ET_OK) return s;
  ET_REQUIRE(h, emb != nullptr, "null embeddings");
  ET_REQUIRE(h, emb->word_embeddings && emb->layernorm_gamma && emb->layernorm_beta, "null embedding table or LayerNorm weight");
  ET_REQUIRE(h, emb->vocab_size >= 1, "vocab_size must be >= 1");
  ET_REQUIRE(h, (emb->token_type_embeddings == nullptr) == (token_type_ids == nullptr),
             "token_type_ids and token_type_embeddings go together");
  ET_REQUIRE(h, emb->token_type_embeddings == nullptr || emb->type_vocab_size >= 1, "type_vocab_size must be >= 1");
  ET_REQUIRE(h, emb->position_embeddings == nullptr || seq_len <= emb->max_position_embeddings,
             "seq_len exceeds max_position_embeddings");
  ET_REQUIRE(h, input_ids && mask && to_tensor && valid_word_num_dev && batch_idx && word_idx, "null tensor pointer");
  ET_REQUIRE(h, workspace != nullptr, "null workspace");
  if (workspace_bytes < et_input_workspace_bytes(batch_size, seq_len))
    return fail(h, ET_WORKSPACE_TOO_SMALL, "et_embedding_input needs et_input_workspace_bytes(batch_size, seq_len)");
  const int H = head_num * size_per_head;
  if (!et::layernorm_row_in_registers(to_dt(dtype), H))
    return fail(h, ET_UNSUPPORTED, "hidden size not supported by the embedding kernel (even, at most 4096)");
  hipStream_t st = (hipStream_t)stream;
  et::launch_scan_index(mask, batch_size * seq_len, nullptr, batch_idx, word_idx, valid_word_num_dev, seq_len,
                        (int32_t*)workspace, st);
  if ((s = check_launch(h, "mask scan")) != ET_OK) return s;
  et::launch_embed_layernorm(to_dt(dtype), to_tensor, input_ids, token_type_ids, batch_idx, word_idx,
                             emb->word_embeddings, emb->vocab_size, emb->token_type_embeddings, emb->type_vocab_size,
                             emb->position_embeddings, emb->max_position_embeddings, emb->layernorm_gamma,
                             emb->layernorm_beta, batch_size * seq_len, H, seq_len, valid_word_num_dev, st);
  if ((s = check_launch(h, "embedding")) != ET_OK) return s;
  if (valid_word_num_host) {
    ET_HIP(h, hipMemcpyAsync(valid_word_num_host, valid_word_num_dev, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    ET_HIP(h, hipStreamSynchronize(st));
  }
  return ET_OK;
}

et_status et_layer(et_handle h, et_dtype dtype, const et_layer_weights* w, const void* from_tensor,
                   const void* to_tensor, const void* attr_mask, const int32_t* valid_word_num_dev,
                   const int32_t* batch_idx, const int32_t* word_idx, void* out, int batch_size, int from_seq_len,
                   int to_seq_len, int head_num, int size_per_head, int valid_word_num_hint, void* workspace,
                   size_t workspace_bytes, void* stream) {
  return et_layer_with_prepared(h, dtype, w, nullptr, from_tensor, to_tensor, attr_mask, valid_word_num_dev, batch_idx,
                                word_idx, out, batch_size, from_seq_len, to_seq_len, head_num, size_per_head,
                                valid_word_num_hint, workspace, workspace_bytes, stream);
}

et_status et_sequence_starts(et_handle h, const int32_t* batch_idx, const int32_t* valid_word_num_dev, int batch_size,
                             int seq_len, int32_t* seq_start, size_t seq_start_bytes, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  if ((s = dims_ok(h, batch_size, seq_len, 1, 1)) != ET_OK) return s;
  ET_REQUIRE(h, batch_idx && valid_word_num_dev && seq_start, "null tensor pointer");
  if (seq_start_bytes < et_seq_workspace_bytes(batch_size))
    return fail(h, ET_WORKSPACE_TOO_SMALL, "the sequence table needs et_seq_workspace_bytes(batch_size)");
  et::launch_seq_start(batch_idx, valid_word_num_dev, batch_size * seq_len, batch_size, seq_start, (hipStream_t)stream);
  return check_launch(h, "sequence starts");
}

et_status et_layer_with_prepared(et_handle h, et_dtype dtype, const et_layer_weights* w, const et_layer_prepared* prep,
                                 const void* from_tensor, const void* to_tensor, const void* attr_mask,
                                 const int32_t* valid_word_num_dev, const int32_t* batch_idx, const int32_t* word_idx,
                                 void* out, int batch_size, int from_seq_len, int to_seq_len, int head_num,
                                 int size_per_head, int valid_word_num_hint, void* workspace, size_t workspace_bytes,
                                 void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, from_seq_len, head_num, size_per_head)) != ET_OK) return s;
  ET_REQUIRE(h, from_seq_len == to_seq_len, "only support from_seq_len == to_seq_len");
  ET_REQUIRE(h, w != nullptr, "null weights");
  ET_REQUIRE(h, w->attr_kernel_Q && w->attr_kernel_K && w->attr_kernel_V && w->attr_bias_Q && w->attr_bias_K &&
                    w->attr_bias_V && w->attr_output_kernel && w->attr_output_bias && w->attr_output_layernorm_gamma &&
                    w->attr_output_layernorm_beta && w->inter_kernel && w->inter_bias && w->output_kernel &&
                    w->output_bias && w->output_layernorm_gamma && w->output_layernorm_beta,
             "null weight pointer");
  ET_REQUIRE(h, from_tensor && to_tensor && attr_mask && valid_word_num_dev && batch_idx && word_idx && out,
             "null tensor pointer");
  ET_REQUIRE(h, out != from_tensor && out != to_tensor, "out must not alias from_tensor / to_tensor");
  ET_REQUIRE(h, workspace != nullptr, "null workspace");
  const int B = batch_size, S = from_seq_len, H = head_num * size_per_head, F = 4 * H;
  ET_REQUIRE(h, valid_word_num_hint >= -1 && valid_word_num_hint <= B * S, "valid_word_num_hint out of range");
  const LayerWs ws = layer_ws(dtype, B, S, head_num, size_per_head);
  if (workspace_bytes < ws.total) return fail(h, ET_WORKSPACE_TOO_SMALL, "et_layer needs et_layer_workspace_bytes(...)");
  const et::DType dt = to_dt(dtype);
  if ((s = batch_fits_grid(h, B)) != ET_OK) return s;
  if (!et::attention_supported(dt, S, size_per_head))
    return fail(h, ET_UNSUPPORTED, "attention needs size_per_head <= 256 and seq_len <= 1024");
  if (!et::gemm_supported(dt, H, H, 3) || !et::gemm_supported(dt, F, H, 1) || !et::gemm_supported(dt, H, F, 1))
    return fail(h, ET_UNSUPPORTED, "hidden size not supported by the GEMM kernels");
  if ((uint64_t)B * S * F * et::elem_size(dt) > 0xffffffffull)
    return fail(h, ET_UNSUPPORTED, "activation matrix larger than 4 GB");
  if (!et::bias_gelu_supported(dt, F) || !et::bias_residual_layernorm_supported(dt, H))
    return fail(h, ET_UNSUPPORTED, "hidden size not supported by the row kernels");
  if (valid_word_num_hint == 0) return ET_OK;
  const int rows = valid_word_num_hint > 0 ? valid_word_num_hint : B * S;
  const int32_t* T = valid_word_num_dev;
  hipStream_t st = (hipStream_t)stream;
  const size_t e = et::elem_size(dt);
  char* base = (char*)workspace;
  void* qkv = base + ws.qkv;
  void* ctx = base + ws.ctx;
  void* attn = base + ws.attn;
  void* inter = base + ws.inter;
  int32_t* seq_start = (int32_t*)(base + ws.seq);

  // The large-M fp16 GEMM reads k-contiguous weights with fewer LDS instructions.  Where the caller prepared such
  // copies they are used wherever that kernel runs; otherwise the wide projections get a transposed copy in the
  // workspace on every call (the caller's weights stay as they are).
  static const et_layer_prepared kNoPrep = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0};
  const et_layer_prepared& pp = prep ? *prep : kNoPrep;
  if (pp.seq_start && pp.seq_start_bytes < et_seq_workspace_bytes(B))
    return fail(h, ET_WORKSPACE_TOO_SMALL, "et_layer_prepared.seq_start needs et_seq_workspace_bytes(batch_size) bytes");
  ET_REQUIRE(h, (pp.attr_kernel_Q_t != nullptr) == (pp.attr_kernel_K_t != nullptr) &&
                    (pp.attr_kernel_Q_t != nullptr) == (pp.attr_kernel_V_t != nullptr),
             "prepared Q, K and V kernels go together");
  const bool can_qkv = et::gemm_takes_transposed_b(dt, rows, 3 * H, H, H, 3);
  const bool can_o = et::gemm_takes_transposed_b(dt, rows, H, H, H, 1);
  const bool can_up = et::gemm_takes_transposed_b(dt, rows, F, F, H, 1);
  const bool can_down = et::gemm_takes_transposed_b(dt, rows, H, H, F, 1);
  const bool t_qkv = can_qkv && (pp.attr_kernel_Q_t || et::gemm_prefers_transposed_b(dt, rows, 3 * H, H, H, 3));
  const bool t_o = can_o && (pp.attr_output_kernel_t || et::gemm_prefers_transposed_b(dt, rows, H, H, H, 1));
  const bool t_up = can_up && (pp.inter_kernel_t || et::gemm_prefers_transposed_b(dt, rows, F, F, H, 1));
  const bool t_down = can_down && (pp.output_kernel_t || et::gemm_prefers_transposed_b(dt, rows, H, H, F, 1));
  char* wt = base + ws.wt;
  const size_t HH = (size_t)H * H * e;
  const void* wt_q = wt; const void* wt_k = wt + HH; const void* wt_v = wt + 2 * HH; const void* wt_o = wt + 3 * HH;
  const void* wt_up = wt + 4 * HH; const void* wt_down = wt + 8 * HH;
  {
    et::TransposeJobs jobs;
    if (t_qkv && pp.attr_kernel_Q_t) {
      wt_q = pp.attr_kernel_Q_t; wt_k = pp.attr_kernel_K_t; wt_v = pp.attr_kernel_V_t;
    } else if (t_qkv) {
      jobs.add(w->attr_kernel_Q, wt, H, H);
      jobs.add(w->attr_kernel_K, wt + HH, H, H);
      jobs.add(w->attr_kernel_V, wt + 2 * HH, H, H);
    }
    if (t_o && pp.attr_output_kernel_t) wt_o = pp.attr_output_kernel_t;
    else if (t_o) jobs.add(w->attr_output_kernel, wt + 3 * HH, H, H);
    if (t_up && pp.inter_kernel_t) wt_up = pp.inter_kernel_t;
    else if (t_up) jobs.add(w->inter_kernel, wt + 4 * HH, H, F);
    if (t_down && pp.output_kernel_t) wt_down = pp.output_kernel_t;
    else if (t_down) jobs.add(w->output_kernel, wt + 8 * HH, F, H);
    // one launch builds the sequence start table and the transposed copies; none when the caller prepared both
    const et::SeqStartJob seq{batch_idx, T, rows, B, seq_start};
    if (pp.seq_start) seq_start = const_cast<int32_t*>(pp.seq_start);
    et::launch_transpose_weights(jobs, st, pp.seq_start ? nullptr : &seq);
  }
  // Every matrix of the layer is read again by the kernel after the one that wrote it.  While the layer's matrices
  // (from, Q/K/V, context, attention output, [T,4H], out) about fit the last-level cache, the GEMMs leave their
  // outputs there (plain stores); beyond that the outputs would only displace the weights and the A rows.
  const bool cached = (double)rows * (7.0 * H + F) * (double)e <= kCachedLayerBytes;
  // Q = from.Wq + bq, K = to.Wk + bk, V = to.Wv + bv into one [T,3H] buffer (bert_transformer_op.cu.cc:105-156)
  et::GemmGroups g3;
  g3.groups = 3;
  g3.c_cached = cached;
  g3.A[0] = from_tensor; g3.A[1] = to_tensor; g3.A[2] = to_tensor;
  g3.B[0] = t_qkv ? wt_q : w->attr_kernel_Q; g3.B[1] = t_qkv ? wt_k : w->attr_kernel_K; g3.B[2] = t_qkv ? wt_v : w->attr_kernel_V;
  g3.bias[0] = w->attr_bias_Q; g3.bias[1] = w->attr_bias_K; g3.bias[2] = w->attr_bias_V;
  g3.b_transposed = t_qkv;
  et::launch_gemm(dt, g3, qkv, 3 * H, rows, H, H, T, st);
  if ((s = check_launch(h, "QKV projection")) != ET_OK) return s;
  // QK^T, softmax, PV, un-pad (:159-192)
  et::launch_attention(dt, qkv, (char*)qkv + (size_t)H * e, (char*)qkv + (size_t)2 * H * e, 1, 3 * H, attr_mask, ctx,
                       seq_start, word_idx, B, S, head_num, size_per_head, softmax_scaler(dtype, size_per_head), st);
  if ((s = check_launch(h, "attention")) != ET_OK) return s;
  // attention output projection + bias + residual(from_tensor) + LayerNorm (:195-213)
  et::GemmGroups g1;
  g1.groups = 1;
  g1.c_cached = cached;
  g1.A[0] = ctx; g1.B[0] = t_o ? wt_o : w->attr_output_kernel; g1.bias[0] = nullptr;
  g1.b_transposed = t_o;
  et::launch_gemm(dt, g1, attn, H, rows, H, H, T, st);
  // Every weight matrix was last read a whole batch ago, and a GEMM's first round of tiles waits for each cold slice of
  // it (13000 rows: FFN-down 63 us with cold weights, 53 with the weights in the last-level cache; 2 .. 3 us for the
  // other projections).  The two LayerNorm kernels request the matrices that come next on their way, for batches in
  // which those are small beside what the kernel moves anyway: this one the FFN-up weights and, while the layer's
  // matrices are small enough for them to survive FFN-up, the FFN-down weights (12-layer BERT-base: -3 % at 4000
  // tokens, -4.4 % at 8000 and 12000, -1 % at 16000); the last one the region the caller names, the next layer's
  // attention weights (another -0.7 .. -1.6 % from 4000 to 40000 tokens, FFN-up included).
  const bool warm_fits = (double)rows * (7.0 * H + F) * (double)e <= kWarmLayerBytes;
  et::WarmList warm1, warm2;
  // (whichever copy the GEMM reads, unless this call has just written it)
  const void* b_up = t_up ? wt_up : w->inter_kernel;
  const void* b_down = t_down ? wt_down : w->output_kernel;
  if (rows >= F && !(t_up && !pp.inter_kernel_t)) warm1.add(b_up, (size_t)H * F * e);
  if (rows >= F && warm_fits && !(t_down && !pp.output_kernel_t)) warm1.add(b_down, (size_t)H * F * e);
  if (rows >= F) warm2.add(pp.warm, pp.warm_bytes);
  et::launch_bias_residual_layernorm(dt, attn, from_tensor, w->attr_output_bias, w->attr_output_layernorm_gamma,
                                     w->attr_output_layernorm_beta, rows, H, T, st, warm1);
  if ((s = check_launch(h, "attention output")) != ET_OK) return s;
  // FFN up + bias + GELU (:215-227, cuda/cuda_kernels.cu:88-150)
  g1.A[0] = attn; g1.B[0] = t_up ? wt_up : w->inter_kernel;
  g1.b_transposed = t_up;
  // bias + GELU are applied to each tile on its way out of the GEMM: no pass of its own over [T,4H]
  g1.bias[0] = w->inter_bias; g1.gelu = true;
  // where both FFN projections run the persistent k-contiguous kernel, [T,4H] goes from one to the other in blocks
  const bool blocked = t_up && t_down && et::gemm_blocked_handover(dt, rows, F, H);
  g1.c_blocked = blocked;
  et::launch_gemm(dt, g1, inter, F, rows, F, H, T, st);
  g1.bias[0] = nullptr; g1.gelu = false; g1.c_blocked = false;
  if ((s = check_launch(h, "FFN up")) != ET_OK) return s;
  // FFN down + bias + residual(LN1 output) + LayerNorm (:229-247)
  g1.A[0] = inter; g1.B[0] = t_down ? wt_down : w->output_kernel;
  g1.b_transposed = t_down;
  g1.a_blocked = blocked;
  et::launch_gemm(dt, g1, out, H, rows, H, F, T, st);
  g1.a_blocked = false;
  et::launch_bias_residual_layernorm(dt, out, attn, w->output_bias, w->output_layernorm_gamma,
                                     w->output_layernorm_beta, rows, H, T, st, warm2);
  if ((s = check_launch(h, "FFN down")) != ET_OK) return s;
  return ET_OK;
}

et_status et_output(et_handle h, et_dtype dtype, const void* from_tensor, const int32_t* valid_word_num_dev,
                    const int32_t* batch_idx, const int32_t* word_idx, void* to_tensor, int batch_size, int seq_len,
                    int head_num, int size_per_head, void* stream) {
  if (head_num < 1 || size_per_head < 1 || (long)head_num * size_per_head >= (1L << 30))
    return fail(h, ET_INVALID_ARGUMENT, "head_num, size_per_head must be >= 1");
  return et_restore(h, dtype, to_tensor, from_tensor, batch_idx, word_idx, valid_word_num_dev, batch_size, seq_len,
                    head_num * size_per_head, stream);
}

et_status et_first_token(et_handle h, et_dtype dtype, const void* from_tensor, const int32_t* valid_word_num_dev,
                         const int32_t* batch_idx, const int32_t* word_idx, void* to_tensor, int batch_size,
                         int seq_len, int hidden_dim, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, seq_len, 1, hidden_dim)) != ET_OK) return s;
  ET_REQUIRE(h, from_tensor && to_tensor && valid_word_num_dev && batch_idx && word_idx, "null tensor pointer");
  const size_t row_bytes = (size_t)hidden_dim * et::elem_size(to_dt(dtype));
  et::launch_first_token(to_tensor, from_tensor, batch_idx, word_idx, valid_word_num_dev, batch_size * seq_len,
                         batch_size, (int)row_bytes, (hipStream_t)stream);
  return check_launch(h, "first token gather");
}

et_status et_exclusive_scan(et_handle h, int32_t* d_out, const int32_t* d_in, int length, void* workspace,
                            size_t workspace_bytes, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, d_out && d_in, "null tensor pointer");
  ET_REQUIRE(h, length >= 1 && length < (1 << 30), "length out of range");
  ET_REQUIRE(h, workspace != nullptr, "null workspace");
  if (workspace_bytes < et_input_workspace_bytes(1, length))
    return fail(h, ET_WORKSPACE_TOO_SMALL, "et_exclusive_scan needs et_input_workspace_bytes(1, length)");
  et::launch_scan_index(d_in, length, d_out, nullptr, nullptr, nullptr, 0, (int32_t*)workspace, (hipStream_t)stream);
  return check_launch(h, "exclusive scan");
}

et_status et_compress(et_handle h, et_dtype dtype, const void* from_tensor, const int32_t* mask,
                      const int32_t* prefix_sum, void* to_tensor, int32_t* batch_idx, int32_t* word_idx,
                      int batch_size, int seq_len, int hidden_dim, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, seq_len, 1, hidden_dim)) != ET_OK) return s;
  ET_REQUIRE(h, from_tensor && mask && prefix_sum && to_tensor && batch_idx && word_idx, "null tensor pointer");
  const size_t row_bytes = (size_t)hidden_dim * et::elem_size(to_dt(dtype));
  if (et::move_chunks(batch_size * seq_len, (int)row_bytes) >= (1ull << 31))
    return fail(h, ET_UNSUPPORTED, "tensor too large for one launch");
  hipStream_t st = (hipStream_t)stream;
  et::launch_index_from_prefix(mask, prefix_sum, batch_idx, word_idx, batch_size, seq_len, st);
  et::launch_compress_rows(from_tensor, to_tensor, batch_idx, word_idx, nullptr, prefix_sum, mask, batch_size, seq_len,
                           (int)row_bytes, st);
  return check_launch(h, "compress");
}

et_status et_restore(et_handle h, et_dtype dtype, void* to_tensor, const void* from_tensor, const int32_t* batch_idx,
                     const int32_t* word_idx, const int32_t* valid_word_num_dev, int batch_size, int seq_len,
                     int hidden_dim, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, seq_len, 1, hidden_dim)) != ET_OK) return s;
  ET_REQUIRE(h, from_tensor && to_tensor && valid_word_num_dev && batch_idx && word_idx, "null tensor pointer");
  const size_t row_bytes = (size_t)hidden_dim * et::elem_size(to_dt(dtype));
  if (et::move_chunks(batch_size * seq_len, (int)row_bytes) >= (1ull << 31))
    return fail(h, ET_UNSUPPORTED, "tensor too large for one launch");
  et::launch_restore_rows(to_tensor, from_tensor, batch_idx, word_idx, valid_word_num_dev, batch_size, seq_len,
                          (int)row_bytes, (hipStream_t)stream);
  return check_launch(h, "restore");
}

et_status et_add_bias_act(et_handle h, et_dtype dtype, void* out, const void* bias, int m, int n,
                          const int32_t* m_dev, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  ET_REQUIRE(h, out && bias, "null tensor pointer");
  ET_REQUIRE(h, m >= 0 && n >= 1, "bad dimensions");
  if (!et::bias_gelu_supported(to_dt(dtype), n)) return fail(h, ET_UNSUPPORTED, "row bytes must be a multiple of 16");
  if (m == 0) return ET_OK;
  et::launch_bias_gelu(to_dt(dtype), out, bias, m, n, m_dev, (hipStream_t)stream);
  return check_launch(h, "bias + gelu");
}

et_status et_add_bias_input_layernorm(et_handle h, et_dtype dtype, void* out, const void* input, const void* bias,
                                      const void* gamma, const void* beta, int m, int n, const int32_t* m_dev,
                                      void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  ET_REQUIRE(h, out && input && bias && gamma && beta, "null tensor pointer");
  ET_REQUIRE(h, m >= 0 && n >= 1, "bad dimensions");
  if (!et::bias_residual_layernorm_supported(to_dt(dtype), n))
    return fail(h, ET_UNSUPPORTED, "row length not supported by the LayerNorm kernel");
  if (m == 0) return ET_OK;
  et::launch_bias_residual_layernorm(to_dt(dtype), out, input, bias, gamma, beta, m, n, m_dev, (hipStream_t)stream);
  return check_launch(h, "bias + residual + layernorm");
}

et_status et_add_qkv_bias_padding(et_handle h, et_dtype dtype, const void* Q, const void* bias_Q, const void* K,
                                  const void* bias_K, const void* V, const void* bias_V, void* q_buf, void* k_buf,
                                  void* v_buf, const int32_t* valid_word_num_dev, int batch_size, int seq_len,
                                  int head_num, int size_per_head, const int32_t* batch_idx, const int32_t* word_idx,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, seq_len, head_num, size_per_head)) != ET_OK) return s;
  ET_REQUIRE(h, Q && K && V && bias_Q && bias_K && bias_V && q_buf && k_buf && v_buf && valid_word_num_dev &&
                    batch_idx && word_idx,
             "null tensor pointer");
  ET_REQUIRE(h, workspace != nullptr, "null workspace");
  if (workspace_bytes < et_seq_workspace_bytes(batch_size))
    return fail(h, ET_WORKSPACE_TOO_SMALL, "needs et_seq_workspace_bytes(batch_size)");
  if (seq_len > 1024) return fail(h, ET_UNSUPPORTED, "seq_len <= 1024");
  hipStream_t st = (hipStream_t)stream;
  et::launch_seq_start(batch_idx, valid_word_num_dev, batch_size * seq_len, batch_size, (int32_t*)workspace, st);
  et::launch_qkv_bias_pad(to_dt(dtype), Q, bias_Q, K, bias_K, V, bias_V, q_buf, k_buf, v_buf, (int32_t*)workspace,
                          word_idx, batch_size, seq_len, head_num, size_per_head, st);
  return check_launch(h, "qkv bias + padding");
}

et_status et_softmax(et_handle h, et_dtype dtype, void* qk_buf, const void* attr_mask, int batch_size, int head_num,
                     int seq_len, float scaler, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, seq_len, head_num, 1)) != ET_OK) return s;
  ET_REQUIRE(h, qk_buf && attr_mask, "null tensor pointer");
  if (seq_len > 1024) return fail(h, ET_UNSUPPORTED, "softmax kernel supports seq_len <= 1024");
  et::launch_softmax(to_dt(dtype), qk_buf, attr_mask, batch_size, head_num, seq_len, scaler, (hipStream_t)stream);
  return check_launch(h, "softmax");
}

et_status et_transpose_rm_padding(et_handle h, et_dtype dtype, const void* src, void* dst,
                                  const int32_t* valid_word_num_dev, int batch_size, int seq_len, int head_num,
                                  int size_per_head, const int32_t* batch_idx, const int32_t* word_idx, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, seq_len, head_num, size_per_head)) != ET_OK) return s;
  ET_REQUIRE(h, src && dst && valid_word_num_dev && batch_idx && word_idx, "null tensor pointer");
  et::launch_transpose_rm_padding(to_dt(dtype), src, dst, valid_word_num_dev, batch_size * seq_len, batch_size,
                                  seq_len, head_num, size_per_head, batch_idx, word_idx, (hipStream_t)stream);
  return check_launch(h, "transpose + remove padding");
}

et_status et_attention(et_handle h, et_dtype dtype, const void* q, const void* k, const void* v, int qkv_layout,
                       int packed_ld, const void* attr_mask, void* dst, const int32_t* valid_word_num_dev,
                       int batch_size, int seq_len, int head_num, int size_per_head, const int32_t* batch_idx,
                       const int32_t* word_idx, void* workspace, size_t workspace_bytes, void* stream) {
  if (h) {
    ET_REQUIRE(h, workspace != nullptr, "null workspace");
    if (workspace_bytes < et_seq_workspace_bytes(batch_size))
      return fail(h, ET_WORKSPACE_TOO_SMALL, "needs et_seq_workspace_bytes(batch_size)");
  }
  return et_attention_with_starts(h, dtype, q, k, v, qkv_layout, packed_ld, attr_mask, dst, valid_word_num_dev,
                                  batch_size, seq_len, head_num, size_per_head, batch_idx, word_idx, nullptr,
                                  (int32_t*)workspace, workspace_bytes, stream);
}

et_status et_attention_with_starts(et_handle h, et_dtype dtype, const void* q, const void* k, const void* v,
                                   int qkv_layout, int packed_ld, const void* attr_mask, void* dst,
                                   const int32_t* valid_word_num_dev, int batch_size, int seq_len, int head_num,
                                   int size_per_head, const int32_t* batch_idx, const int32_t* word_idx,
                                   const int32_t* seq_start, int32_t* seq_start_scratch, size_t seq_table_bytes,
                                   void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  if ((s = dims_ok(h, batch_size, seq_len, head_num, size_per_head)) != ET_OK) return s;
  ET_REQUIRE(h, q && k && v && attr_mask && dst && valid_word_num_dev && batch_idx && word_idx, "null tensor pointer");
  ET_REQUIRE(h, qkv_layout == 0 || qkv_layout == 1, "qkv_layout must be 0 (padded) or 1 (packed)");
  ET_REQUIRE(h, qkv_layout == 0 || packed_ld >= head_num * size_per_head, "packed_ld smaller than the hidden size");
  ET_REQUIRE(h, seq_start != nullptr || seq_start_scratch != nullptr, "null sequence start table");
  if (seq_table_bytes < et_seq_workspace_bytes(batch_size))
    return fail(h, ET_WORKSPACE_TOO_SMALL, "the sequence table needs et_seq_workspace_bytes(batch_size)");
  if ((s = batch_fits_grid(h, batch_size)) != ET_OK) return s;
  if (!et::attention_supported(to_dt(dtype), seq_len, size_per_head))
    return fail(h, ET_UNSUPPORTED, "attention needs size_per_head <= 256 and seq_len <= 1024");
  hipStream_t st = (hipStream_t)stream;
  if (!seq_start) {
    et::launch_seq_start(batch_idx, valid_word_num_dev, batch_size * seq_len, batch_size, seq_start_scratch, st);
    seq_start = seq_start_scratch;
  }
  et::launch_attention(to_dt(dtype), q, k, v, qkv_layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch_size,
                       seq_len, head_num, size_per_head, softmax_scaler(dtype, size_per_head), st);
  return check_launch(h, "attention");
}

namespace {

et_status gemm_impl(et_handle h, et_dtype dtype, const void* A, const void* B, void* C, const void* bias, int m, int n,
                    int k, const int32_t* m_dev, void* stream, bool gelu, const char* what) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype_ok(dtype), "dtype must be ET_FP32 or ET_FP16");
  ET_REQUIRE(h, A && B && C, "null tensor pointer");
  ET_REQUIRE(h, !gelu || bias, "null bias");
  ET_REQUIRE(h, m >= 0 && n >= 1 && k >= 1, "bad dimensions");
  if (!et::gemm_supported(to_dt(dtype), n, k, 1))
    return fail(h, ET_UNSUPPORTED, "GEMM dimensions out of range");
  if ((uint64_t)m * k * et::elem_size(to_dt(dtype)) > 0xffffffffull)
    return fail(h, ET_UNSUPPORTED, "A larger than 4 GB");
  if (m == 0) return ET_OK;
  et::GemmGroups g;
  g.groups = 1;
  g.A[0] = A; g.B[0] = B; g.bias[0] = bias;
  g.gelu = gelu;
  et::launch_gemm(to_dt(dtype), g, C, n, m, n, k, m_dev, (hipStream_t)stream);
  return check_launch(h, what);
}

}  // namespace

et_status et_gemm(et_handle h, et_dtype dtype, const void* A, const void* B, void* C, const void* bias, int m, int n,
                  int k, const int32_t* m_dev, void* stream) {
  return gemm_impl(h, dtype, A, B, C, bias, m, n, k, m_dev, stream, false, "gemm");
}

et_status et_gemm_bias_gelu(et_handle h, et_dtype dtype, const void* A, const void* B, void* C, const void* bias, int m,
                            int n, int k, const int32_t* m_dev, void* stream) {
  return gemm_impl(h, dtype, A, B, C, bias, m, n, k, m_dev, stream, true, "gemm + bias + gelu");
}

et_status et_transpose_weight(et_handle h, et_dtype dtype, const void* src, void* dst, int k, int n, void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype == ET_FP16, "dtype must be ET_FP16");
  ET_REQUIRE(h, src && dst && src != dst, "null or aliased tensor pointer");
  ET_REQUIRE(h, k >= 1 && n >= 1 && k % 8 == 0 && n % 8 == 0, "k and n must be positive multiples of 8");
  et::TransposeJobs jobs;
  jobs.add(src, dst, k, n);
  et::launch_transpose_weights(jobs, (hipStream_t)stream);
  return check_launch(h, "weight transpose");
}

namespace {

et_status gemm_bt_impl(et_handle h, et_dtype dtype, const void* A, const void* Bt, void* C, const void* bias, int m, int n,
                       int k, const int32_t* m_dev, void* stream, bool gelu, const char* what) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, dtype == ET_FP16, "dtype must be ET_FP16");
  ET_REQUIRE(h, A && Bt && C, "null tensor pointer");
  ET_REQUIRE(h, !gelu || bias, "null bias");
  ET_REQUIRE(h, m >= 0 && n >= 1 && k >= 1, "bad dimensions");
  if ((uint64_t)m * k * 2 > 0xffffffffull) return fail(h, ET_UNSUPPORTED, "A larger than 4 GB");
  if (!et::gemm_takes_transposed_b(et::DType::F16, m, n, n, k, 1))
    return fail(h, ET_UNSUPPORTED,
                std::string(what) + " needs k % 64 == 0 and n % 8 == 0");
  et::GemmGroups g;
  g.groups = 1;
  g.A[0] = A; g.B[0] = Bt; g.bias[0] = bias;
  g.b_transposed = true;
  g.gelu = gelu;
  g.c_cached = (double)m * ((double)k + n) * 2.0 <= kCachedCallBytes;     // A and C together: a small call
  et::launch_gemm(et::DType::F16, g, C, n, m, n, k, m_dev, (hipStream_t)stream);
  return check_launch(h, what);
}

}  // namespace

et_status et_gemm_bt(et_handle h, et_dtype dtype, const void* A, const void* Bt, void* C, const void* bias, int m, int n,
                     int k, const int32_t* m_dev, void* stream) {
  return gemm_bt_impl(h, dtype, A, Bt, C, bias, m, n, k, m_dev, stream, false, "et_gemm_bt");
}

et_status et_gemm_bt_bias_gelu(et_handle h, et_dtype dtype, const void* A, const void* Bt, void* C, const void* bias,
                               int m, int n, int k, const int32_t* m_dev, void* stream) {
  return gemm_bt_impl(h, dtype, A, Bt, C, bias, m, n, k, m_dev, stream, true, "et_gemm_bt_bias_gelu");
}

namespace {
int current_cu_count() {
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess || prop.multiProcessorCount <= 0)
    return 256;
  return prop.multiProcessorCount;
}
}  // namespace

size_t et_calibrate_mfma_sink_bytes(et_handle h) {
  Entry entry(h);
  if (entry.status != ET_OK) return 0;
  return et::mfma_ceiling_sink_bytes(current_cu_count());
}

et_status et_calibrate_mfma(et_handle h, int random_operands, int iters, void* sink, size_t sink_bytes, double* flops,
                            void* stream) {
  Entry entry(h);
  et_status s = entry.status;
  if (s != ET_OK) return s;
  ET_REQUIRE(h, sink && flops, "null pointer");
  ET_REQUIRE(h, iters >= 1 && iters <= (1 << 22), "iters must be in 1 .. 4194304");
  const int cus = current_cu_count();
  if (sink_bytes < et::mfma_ceiling_sink_bytes(cus)) return fail(h, ET_WORKSPACE_TOO_SMALL, "sink buffer too small");
  *flops = et::launch_mfma_ceiling(random_operands != 0, cus, iters, (float*)sink, (hipStream_t)stream);
  return check_launch(h, "MFMA calibration");
}

}  // extern "C"
