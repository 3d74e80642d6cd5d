// Internal launcher interface between the C ABI (et_api.cpp) and the gfx950 kernels.
// Every launcher enqueues on `stream` and returns; none allocates.  Row counts that live on
// the device are passed as `rows_dev` (may be null) next to a host-side upper bound.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace et {

enum class DType : int { F32 = 0, F16 = 1 };
inline size_t elem_size(DType t) { return t == DType::F32 ? 4 : 2; }

// Kernels that need more than 64 KB of dynamic LDS raise the limit once per (kernel, device): the attribute belongs
// to the device a module is loaded on, and a process may hold handles on several GPUs.  (et_api.cpp)
void allow_dynamic_lds(const void* kernel, int bytes);
// The error of a failed allow_dynamic_lds on this thread since the last call (hipSuccess if none); clears it.
hipError_t take_attribute_error();

// ---- input_output.hip --------------------------------------------------------------------
// Number of int32 words of scratch the scan needs for `length` elements.
size_t scan_scratch_words(int length);
// Exclusive prefix sum of `in`; optionally (seq_len > 0) also writes batch_idx / word_idx for
// every element > 0 and the valid-token count.  prefix_out may be null.
void launch_scan_index(const int32_t* in, int length, int32_t* prefix_out, int32_t* batch_idx,
                       int32_t* word_idx, int32_t* valid_word_num, int seq_len, int32_t* scratch,
                       hipStream_t stream);
// batch_idx / word_idx from mask + an existing prefix sum.
void launch_index_from_prefix(const int32_t* mask, const int32_t* prefix, int32_t* batch_idx,
                              int32_t* word_idx, int batch, int seq_len, hipStream_t stream);
// to[t,:] = from[batch_idx[t]*S + word_idx[t], :] for t < T.  T comes from *rows_dev when given,
// otherwise from prefix[last] + (mask[last] == 1).
void launch_compress_rows(const void* from, void* to, const int32_t* batch_idx, const int32_t* word_idx,
                          const int32_t* rows_dev, const int32_t* prefix, const int32_t* mask,
                          int batch, int seq_len, int row_bytes, hipStream_t stream);
// Chunks (16, 4 or 2 bytes: the widest piece row_bytes is a whole number of) the two movers below index for n_pos rows;
// must stay below 2^31.
size_t move_chunks(int n_pos, int row_bytes);
// to[B*S rows] = 0 at padding, from[t] at batch_idx[t]*S + word_idx[t]; indices ascending.
void launch_restore_rows(void* to, const void* from, const int32_t* batch_idx, const int32_t* word_idx,
                         const int32_t* rows_dev, int batch, int seq_len, int row_bytes, hipStream_t stream);
// to[b,:] = packed row at position 0 of sequence b (zeros if there is none); indices ascending.
void launch_first_token(void* to, const void* from, const int32_t* batch_idx, const int32_t* word_idx,
                        const int32_t* rows_dev, int rows_bound, int batch, int row_bytes, hipStream_t stream);
// The sequence table of a batch, 2 B + 1 words: seq_start[b] = first packed row of sequence b, b in [0,B];
// seq_start[B] = T; then the B sequence numbers in the order the attention kernels serve them (longest first).
inline size_t seq_table_words(int batch) { return 2 * (size_t)batch + 1; }
void launch_seq_start(const int32_t* batch_idx, const int32_t* rows_dev, int rows_bound, int batch,
                      int32_t* seq_start, hipStream_t stream);
// second half of the table from its first half (for tables whose first half another kernel wrote)
void launch_seq_order(int32_t* seq_table, int batch, hipStream_t stream);

// ---- row_kernels.hip ---------------------------------------------------------------------
bool bias_gelu_supported(DType t, int n);
void launch_bias_gelu(DType t, void* out, const void* bias, int m, int n, const int32_t* rows_dev,
                      hipStream_t stream);
bool bias_residual_layernorm_supported(DType t, int n);
// rows the wave-per-row kernels keep in registers (n a multiple of 2 in fp16, up to 4096 elements)
bool layernorm_row_in_registers(DType t, int n);
// Regions whose 128-byte lines a kernel requests on its way (pulled into the last-level cache) for a later kernel that
// would otherwise read them cold.
struct WarmList {
  static constexpr int kMax = 3;
  const uint32_t* p[kMax] = {nullptr, nullptr, nullptr};
  int lines[kMax] = {0, 0, 0};
  int total = 0;
  void add(const void* region, size_t bytes);
};
void launch_bias_residual_layernorm(DType t, void* out, const void* input, const void* bias,
                                    const void* gamma, const void* beta, int m, int n,
                                    const int32_t* rows_dev, hipStream_t stream, const WarmList& warm = WarmList());

// out[t,:] = LayerNorm(word[ids[p]] + type[type_ids[p]] + pos[word_idx[t]]) * gamma + beta for packed row t at padded
// position p = batch_idx[t]*seq_len + word_idx[t]; eps 1e-12.  type_ids/type_table and pos_table may be null.
// n must satisfy bias_residual_layernorm_supported.
void launch_embed_layernorm(DType t, void* out, const int32_t* ids, const int32_t* type_ids, const int32_t* batch_idx,
                            const int32_t* word_idx, const void* word_table, int vocab, const void* type_table,
                            int type_vocab, const void* pos_table, int max_pos, const void* gamma, const void* beta,
                            int m, int n, int seq_len, const int32_t* rows_dev, hipStream_t stream);

// ---- attention.hip -----------------------------------------------------------------------
void launch_qkv_bias_pad(DType t, const void* Q, const void* bQ, const void* K, const void* bK,
                         const void* V, const void* bV, void* q_buf, void* k_buf, void* v_buf,
                         const int32_t* seq_start, const int32_t* word_idx, int batch, int seq_len,
                         int heads, int d, hipStream_t stream);
void launch_softmax(DType t, void* qk, const void* attr_mask, int batch, int heads, int seq_len,
                    float scaler, hipStream_t stream);
void launch_transpose_rm_padding(DType t, const void* src, void* dst, const int32_t* rows_dev,
                                 int rows_bound, int batch, int seq_len, int heads, int d,
                                 const int32_t* batch_idx, const int32_t* word_idx, hipStream_t stream);
bool attention_supported(DType t, int seq_len, int d);
// layout 0: padded [B,heads,S,d]; layout 1: packed rows with leading dimension packed_ld.
void launch_attention(DType t, const void* q, const void* k, const void* v, int layout, int packed_ld,
                      const void* attr_mask, void* dst, const int32_t* seq_start, const int32_t* word_idx,
                      int batch, int seq_len, int heads, int d, float scaler, hipStream_t stream);

// ---- gemm.hip ----------------------------------------------------------------------------
// Up to three independent column groups share one launch (the Q/K/V projections): group g
// computes C[:, g*n : (g+1)*n] = A[g] . B[g] (+ bias[g]) into a row-major C with leading
// dimension ldc.  groups == 1 is the plain GEMM.
struct GemmGroups {
  const void* A[3];
  const void* B[3];
  const void* bias[3];
  int groups;
  // true: B[g] holds the transpose, [n][k] row-major (see launch_transpose_weights); only where
  // gemm_takes_transposed_b() says so
  bool b_transposed = false;
  // C = gelu(A.B + bias): bias + GELU as in launch_bias_gelu, same rounding points, applied to each tile on its way
  // out; bias[g] must be set
  bool gelu = false;
  // Hand-over of a wide intermediate between two launches of the persistent k-contiguous kernel (the FFN's [T, 4H]
  // matrix): the producer writes C, the consumer reads A, with every tile of 256 rows stored as consecutive blocks of
  // [256 rows][64 columns] (32 KB each) instead of row-major, so that the consumer's operand fetches, 128 bytes per row
  // and pair of k-steps, are contiguous in memory instead of one row stride apart.  Only where
  // gemm_blocked_handover() says so; the matrix must be allocated for a whole number of 256-row tiles.
  bool c_blocked = false, a_blocked = false;
  // C is read again by the next kernels while it can still be in the last-level cache (the working set of the layer
  // or of the call fits it a few times over): the persistent kernel then stores C with plain stores.  Its non-temporal
  // stores are the better choice when C would only push the weights and the A rows out of that cache.
  bool c_cached = false;
};
// any n, k >= 1 (the MFMA kernels need k % 32 == 0, n % 8 == 0 in fp16 and k % 16 == 0, n % 4 == 0 in fp32; other
// shapes run the element-wise kernel of generic.hip)
bool gemm_supported(DType t, int n, int k, int groups);
// True when both C = A.B1 ([m, wide] from k = narrow) and the product that consumes it (k = wide, n = narrow) run the
// persistent k-contiguous kernel, given k-contiguous copies of both weights.
bool gemm_blocked_handover(DType t, int m_bound, int wide, int narrow);
// The large-M fp16 kernel is faster when B comes k-contiguous ([n][k]): both operands then reach the
// MFMA with 128-bit LDS reads and no register transpose.  True when launch_gemm would use that kernel.
bool gemm_takes_transposed_b(DType t, int m_bound, int ldc, int n, int k, int groups);
// ... and where the encoder layer finds a per-call copy worth its time (everywhere it can be used).
bool gemm_prefers_transposed_b(DType t, int m_bound, int ldc, int n, int k, int groups);
// dst[j] ([n][k], row-major) = transpose of src[j] ([k][n], row-major), fp16, one launch for all jobs.
struct TransposeJobs {
  static constexpr int kMax = 6;
  const void* src[kMax];
  void* dst[kMax];
  int k[kMax], n[kMax];
  int count = 0;
  void add(const void* s, void* d, int k_, int n_) { src[count] = s; dst[count] = d; k[count] = k_; n[count] = n_; ++count; }
};
// The layer needs the per-sequence start table as well; `seq` (optional) makes the same launch build it, which saves a
// launch per layer.
struct SeqStartJob {
  const int32_t* batch_idx;
  const int32_t* rows_dev;
  int rows_bound, batch;
  int32_t* seq_start;
};
void launch_transpose_weights(const TransposeJobs& jobs, hipStream_t stream, const SeqStartJob* seq = nullptr);
void launch_gemm(DType t, const GemmGroups& g, void* C, int ldc, int m_bound, int n, int k,
                 const int32_t* rows_dev, hipStream_t stream);

// ---- generic.hip: element-wise kernels for the shapes the tuned kernels do not take ------------------------------
// (rows or head rows that are no whole number of 16-byte pieces, GEMM k / n the MFMA tiles cannot take); the launchers
// above fall back to them by themselves.
void launch_gemm_generic(DType t, const GemmGroups& g, void* C, int ldc, int m_bound, int n, int k,
                         const int32_t* rows_dev, hipStream_t stream);
void launch_bias_gelu_generic(DType t, void* out, const void* bias, int m, int n, const int32_t* rows_dev,
                              hipStream_t stream);
void launch_layernorm_generic(DType t, void* out, const void* input, const void* bias, const void* gamma,
                              const void* beta, int m, int n, const int32_t* rows_dev, float eps, hipStream_t stream);
void launch_qkv_bias_pad_generic(DType t, const void* Q, const void* bQ, const void* K, const void* bK, const void* V,
                                 const void* bV, void* q_buf, void* k_buf, void* v_buf, const int32_t* seq_start,
                                 const int32_t* word_idx, int batch, int seq_len, int heads, int d, hipStream_t stream);
void launch_transpose_rm_padding_generic(DType t, const void* src, void* dst, const int32_t* rows_dev, int rows_bound,
                                         int seq_len, int heads, int d, const int32_t* batch_idx,
                                         const int32_t* word_idx, hipStream_t stream);

// ---- calibrate.hip: measurement aid ---------------------------------------------------------------------
// One launch of `iters` k-steps of the large fp16 GEMM's inner loop (MFMAs + LDS operand reads, no global memory) on
// `cus` workgroups of 8 wavefronts, with zero or random operands; returns the floating-point operations of the launch.
// `sink` receives one float per thread (mfma_ceiling_sink_bytes).
size_t mfma_ceiling_sink_bytes(int cus);
double launch_mfma_ceiling(bool random_operands, int cus, int iters, float* sink, hipStream_t stream);

}  // namespace et
