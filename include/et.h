/*
 * et.h -- C ABI of the MI355X (gfx950) padding-free BERT encoder library, libet_hip.so.
 *
 * The entry points replace, one for one, the GPU functors behind the three TensorFlow ops
 * of bytedance/effective_transformer and the kernel launchers those functors call.  Paths
 * in the comments are relative to the reference tree.
 *
 * Conventions
 *   - extern "C", plain pointers and sizes, POD structs; no exception crosses the boundary.
 *   - Every pointer named *_dev / every tensor argument is DEVICE memory owned by the caller
 *     (inputs, outputs, weights and workspace).  No entry point allocates or frees device
 *     memory.
 *   - Every call returns an et_status; et_last_error() gives the message of the last failure
 *     on that handle (replaces the reference's std::runtime_error -> errors::Internal path,
 *     common.h:73-81, tf_op/bert_transformer_op.cu.cc:251-258).
 *   - Work is enqueued on the hipStream_t passed as `stream` (an opaque void* here) and is
 *     asynchronous unless a host output (valid_word_num_host) is requested.
 *   - Dense kernels are [in,out] row-major, biases / gamma / beta are [out]
 *     (tf_op/bert_transformer_op.cu.cc:110-119).
 *   - One handle may be used from several threads: calls on it are serialised by an
 *     internal mutex (the reference's cublas_mutex_, tf_op/bert_transformer_op.cc:213).
 */
#ifndef ET_H_
#define ET_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum et_status {
  ET_OK = 0,
  ET_INVALID_ARGUMENT = 1,    /* null pointer, bad dimension, from_seq_len != to_seq_len ... */
  ET_WORKSPACE_TOO_SMALL = 2,
  ET_UNSUPPORTED = 3,         /* shape outside what the kernels are built for */
  ET_LAUNCH_FAILURE = 4,      /* hipGetLastError() after a launch */
  ET_RUNTIME_ERROR = 5        /* any other HIP runtime error */
} et_status;

/* OperationType{FP32,HALF}, common.h:26 */
typedef enum et_dtype { ET_FP32 = 0, ET_FP16 = 1 } et_dtype;

typedef struct et_context* et_handle;

/* Handle life cycle.  Replaces the per-op state created in the OpKernel constructors
 * (cublasCreate at tf_op/bert_transformer_op.cc:171).  `device` is a HIP device ordinal. */
et_status et_create(et_handle* out, int device);
et_status et_destroy(et_handle h);
/* Message of the last failing call on `h` (or, when h is NULL, of the last call on this thread that failed without a
 * handle: et_create, a NULL handle argument).  Never NULL.  With several threads on one handle every thread reads the
 * message of ITS OWN last failing call as long as that call was its most recent failure; a thread that has not failed
 * on `h` gets the handle's last message from any thread.  The pointer stays valid until the calling thread's next
 * failing call or next et_last_error. */
const char* et_last_error(et_handle h);
const char* et_status_string(et_status s);
/* 1 when the library was built for the architecture of `device` and a kernel runs there. */
int et_device_ok(int device);

/* The 16 per-layer tensors, named as the fields of EncoderInitParam<T>
 * (tf_op/bert_transformer_op.h:66-96).  All device pointers of the layer's dtype. */
typedef struct et_layer_weights {
  const void* attr_kernel_Q;               /* [H,H]  */
  const void* attr_kernel_K;               /* [H,H]  */
  const void* attr_kernel_V;               /* [H,H]  */
  const void* attr_bias_Q;                 /* [H]    */
  const void* attr_bias_K;                 /* [H]    */
  const void* attr_bias_V;                 /* [H]    */
  const void* attr_output_kernel;          /* [H,H]  */
  const void* attr_output_bias;            /* [H]    */
  const void* attr_output_layernorm_gamma; /* [H]    */
  const void* attr_output_layernorm_beta;  /* [H]    */
  const void* inter_kernel;                /* [H,4H] */
  const void* inter_bias;                  /* [4H]   */
  const void* output_kernel;               /* [4H,H] */
  const void* output_bias;                 /* [H]    */
  const void* output_layernorm_gamma;      /* [H]    */
  const void* output_layernorm_beta;       /* [H]    */
} et_layer_weights;

/* Workspace sizes in bytes (sized by element type; the reference sizes its layer buffer in
 * bytes but indexes it in elements, tf_op/bert_transformer_op.cu.cc:75-96). */
size_t et_input_workspace_bytes(int batch_size, int seq_len);
size_t et_layer_workspace_bytes(et_dtype dtype, int batch_size, int seq_len, int head_num, int size_per_head);
/* size of the sequence table of a batch (et_sequence_starts; also the scratch of the kernel-level entry points that
 * build one): 2 * batch_size + 1 int32, rounded up to 256 bytes */
size_t et_seq_workspace_bytes(int batch_size);

/* ---- the three ops ------------------------------------------------------------------ */

/* EffectiveTransformerInputOpFunctor::Compute, tf_op/bert_transformer_op.cu.cc:266-331
 * (op registered at tf_op/bert_transformer_op.cc:249-274).
 *   from_tensor [B,S,H], mask int32 [B,S] (0/1)  ->
 *   to_tensor (first T rows of [B*S,H] defined), valid_word_num_dev int32[1],
 *   batch_idx / word_idx int32[B*S] (first T defined).
 * valid_word_num_host: optional; when non-NULL the call synchronises the stream and stores T
 * there (the reference always synchronises, :306-310). */
et_status et_input(et_handle h, et_dtype dtype, const void* from_tensor, const int32_t* mask,
                   void* to_tensor, int32_t* valid_word_num_dev, int32_t* batch_idx, int32_t* word_idx,
                   int batch_size, int seq_len, int head_num, int size_per_head,
                   void* workspace, size_t workspace_bytes, void* stream, int32_t* valid_word_num_host);

/* et_input for callers that cannot allocate device memory or hand over a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same kernels, same
 * outputs as et_input bit for bit; the scan's scratch (one int32 per 1024 mask positions) lives in an array
 * inside the library's device image (32 KB), one copy per GPU for the life of the process, so the call takes no workspace and
 * allocates nothing.  Limit: batch_size * seq_len <= 1048576 positions (ET_UNSUPPORTED beyond; use et_input).  Never
 * synchronises (no host count).  The array is cut into 8 slots; a handle takes a free slot of its GPU in et_create and
 * returns it in et_destroy (a ninth live handle on one GPU has none: ET_UNSUPPORTED), so calls on different handles
 * never share scratch.  The calls of ONE handle do: queued on one stream they run in order; a call on another stream
 * than the handle's previous one is refused with ET_INVALID_ARGUMENT while that previous stream still has work in
 * flight.  Replays of captured graphs that hold such calls are not seen by that check: replays of one handle's calls
 * that overlap on the GPU race. */
et_status et_input_static(et_handle h, et_dtype dtype, const void* from_tensor, const int32_t* mask,
                          void* to_tensor, int32_t* valid_word_num_dev, int32_t* batch_idx, int32_t* word_idx,
                          int batch_size, int seq_len, int head_num, int size_per_head, void* stream);

/* EffectiveTransformerOpFunctor::Compute, tf_op/bert_transformer_op.cu.cc:33-260
 * (op registered at tf_op/bert_transformer_op.cc:44-77): one encoder layer on packed tokens.
 *   from_tensor, to_tensor [T,H] packed; attr_mask [B,S,S] of dtype (1 = attend);
 *   out [T,H] packed (rows >= T untouched).
 * valid_word_num_hint: T when the host knows it (grids are sized exactly), any upper bound of T
 * that the caller vouches for (grids are sized for that many rows; rows beyond it would not be
 * computed), or -1: grids are then sized for B*S rows.  Every kernel bounds itself by
 * *valid_word_num_dev, so the call never blocks the host (the reference copies T back every
 * layer, :99-101).
 * from_seq_len must equal to_seq_len (tf_op/bert_transformer_op.cc:130-131).  `out` must not
 * alias from_tensor/to_tensor.  Shapes: seq_len <= 1024, batch_size <= 65535, any size_per_head from 1 to 256 (see
 * et_attention), head_num * size_per_head <= 1048576 (every entry point), activations below 4 GB per matrix.  The tuned kernels take head size 64 and hidden sizes in multiples of 32 (fp16) or 16 (fp32); every
 * other shape runs element-wise kernels with the same arithmetic (the reference's kernels index by element too,
 * cuda/attention.cu:190-219). */
et_status et_layer(et_handle h, et_dtype dtype, const et_layer_weights* weights,
                   const void* from_tensor, const void* to_tensor, const void* attr_mask,
                   const int32_t* valid_word_num_dev, const int32_t* batch_idx, const int32_t* word_idx,
                   void* out, int batch_size, int from_seq_len, int to_seq_len, int head_num, int size_per_head,
                   int valid_word_num_hint, void* workspace, size_t workspace_bytes, void* stream);

/* What a caller that keeps a layer's weights constant can prepare once instead of having et_layer redo it on every
 * call.  No counterpart in the reference, whose op receives the weights as inputs of every call (tf_op/
 * bert_transformer_op.cc:44-77) and rebuilds nothing across calls either.  Every member may be NULL.
 *   *_t: the dense kernel handed over [out,in] (k-contiguous), i.e. et_transpose_weight of the [in,out] tensor, fp16
 *        only.  Used where et_layer would run its large-M GEMM (it then skips its per-call transposition; Q, K and V
 *        go together); ignored for batches that run the small-M kernels, which read the [in,out] tensors.
 *   seq_start, seq_start_bytes: the sequence table et_sequence_starts wrote for THIS batch and the size of its buffer
 *        (at least et_seq_workspace_bytes(batch_size), ET_WORKSPACE_TOO_SMALL below); the same table serves every
 *        layer of the batch.
 *   warm, warm_bytes: a region that the layer's last kernel requests line by line on its way, so that whoever reads it
 *        next finds it in the last-level cache: the k-contiguous copies of the NEXT layer's attention kernels, whose
 *        GEMMs would otherwise wait for weights last read a whole batch ago.  Only used for batches large enough that
 *        the region is small beside what that kernel moves anyway. */
typedef struct et_layer_prepared {
  const void* attr_kernel_Q_t;       /* [H,H]  */
  const void* attr_kernel_K_t;       /* [H,H]  */
  const void* attr_kernel_V_t;       /* [H,H]  */
  const void* attr_output_kernel_t;  /* [H,H]  */
  const void* inter_kernel_t;        /* [4H,H] */
  const void* output_kernel_t;       /* [H,4H] */
  const int32_t* seq_start;          /* [2B+1] */
  const void* warm;                  /* see above; 128-byte aligned */
  size_t warm_bytes;
  size_t seq_start_bytes;            /* bytes behind seq_start (checked when seq_start is set) */
} et_layer_prepared;

/* The sequence table of a batch, from the index arrays et_input produced: seq_start[b] = first packed row of sequence
 * b for b in [0,B), seq_start[B] = T, followed by the B sequence numbers in the order the attention kernels serve them
 * (by length, longest first: workgroups of similar duration run side by side and the long ones start first).
 * seq_start must hold et_seq_workspace_bytes(batch_size) bytes (2 B + 1 int32); seq_start_bytes is the size of the
 * caller's buffer, ET_WORKSPACE_TOO_SMALL when it is less.  No counterpart in the reference (its attention works on
 * padded buffers). */
et_status et_sequence_starts(et_handle h, const int32_t* batch_idx, const int32_t* valid_word_num_dev, int batch_size,
                             int seq_len, int32_t* seq_start, size_t seq_start_bytes, void* stream);

/* et_layer with prepared data (see et_layer_prepared; NULL = et_layer).  Same results, bit for bit. */
et_status et_layer_with_prepared(et_handle h, et_dtype dtype, const et_layer_weights* weights,
                                 const et_layer_prepared* prepared, const void* from_tensor, const void* to_tensor,
                                 const void* attr_mask, const int32_t* valid_word_num_dev, const int32_t* batch_idx,
                                 const int32_t* word_idx, void* out, int batch_size, int from_seq_len, int to_seq_len,
                                 int head_num, int size_per_head, int valid_word_num_hint, void* workspace,
                                 size_t workspace_bytes, void* stream);

/* EffectiveTransformerOutputOpFunctor::Compute, tf_op/bert_transformer_op.cu.cc:339-373
 * (op registered at tf_op/bert_transformer_op.cc:359-380): to_tensor [B,S,H] = 0 at padding,
 * from_tensor row t at (batch_idx[t], word_idx[t]).  batch_idx/word_idx must be those written
 * by et_input (ascending in b*S+s). */
et_status et_output(et_handle h, et_dtype dtype, const void* from_tensor, const int32_t* valid_word_num_dev,
                    const int32_t* batch_idx, const int32_t* word_idx, void* to_tensor,
                    int batch_size, int seq_len, int head_num, int size_per_head, void* stream);

/* ---- the step in front of the path --------------------------------------------------- */

/* The tables of the BERT embedding block (sample/tensorflow/modeling.py:171-194: `word_embeddings`,
 * `token_type_embeddings`, `position_embeddings`, then `LayerNorm/{gamma,beta}`), row-major in dtype. */
typedef struct et_embedding_weights {
  const void* word_embeddings;        /* [vocab_size, H]                         */
  const void* token_type_embeddings;  /* [type_vocab_size, H] or NULL            */
  const void* position_embeddings;    /* [max_position_embeddings, H] or NULL    */
  const void* layernorm_gamma;        /* [H]                                     */
  const void* layernorm_beta;         /* [H]                                     */
  int vocab_size, type_vocab_size, max_position_embeddings;
} et_embedding_weights;

/* Embedding lookup + post-processing fused with et_input: what embedding_lookup, embedding_postprocessor
 * (sample/tensorflow/modeling.py:380-521, dropout off) and EffectiveTransformerInputOpFunctor::Compute
 * (tf_op/bert_transformer_op.cu.cc:266-331) do one after the other, without the padded [B,S,H] tensor in between --
 * the reference notes that the compress belongs in front of the embedding (:295-296).
 *   input_ids, token_type_ids (may be NULL), mask: int32 [B,S]  ->
 *   to_tensor row t = LayerNorm(word[id] + type[type_id] + position[s]) (eps 1e-12) for the t-th valid (b,s);
 *   valid_word_num_dev, batch_idx, word_idx exactly as et_input writes them.
 * Ids outside their table contribute a zero row.  workspace: et_input_workspace_bytes(B, S). */
et_status et_embedding_input(et_handle h, et_dtype dtype, const et_embedding_weights* embeddings,
                             const int32_t* input_ids, const int32_t* token_type_ids, const int32_t* mask,
                             void* to_tensor, int32_t* valid_word_num_dev, int32_t* batch_idx, int32_t* word_idx,
                             int batch_size, int seq_len, int head_num, int size_per_head,
                             void* workspace, size_t workspace_bytes, void* stream, int32_t* valid_word_num_host);

/* The consumer side of the same fusion: the first token of every sequence straight from the packed matrix, i.e.
 * what `sequence_output[:, 0:1, :]` (the pooler's input, sample/tensorflow/modeling.py:224-232) reads after
 * EffectiveTransformerOutput, without materialising the padded [B,S,H] tensor.
 *   from_tensor [T,H] packed, batch_idx / word_idx as written by et_input  ->  to_tensor [B,H]
 * (zeros for a sequence whose position 0 holds no token). */
et_status et_first_token(et_handle h, et_dtype dtype, const void* from_tensor, const int32_t* valid_word_num_dev,
                         const int32_t* batch_idx, const int32_t* word_idx, void* to_tensor,
                         int batch_size, int seq_len, int hidden_dim, void* stream);

/* ---- kernel-level entry points (unit tests, profiling in isolation) ----------------- */

/* exclusiveScan_kernelLauncher, cuda/cuda_kernels.h:29 (cuda/cuda_kernels.cu:709-718).
 * workspace: et_input_workspace_bytes(1, length). */
et_status et_exclusive_scan(et_handle h, int32_t* d_out, const int32_t* d_in, int length,
                            void* workspace, size_t workspace_bytes, void* stream);

/* compressBertInput_kernelLauncher, cuda/cuda_kernels.h:31-35 (cuda/cuda_kernels.cu:278-384). */
et_status et_compress(et_handle h, et_dtype dtype, const void* from_tensor, const int32_t* mask,
                      const int32_t* prefix_sum, void* to_tensor, int32_t* batch_idx, int32_t* word_idx,
                      int batch_size, int seq_len, int hidden_dim, void* stream);

/* restoreBertOutput_kernelLauncher, cuda/cuda_kernels.h:37-41 (cuda/cuda_kernels.cu:389-468),
 * fused with the zero fill the output op does first (tf_op/bert_transformer_op.cu.cc:354-355). */
et_status et_restore(et_handle h, et_dtype dtype, void* to_tensor, const void* from_tensor,
                     const int32_t* batch_idx, const int32_t* word_idx, const int32_t* valid_word_num_dev,
                     int batch_size, int seq_len, int hidden_dim, void* stream);

/* add_bias_act_kernelLauncher, cuda/cuda_kernels.h:22-23 (cuda/cuda_kernels.cu:88-150):
 * out[m,n] = gelu_tanh(out + bias), in place.  m_dev (optional) bounds the rows on the device. */
et_status et_add_bias_act(et_handle h, et_dtype dtype, void* out, const void* bias, int m, int n,
                          const int32_t* m_dev, void* stream);

/* add_bias_input_layernorm_kernelLauncher, cuda/cuda_kernels.h:25-27 (cuda/cuda_kernels.cu:157-271):
 * out[m,n] = LayerNorm(out + input + bias) * gamma + beta, eps 1e-6, in place. */
et_status et_add_bias_input_layernorm(et_handle h, et_dtype dtype, void* out, const void* input,
                                      const void* bias, const void* gamma, const void* beta,
                                      int m, int n, const int32_t* m_dev, void* stream);

/* add_QKV_bias_padding_kernelLauncher, cuda/attention.h:25-35 (cuda/attention.cu:105-242), fused
 * with the zero fill that precedes it (tf_op/bert_transformer_op.cu.cc:146):
 * q/k/v_buf [B,heads,S,d] = 0 at padding, src[t] + bias at (batch_idx[t], :, word_idx[t], :).
 * workspace: et_seq_workspace_bytes(B). */
et_status et_add_qkv_bias_padding(et_handle h, et_dtype dtype,
                                  const void* Q, const void* bias_Q, const void* K, const void* bias_K,
                                  const void* V, const void* bias_V, void* q_buf, void* k_buf, void* v_buf,
                                  const int32_t* valid_word_num_dev, int batch_size, int seq_len,
                                  int head_num, int size_per_head,
                                  const int32_t* batch_idx, const int32_t* word_idx,
                                  void* workspace, size_t workspace_bytes, void* stream);

/* softmax_kernel_kernelLauncher, cuda/attention.h:37-42 (cuda/attention.cu:249-382): in-place
 * masked, scaled softmax of qk_buf [B,heads,S,S] with attr_mask [B,S,S], S <= 1024 (the reach of the reference's
 * launcher, :345-356).  As in the reference the row maximum is clamped below at 0 for S < 1024 and is the true maximum
 * at S = 1024 (:77-95, 267-270). */
et_status et_softmax(et_handle h, et_dtype dtype, void* qk_buf, const void* attr_mask,
                     int batch_size, int head_num, int seq_len, float scaler, void* stream);

/* transpose_rm_padding_kernelLauncher, cuda/attention.h:44-51 (cuda/attention.cu:387-492):
 * src [B,heads,S,d] -> dst packed [T,heads*d]. */
et_status et_transpose_rm_padding(et_handle h, et_dtype dtype, const void* src, void* dst,
                                  const int32_t* valid_word_num_dev, int batch_size, int seq_len,
                                  int head_num, int size_per_head,
                                  const int32_t* batch_idx, const int32_t* word_idx, void* stream);

/* The attention block of the layer in one kernel: batched QK^T, masked softmax, batched PV and
 * un-padding (tf_op/bert_transformer_op.cu.cc:159-192).
 *   qkv_layout 0: q/k/v are the padded [B,heads,S,d] buffers add_QKV_bias_padding writes;
 *   qkv_layout 1: q/k/v point into packed token-major rows (row t, column head*d + j) with row
 *                 stride `packed_ld` elements (bias already added).
 *   dst packed [T,heads*d].  workspace: et_seq_workspace_bytes(B).
 * seq_len <= 1024; size_per_head from 1 to 256.  size_per_head = 64 (head rows on 16-byte boundaries) runs the MFMA
 * kernels, every other head size a slower general kernel with the same arithmetic. */
et_status et_attention(et_handle h, et_dtype dtype, const void* q, const void* k, const void* v, int qkv_layout,
                       int packed_ld, const void* attr_mask, void* dst,
                       const int32_t* valid_word_num_dev, int batch_size, int seq_len,
                       int head_num, int size_per_head,
                       const int32_t* batch_idx, const int32_t* word_idx,
                       void* workspace, size_t workspace_bytes, void* stream);

/* et_attention with the sequence start table of et_sequence_starts handed in (seq_start; one table serves
 * every layer of a batch, as in et_layer_with_prepared), so that the call is the attention kernel alone.  With
 * seq_start NULL the table is built into seq_start_scratch first, which is what et_attention does.  seq_table_bytes is
 * the size of whichever of the two buffers is used: ET_WORKSPACE_TOO_SMALL below et_seq_workspace_bytes(B).  No
 * counterpart in the reference, whose attention works on padded buffers. */
et_status et_attention_with_starts(et_handle h, et_dtype dtype, const void* q, const void* k, const void* v,
                                   int qkv_layout, int packed_ld, const void* attr_mask, void* dst,
                                   const int32_t* valid_word_num_dev, int batch_size, int seq_len, int head_num,
                                   int size_per_head, const int32_t* batch_idx, const int32_t* word_idx,
                                   const int32_t* seq_start, int32_t* seq_start_scratch, size_t seq_table_bytes,
                                   void* stream);

/* Replaces the cublasGemmEx call sites (tf_op/bert_transformer_op.cu.cc:110-141, 200-240):
 * C[m,n] = A[m,k] . B[k,n], all row-major, alpha = 1, beta = 0, fp32 accumulation, C of dtype.
 * bias (optional, [n]) is added to the rounded product (in the element type, as the reference's
 * following kernel would).  m_dev (optional) bounds the rows on the device.  Any m, n, k: the MFMA kernels take
 * k % 32 == 0, n % 8 == 0 (fp16) / k % 16 == 0, n % 4 == 0 (fp32), other shapes an element-wise kernel. */
et_status et_gemm(et_handle h, et_dtype dtype, const void* A, const void* B, void* C, const void* bias,
                  int m, int n, int k, const int32_t* m_dev, void* stream);

/* C[m,n] = gelu(A[m,k] . B[k,n] + bias[n]): et_gemm followed by et_add_bias_act in one launch, same arithmetic and
 * rounding points as the two calls in a row (reference: the cublasGemmEx call and the add_bias_act launch behind it,
 * tf_op/bert_transformer_op.cu.cc:215-227, cuda/cuda_kernels.cu:29-51, 88-150).  bias is required. */
et_status et_gemm_bias_gelu(et_handle h, et_dtype dtype, const void* A, const void* B, void* C, const void* bias,
                            int m, int n, int k, const int32_t* m_dev, void* stream);

/* dst[n][k] = transpose of src[k][n] (both row-major), fp16 only.  No counterpart in the reference, which hands the
 * TF dense kernels [in,out] to cuBLAS as they are; et_layer does this internally for its large-M GEMMs. */
et_status et_transpose_weight(et_handle h, et_dtype dtype, const void* src, void* dst, int k, int n, void* stream);

/* et_gemm with the second operand k-contiguous: C[m,n] = A[m,k] . Bt[n,k]^T (+ bias), fp16 only.  This is the kernel
 * et_layer runs where it has such a copy of a weight (same cublasGemmEx call sites as et_gemm): a persistent kernel
 * from 128 tiles of 256x256 on, one tile of 32x64 .. 128x128 per workgroup below that.  Same bits as et_gemm on the
 * same operands.  ET_UNSUPPORTED for k % 64 != 0 or n % 8 != 0. */
et_status et_gemm_bt(et_handle h, et_dtype dtype, const void* A, const void* Bt, void* C, const void* bias,
                     int m, int n, int k, const int32_t* m_dev, void* stream);

/* C[m,n] = gelu(A[m,k] . Bt[n,k]^T + bias[n]): et_gemm_bt with et_add_bias_act applied to each tile on its way out,
 * same arithmetic and rounding points as the two calls in a row (reference: the cublasGemmEx call and the
 * add_bias_act launch that follows it, tf_op/bert_transformer_op.cu.cc:215-227, cuda/cuda_kernels.cu:29-51, 88-150).
 * This is what et_layer runs for the first FFN projection where it has a k-contiguous copy of the weight.  fp16 only,
 * bias required; shapes as for et_gemm_bt. */
et_status et_gemm_bt_bias_gelu(et_handle h, et_dtype dtype, const void* A, const void* Bt, void* C, const void* bias,
                               int m, int n, int k, const int32_t* m_dev, void* stream);

/* Measurement aid, no counterpart in the reference and no part of the encoder path: one launch of `iters` k-steps of
 * the large fp16 GEMM's inner loop (per wavefront 32 v_mfma_f32_16x16x32_f16 and 12 16-byte LDS operand reads, 8
 * wavefronts on every CU, no global memory traffic) with operands that are all zero (random_operands == 0) or random
 * halves.  *flops receives the floating-point operations of the launch; the caller times it with events on `stream`.
 * The rate with random operands is the ceiling a GEMM on real data runs under on this part (switching activity costs
 * clock), which is what bench.py --calibrate-mfma reports beside the data-sheet peak.  `sink` is a device buffer of
 * et_calibrate_mfma_sink_bytes() bytes that receives one float per thread. */
size_t et_calibrate_mfma_sink_bytes(et_handle h);
et_status et_calibrate_mfma(et_handle h, int random_operands, int iters, void* sink, size_t sink_bytes, double* flops,
                            void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ET_H_ */
