// Attention side of the encoder layer on gfx950.
//   qkv_bias_pad      : [T,H] + bias -> zero-padded [B,heads,S,d]   (reference: cuda/attention.cu:105-242,
//                                                                    zero fill tf_op/bert_transformer_op.cu.cc:146)
//   softmax           : masked, scaled softmax in place             (cuda/attention.cu:249-382)
//   transpose_rm_pad  : [B,heads,S,d] -> packed [T,H]               (cuda/attention.cu:387-492)
//   attention (fused) : QK^T, masked softmax, PV and un-padding in one kernel
//                       (tf_op/bert_transformer_op.cu.cc:159-192); reads Q/K/V either from the padded
//                       buffers or straight from packed token rows, writes packed [T,H].
//
// Softmax semantics (both kernels): t = qk*scale + (1-mask)*(-10000); m = max(max_k t, 0);
// e = exp(t-m); p = e / (sum e + 1e-6).  In fp16 the score is rounded to half before the softmax
// and the probability after it, as the reference stores both in half.
#include "et_device.hpp"
#include "kernels.hpp"

namespace et {

namespace {

constexpr float kLog2e = 1.4426950408889634f;

template <typename T> struct Chunk16;
template <> struct Chunk16<float> {
  typedef float4v vec;
  float4v v;
  static constexpr int kElems = 4;
};
template <> struct Chunk16<_Float16> {
  typedef half8 vec;
  half8 v;
  static constexpr int kElems = 8;
};

// ------------------------------------------------------------------------------------------
// add bias + head split + re-pad, one workgroup per (sequence, matrix).  Every 16-byte chunk of
// the padded destination is written once: bias-added data where a token exists, zero elsewhere.
// ------------------------------------------------------------------------------------------
constexpr int kPadThreads = 256;
constexpr int kPadMaxSeq = 1024;

template <typename T>
__global__ __launch_bounds__(kPadThreads) void qkv_bias_pad_kernel(
    const T* __restrict__ Q, const T* __restrict__ bQ, const T* __restrict__ K, const T* __restrict__ bK,
    const T* __restrict__ V, const T* __restrict__ bV, T* __restrict__ q_buf, T* __restrict__ k_buf,
    T* __restrict__ v_buf, const int32_t* __restrict__ seq_start, const int32_t* __restrict__ word_idx, int seq_len,
    int heads, int d) {
  using C = Chunk16<T>;
  __shared__ int tok_of_pos[kPadMaxSeq];
  const int b = blockIdx.x;
  const int mat = blockIdx.y;
  const T* src = mat == 0 ? Q : (mat == 1 ? K : V);
  const T* bias = mat == 0 ? bQ : (mat == 1 ? bK : bV);
  T* dst = mat == 0 ? q_buf : (mat == 1 ? k_buf : v_buf);
  for (int s = threadIdx.x; s < seq_len; s += kPadThreads) tok_of_pos[s] = -1;
  __syncthreads();
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  for (int t = t0 + threadIdx.x; t < t1; t += kPadThreads) {
    const int s = word_idx[t];
    if (s >= 0 && s < seq_len) tok_of_pos[s] = t;
  }
  __syncthreads();
  const int cpd = d / C::kElems;           // chunks per head row
  const int cph = heads * cpd;             // chunks per token row
  const int total = heads * seq_len * cpd;
  C* out = reinterpret_cast<C*>(dst) + (size_t)b * total;
  const C* in = reinterpret_cast<const C*>(src);
  const C* bi = reinterpret_cast<const C*>(bias);
  for (int i = threadIdx.x; i < total; i += kPadThreads) {
    const int c = i % cpd;
    const int s = (i / cpd) % seq_len;
    const int head = i / (cpd * seq_len);
    const int t = tok_of_pos[s];
    C val;
    if (t >= 0) {
      val.v = in[(size_t)t * cph + head * cpd + c].v + bi[head * cpd + c].v;
    } else {
#pragma unroll
      for (int j = 0; j < C::kElems; ++j) val.v[j] = (T)0;
    }
    out[i] = val;
  }
}

// ------------------------------------------------------------------------------------------
// stand-alone softmax: one wavefront per (b, head, q) row, up to 1024 keys.
// ------------------------------------------------------------------------------------------
constexpr int kSmThreads = 256;
constexpr int kSmMaxIters = 16;

template <typename T>
__global__ __launch_bounds__(kSmThreads) void softmax_kernel(T* __restrict__ qk, const T* __restrict__ attr_mask,
                                                             int rows_total, int heads, int seq_len, float scaler) {
  const int lane = threadIdx.x & (kWave - 1);
  const int row = blockIdx.x * (kSmThreads / kWave) + threadIdx.x / kWave;
  if (row >= rows_total) return;          // wave-uniform
  const int q = row % seq_len;
  const int b = row / (seq_len * heads);
  T* x = qk + (size_t)row * seq_len;
  const T* mk = attr_mask + ((size_t)b * seq_len + q) * seq_len;
  float t[kSmMaxIters];
  // the maximum is clamped below at 0, except at 1024 keys, where the reference's max reduction has no idle lane
  float mx = seq_len < 1024 ? 0.f : -INFINITY;
#pragma unroll
  for (int i = 0; i < kSmMaxIters; ++i) {
    const int k = lane + i * kWave;
    t[i] = -INFINITY;
    if (k < seq_len) {
      t[i] = (float)x[k] * scaler + (1.0f - (float)mk[k]) * -10000.0f;
      mx = fmaxf(mx, t[i]);
    }
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < kSmMaxIters; ++i) {
    t[i] = __builtin_amdgcn_exp2f((t[i] - mx) * kLog2e);   // exp2(-inf) = 0 for absent keys
    sum += t[i];
  }
  sum = wave_sum(sum) + 1e-6f;
#pragma unroll
  for (int i = 0; i < kSmMaxIters; ++i) {
    const int k = lane + i * kWave;
    if (k < seq_len) x[k] = (T)(t[i] / sum);
  }
}

// ------------------------------------------------------------------------------------------
// un-pad + head merge: gather flattened over (packed row, 16-byte chunk).
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void transpose_rm_padding_kernel(
    const T* __restrict__ src, T* __restrict__ dst, const int32_t* __restrict__ rows_dev, int rows_bound, int seq_len,
    int heads, int cpd, const int32_t* __restrict__ batch_idx, const int32_t* __restrict__ word_idx) {
  using C = Chunk16<T>;
  const int rows = rows_dev ? min(*rows_dev, rows_bound) : rows_bound;
  const int cph = heads * cpd;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)rows * cph) return;
  const int t = (int)(i / cph);
  const int c = (int)(i - (long)t * cph);
  const int head = c / cpd;
  const int cc = c - head * cpd;
  const int b = batch_idx[t], s = word_idx[t];
  reinterpret_cast<C*>(dst)[i] =
      reinterpret_cast<const C*>(src)[(((size_t)b * heads + head) * seq_len + s) * cpd + cc];
}

// ------------------------------------------------------------------------------------------
// fused attention, size_per_head = 64, seq_len <= 128 (longer sequences: attention_long_kernel below).
//
// One workgroup (4 wavefronts) per (sequence, group of heads).  What does not depend on the
// head is done once: token positions, the zero fill of key/value slots without a token (so that a
// mask that attends to a padded key sees the zero score / zero value the reference's padded buffers
// hold) and the mask rows of each wavefront's queries, which stay in registers.  Per head the K rows
// and the transpose of the V rows are staged in LDS at their padded positions, Q rows beside them,
// while the next head's rows are already in flight into registers.  Each wavefront takes 16-query tiles:
//   S^T = K Q^T   on v_mfma_f32_16x16x32_f16 / v_mfma_f32_16x16x4_f32 -> a lane owns one query
//                 column and 4 keys of every 16-key tile,
//   softmax       over the lane's values + 2 cross-lane steps (lanes l, l^16, l^32, l^48 share a query),
//   O^T = V^T P^T where the lane's own probability registers already are the B operand,
//   then the lane writes 4 consecutive features of its query's packed output row.
// Key tiles that hold no token skip their MFMAs (score 0, value 0) but still go through the
// masked softmax, so the result equals the padded computation exactly.
// ------------------------------------------------------------------------------------------
constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / kWave;
constexpr int kD = 64;

template <typename T> struct AttnCfg;
template <> struct AttnCfg<_Float16> {
  static constexpr int kQkStride = kD + 8;   // halves; 144-byte rows keep 16-byte reads of 8 consecutive rows on distinct banks
  static constexpr int kVtPad = 4;           // halves
  // fp16 keeps V row-major ([key][feature]) and transposes 8x4 blocks in registers: 160-byte rows put the four
  // key groups of an 8-byte operand read 128 bytes apart modulo the 256-byte bank span
  static constexpr int kVStride = kD + 16;
};
template <> struct AttnCfg<float> {
  static constexpr int kQkStride = kD + 4;   // floats; 272-byte rows
  static constexpr int kVtPad = 4;           // floats
};

template <typename T, int NKT>
struct AttnSmem {
  static constexpr int kSp = NKT * 16;
  static constexpr int kVtStride = kSp + AttnCfg<T>::kVtPad;
  static constexpr size_t kQBytes = (size_t)kSp * AttnCfg<T>::kQkStride * sizeof(T);
  static constexpr size_t kVtBytes =
      sizeof(T) == 2 ? (size_t)kSp * AttnCfg<_Float16>::kVStride * sizeof(T) : (size_t)kD * kVtStride * sizeof(T);
  static constexpr size_t kBytes = 2 * kQBytes + kVtBytes + kSp * sizeof(int);
};

// Reductions over the four 16-lane rows of a wavefront (lanes l, l ^ 16, l ^ 32, l ^ 48), the result in all of them.
// v_permlane16_swap exchanges the odd rows of its first operand with the even rows of its second, v_permlane32_swap
// the upper half of the first with the lower half of the second: with both operands a copy of v, the two results hold
// the two rows (halves) that have to be combined, in every lane, without a trip through the LDS crossbar.  The
// operands of each combination are those of the xor shuffle, in one order or the other: same bits.
// (Written as inline assembly on two float copies: with the compiler's builtin, and with integer copies handed back
// as a vector, the second result was lost when both operands hold the same value.  The wait states in front are
// those the compiler itself puts between a VALU write and this instruction.)
__device__ __forceinline__ float xor_lanes_16_32_max(float v) {
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  v = fmaxf(a, b);
  a = v;
  b = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return fmaxf(a, b);
}
__device__ __forceinline__ float xor_lanes_16_32_sum(float v) {
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  v = a + b;
  a = v;
  b = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return a + b;
}

// WAVES: wavefronts per workgroup (4; a wavefront serves NKT / WAVES query tiles at 128 keys).  CPT = 16-byte chunks of
// one matrix a thread moves per head (ceil(seq rows * chunks per row / threads)).
// PF: keep the next head's Q/K/V chunks in registers while the current head is computed.
template <typename T, int NKT, int WAVES, int CPT, bool PF>
__global__ __launch_bounds__(WAVES * kWave) void attention_kernel(
    const T* __restrict__ q_src, const T* __restrict__ k_src, const T* __restrict__ v_src, int layout, int packed_ld,
    const T* __restrict__ attr_mask, T* __restrict__ dst, const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ word_idx, int batch, int seq_len, int heads, int heads_per_wg, float scaler) {
  using Cfg = AttnCfg<T>;
  using Sm = AttnSmem<T, NKT>;
  using C = Chunk16<T>;
  constexpr int kQS = Cfg::kQkStride;
  constexpr int kVS = Sm::kVtStride;
  constexpr int kVR = AttnCfg<_Float16>::kVStride;   // fp16: stride of the row-major V tile
  constexpr int kSp = Sm::kSp;
  constexpr int kCpr = kD / C::kElems;       // 16-byte chunks per head row
  constexpr int kThreads = WAVES * kWave;
  constexpr int QPW = NKT > WAVES ? NKT / WAVES : 1;   // query tiles per wavefront
  typedef T mask4 __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* Qs = reinterpret_cast<T*>(smem_raw);
  T* Ks = reinterpret_cast<T*>(smem_raw + Sm::kQBytes);
  T* Vt = reinterpret_cast<T*>(smem_raw + 2 * Sm::kQBytes);
  int* tok_of_pos = reinterpret_cast<int*>(smem_raw + 2 * Sm::kQBytes + Sm::kVtBytes);

  // workgroups are dealt out in the order of the table's second half: sequences of similar length side by side, the
  // longest first
  const int b = min(max(seq_start[batch + 1 + blockIdx.y], 0), batch - 1);
  const int h_begin = blockIdx.x * heads_per_wg;
  const int h_end = min(h_begin + heads_per_wg, heads);
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  const int len = t1 - t0;
  if (len <= 0) return;
  const int H = heads * kD;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int l16 = lane & 15;
  const int g = lane >> 4;

  // ---- everything that does not depend on the head: issued up front, all loads in flight together ----
  // positions are ascending inside a sequence: the last token bounds the occupied 16-row tiles
  const int last_pos_raw = word_idx[t1 - 1];
  int my_t[CPT], my_pos[CPT], my_c[CPT];
#pragma unroll
  for (int k = 0; k < CPT; ++k) {
    const int i = threadIdx.x + k * kThreads;
    const int tt = i / kCpr;
    my_c[k] = i - tt * kCpr;
    my_t[k] = tt < len ? t0 + tt : -1;
    my_pos[k] = tt < len ? word_idx[t0 + tt] : -1;
  }
  // the mask rows of this wavefront's queries stay in registers for all heads
  mask4 mreg[QPW][NKT];
  const bool vec_mask = (seq_len & 3) == 0;
#pragma unroll
  for (int qi = 0; qi < QPW; ++qi) {
    const int q = (wave + qi * WAVES) * 16 + l16;
    const T* mrow = attr_mask + ((size_t)b * seq_len + min(q, seq_len - 1)) * seq_len;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) {
      const int key0 = kt * 16 + g * 4;
      mask4 m4 = {(T)0, (T)0, (T)0, (T)0};
      if (vec_mask) {
        if (key0 < seq_len) m4 = *reinterpret_cast<const mask4*>(mrow + key0);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (key0 + r < seq_len) m4[r] = mrow[key0 + r];
      }
      mreg[qi][kt] = m4;
    }
  }
  using V16 = typename C::vec;
  V16 rq[CPT], rk[CPT], rv[CPT];
  // 16-byte chunk k of this thread for `head`: element offset into the source matrices.  Packed rows are addressed by
  // the token alone, so their loads leave without waiting for the positions (one step less in the chain of dependent
  // loads a workgroup starts with: -1.6 us per launch at 1000 x 64 tokens); a position outside the sequence is only
  // sorted out when the chunk goes to LDS.
#define ET_ATTN_LOAD_HEAD(head_)                                                                            \
  _Pragma("unroll") for (int k = 0; k < CPT; ++k) {                                                         \
    if (my_t[k] >= 0 && (layout == 1 || (my_pos[k] >= 0 && my_pos[k] < seq_len))) {                         \
      const size_t off = layout == 1                                                                        \
                             ? (size_t)my_t[k] * packed_ld + (head_) * kD + my_c[k] * C::kElems             \
                             : (((size_t)b * heads + (head_)) * seq_len + my_pos[k]) * kD + my_c[k] * C::kElems; \
      rq[k] = *reinterpret_cast<const V16*>(q_src + off);                                                   \
      rk[k] = *reinterpret_cast<const V16*>(k_src + off);                                                   \
      rv[k] = *reinterpret_cast<const V16*>(v_src + off);                                                   \
    }                                                                                                       \
  }
  if (PF) { ET_ATTN_LOAD_HEAD(h_begin) }

  const int last_pos = min(max(last_pos_raw, 0), seq_len - 1);
  const int n_tiles = last_pos / 16 + 1;    // 16-row tiles that hold at least one token (queries and keys)

  // mask value -> additive bias, once for all heads: (1 - m) * -10000 in float as the reference computes it, kept in
  // the element type (exact for 0/1 masks); keys beyond seq_len do not exist
#pragma unroll
  for (int qi = 0; qi < QPW; ++qi)
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        mreg[qi][kt][r] = kt * 16 + g * 4 + r < seq_len ? (T)((1.0f - (float)mreg[qi][kt][r]) * -10000.0f) : (T)-INFINITY;

  // ---- position table, then zero the key / value slots that hold no token (once: heads only overwrite tokens) ----
  for (int i = threadIdx.x; i < kSp; i += kThreads) tok_of_pos[i] = -1;
  __syncthreads();
#pragma unroll
  for (int k = 0; k < CPT; ++k)
    if (my_t[k] >= 0 && my_c[k] == 0 && my_pos[k] >= 0 && my_pos[k] < seq_len) tok_of_pos[my_pos[k]] = my_t[k];
  __syncthreads();
  {
    // the fp16 P.V contraction runs over pairs of key tiles, so an odd tile count drags one more tile of Vt in
    const int rows = min(kSp, ((n_tiles + 1) / 2) * 32);
    // K: row `pos` (kQS elements), Vt: column `pos` of every feature row
    for (int i = threadIdx.x; i < rows * (kD / 2); i += kThreads) {
      const int pos = i / (kD / 2), w = i - pos * (kD / 2);
      if (tok_of_pos[pos] < 0) {
        if (sizeof(T) == 2) {
          reinterpret_cast<uint32_t*>(Ks + pos * kQS)[w] = 0u;                // 2 halves
          reinterpret_cast<uint32_t*>(Vt + pos * kVR)[w] = 0u;                // V is row-major for fp16
        } else {
          Ks[pos * kQS + 2 * w] = (T)0; Ks[pos * kQS + 2 * w + 1] = (T)0;
          Vt[(2 * w) * kVS + pos] = (T)0;
          Vt[(2 * w + 1) * kVS + pos] = (T)0;
        }
      }
    }
  }

  // where each of this lane's queries writes its output row (head 0; null without a token): the same for every head
  T* out_row[QPW];
#pragma unroll
  for (int qi = 0; qi < QPW; ++qi) {
    const int qt = wave + qi * WAVES;
    const int tq = qt < n_tiles ? tok_of_pos[qt * 16 + l16] : -1;
    out_row[qi] = tq >= 0 ? dst + (size_t)tq * H + g * (sizeof(T) == 2 ? 16 : 4) : nullptr;
  }

  for (int head = h_begin; head < h_end; ++head) {
    if (!PF) { ET_ATTN_LOAD_HEAD(head) }
    if (head != h_begin) __syncthreads();      // every wavefront is done with the previous head's tiles
#pragma unroll
    for (int k = 0; k < CPT; ++k) {
      const int pos = my_pos[k];
      if (my_t[k] >= 0 && pos >= 0 && pos < seq_len) {
        const int c = my_c[k];
        *reinterpret_cast<V16*>(Qs + pos * kQS + c * C::kElems) = rq[k];
        *reinterpret_cast<V16*>(Ks + pos * kQS + c * C::kElems) = rk[k];
        if constexpr (sizeof(T) == 2) {
          *reinterpret_cast<V16*>(Vt + pos * kVR + c * C::kElems) = rv[k];
        } else {
#pragma unroll
          for (int j = 0; j < C::kElems; ++j) Vt[(c * C::kElems + j) * kVS + pos] = rv[k][j];
        }
      }
    }
    __syncthreads();
    if (PF && head + 1 < h_end) { ET_ATTN_LOAD_HEAD(head + 1) }   // flies while this head is computed

#pragma unroll
    for (int qi = 0; qi < QPW; ++qi) {
      const int qt = wave + qi * WAVES;
      if (qt >= n_tiles) break;               // wave-uniform
      const int q = qt * 16 + l16;            // this lane's query position
      float s[NKT][4];
      // ---- S^T = K Q^T -------------------------------------------------------------------
      if constexpr (sizeof(T) == 2) {
        half8 bq[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) bq[ks] = *reinterpret_cast<const half8*>(Qs + q * kQS + ks * 32 + g * 8);
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
          float4v acc = {0.f, 0.f, 0.f, 0.f};
          if (kt < n_tiles) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
              const half8 a = *reinterpret_cast<const half8*>(Ks + (kt * 16 + l16) * kQS + ks * 32 + g * 8);
              acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bq[ks], acc, 0, 0, 0);
            }
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) s[kt][r] = h2f(f2h(acc[r]));   // the score is stored in half
        }
      } else {
        float bq[16];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float4v v4 = *reinterpret_cast<const float4v*>(Qs + q * kQS + g * 16 + i * 4);
#pragma unroll
          for (int j = 0; j < 4; ++j) bq[i * 4 + j] = v4[j];
        }
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
          float4v acc = {0.f, 0.f, 0.f, 0.f};
          if (kt < n_tiles) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float4v a4 = *reinterpret_cast<const float4v*>(Ks + (kt * 16 + l16) * kQS + g * 16 + i * 4);
#pragma unroll
              for (int j = 0; j < 4; ++j)
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[j], bq[i * 4 + j], acc, 0, 0, 0);
            }
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) s[kt][r] = acc[r];
        }
      }
      // ---- masked softmax over the keys of query q ------------------------------------------
      float mx = 0.f;                          // clamp of the maximum at 0
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float tv = s[kt][r] * scaler + (float)mreg[qi][kt][r];   // mreg: (1 - mask) * -10000, -inf beyond seq_len
          s[kt][r] = tv;
          mx = fmaxf(mx, tv);
        }
      mx = xor_lanes_16_32_max(mx) * kLog2e;
      float sum = 0.f;
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          s[kt][r] = __builtin_amdgcn_exp2f(s[kt][r] * kLog2e - mx);
          sum += s[kt][r];
        }
      sum = xor_lanes_16_32_sum(sum) + 1e-6f;
      const float inv = 1.0f / sum;
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) s[kt][r] *= inv;
      // ---- O^T = V^T P^T --------------------------------------------------------------------
      float4v o[4];
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) o[dt] = float4v{0.f, 0.f, 0.f, 0.f};
      if constexpr (sizeof(T) == 2) {
        // A operand j = V^T rows {4*l + j}: the lane reads 4 consecutive features of its 8 keys (the keys its
        // probability registers belong to) and transposes the 8x4 block with v_perm_b32
#pragma unroll
        for (int ks = 0; ks < NKT / 2; ++ks) {
          if (2 * ks < n_tiles) {
            half8 p;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              p[r] = f2h(s[2 * ks][r]);
              p[4 + r] = f2h(s[2 * ks + 1][r]);
            }
            typedef uint32_t u2 __attribute__((ext_vector_type(2)));
            typedef uint32_t u4 __attribute__((ext_vector_type(4)));
            u2 raw[8];
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
              const int key = ks * 32 + (kk >> 2) * 16 + g * 4 + (kk & 3);
              raw[kk] = *reinterpret_cast<const u2*>(Vt + key * kVR + l16 * 4);
            }
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
              u4 lo, hi;
#pragma unroll
              for (int q4 = 0; q4 < 4; ++q4) {
                lo[q4] = __builtin_amdgcn_perm(raw[2 * q4 + 1][jj], raw[2 * q4][jj], 0x05040100u);
                hi[q4] = __builtin_amdgcn_perm(raw[2 * q4 + 1][jj], raw[2 * q4][jj], 0x07060302u);
              }
              o[2 * jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, lo), p, o[2 * jj], 0, 0, 0);
              o[2 * jj + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, hi), p, o[2 * jj + 1], 0, 0, 0);
            }
          }
        }
      } else {
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
          if (kt < n_tiles) {
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) {
              const float4v a4 = *reinterpret_cast<const float4v*>(Vt + (dt * 16 + l16) * kVS + kt * 16 + g * 4);
#pragma unroll
              for (int r = 0; r < 4; ++r)
                o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[r], s[kt][r], o[dt], 0, 0, 0);
            }
          }
        }
      }
      // ---- write the lane's 16 features of its query's packed row --------------------------
      if (out_row[qi] != nullptr) {
        if constexpr (sizeof(T) == 2) {
          // o[j][r] is feature 16*g + 4*r + j: 16 consecutive features
          half8 v0, v1;
#pragma unroll
          for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              v0[4 * r + j] = f2h(o[j][r]);
              v1[4 * r + j] = f2h(o[j][2 + r]);
            }
          T* orow = out_row[qi] + head * kD;
          *reinterpret_cast<half8*>(orow) = v0;
          *reinterpret_cast<half8*>(orow + 8) = v1;
        } else {
          T* orow = out_row[qi] + head * kD;
#pragma unroll
          for (int dt = 0; dt < 4; ++dt) {
            typedef T out4 __attribute__((ext_vector_type(4)));
            out4 v;
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = (T)o[dt][r];
            *reinterpret_cast<out4*>(orow + dt * 16) = v;
          }
        }
      }
    }
  }
}

#undef ET_ATTN_LOAD_HEAD

template <typename T, int NKT>
void attention_launch(const void* q, const void* k, const void* v, int layout, int packed_ld, const void* attr_mask,
                      void* dst, const int32_t* seq_start, const int32_t* word_idx, int batch, int seq_len, int heads,
                      float scaler, hipStream_t stream) {
  using Sm = AttnSmem<T, NKT>;
  constexpr int kCpr = kD * (int)sizeof(T) / 16;
  // Four wavefronts.  Eight at 128 keys in fp16 (one query tile per wavefront, 128 registers, two workgroups per CU)
  // run the kernel alone 6 % faster on a batch with few long sequences and no faster inside the layer.
  constexpr int WAVES = 4;
  constexpr int kThreads = WAVES * kWave;
  constexpr int CPT = (NKT * 16 * kCpr + kThreads - 1) / kThreads;
  constexpr bool PF = CPT <= 4;                // more than 4 chunks x 3 matrices in flight would not fit the registers
  auto kern = attention_kernel<T, NKT, WAVES, CPT, PF>;
  allow_dynamic_lds(reinterpret_cast<const void*>(kern), (int)Sm::kBytes);
  // A workgroup serves several heads of one sequence: mask rows, positions and zero fill are shared by them, and the
  // chain of dependent loads a workgroup starts with (sequence start, positions, rows) is paid once.  Up to 6 heads
  // (4 in fp32; 8 for the 128-key kernel, whose start is the longest), in equal groups, as long as about two workgroups per CU
  // remain: measured best on batches of 100 x 32, 1000 x 64 and 256 x 128 tokens.
  int hpw = 1;
  for (int h = NKT >= 8 ? 8 : (sizeof(T) == 2 ? 6 : 4); h > 1; --h)
    if (heads % h == 0 && (long)batch * (heads / h) >= 512) {
      hpw = h;
      break;
    }
  dim3 grid((heads + hpw - 1) / hpw, batch);
  kern<<<grid, kThreads, Sm::kBytes, stream>>>((const T*)q, (const T*)k, (const T*)v, layout, packed_ld,
                                                   (const T*)attr_mask, (T*)dst, seq_start, word_idx, batch, seq_len,
                                                   heads, hpw, scaler);
}


// ------------------------------------------------------------------------------------------
// fused attention for 128 < seq_len <= 512: one workgroup (4 wavefronts) per (64 queries, head, sequence).
// The scores of a wavefront's 16 queries against all keys stay in registers (4 per lane and 16-key tile); K and
// V pass through LDS in chunks of 128 keys (K chunks first, the softmax over the registers, then V chunks), so the
// LDS footprint does not grow with the sequence.  Q comes straight from global memory: the MFMA operand of a lane
// is 16 (fp16) or 64 (fp32) contiguous bytes of its query's row.  Arithmetic and rounding points are those of
// the kernel above; key tiles beyond the last token skip their MFMAs (score 0, value 0).
// ------------------------------------------------------------------------------------------
constexpr int kLongChunkTiles = 8;                 // 128 keys per LDS chunk
constexpr int kLongChunk = kLongChunkTiles * 16;

template <typename T>
struct LongSmem {
  static constexpr int kQS = AttnCfg<T>::kQkStride;
  static constexpr int kVR = AttnCfg<_Float16>::kVStride;              // fp16 V rows
  static constexpr int kVS = kLongChunk + AttnCfg<T>::kVtPad;          // fp32 V^T rows
  static constexpr size_t kKBytes = (size_t)kLongChunk * kQS * sizeof(T);
  static constexpr size_t kVBytes = sizeof(T) == 2 ? (size_t)kLongChunk * kVR * sizeof(T) : (size_t)kD * kVS * sizeof(T);
  static constexpr size_t kTileBytes = kKBytes > kVBytes ? kKBytes : kVBytes;   // K and V chunks take turns
};

template <typename T, int NKT>
__global__ __launch_bounds__(kAttnThreads) void attention_long_kernel(
    const T* __restrict__ q_src, const T* __restrict__ k_src, const T* __restrict__ v_src, int layout, int packed_ld,
    const T* __restrict__ attr_mask, T* __restrict__ dst, const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ word_idx, int batch, int seq_len, int heads, float scaler) {
  using Sm = LongSmem<T>;
  using C = Chunk16<T>;
  using V16 = typename C::vec;
  constexpr int kQS = Sm::kQS, kVR = Sm::kVR, kVS = Sm::kVS;
  constexpr int kSp = NKT * 16;
  constexpr int kCpr = kD / C::kElems;
  constexpr int kChunks = NKT / kLongChunkTiles;
  constexpr int CPT = kLongChunk * kCpr / kAttnThreads;      // 16-byte pieces of a chunk per thread
  typedef T mask4 __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* Ks = reinterpret_cast<T*>(smem_raw);                    // K chunk, later V chunk
  T* Vs = Ks;
  int* tok_of_pos = reinterpret_cast<int*>(smem_raw + Sm::kTileBytes);

  const int b = min(max(seq_start[batch + 1 + blockIdx.z], 0), batch - 1), head = blockIdx.y, qblock = blockIdx.x;
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  const int len = t1 - t0;
  if (len <= 0) return;
  const int H = heads * kD;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int l16 = lane & 15, g = lane >> 4;

  const int last_pos = min(max(word_idx[t1 - 1], 0), seq_len - 1);
  const int n_tiles = last_pos / 16 + 1;                     // 16-row tiles that hold at least one token
  if (qblock * 4 >= n_tiles) return;                         // no token among this workgroup's queries
  for (int i = threadIdx.x; i < kSp; i += kAttnThreads) tok_of_pos[i] = -1;
  __syncthreads();
  for (int tt = threadIdx.x; tt < len; tt += kAttnThreads) {
    const int pos = word_idx[t0 + tt];
    if (pos >= 0 && pos < seq_len) tok_of_pos[pos] = t0 + tt;
  }
  __syncthreads();

  // element offset of (token t / position pos, this head) in the source matrices
  auto src_off = [&](int t, int pos) -> size_t {
    return layout == 1 ? (size_t)t * packed_ld + head * kD : (((size_t)b * heads + head) * seq_len + pos) * kD;
  };
  // stage rows [c0, c0 + 128) of `src` row-major (stride `stride` elements) into LDS, zeros where no token sits
  auto stage_rows = [&](const T* __restrict__ src, T* lds, int stride, int c0) {
    V16 r[CPT];
    int tk[CPT];
#pragma unroll
    for (int k = 0; k < CPT; ++k) {
      const int i = threadIdx.x + k * kAttnThreads;
      const int row = i / kCpr, c = i - row * kCpr;
      const int pos = c0 + row;
      tk[k] = pos < kSp ? tok_of_pos[pos] : -1;
#pragma unroll
      for (int j = 0; j < C::kElems; ++j) r[k][j] = (T)0;
      if (tk[k] >= 0) r[k] = *reinterpret_cast<const V16*>(src + src_off(tk[k], pos) + c * C::kElems);
    }
#pragma unroll
    for (int k = 0; k < CPT; ++k) {
      const int i = threadIdx.x + k * kAttnThreads;
      const int row = i / kCpr, c = i - row * kCpr;
      *reinterpret_cast<V16*>(lds + row * stride + c * C::kElems) = r[k];
    }
  };

  const int qt = qblock * 4 + wave;                          // this wavefront's 16-query tile
  const bool active = qt < n_tiles;                          // wave-uniform
  const int q = qt * 16 + l16;
  const int tq = (active && q < kSp) ? tok_of_pos[q] : -1;
  const T* mrow = attr_mask + ((size_t)b * seq_len + min(q, seq_len - 1)) * seq_len;
  const bool vec_mask = (seq_len & 3) == 0;

  // Q operand of this lane (zeros for a query position without a token: its result is never stored)
  half8 bqh[2];
  float bqf[16];
  if constexpr (sizeof(T) == 2) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int j = 0; j < 8; ++j) bqh[ks][j] = (_Float16)0;
      if (tq >= 0) bqh[ks] = *reinterpret_cast<const half8*>(q_src + src_off(tq, q) + ks * 32 + g * 8);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float4v v4 = {0.f, 0.f, 0.f, 0.f};
      if (tq >= 0) v4 = *reinterpret_cast<const float4v*>(q_src + src_off(tq, q) + g * 16 + i * 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) bqf[i * 4 + j] = v4[j];
    }
  }

  // ---- S^T = K Q^T chunk by chunk, bias added on the way ------------------------------------------
  float s[NKT][4];
#pragma unroll
  for (int ch = 0; ch < kChunks; ++ch) {
    const bool chunk_has_tokens = ch * kLongChunkTiles < n_tiles;       // workgroup-uniform
    if (chunk_has_tokens) {
      __syncthreads();                                                  // previous chunk fully consumed
      stage_rows(k_src, Ks, kQS, ch * kLongChunk);
      __syncthreads();
    }
    if (active) {
#pragma unroll
      for (int kc = 0; kc < kLongChunkTiles; ++kc) {
        const int kt = ch * kLongChunkTiles + kc;
        float4v acc = {0.f, 0.f, 0.f, 0.f};
        if (kt < n_tiles) {
          if constexpr (sizeof(T) == 2) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
              const half8 a = *reinterpret_cast<const half8*>(Ks + (kc * 16 + l16) * kQS + ks * 32 + g * 8);
              acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bqh[ks], acc, 0, 0, 0);
            }
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float4v a4 = *reinterpret_cast<const float4v*>(Ks + (kc * 16 + l16) * kQS + g * 16 + i * 4);
#pragma unroll
              for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[j], bqf[i * 4 + j], acc, 0, 0, 0);
            }
          }
        }
        const int key0 = kt * 16 + g * 4;
        mask4 m4 = {(T)0, (T)0, (T)0, (T)0};
        if (vec_mask) {
          if (key0 < seq_len) m4 = *reinterpret_cast<const mask4*>(mrow + key0);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (key0 + r < seq_len) m4[r] = mrow[key0 + r];
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float sc = sizeof(T) == 2 ? h2f(f2h(acc[r])) : acc[r];      // the score is stored in the element type
          s[kt][r] = key0 + r < seq_len ? sc * scaler + (1.0f - (float)m4[r]) * -10000.0f : -INFINITY;
        }
      }
    }
  }

  // ---- masked softmax over the registers ---------------------------------------------------------------
  if (active) {
    float mx = 0.f;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[kt][r]);
    mx = xor_lanes_16_32_max(mx) * kLog2e;
    float sum = 0.f;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[kt][r] = __builtin_amdgcn_exp2f(s[kt][r] * kLog2e - mx);
        sum += s[kt][r];
      }
    sum = xor_lanes_16_32_sum(sum) + 1e-6f;
    const float inv = 1.0f / sum;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) s[kt][r] *= inv;
  }

  // ---- O^T = V^T P^T chunk by chunk ----------------------------------------------------------------------
  float4v o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) o[dt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ch = 0; ch < kChunks; ++ch) {
    if (ch * kLongChunkTiles >= n_tiles) break;                         // workgroup-uniform: no token, value 0
    __syncthreads();
    if constexpr (sizeof(T) == 2) {
      stage_rows(v_src, Vs, kVR, ch * kLongChunk);
    } else {
      // fp32 keeps V^T: feature rows, key columns
#pragma unroll
      for (int k = 0; k < CPT; ++k) {
        const int i = threadIdx.x + k * kAttnThreads;
        const int row = i / kCpr, c = i - row * kCpr;
        const int pos = ch * kLongChunk + row;
        const int tk = pos < kSp ? tok_of_pos[pos] : -1;
        V16 r = {0.f, 0.f, 0.f, 0.f};
        if (tk >= 0) r = *reinterpret_cast<const V16*>(v_src + src_off(tk, pos) + c * C::kElems);
#pragma unroll
        for (int j = 0; j < C::kElems; ++j) Vs[(c * C::kElems + j) * kVS + row] = r[j];
      }
    }
    __syncthreads();
    if (!active) continue;
    if constexpr (sizeof(T) == 2) {
#pragma unroll
      for (int kp = 0; kp < kLongChunkTiles / 2; ++kp) {
        const int kt = ch * kLongChunkTiles + 2 * kp;
        if (kt < n_tiles) {
          half8 p;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            p[r] = f2h(s[kt][r]);
            p[4 + r] = f2h(s[kt + 1][r]);
          }
          typedef uint32_t u2 __attribute__((ext_vector_type(2)));
          typedef uint32_t u4 __attribute__((ext_vector_type(4)));
          u2 raw[8];
#pragma unroll
          for (int kk = 0; kk < 8; ++kk) {
            const int key = kp * 32 + (kk >> 2) * 16 + g * 4 + (kk & 3);
            raw[kk] = *reinterpret_cast<const u2*>(Vs + key * kVR + l16 * 4);
          }
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            u4 lo, hi;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
              lo[q4] = __builtin_amdgcn_perm(raw[2 * q4 + 1][jj], raw[2 * q4][jj], 0x05040100u);
              hi[q4] = __builtin_amdgcn_perm(raw[2 * q4 + 1][jj], raw[2 * q4][jj], 0x07060302u);
            }
            o[2 * jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, lo), p, o[2 * jj], 0, 0, 0);
            o[2 * jj + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, hi), p, o[2 * jj + 1], 0, 0, 0);
          }
        }
      }
    } else {
#pragma unroll
      for (int kc = 0; kc < kLongChunkTiles; ++kc) {
        const int kt = ch * kLongChunkTiles + kc;
        if (kt < n_tiles) {
#pragma unroll
          for (int dt = 0; dt < 4; ++dt) {
            const float4v a4 = *reinterpret_cast<const float4v*>(Vs + (dt * 16 + l16) * kVS + kc * 16 + g * 4);
#pragma unroll
            for (int r = 0; r < 4; ++r) o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[r], s[kt][r], o[dt], 0, 0, 0);
          }
        }
      }
    }
  }

  if (tq >= 0) {
    if constexpr (sizeof(T) == 2) {
      half8 v0, v1;
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v0[4 * r + j] = f2h(o[j][r]);
          v1[4 * r + j] = f2h(o[j][2 + r]);
        }
      T* orow = dst + (size_t)tq * H + head * kD + g * 16;
      *reinterpret_cast<half8*>(orow) = v0;
      *reinterpret_cast<half8*>(orow + 8) = v1;
    } else {
      T* orow = dst + (size_t)tq * H + head * kD + g * 4;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        float4v v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = o[dt][r];
        *reinterpret_cast<float4v*>(orow + dt * 16) = v;
      }
    }
  }
}

template <typename T, int NKT>
void attention_long_launch(const void* q, const void* k, const void* v, int layout, int packed_ld, const void* attr_mask,
                           void* dst, const int32_t* seq_start, const int32_t* word_idx, int batch, int seq_len, int heads,
                           float scaler, hipStream_t stream) {
  const size_t smem = LongSmem<T>::kTileBytes + (size_t)NKT * 16 * sizeof(int);
  auto kern = attention_long_kernel<T, NKT>;
  dim3 grid((seq_len + 63) / 64, heads, batch);               // blocks of 64 queries that can hold a token
  kern<<<grid, kAttnThreads, smem, stream>>>((const T*)q, (const T*)k, (const T*)v, layout, packed_ld, (const T*)attr_mask,
                                             (T*)dst, seq_start, word_idx, batch, seq_len, heads, scaler);
}

// ------------------------------------------------------------------------------------------
// K / V rows brought into LDS by DMA (the resident-key kernels below): rows of 128 bytes without padding, one
// `buffer_load ... lds` instruction fills eight of them (lane -> row lane / 8, 16-byte chunk lane & 7).  A row without
// a token is requested beyond its buffer descriptor's range and arrives as zeros.
// Which key a row of an MFMA tile stands for is free as long as K, the mask and V agree: row m of the first tile of a
// pair (32 keys from `base`) is key base + (m >> 2) * 8 + (m & 3), of the second tile 4 keys further.  A lane's scores
// of a pair are then 8 consecutive keys: one 16-byte load of its mask row, and the P operand of the P.V MFMA is in
// natural key order.  Key row `key` lies in slot key ^ ((key >> 3) & 1) (the two rows of a half-wave of the 8-byte V
// reads, 8 keys apart, land on different halves of the banks), and the 16-byte chunks of a slot are XOR-swizzled with
// slot bits 1, 3 and 4 (the 16 rows x one chunk of a K operand read cover all 64 banks).
// ------------------------------------------------------------------------------------------
#define ET_ATTN_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
__device__ __forceinline__ int wide_slot(int key) { return key ^ ((key >> 3) & 1); }
__device__ __forceinline__ int wide_swizzle(int slot) { return ((slot >> 1) & 1) | ((slot >> 2) & 6); }
// s_waitcnt immediates of gfx9: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]
__device__ __forceinline__ void wide_wait_dma() { __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8) | (0 << 14)); }
__device__ __forceinline__ void wide_wait_lds() { __builtin_amdgcn_s_waitcnt(15 | (7 << 4) | (0 << 8) | (3 << 14)); }
// barrier without the fence of __syncthreads(), which would wait for every DMA in flight
__device__ __forceinline__ void wide_barrier() { asm volatile("s_barrier" ::: "memory"); }

// ------------------------------------------------------------------------------------------
// fp16 fused attention for 128 < seq_len <= 512 with K and V of the whole sequence resident in LDS: one workgroup of
// 8 wavefronts per (head, sequence) (or per share of its query tiles, see `qsplit`).  K and V arrive once by DMA (64 +
// 64 KB at 512 keys, all requests in flight at once, layout above) instead of once per block of 64 queries, and after
// that one barrier the wavefronts run their 16-query tiles independently: S^T = K Q^T over all key tiles, the softmax
// over the registers, O^T = V^T P^T.  Arithmetic and rounding points per element are those of attention_long_kernel.
// ------------------------------------------------------------------------------------------
constexpr int kResThreads = 512;
[[maybe_unused]] constexpr int kResWaves = kResThreads / kWave;

template <int NKT>
struct ResSmem {
  static constexpr int kSp = NKT * 16;
  static constexpr size_t kKBytes = (size_t)kSp * 128;
  static constexpr size_t kVBytes = (size_t)kSp * 128;
  static constexpr size_t kBytes = kKBytes + kVBytes + (size_t)kSp * sizeof(int);
};

template <int NKT>
__global__ __launch_bounds__(kResThreads) __attribute__((amdgpu_waves_per_eu(NKT <= 16 ? 4 : 2, NKT <= 16 ? 4 : 2)))
void attention_resident_kernel(
    const _Float16* __restrict__ q_src, const _Float16* __restrict__ k_src, const _Float16* __restrict__ v_src, int layout,
    int packed_ld, const _Float16* __restrict__ attr_mask, _Float16* __restrict__ dst,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ word_idx, int batch, int seq_len, int heads,
    int qsplit, float scaler) {
#if defined(__HIP_DEVICE_COMPILE__)   // device-only types in the body; the host pass only needs the stub
  using T = _Float16;
  using Sm = ResSmem<NKT>;
  constexpr int kSp = Sm::kSp;

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  unsigned char* ks = smem_raw;
  unsigned char* vs = smem_raw + Sm::kKBytes;
  int* tok_of_pos = reinterpret_cast<int*>(smem_raw + Sm::kKBytes + Sm::kVBytes);

  const int b = min(max(seq_start[batch + 1 + blockIdx.y], 0), batch - 1);
  const int head = blockIdx.x / qsplit, part = blockIdx.x - head * qsplit;
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  const int len = t1 - t0;
  if (len <= 0) return;
  const int H = heads * kD;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int l16 = lane & 15, g = lane >> 4;

  const int last_pos = min(max(word_idx[t1 - 1], 0), seq_len - 1);
  const int n_tiles = last_pos / 16 + 1;                     // 16-row tiles that hold at least one token
  if (part >= n_tiles) return;                               // no query tile for this share (workgroup-uniform)
  for (int i = threadIdx.x; i < kSp; i += kResThreads) tok_of_pos[i] = -1;
  __syncthreads();
  for (int tt = threadIdx.x; tt < len; tt += kResThreads) {
    const int pos = word_idx[t0 + tt];
    if (pos >= 0 && pos < seq_len) tok_of_pos[pos] = tt;     // relative to the sequence's first packed row
  }
  __syncthreads();

  // K and V rows of every group of four key tiles that holds a token (the loops below run over such groups)
  const int n_groups = (n_tiles + 3) / 4;
  {
    const int rows_in = min(kSp, n_groups * 64);
    const T* kbase = layout == 1 ? k_src + (size_t)t0 * packed_ld + head * kD : k_src + ((size_t)b * heads + head) * seq_len * kD;
    const T* vbase = layout == 1 ? v_src + (size_t)t0 * packed_ld + head * kD : v_src + ((size_t)b * heads + head) * seq_len * kD;
    const uint32_t bytes = layout == 1 ? ((uint32_t)(len - 1) * (uint32_t)packed_ld + kD) * 2u : (uint32_t)seq_len * kD * 2u;
    const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(kbase), 0, (int)bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(vbase), 0, (int)bytes, 0x00020000);
    for (int i = wave; i < rows_in / 8; i += kResWaves) {
      const int slot = i * 8 + (lane >> 3);
      const int key = wide_slot(slot);
      const int c = (lane & 7) ^ wide_swizzle(slot);
      const int tk = tok_of_pos[key];
      const uint32_t row_off = layout == 1 ? (uint32_t)tk * (uint32_t)packed_ld : (uint32_t)key * kD;
      const uint32_t voff = tk >= 0 ? (row_off + (uint32_t)c * 8u) * 2u : 0x80000000u;      // out of range: zeros
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, ET_ATTN_LDS_PTR(ks + i * 1024), 16, voff, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, ET_ATTN_LDS_PTR(vs + i * 1024), 16, voff, 0, 0, 0);
    }
  }
  wide_wait_dma();
  __syncthreads();

  // Operand addresses: a lane-dependent base plus a compile-time offset per tile.  The slot flip touches bit 0 of the
  // row and the swizzle bits 1, 3, 4, none of which the tile's part of the row number (multiples of 32, +4 for the
  // second tile of a pair) reaches, so both are constants of the lane.
  //   K, row l16 of a tile: key row L = (l16 >> 2) * 8 + (l16 & 3) within the pair, chunk ks * 4 + g
  const unsigned char* kbase_ks[2];
  {
    const int L = wide_slot((l16 >> 2) * 8 + (l16 & 3));
    const int sw = wide_swizzle(L);
#pragma unroll
    for (int ks2 = 0; ks2 < 2; ++ks2) kbase_ks[ks2] = ks + L * 128 + (((ks2 * 4 + g) ^ sw) * 16);
  }
  //   V, key g * 8 + kk of a pair (kk = 4 a + 2 b + c), features 4 l16 ..: base by (b, c), offset 512 a
  const unsigned char* vbase_bc[2][2];
#pragma unroll
  for (int bb = 0; bb < 2; ++bb)
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      const int slot = wide_slot(g * 8 + 2 * bb + cc);
      vbase_bc[bb][cc] = vs + slot * 128 + (((l16 >> 1) ^ wide_swizzle(slot)) * 16) + (l16 & 1) * 8;
    }

  const bool vec_mask = (seq_len & 7) == 0;                  // mask rows start at multiples of 16 bytes
  for (int qt = part + qsplit * wave; qt < n_tiles; qt += qsplit * kResWaves) {
    const int q = qt * 16 + l16;
    const int tq = tok_of_pos[q];
    const T* mrow = attr_mask + ((size_t)b * seq_len + min(q, seq_len - 1)) * seq_len;
    // Q operand of this lane (zeros for a query position without a token: its result is never stored)
    half8 bqh[2];
#pragma unroll
    for (int ks2 = 0; ks2 < 2; ++ks2) {
#pragma unroll
      for (int j = 0; j < 8; ++j) bqh[ks2][j] = (_Float16)0;
      if (tq >= 0) {
        const size_t qo = layout == 1 ? (size_t)(t0 + tq) * packed_ld + head * kD
                                      : (((size_t)b * heads + head) * seq_len + q) * kD;
        bqh[ks2] = *reinterpret_cast<const half8*>(q_src + qo + ks2 * 32 + g * 8);
      }
    }

    // ---- the additive bias of the mask row first: the whole row requested before any of it is converted --------
    float s[NKT][4];                                         // s[2 P], s[2 P + 1]: keys 32 P + 8 g + 0..3, + 4..7
    // (opaque to the compiler, or it would keep the clamped offsets of all pairs in registers across query tiles)
    int g8 = g * 8;
    asm volatile("" : "+v"(g8));
    // (1 - m) * -10000 as one fma: 1 - m is exact in float for a half m, so both forms round the same real number once
    if (vec_mask) {
      half8 m8[NKT / 2];
#pragma unroll
      for (int kp = 0; kp < NKT / 2; ++kp) m8[kp] = *reinterpret_cast<const half8*>(mrow + min(kp * 32 + g8, seq_len - 8));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kp = 0; kp < NKT / 2; ++kp) {
        const int key0 = kp * 32 + g8;
        if ((kp + 1) * 32 <= seq_len) {                      // wave-uniform: every key of the pair exists
#pragma unroll
          for (int j = 0; j < 8; ++j) s[2 * kp + (j >> 2)][j & 3] = __builtin_fmaf((float)m8[kp][j], 10000.0f, -10000.0f);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            s[2 * kp + (j >> 2)][j & 3] = key0 < seq_len ? __builtin_fmaf((float)m8[kp][j], 10000.0f, -10000.0f) : -INFINITY;
        }
      }
    } else {
#pragma unroll
      for (int kp = 0; kp < NKT / 2; ++kp) {
        const int key0 = kp * 32 + g8;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const T m = mrow[min(key0 + j, seq_len - 1)];
          s[2 * kp + (j >> 2)][j & 3] = key0 + j < seq_len ? __builtin_fmaf((float)m, 10000.0f, -10000.0f) : -INFINITY;
        }
        if (kp % 2 == 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- S^T = K Q^T, four key tiles at a time (rows without a token are zero: score 0) ---------------------
#pragma unroll
    for (int kg = 0; kg < NKT / 4; ++kg) {
      if (kg < n_groups) {
#pragma unroll
        for (int kc = 0; kc < 4; ++kc) {
          const int kt = kg * 4 + kc;
          // row l16 of tile kt: pair kt >> 1, first or second tile kt & 1 (4 rows further)
          float4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks2 = 0; ks2 < 2; ++ks2) {
            const half8 a = *reinterpret_cast<const half8*>(kbase_ks[ks2] + ((kt & ~1) * 16 + (kt & 1) * 4) * 128);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bqh[ks2], acc, 0, 0, 0);
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float sc = h2f(f2h(acc[r]));                         // the score is stored in half
            s[kt][r] = sc * scaler + s[kt][r];                         // -inf stays -inf for keys that do not exist
          }
        }
      }
    }

    // ---- masked softmax over the registers ------------------------------------------------------------
    {
      float mx = 0.f;
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[kt][r]);
      mx = xor_lanes_16_32_max(mx) * kLog2e;
      float sum = 0.f;
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          s[kt][r] = __builtin_amdgcn_exp2f(s[kt][r] * kLog2e - mx);
          sum += s[kt][r];
        }
      sum = xor_lanes_16_32_sum(sum) + 1e-6f;
      const float inv = 1.0f / sum;
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) s[kt][r] *= inv;
    }

    // ---- O^T = V^T P^T over pairs of key tiles ----------------------------------------------------------
    float4v o[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) o[dt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kp = 0; kp < NKT / 2; ++kp) {
      const int kt = 2 * kp;
      if (kp / 2 < n_groups) {
        half8 p;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          p[r] = f2h(s[kt][r]);
          p[4 + r] = f2h(s[kt + 1][r]);
        }
        typedef uint32_t u2 __attribute__((ext_vector_type(2)));
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        u2 raw[8];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
          raw[kk] = *reinterpret_cast<const u2*>(vbase_bc[(kk >> 1) & 1][kk & 1] + (kp * 32 + (kk & 4)) * 128);
        }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          u4 lo, hi;
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            lo[q4] = __builtin_amdgcn_perm(raw[2 * q4 + 1][jj], raw[2 * q4][jj], 0x05040100u);
            hi[q4] = __builtin_amdgcn_perm(raw[2 * q4 + 1][jj], raw[2 * q4][jj], 0x07060302u);
          }
          o[2 * jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, lo), p, o[2 * jj], 0, 0, 0);
          o[2 * jj + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, hi), p, o[2 * jj + 1], 0, 0, 0);
        }
      }
    }

    if (tq >= 0) {
      half8 v0, v1;
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v0[4 * r + j] = f2h(o[j][r]);
          v1[4 * r + j] = f2h(o[j][2 + r]);
        }
      T* orow = dst + (size_t)(t0 + tq) * H + head * kD + g * 16;
      *reinterpret_cast<half8*>(orow) = v0;
      *reinterpret_cast<half8*>(orow + 8) = v1;
    }
  }
#endif
}

inline int attention_cu_count() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
    return 256;
  return n;
}

template <int NKT>
void attention_resident_launch(const void* q, const void* k, const void* v, int layout, int packed_ld,
                               const void* attr_mask, void* dst, const int32_t* seq_start, const int32_t* word_idx,
                               int batch, int seq_len, int heads, float scaler, hipStream_t stream) {
  using Sm = ResSmem<NKT>;
  auto kern = attention_resident_kernel<NKT>;
  allow_dynamic_lds(reinterpret_cast<const void*>(kern), (int)Sm::kBytes);
  // few (head, sequence) pairs: the query tiles of a pair are dealt to 2 or 4 workgroups, each staging K and V itself
  const long pairs = (long)heads * batch;
  const int cus = attention_cu_count();
  const int qsplit = pairs >= cus ? 1 : (2 * pairs >= cus ? 2 : 4);
  dim3 grid(heads * qsplit, batch);
  kern<<<grid, kResThreads, Sm::kBytes, stream>>>((const _Float16*)q, (const _Float16*)k, (const _Float16*)v, layout,
                                                 packed_ld, (const _Float16*)attr_mask, (_Float16*)dst, seq_start,
                                                 word_idx, batch, seq_len, heads, qsplit, scaler);
}

// ------------------------------------------------------------------------------------------
// fused attention for 512 < seq_len <= 1024: the chunked kernel above with the keys of a query tile split over two
// wavefronts.  One workgroup of 8 wavefronts per (64 queries, head, sequence): wavefront w serves query tile w & 3 and
// the key half w >> 2 (512 keys: 4 scores per lane and key tile, 128 VGPRs).  K and V pass through LDS in chunks of
// 128 keys per half, both halves in the same step.  The two halves of a query tile exchange their maxima and their
// sums through LDS (sum = first half + second half, the same on both sides), and the second half hands its part of
// O over for the first to add and store.  Arithmetic and rounding points per element are those of the other kernels;
// at 1024 keys the maximum is not clamped at 0 (see attention_generic_kernel).
// ------------------------------------------------------------------------------------------
constexpr int kSplitThreads = 512;
constexpr int kSplitHalfTiles = 32;               // key tiles per wavefront
constexpr int kSplitKeys = 2 * kSplitHalfTiles * 16;

template <typename T>
__global__ __launch_bounds__(kSplitThreads) void attention_split_kernel(
    const T* __restrict__ q_src, const T* __restrict__ k_src, const T* __restrict__ v_src, int layout, int packed_ld,
    const T* __restrict__ attr_mask, T* __restrict__ dst, const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ word_idx, int batch, int seq_len, int heads, float scaler) {
  static_assert(sizeof(T) == 4, "fp32 only: fp16 beyond 512 positions runs attention_wide_kernel");
  using Sm = LongSmem<T>;
  using C = Chunk16<T>;
  using V16 = typename C::vec;
  constexpr int kQS = Sm::kQS, kVS = Sm::kVS;
  constexpr int kCpr = kD / C::kElems;
  constexpr int NKT = kSplitHalfTiles;
  constexpr int kChunks = NKT / kLongChunkTiles;             // 4 steps of 128 keys per half
  constexpr int CPT = kLongChunk * kCpr / kAttnThreads;      // 16-byte pieces of a chunk per thread of a half
  typedef T mask4 __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  int* tok_of_pos = reinterpret_cast<int*>(smem_raw + 2 * Sm::kTileBytes);
  float* red = reinterpret_cast<float*>(smem_raw + 2 * Sm::kTileBytes + kSplitKeys * sizeof(int));   // [2][4 tiles][2 halves][16]

  const int b = min(max(seq_start[batch + 1 + blockIdx.z], 0), batch - 1), head = blockIdx.y, qblock = blockIdx.x;
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  const int len = t1 - t0;
  if (len <= 0) return;
  const int H = heads * kD;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int tile_w = wave & 3, half = wave >> 2;
  const int l16 = lane & 15, g = lane >> 4;
  // this half's staging threads (256 per half) and its chunk buffer
  const int tid_h = threadIdx.x & (kAttnThreads - 1);
  T* Ks = reinterpret_cast<T*>(smem_raw + half * Sm::kTileBytes);
  T* Vs = Ks;
  const int kt_base = half * NKT;                            // first key tile of this half

  const int last_pos = min(max(word_idx[t1 - 1], 0), seq_len - 1);
  const int n_tiles = last_pos / 16 + 1;                     // 16-row tiles that hold at least one token
  if (qblock * 4 >= n_tiles) return;                         // no token among this workgroup's queries
  for (int i = threadIdx.x; i < kSplitKeys; i += kSplitThreads) tok_of_pos[i] = -1;
  __syncthreads();
  for (int tt = threadIdx.x; tt < len; tt += kSplitThreads) {
    const int pos = word_idx[t0 + tt];
    if (pos >= 0 && pos < seq_len) tok_of_pos[pos] = t0 + tt;
  }
  __syncthreads();

  auto src_off = [&](int t, int pos) -> size_t {
    return layout == 1 ? (size_t)t * packed_ld + head * kD : (((size_t)b * heads + head) * seq_len + pos) * kD;
  };
  // rows [c0, c0 + 128) of `src`, zeros where no token sits: global memory -> registers -> this half's buffer
  // (row-major, stride `stride` elements)
  auto stage_rows = [&](const T* __restrict__ src, T* lds, int stride, int c0) {
    V16 r[CPT];
#pragma unroll
    for (int k = 0; k < CPT; ++k) {
      const int i = tid_h + k * kAttnThreads;
      const int row = i / kCpr, c = i - row * kCpr;
      const int pos = c0 + row;
      const int tk = pos < kSplitKeys ? tok_of_pos[pos] : -1;
#pragma unroll
      for (int j = 0; j < C::kElems; ++j) r[k][j] = (T)0;
      if (tk >= 0) r[k] = *reinterpret_cast<const V16*>(src + src_off(tk, pos) + c * C::kElems);
    }
#pragma unroll
    for (int k = 0; k < CPT; ++k) {
      const int i = tid_h + k * kAttnThreads;
      const int row = i / kCpr, c = i - row * kCpr;
      *reinterpret_cast<V16*>(lds + row * stride + c * C::kElems) = r[k];
    }
  };

  const int qt = qblock * 4 + tile_w;                        // this wavefront's 16-query tile
  const bool active = qt < n_tiles;                          // wave-uniform
  const int q = qt * 16 + l16;
  const int tq = (active && q < kSplitKeys) ? tok_of_pos[q] : -1;
  const T* mrow = attr_mask + ((size_t)b * seq_len + min(q, seq_len - 1)) * seq_len;
  const bool vec_mask = (seq_len & 3) == 0;

  // Q operand of this lane (zeros for a query position without a token: its result is never stored)
  float bqf[16];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float4v v4 = {0.f, 0.f, 0.f, 0.f};
    if (tq >= 0) v4 = *reinterpret_cast<const float4v*>(q_src + src_off(tq, q) + g * 16 + i * 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) bqf[i * 4 + j] = v4[j];
  }

  // ---- the additive bias of this half of the mask row (no branch between the loads) -------------------------
  float s[NKT][4];
  {
    int g4 = g * 4;
    asm volatile("" : "+v"(g4));       // opaque: the clamped offsets are recomputed, not kept in registers
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) {
      const int key0 = (kt_base + kt) * 16 + g4;
      if (vec_mask) {
        const mask4 m4 = *reinterpret_cast<const mask4*>(mrow + min(key0, seq_len - 4));
#pragma unroll
        for (int r = 0; r < 4; ++r) s[kt][r] = key0 < seq_len ? (1.0f - (float)m4[r]) * -10000.0f : -INFINITY;
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const T m = mrow[min(key0 + r, seq_len - 1)];
          s[kt][r] = key0 + r < seq_len ? (1.0f - (float)m) * -10000.0f : -INFINITY;
        }
      }
      if (kt % 4 == 3) __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- S^T = K Q^T chunk by chunk -------------------------------------------------------------------------
#pragma unroll
  for (int ch = 0; ch < kChunks; ++ch) {
    if (ch * kLongChunkTiles >= n_tiles) break;                          // workgroup-uniform: no token in either half
    const bool chunk_has_tokens = kt_base + ch * kLongChunkTiles < n_tiles;   // uniform over this half's 4 wavefronts
    __syncthreads();                                                     // previous chunks fully consumed
    if (chunk_has_tokens) stage_rows(k_src, Ks, kQS, (kt_base + ch * kLongChunkTiles) * 16);
    __syncthreads();
    if (active && chunk_has_tokens) {
#pragma unroll
      for (int kc = 0; kc < kLongChunkTiles; ++kc) {
        const int ktl = ch * kLongChunkTiles + kc;
        if (kt_base + ktl < n_tiles) {
          float4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float4v a4 = *reinterpret_cast<const float4v*>(Ks + (kc * 16 + l16) * kQS + g * 16 + i * 4);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[j], bqf[i * 4 + j], acc, 0, 0, 0);
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) s[ktl][r] = acc[r] * scaler + s[ktl][r];
        }
      }
    }
  }

  // ---- masked softmax: each half over its registers, maxima and sums exchanged through LDS --------------------
  float* red_max = red;
  float* red_sum = red + 4 * 2 * 16;
  {
    float mx = seq_len < kSplitKeys ? 0.f : -INFINITY;       // the clamp at 0 holds below 1024 keys
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[kt][r]);
    mx = xor_lanes_16_32_max(mx);
    if (g == 0) red_max[(tile_w * 2 + half) * 16 + l16] = mx;
  }
  __syncthreads();
  float inv;
  {
    const float mx = fmaxf(red_max[(tile_w * 2) * 16 + l16], red_max[(tile_w * 2 + 1) * 16 + l16]) * kLog2e;
    float sum = 0.f;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[kt][r] = __builtin_amdgcn_exp2f(s[kt][r] * kLog2e - mx);
        sum += s[kt][r];
      }
    sum = xor_lanes_16_32_sum(sum);
    if (g == 0) red_sum[(tile_w * 2 + half) * 16 + l16] = sum;
  }
  __syncthreads();
  {
    const float sum = red_sum[(tile_w * 2) * 16 + l16] + red_sum[(tile_w * 2 + 1) * 16 + l16] + 1e-6f;
    inv = 1.0f / sum;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) s[kt][r] *= inv;
  }

  // ---- O^T = V^T P^T chunk by chunk, each half over its keys ---------------------------------------------------
  float4v o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) o[dt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ch = 0; ch < kChunks; ++ch) {
    if (ch * kLongChunkTiles >= n_tiles) break;                         // workgroup-uniform
    const bool chunk_has_tokens = kt_base + ch * kLongChunkTiles < n_tiles;
    __syncthreads();
    if (chunk_has_tokens) {
      // V^T in LDS: feature rows, key columns
#pragma unroll
      for (int k = 0; k < CPT; ++k) {
        const int i = tid_h + k * kAttnThreads;
        const int row = i / kCpr, c = i - row * kCpr;
        const int pos = (kt_base + ch * kLongChunkTiles) * 16 + row;
        const int tk = pos < kSplitKeys ? tok_of_pos[pos] : -1;
        V16 r = {0.f, 0.f, 0.f, 0.f};
        if (tk >= 0) r = *reinterpret_cast<const V16*>(v_src + src_off(tk, pos) + c * C::kElems);
#pragma unroll
        for (int j = 0; j < C::kElems; ++j) Vs[(c * C::kElems + j) * kVS + row] = r[j];
      }
    }
    __syncthreads();
    if (!active || !chunk_has_tokens) continue;
#pragma unroll
    for (int kc = 0; kc < kLongChunkTiles; ++kc) {
      const int ktl = ch * kLongChunkTiles + kc;
      if (kt_base + ktl < n_tiles) {
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
          const float4v a4 = *reinterpret_cast<const float4v*>(Vs + (dt * 16 + l16) * kVS + kc * 16 + g * 4);
#pragma unroll
          for (int r = 0; r < 4; ++r) o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[r], s[ktl][r], o[dt], 0, 0, 0);
        }
      }
    }
  }

  // ---- the second half hands its part of O over (through the chunk buffers, free now), the first adds and stores --
  __syncthreads();
  float4v* xo = reinterpret_cast<float4v*>(smem_raw);        // [4 tiles][64 lanes][4]
  if (half == 1) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) xo[(tile_w * kWave + lane) * 4 + dt] = o[dt];
  }
  __syncthreads();
  if (half == 0 && tq >= 0) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      const float4v other = xo[(tile_w * kWave + lane) * 4 + dt];
#pragma unroll
      for (int r = 0; r < 4; ++r) o[dt][r] += other[r];
    }
    T* orow = dst + (size_t)tq * H + head * kD + g * 4;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      float4v v;
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = o[dt][r];
      *reinterpret_cast<float4v*>(orow + dt * 16) = v;
    }
  }
}

// ------------------------------------------------------------------------------------------
// fp16, 512 < seq_len <= 1024: the split kernel above with K of the whole sequence in LDS at once, then V in its place.
// The score registers allow one workgroup per CU either way, so the workgroup takes 128 KB of LDS: every K row (128
// bytes) arrives by DMA, all requests in flight together with the mask row and Q, instead of chunk after chunk through
// registers with a fetch latency each; V follows into the same rows while the softmax runs.  A row without a token is
// requested beyond its buffer descriptor's range and arrives as zeros.
// Rows, key order and swizzle as described above the resident-key kernel.  Arithmetic and rounding points per element
// are those of the split kernel.
// ------------------------------------------------------------------------------------------
constexpr int kWideKvBytes = kSplitKeys * 128;
constexpr int kWideSmem = kWideKvBytes + kSplitKeys * (int)sizeof(int) + 2 * 4 * 2 * 16 * (int)sizeof(float);

__global__ __launch_bounds__(kSplitThreads) void attention_wide_kernel(
    const _Float16* __restrict__ q_src, const _Float16* __restrict__ k_src, const _Float16* __restrict__ v_src, int layout,
    int packed_ld, const _Float16* __restrict__ attr_mask, _Float16* __restrict__ dst, const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ word_idx, int batch, int seq_len, int heads, float scaler) {
#if defined(__HIP_DEVICE_COMPILE__)   // device-only types in the body; the host pass only needs the stub
  using T = _Float16;
  constexpr int NKT = kSplitHalfTiles;

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  unsigned char* kv = smem_raw;
  int* tok_of_pos = reinterpret_cast<int*>(smem_raw + kWideKvBytes);
  float* red = reinterpret_cast<float*>(smem_raw + kWideKvBytes + kSplitKeys * sizeof(int));   // [2][4 tiles][2 halves][16]

  const int b = min(max(seq_start[batch + 1 + blockIdx.z], 0), batch - 1), head = blockIdx.y, qblock = blockIdx.x;
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  const int len = t1 - t0;
  if (len <= 0) return;
  const int H = heads * kD;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int tile_w = wave & 3, half = wave >> 2;
  const int l16 = lane & 15, g = lane >> 4;
  const int kt_base = half * NKT;                            // first key tile of this half

  const int last_pos = min(max(word_idx[t1 - 1], 0), seq_len - 1);
  const int n_tiles = last_pos / 16 + 1;                     // 16-row tiles that hold at least one token
  if (qblock * 4 >= n_tiles) return;                         // no token among this workgroup's queries
  for (int i = threadIdx.x; i < kSplitKeys; i += kSplitThreads) tok_of_pos[i] = -1;
  __syncthreads();
  for (int tt = threadIdx.x; tt < len; tt += kSplitThreads) {
    const int pos = word_idx[t0 + tt];
    if (pos >= 0 && pos < seq_len) tok_of_pos[pos] = tt;     // relative to the sequence's first packed row
  }
  __syncthreads();

  // Rows come in whole groups of four key tiles (what a step of the QK loop reads).  One DMA instruction fills eight
  // slots; lane -> slot 8 i + lane / 8, 16-byte chunk (lane & 7) ^ swizzle.
  const int rows_in = min((n_tiles + 3) / 4 * 64, kSplitKeys);
  auto stage = [&](const T* __restrict__ src) {
    const T* base = layout == 1 ? src + (size_t)t0 * packed_ld + head * kD : src + ((size_t)b * heads + head) * seq_len * kD;
    const uint32_t bytes = layout == 1 ? ((uint32_t)(len - 1) * (uint32_t)packed_ld + kD) * 2u : (uint32_t)seq_len * kD * 2u;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(base), 0, (int)bytes, 0x00020000);
    for (int i = wave; i < rows_in / 8; i += kSplitThreads / kWave) {
      const int slot = i * 8 + (lane >> 3);
      const int key = wide_slot(slot);
      const int c = (lane & 7) ^ wide_swizzle(slot);
      const int tk = tok_of_pos[key];
      const uint32_t row_off = layout == 1 ? (uint32_t)tk * (uint32_t)packed_ld : (uint32_t)key * kD;
      const uint32_t voff = tk >= 0 ? (row_off + (uint32_t)c * 8u) * 2u : 0x80000000u;      // out of range: zeros
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, ET_ATTN_LDS_PTR(kv + i * 1024), 16, voff, 0, 0, 0);
    }
  };
  stage(k_src);

  const int qt = qblock * 4 + tile_w;                        // this wavefront's 16-query tile
  const bool active = qt < n_tiles;                          // wave-uniform
  const int q = qt * 16 + l16;
  const int tq = (active && q < kSplitKeys) ? tok_of_pos[q] : -1;
  const T* mrow = attr_mask + ((size_t)b * seq_len + min(q, seq_len - 1)) * seq_len;
  const bool vec_mask = (seq_len & 7) == 0;                  // mask rows start at multiples of 16 bytes
  auto q_off = [&](int tk, int pos) -> size_t {
    return layout == 1 ? (size_t)(t0 + tk) * packed_ld + head * kD : (((size_t)b * heads + head) * seq_len + pos) * kD;
  };

  // Q operand of this lane (zeros for a query position without a token: its result is never stored)
  half8 bqh[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
    for (int j = 0; j < 8; ++j) bqh[ks][j] = (_Float16)0;
    if (tq >= 0) bqh[ks] = *reinterpret_cast<const half8*>(q_src + q_off(tq, q) + ks * 32 + g * 8);
  }

  // ---- the additive bias of this half of the mask row: all loads of the row in flight before the first use -------
  float s[NKT][4];                                           // s[2 P], s[2 P + 1]: keys base + 8 g + 0..3, + 4..7 of pair P
  // (1 - m) * -10000 as one fma: 1 - m is exact in float for a half m, so both forms round the same real number once
  {
    int g8 = g * 8;
    asm volatile("" : "+v"(g8));       // opaque: the clamped offsets are recomputed, not kept in registers
    if (vec_mask) {
      half8 m8[NKT / 2];
#pragma unroll
      for (int kp = 0; kp < NKT / 2; ++kp)
        m8[kp] = *reinterpret_cast<const half8*>(mrow + min((kt_base + 2 * kp) * 16 + g8, seq_len - 8));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kp = 0; kp < NKT / 2; ++kp) {
        const int key0 = (kt_base + 2 * kp) * 16 + g8;
        if ((kt_base + 2 * kp + 2) * 16 <= seq_len) {        // wave-uniform: every key of the pair exists
#pragma unroll
          for (int j = 0; j < 8; ++j) s[2 * kp + (j >> 2)][j & 3] = __builtin_fmaf((float)m8[kp][j], 10000.0f, -10000.0f);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            s[2 * kp + (j >> 2)][j & 3] = key0 < seq_len ? __builtin_fmaf((float)m8[kp][j], 10000.0f, -10000.0f) : -INFINITY;
        }
      }
    } else {
#pragma unroll
      for (int kp = 0; kp < NKT / 2; ++kp) {
        const int key0 = (kt_base + 2 * kp) * 16 + g8;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const T m = mrow[min(key0 + j, seq_len - 1)];
          s[2 * kp + (j >> 2)][j & 3] = key0 + j < seq_len ? __builtin_fmaf((float)m, 10000.0f, -10000.0f) : -INFINITY;
        }
        if (kp % 4 == 3) __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // operand addresses: a lane-dependent base (this half's first row included) plus a compile-time offset per tile
  const unsigned char* kbase_ks[2];
  const unsigned char* vbase_bc[2][2];
  {
    const int L = wide_slot((l16 >> 2) * 8 + (l16 & 3));
    const int sw = wide_swizzle(L);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) kbase_ks[ks] = kv + (kt_base * 16 + L) * 128 + (((ks * 4 + g) ^ sw) * 16);
#pragma unroll
    for (int bb = 0; bb < 2; ++bb)
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        const int slot = wide_slot(g * 8 + 2 * bb + cc);
        vbase_bc[bb][cc] = kv + (kt_base * 16 + slot) * 128 + (((l16 >> 1) ^ wide_swizzle(slot)) * 16) + (l16 & 1) * 8;
      }
  }
  wide_wait_dma();
  __syncthreads();                                           // K is in place

  // ---- S^T = K Q^T, four key tiles at a time -----------------------------------------------------------------------
  if (active) {
#pragma unroll
    for (int kg = 0; kg < NKT / 4; ++kg) {
      if (kt_base + kg * 4 < n_tiles) {                      // wave-uniform; the rows of a started group are all staged
        half8 a[4][2];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          // row l16 of tile t of the group: pair t >> 1, first or second tile t & 1 (4 rows further)
#pragma unroll
          for (int ks = 0; ks < 2; ++ks)
            a[t][ks] = *reinterpret_cast<const half8*>(kbase_ks[ks] + ((kg * 4 + (t & ~1)) * 16 + (t & 1) * 4) * 128);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          float4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < 2; ++ks) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t][ks], bqh[ks], acc, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float sc = h2f(f2h(acc[r]));                 // the score is stored in half
            s[kg * 4 + t][r] = sc * scaler + s[kg * 4 + t][r];
          }
        }
      }
    }
  }
  __syncthreads();                                           // every wavefront has read K for the last time
  stage(v_src);                                              // arrives while the softmax runs

  // ---- masked softmax: each half over its registers, maxima and sums exchanged through LDS --------------------
  float* red_max = red;
  float* red_sum = red + 4 * 2 * 16;
  {
    float mx = seq_len < kSplitKeys ? 0.f : -INFINITY;       // the clamp at 0 holds below 1024 keys
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[kt][r]);
    mx = xor_lanes_16_32_max(mx);
    if (g == 0) red_max[(tile_w * 2 + half) * 16 + l16] = mx;
  }
  wide_wait_lds();
  wide_barrier();
  {
    const float mx = fmaxf(red_max[(tile_w * 2) * 16 + l16], red_max[(tile_w * 2 + 1) * 16 + l16]) * kLog2e;
    float sum = 0.f;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[kt][r] = __builtin_amdgcn_exp2f(s[kt][r] * kLog2e - mx);
        sum += s[kt][r];
      }
    sum = xor_lanes_16_32_sum(sum);
    if (g == 0) red_sum[(tile_w * 2 + half) * 16 + l16] = sum;
  }
  wide_wait_lds();
  wide_barrier();
  {
    const float sum = red_sum[(tile_w * 2) * 16 + l16] + red_sum[(tile_w * 2 + 1) * 16 + l16] + 1e-6f;
    const float inv = 1.0f / sum;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) s[kt][r] *= inv;
  }
  wide_wait_dma();
  __syncthreads();                                           // V is in place

  // ---- O^T = V^T P^T, each half over its keys, two key tiles (one MFMA k range) at a time ------------------------
  float4v o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) o[dt] = float4v{0.f, 0.f, 0.f, 0.f};
  if (active) {
#pragma unroll
    for (int kp = 0; kp < NKT / 2; ++kp) {
      if (kt_base + 2 * kp < n_tiles) {                      // wave-uniform
        half8 p;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          p[r] = f2h(s[2 * kp][r]);
          p[4 + r] = f2h(s[2 * kp + 1][r]);
        }
        typedef uint32_t u2 __attribute__((ext_vector_type(2)));
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        u2 raw[8];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
          raw[kk] = *reinterpret_cast<const u2*>(vbase_bc[(kk >> 1) & 1][kk & 1] + (kp * 32 + (kk & 4)) * 128);
        }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          u4 lo, hi;
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            lo[q4] = __builtin_amdgcn_perm(raw[2 * q4 + 1][jj], raw[2 * q4][jj], 0x05040100u);
            hi[q4] = __builtin_amdgcn_perm(raw[2 * q4 + 1][jj], raw[2 * q4][jj], 0x07060302u);
          }
          o[2 * jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, lo), p, o[2 * jj], 0, 0, 0);
          o[2 * jj + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, hi), p, o[2 * jj + 1], 0, 0, 0);
        }
      }
    }
  }

  // ---- the second half hands its part of O over (through the K/V rows, free now), the first adds and stores ------
  __syncthreads();
  float4v* xo = reinterpret_cast<float4v*>(smem_raw);        // [4 tiles][64 lanes][4]
  if (half == 1) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) xo[(tile_w * kWave + lane) * 4 + dt] = o[dt];
  }
  __syncthreads();
  if (half == 0 && tq >= 0) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      const float4v other = xo[(tile_w * kWave + lane) * 4 + dt];
#pragma unroll
      for (int r = 0; r < 4; ++r) o[dt][r] += other[r];
    }
    half8 v0, v1;
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v0[4 * r + j] = f2h(o[j][r]);
        v1[4 * r + j] = f2h(o[j][2 + r]);
      }
    T* orow = dst + (size_t)(t0 + tq) * H + head * kD + g * 16;
    *reinterpret_cast<half8*>(orow) = v0;
    *reinterpret_cast<half8*>(orow + 8) = v1;
  }
#endif
}

// 512 < seq_len <= 1024, head size 64: fp32 runs the chunked split kernel, fp16 the kernel with the whole sequence in LDS
template <typename T>
void attention_split_launch(const void* q, const void* k, const void* v, int layout, int packed_ld, const void* attr_mask,
                            void* dst, const int32_t* seq_start, const int32_t* word_idx, int batch, int seq_len, int heads,
                            float scaler, hipStream_t stream) {
  dim3 grid((seq_len + 63) / 64, heads, batch);              // blocks of 64 queries that can hold a token
  if constexpr (sizeof(T) == 2) {
    allow_dynamic_lds(reinterpret_cast<const void*>(attention_wide_kernel), kWideSmem);
    attention_wide_kernel<<<grid, kSplitThreads, kWideSmem, stream>>>(
        (const _Float16*)q, (const _Float16*)k, (const _Float16*)v, layout, packed_ld, (const _Float16*)attr_mask,
        (_Float16*)dst, seq_start, word_idx, batch, seq_len, heads, scaler);
  } else {
    const size_t smem = 2 * LongSmem<T>::kTileBytes + (size_t)kSplitKeys * sizeof(int) + 2 * 4 * 2 * 16 * sizeof(float);
    auto kern = attention_split_kernel<T>;
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), (int)smem);
    kern<<<grid, kSplitThreads, smem, stream>>>((const T*)q, (const T*)k, (const T*)v, layout, packed_ld,
                                                (const T*)attr_mask, (T*)dst, seq_start, word_idx, batch, seq_len, heads,
                                                scaler);
  }
}

// ------------------------------------------------------------------------------------------
// fused attention for every shape the MFMA kernels above are not built for: size_per_head other than 64 (any
// multiple of 16 bytes up to 256 elements) and 512 < seq_len <= 1024.  One wavefront per (query, head): the lanes
// split the keys for the scores (full dot products in float, rounded to the element type as the reference stores
// them), the softmax runs on wave reductions, then the lanes split the features for P.V, skipping keys whose
// probability is 0.  Same arithmetic and rounding points as the other kernels; at seq_len = 1024 the reference's block
// of 1024 threads leaves no idle lane in its max reduction, so the clamp of the maximum at 0 disappears there
// (cuda/attention.cu:77-95, 267-270, 345-356: below 1024 the filler -1e-20 of the out-of-range threads acts as the clamp).
// ------------------------------------------------------------------------------------------
constexpr int kGenMaxSeq = 1024;
constexpr int kGenMaxD = 256;

template <typename T>
__global__ __launch_bounds__(kAttnThreads) void attention_generic_kernel(
    const T* __restrict__ q_src, const T* __restrict__ k_src, const T* __restrict__ v_src, int layout, int packed_ld,
    const T* __restrict__ attr_mask, T* __restrict__ dst, const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ word_idx, int batch, int seq_len, int heads, int d, int rows_16b, float scaler) {
  using C = Chunk16<T>;
  using V16 = typename C::vec;
  constexpr int kPerLane = kGenMaxSeq / kWave;             // keys per lane
  __shared__ int tok_of_pos[kGenMaxSeq];
  __shared__ float prob[kAttnWaves][kGenMaxSeq];
  __shared__ float qrow[kAttnWaves][kGenMaxD];

  const int b = min(max(seq_start[batch + 1 + blockIdx.z], 0), batch - 1), head = blockIdx.y;
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  const int len = t1 - t0;
  if (len <= 0) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int H = heads * d;
  for (int i = threadIdx.x; i < seq_len; i += kAttnThreads) tok_of_pos[i] = -1;
  __syncthreads();
  for (int tt = threadIdx.x; tt < len; tt += kAttnThreads) {
    const int pos = word_idx[t0 + tt];
    if (pos >= 0 && pos < seq_len) tok_of_pos[pos] = t0 + tt;
  }
  __syncthreads();
  const int q = blockIdx.x * kAttnWaves + wave;            // this wavefront's query position
  if (q >= seq_len) return;
  const int tq = tok_of_pos[q];
  if (tq < 0) return;                                      // no token: the reference drops this row
  auto src_off = [&](int t, int pos) -> size_t {
    return layout == 1 ? (size_t)t * packed_ld + head * d : (((size_t)b * heads + head) * seq_len + pos) * d;
  };
  for (int j = lane; j < d; j += kWave) qrow[wave][j] = (float)q_src[src_off(tq, q) + j];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  // ---- scores of the lane's keys: key = lane + 64 i --------------------------------------------------------
  const T* mrow = attr_mask + ((size_t)b * seq_len + q) * seq_len;
  float t[kPerLane];
  float mx = seq_len < kGenMaxSeq ? 0.f : -INFINITY;       // the clamp at 0 holds below 1024 keys
#pragma unroll
  for (int i = 0; i < kPerLane; ++i) {
    const int key = lane + i * kWave;
    t[i] = -INFINITY;
    if (key < seq_len) {
      const int tk = tok_of_pos[key];
      float dot = 0.f;
      if (tk >= 0) {
        const T* krow = k_src + src_off(tk, key);
        if (rows_16b) {                                    // wave-uniform: head rows of whole, aligned 16-byte pieces
          for (int c = 0; c < d; c += C::kElems) {
            const V16 kv = *reinterpret_cast<const V16*>(krow + c);
#pragma unroll
            for (int j = 0; j < C::kElems; ++j) dot += qrow[wave][c + j] * (float)kv[j];
          }
        } else {
          for (int c = 0; c < d; ++c) dot += qrow[wave][c] * (float)krow[c];
        }
      }
      const float sc = (float)(T)dot;                      // the score is stored in the element type
      t[i] = sc * scaler + (1.0f - (float)mrow[key]) * -10000.0f;
      mx = fmaxf(mx, t[i]);
    }
  }
  mx = wave_max(mx) * kLog2e;
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < kPerLane; ++i) {
    t[i] = __builtin_amdgcn_exp2f(t[i] * kLog2e - mx);     // exp2(-inf) = 0 for absent keys
    sum += t[i];
  }
  sum = wave_sum(sum) + 1e-6f;
  const float inv = 1.0f / sum;
#pragma unroll
  for (int i = 0; i < kPerLane; ++i) {
    const int key = lane + i * kWave;
    if (key < seq_len) prob[wave][key] = (float)(T)(t[i] * inv);     // the probability is stored in the element type
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  // ---- P.V: feature = lane + 64 i ------------------------------------------------------------------------------
  constexpr int kFeat = kGenMaxD / kWave;
  float acc[kFeat];
#pragma unroll
  for (int i = 0; i < kFeat; ++i) acc[i] = 0.f;
  for (int key = 0; key < seq_len; ++key) {
    const int tk = tok_of_pos[key];
    const float pk = prob[wave][key];
    if (tk < 0 || pk == 0.f) continue;                     // wave-uniform: a zero value or a zero weight
    const T* vrow = v_src + src_off(tk, key);
#pragma unroll
    for (int i = 0; i < kFeat; ++i) {
      const int j = lane + i * kWave;
      if (j < d) acc[i] += pk * (float)vrow[j];
    }
  }
#pragma unroll
  for (int i = 0; i < kFeat; ++i) {
    const int j = lane + i * kWave;
    if (j < d) dst[(size_t)tq * H + head * d + j] = (T)acc[i];
  }
}

// true when every head row of Q, K and V starts on a 16-byte boundary and is a whole number of 16-byte pieces (what the
// MFMA kernels and the vector loads of the generic one assume)
template <typename T>
bool head_rows_16b(const void* q, const void* k, const void* v, int layout, int packed_ld, int d) {
  const bool ptrs = ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v)) & 15) == 0;
  return ptrs && ((size_t)d * sizeof(T)) % 16 == 0 && (layout != 1 || ((size_t)packed_ld * sizeof(T)) % 16 == 0);
}

template <typename T>
void attention_generic_launch(const void* q, const void* k, const void* v, int layout, int packed_ld, const void* attr_mask,
                              void* dst, const int32_t* seq_start, const int32_t* word_idx, int batch, int seq_len,
                              int heads, int d, float scaler, hipStream_t stream) {
  dim3 grid((seq_len + kAttnWaves - 1) / kAttnWaves, heads, batch);
  attention_generic_kernel<T><<<grid, kAttnThreads, 0, stream>>>((const T*)q, (const T*)k, (const T*)v, layout, packed_ld,
                                                                 (const T*)attr_mask, (T*)dst, seq_start, word_idx, batch,
                                                                 seq_len, heads, d,
                                                                 head_rows_16b<T>(q, k, v, layout, packed_ld, d) ? 1 : 0,
                                                                 scaler);
}

template <typename T>
void attention_dispatch(const void* q, const void* k, const void* v, int layout, int packed_ld, const void* attr_mask,
                        void* dst, const int32_t* seq_start, const int32_t* word_idx, int batch, int seq_len, int heads,
                        int d, float scaler, hipStream_t stream) {
  if (d != kD || !head_rows_16b<T>(q, k, v, layout, packed_ld, d))
    attention_generic_launch<T>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads, d,
                                scaler, stream);
  else if (seq_len > 512)
    attention_split_launch<T>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads,
                              scaler, stream);
  else if (sizeof(T) == 2 && seq_len > 384)
    attention_resident_launch<32>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads,
                                  scaler, stream);
  else if (sizeof(T) == 2 && seq_len > 256)
    attention_resident_launch<24>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads,
                                  scaler, stream);
  else if (sizeof(T) == 2 && seq_len > 128)
    attention_resident_launch<16>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads,
                                  scaler, stream);
  else if (seq_len > 256)
    attention_long_launch<T, 32>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads,
                                 scaler, stream);
  else if (seq_len > 128)
    attention_long_launch<T, 16>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads,
                                 scaler, stream);
  else if (seq_len <= 32)
    attention_launch<T, 2>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads,
                           scaler, stream);
  else if (seq_len <= 64)
    attention_launch<T, 4>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads,
                           scaler, stream);
  else
    attention_launch<T, 8>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads,
                           scaler, stream);
}

}  // namespace

void launch_qkv_bias_pad(DType t, const void* Q, const void* bQ, const void* K, const void* bK, const void* V,
                         const void* bV, void* q_buf, void* k_buf, void* v_buf, const int32_t* seq_start,
                         const int32_t* word_idx, int batch, int seq_len, int heads, int d, hipStream_t stream) {
  if (((size_t)d * elem_size(t)) % 16 != 0) {      // head rows that are no whole number of 16-byte pieces
    launch_qkv_bias_pad_generic(t, Q, bQ, K, bK, V, bV, q_buf, k_buf, v_buf, seq_start, word_idx, batch, seq_len, heads,
                                d, stream);
    return;
  }
  dim3 grid(batch, 3);
  if (t == DType::F32)
    qkv_bias_pad_kernel<float><<<grid, kPadThreads, 0, stream>>>(
        (const float*)Q, (const float*)bQ, (const float*)K, (const float*)bK, (const float*)V, (const float*)bV,
        (float*)q_buf, (float*)k_buf, (float*)v_buf, seq_start, word_idx, seq_len, heads, d);
  else
    qkv_bias_pad_kernel<_Float16><<<grid, kPadThreads, 0, stream>>>(
        (const _Float16*)Q, (const _Float16*)bQ, (const _Float16*)K, (const _Float16*)bK, (const _Float16*)V,
        (const _Float16*)bV, (_Float16*)q_buf, (_Float16*)k_buf, (_Float16*)v_buf, seq_start, word_idx, seq_len, heads,
        d);
}

void launch_softmax(DType t, void* qk, const void* attr_mask, int batch, int heads, int seq_len, float scaler,
                    hipStream_t stream) {
  const int rows = batch * heads * seq_len;
  const int grid = (rows + kSmThreads / kWave - 1) / (kSmThreads / kWave);
  if (t == DType::F32)
    softmax_kernel<float><<<grid, kSmThreads, 0, stream>>>((float*)qk, (const float*)attr_mask, rows, heads, seq_len,
                                                           scaler);
  else
    softmax_kernel<_Float16><<<grid, kSmThreads, 0, stream>>>((_Float16*)qk, (const _Float16*)attr_mask, rows, heads,
                                                              seq_len, scaler);
}

void launch_transpose_rm_padding(DType t, const void* src, void* dst, const int32_t* rows_dev, int rows_bound,
                                 int batch, int seq_len, int heads, int d, const int32_t* batch_idx,
                                 const int32_t* word_idx, hipStream_t stream) {
  (void)batch;
  if (((size_t)d * elem_size(t)) % 16 != 0) {
    launch_transpose_rm_padding_generic(t, src, dst, rows_dev, rows_bound, seq_len, heads, d, batch_idx, word_idx, stream);
    return;
  }
  const int cpd = (int)((size_t)d * elem_size(t) / 16);
  const long total = (long)rows_bound * heads * cpd;
  const int grid = (int)((total + 255) / 256);
  if (grid == 0) return;
  if (t == DType::F32)
    transpose_rm_padding_kernel<float><<<grid, 256, 0, stream>>>((const float*)src, (float*)dst, rows_dev, rows_bound,
                                                                 seq_len, heads, cpd, batch_idx, word_idx);
  else
    transpose_rm_padding_kernel<_Float16><<<grid, 256, 0, stream>>>((const _Float16*)src, (_Float16*)dst, rows_dev,
                                                                    rows_bound, seq_len, heads, cpd, batch_idx,
                                                                    word_idx);
}

bool attention_supported(DType t, int seq_len, int d) {
  (void)t;
  return d >= 1 && d <= kGenMaxD && seq_len >= 1 && seq_len <= kGenMaxSeq;
}

void launch_attention(DType t, const void* q, const void* k, const void* v, int layout, int packed_ld,
                      const void* attr_mask, void* dst, const int32_t* seq_start, const int32_t* word_idx, int batch,
                      int seq_len, int heads, int d, float scaler, hipStream_t stream) {
  if (t == DType::F32)
    attention_dispatch<float>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len, heads, d,
                              scaler, stream);
  else
    attention_dispatch<_Float16>(q, k, v, layout, packed_ld, attr_mask, dst, seq_start, word_idx, batch, seq_len,
                                 heads, d, scaler, stream);
}

}  // namespace et
