// Row kernels of the encoder layer on gfx950, both HBM-bound:
//   out = gelu_tanh(out + bias)                       (reference: cuda/cuda_kernels.cu:29-51, 88-150)
//   out = LayerNorm(out + input + bias) * gamma + beta (reference: cuda/cuda_kernels.cu:157-271)
// Arithmetic and rounding points follow the reference: fp32 rows are computed in float; fp16
// rows add in half (packed v_pk_add_f16), take statistics / the tanh polynomial in float and
// round once on the way out.
#include "et_device.hpp"
#include "kernels.hpp"

namespace et {

namespace {

// ------------------------------------------------------------------------------------------
// bias + GELU (arithmetic in et_device.hpp, shared with the GEMM epilogue that fuses it)
// ------------------------------------------------------------------------------------------
constexpr int kGeluThreads = 128;
constexpr int kGeluRows = 16;     // rows per workgroup
constexpr int kGeluInFlight = 4;  // rows loaded before any is computed

template <typename T> struct GeluChunk;

template <> struct GeluChunk<float> {
  float4v v;
  __device__ __forceinline__ void apply(const GeluChunk<float>& b) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float x = v[i] + b.v[i];
      v[i] = x * gelu_cdf(x, x * x * x);
    }
  }
};

template <> struct GeluChunk<_Float16> {
  half8 v;
  __device__ __forceinline__ void apply(const GeluChunk<_Float16>& b) {
    v = bias_gelu_half<half8, 8>(v, b.v);
  }
};

template <typename T>
__global__ __launch_bounds__(kGeluThreads) void bias_gelu_kernel(T* __restrict__ out, const T* __restrict__ bias, int m,
                                                                 int cpr, const int32_t* __restrict__ rows_dev) {
  using Chunk = GeluChunk<T>;
  static_assert(sizeof(Chunk) == 16, "one 128-bit access per lane");
  const int rows = rows_dev ? min(*rows_dev, m) : m;
  const int c = blockIdx.x * kGeluThreads + threadIdx.x;
  const int r0 = blockIdx.y * kGeluRows;
  if (c >= cpr || r0 >= rows) return;
  Chunk* base = reinterpret_cast<Chunk*>(out) + c;
  const Chunk b = reinterpret_cast<const Chunk*>(bias)[c];
  const int r1 = min(r0 + kGeluRows, rows);
  for (int r = r0; r < r1; r += kGeluInFlight) {
    Chunk x[kGeluInFlight];
    // no predication: rows past the end repeat the last row (same input, same result, same store), so the four
    // loads are in flight together
    Chunk* p[kGeluInFlight];
#pragma unroll
    for (int u = 0; u < kGeluInFlight; ++u) {
      p[u] = base + (size_t)min(r + u, r1 - 1) * cpr;
      x[u] = *p[u];
    }
#pragma unroll
    for (int u = 0; u < kGeluInFlight; ++u) {
      x[u].apply(b);
      *p[u] = x[u];
    }
  }
}

// ------------------------------------------------------------------------------------------
// bias + residual + LayerNorm: one wavefront per row, the row lives in registers between the
// two statistics passes, both reductions are 64-lane DPP sums (no LDS, no barrier).
// ------------------------------------------------------------------------------------------
constexpr int kLnThreads = 256;
constexpr int kLnWaves = kLnThreads / kWave;

template <typename T, int VEC> struct RowVec;
template <int VEC> struct RowVec<float, VEC> {
  typedef float type __attribute__((ext_vector_type(VEC)));
};
template <int VEC> struct RowVec<_Float16, VEC> {
  typedef _Float16 type __attribute__((ext_vector_type(VEC)));
};

// VEC elements per lane per access, ITERS accesses per row: the row has n <= 64*VEC*ITERS
// elements, n % VEC == 0.
template <typename T, int VEC, int ITERS>
__global__ __launch_bounds__(kLnThreads) void bias_residual_layernorm_kernel(
    T* __restrict__ out, const T* __restrict__ input, const T* __restrict__ bias, const T* __restrict__ gamma,
    const T* __restrict__ beta, int m, int n, const int32_t* __restrict__ rows_dev, WarmList warm) {
  using V = typename RowVec<T, VEC>::type;
  const int rows = rows_dev ? min(*rows_dev, m) : m;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = blockIdx.x * kLnWaves + threadIdx.x / kWave;
  const int nwaves = gridDim.x * kLnWaves;
  const int vpr = n / VEC;                       // vectors per row

  // `warm`: regions (weight matrices) that one of the next kernels would read cold; one word of each of their 128-byte
  // lines is requested here, which pulls the line into the last-level cache.  The values are only looked at behind
  // the row loop, so no wavefront waits for them.
  uint32_t warm0 = 0, warm1 = 0;
  if (warm.total > 0) {
    const int tid = blockIdx.x * kLnThreads + threadIdx.x, nth = gridDim.x * kLnThreads;
    auto word = [&](int i) {
      int r = 0;
      while (r + 1 < WarmList::kMax && i >= warm.lines[r]) i -= warm.lines[r++];
      return warm.p[r][(size_t)i * 32];
    };
    if (tid < warm.total) warm0 = word(tid);
    for (int i = tid + nth; i < warm.total; i += nth) warm1 ^= word(i);
  }

  V b[ITERS], g[ITERS], be[ITERS];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = lane + i * kWave;
    if (c < vpr) {
      b[i] = reinterpret_cast<const V*>(bias)[c];
      g[i] = reinterpret_cast<const V*>(gamma)[c];
      be[i] = reinterpret_cast<const V*>(beta)[c];
    }
  }
  const float inv_n = 1.0f / (float)n;

  for (int r = wave; r < rows; r += nwaves) {
    V* orow = reinterpret_cast<V*>(out + (size_t)r * n);
    const V* irow = reinterpret_cast<const V*>(input + (size_t)r * n);
    V xo[ITERS], xi[ITERS];
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = lane + i * kWave;
      if (c < vpr) {
        xo[i] = orow[c];
        xi[i] = irow[c];
      }
    }
    float x[ITERS][VEC];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = lane + i * kWave;
      // (out + input) + bias in the element type: float adds for fp32, two half roundings for fp16
      const V s = (xo[i] + xi[i]) + b[i];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        x[i][j] = c < vpr ? (float)s[j] : 0.f;
        sum += x[i][j];
      }
    }
    const float mean = wave_sum(sum) * inv_n;
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = lane + i * kWave;
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float dlt = x[i][j] - mean;
        sq += c < vpr ? dlt * dlt : 0.f;
      }
    }
    const float rstd = __builtin_amdgcn_rsqf(wave_sum(sq) * inv_n + 1e-6f);
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = lane + i * kWave;
      if (c < vpr) {
        V y;
#pragma unroll
        for (int j = 0; j < VEC; ++j) y[j] = (T)(((x[i][j] - mean) * rstd) * (float)g[i][j] + (float)be[i][j]);
        orow[c] = y;
      }
    }
  }
  // The requested words are consumed here, behind the row loop, by an empty instruction sequence: the loads cannot be
  // dropped, and nothing that depends on a corrupt row count decides whether they stay.
  asm volatile("" ::"v"(warm0), "v"(warm1));
}

// ------------------------------------------------------------------------------------------
// Embedding lookup + post-processing written straight into the packed token matrix (reference graph:
// sample/tensorflow/modeling.py:380-521): row t = LayerNorm(word[ids[p]] + type[type_ids[p]] + pos[s]) for the t-th
// valid position p = (b, s).  One wavefront per packed row, same register-resident two-pass LayerNorm as above with
// the TF layer_norm epsilon; ids outside a table read as a zero row (what tf.gather does on a GPU).
// ------------------------------------------------------------------------------------------
template <typename T, int VEC, int ITERS>
__global__ __launch_bounds__(kLnThreads) void embed_layernorm_kernel(
    T* __restrict__ out, const int32_t* __restrict__ ids, const int32_t* __restrict__ type_ids,
    const int32_t* __restrict__ batch_idx, const int32_t* __restrict__ word_idx, const T* __restrict__ word_table,
    int vocab, const T* __restrict__ type_table, int type_vocab, const T* __restrict__ pos_table, int max_pos,
    const T* __restrict__ gamma, const T* __restrict__ beta, int m, int n, int seq_len,
    const int32_t* __restrict__ rows_dev) {
  using V = typename RowVec<T, VEC>::type;
  const int rows = rows_dev ? min(*rows_dev, m) : m;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = blockIdx.x * kLnWaves + threadIdx.x / kWave;
  const int nwaves = gridDim.x * kLnWaves;
  const int vpr = n / VEC;

  V g[ITERS], be[ITERS];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = lane + i * kWave;
    if (c < vpr) {
      g[i] = reinterpret_cast<const V*>(gamma)[c];
      be[i] = reinterpret_cast<const V*>(beta)[c];
    }
  }
  const float inv_n = 1.0f / (float)n;

  for (int r = wave; r < rows; r += nwaves) {
    const int b = batch_idx[r], sp = word_idx[r];
    const int p = b * seq_len + sp;
    const int id = ids[p];
    const int tt = type_ids ? type_ids[p] : 0;
    const bool id_ok = id >= 0 && id < vocab;
    const bool tt_ok = type_table != nullptr && tt >= 0 && tt < type_vocab;
    const bool pos_ok = pos_table != nullptr && sp < max_pos;
    const V* wrow = reinterpret_cast<const V*>(word_table + (size_t)(id_ok ? id : 0) * n);
    const V* trow = reinterpret_cast<const V*>(type_table + (size_t)(tt_ok ? tt : 0) * n);
    const V* prow = reinterpret_cast<const V*>(pos_table + (size_t)(pos_ok ? sp : 0) * n);
    float x[ITERS][VEC];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = lane + i * kWave;
      V s;
#pragma unroll
      for (int j = 0; j < VEC; ++j) s[j] = (T)0;
      if (c < vpr) {
        if (id_ok) s = wrow[c];
        if (tt_ok) s = s + trow[c];             // element-type adds in the order of the graph: word, += type, += position
        if (pos_ok) s = s + prow[c];
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        x[i][j] = c < vpr ? (float)s[j] : 0.f;
        sum += x[i][j];
      }
    }
    const float mean = wave_sum(sum) * inv_n;
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = lane + i * kWave;
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float dlt = x[i][j] - mean;
        sq += c < vpr ? dlt * dlt : 0.f;
      }
    }
    const float rstd = __builtin_amdgcn_rsqf(wave_sum(sq) * inv_n + 1e-12f);
    V* orow = reinterpret_cast<V*>(out + (size_t)r * n);
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = lane + i * kWave;
      if (c < vpr) {
        V y;
#pragma unroll
        for (int j = 0; j < VEC; ++j) y[j] = (T)(((x[i][j] - mean) * rstd) * (float)g[i][j] + (float)be[i][j]);
        orow[c] = y;
      }
    }
  }
}

template <typename T>
bool ln_pick(int n, int& vec, int& iters) {
  const int max_vec = 16 / (int)sizeof(T);
  for (int v = max_vec; v >= max_vec / 4 && v >= 1; v /= 2) {
    if (n % v) continue;
    const int it = (n / v + kWave - 1) / kWave;
    if (it <= 8) {
      vec = v;
      iters = it;
      return true;
    }
  }
  return false;
}

template <typename T, int VEC>
void ln_launch_iters(int iters, int grid, hipStream_t stream, T* out, const T* input, const T* bias, const T* gamma,
                     const T* beta, int m, int n, const int32_t* rows_dev, const WarmList& warm) {
#define ET_LN_CASE(I)                                                                                          \
  case I:                                                                                                      \
    bias_residual_layernorm_kernel<T, VEC, I><<<grid, kLnThreads, 0, stream>>>(out, input, bias, gamma, beta, m, n, \
                                                                               rows_dev, warm);                \
    break;
  switch (iters) {
    ET_LN_CASE(1)
    ET_LN_CASE(2)
    ET_LN_CASE(3)
    ET_LN_CASE(4)
    ET_LN_CASE(5)
    ET_LN_CASE(6)
    ET_LN_CASE(7)
    ET_LN_CASE(8)
  }
#undef ET_LN_CASE
}

template <typename T>
void ln_launch(void* out, const void* input, const void* bias, const void* gamma, const void* beta, int m, int n,
               const int32_t* rows_dev, hipStream_t stream, const WarmList& warm) {
  int vec = 0, iters = 0;
  if (!ln_pick<T>(n, vec, iters)) return;
  // enough wavefronts to fill 256 CUs several times over; rows beyond that are looped
  const int grid = (int)min((long)(m + kLnWaves - 1) / kLnWaves, 256L * 8);
  T* o = (T*)out;
  const T *i = (const T*)input, *b = (const T*)bias, *g = (const T*)gamma, *be = (const T*)beta;
  constexpr int MV = 16 / (int)sizeof(T);
  if (vec == MV)
    ln_launch_iters<T, MV>(iters, grid, stream, o, i, b, g, be, m, n, rows_dev, warm);
  else if (vec == MV / 2)
    ln_launch_iters<T, MV / 2>(iters, grid, stream, o, i, b, g, be, m, n, rows_dev, warm);
  else
    ln_launch_iters<T, MV / 4>(iters, grid, stream, o, i, b, g, be, m, n, rows_dev, warm);
}

struct EmbedArgs {
  void* out;
  const int32_t *ids, *type_ids, *batch_idx, *word_idx;
  const void *word_table, *type_table, *pos_table, *gamma, *beta;
  int vocab, type_vocab, max_pos, m, n, seq_len;
  const int32_t* rows_dev;
};

template <typename T, int VEC>
void embed_launch_iters(int iters, int grid, hipStream_t stream, const EmbedArgs& a) {
#define ET_EMB_CASE(I)                                                                                              \
  case I:                                                                                                           \
    embed_layernorm_kernel<T, VEC, I><<<grid, kLnThreads, 0, stream>>>(                                             \
        (T*)a.out, a.ids, a.type_ids, a.batch_idx, a.word_idx, (const T*)a.word_table, a.vocab,                     \
        (const T*)a.type_table, a.type_vocab, (const T*)a.pos_table, a.max_pos, (const T*)a.gamma, (const T*)a.beta, \
        a.m, a.n, a.seq_len, a.rows_dev);                                                                           \
    break;
  switch (iters) {
    ET_EMB_CASE(1)
    ET_EMB_CASE(2)
    ET_EMB_CASE(3)
    ET_EMB_CASE(4)
    ET_EMB_CASE(5)
    ET_EMB_CASE(6)
    ET_EMB_CASE(7)
    ET_EMB_CASE(8)
  }
#undef ET_EMB_CASE
}

template <typename T>
void embed_launch(const EmbedArgs& a, hipStream_t stream) {
  int vec = 0, iters = 0;
  if (!ln_pick<T>(a.n, vec, iters)) return;
  const int grid = (int)min((long)(a.m + kLnWaves - 1) / kLnWaves, 256L * 8);
  constexpr int MV = 16 / (int)sizeof(T);
  if (vec == MV)
    embed_launch_iters<T, MV>(iters, grid, stream, a);
  else if (vec == MV / 2)
    embed_launch_iters<T, MV / 2>(iters, grid, stream, a);
  else
    embed_launch_iters<T, MV / 4>(iters, grid, stream, a);
}

}  // namespace

void launch_embed_layernorm(DType t, void* out, const int32_t* ids, const int32_t* type_ids, const int32_t* batch_idx,
                            const int32_t* word_idx, const void* word_table, int vocab, const void* type_table,
                            int type_vocab, const void* pos_table, int max_pos, const void* gamma, const void* beta,
                            int m, int n, int seq_len, const int32_t* rows_dev, hipStream_t stream) {
  if (m <= 0) return;
  EmbedArgs a{out, ids, type_ids, batch_idx, word_idx, word_table, type_table, pos_table, gamma, beta,
              vocab, type_vocab, max_pos, m, n, seq_len, rows_dev};
  if (t == DType::F32)
    embed_launch<float>(a, stream);
  else
    embed_launch<_Float16>(a, stream);
}

bool bias_gelu_supported(DType t, int n) {
  (void)t;
  return n > 0;
}

void launch_bias_gelu(DType t, void* out, const void* bias, int m, int n, const int32_t* rows_dev, hipStream_t stream) {
  if (((size_t)n * elem_size(t)) % 16 != 0) {      // rows that are no whole number of 16-byte pieces
    launch_bias_gelu_generic(t, out, bias, m, n, rows_dev, stream);
    return;
  }
  const int cpr = (int)((size_t)n * elem_size(t) / 16);
  dim3 grid((cpr + kGeluThreads - 1) / kGeluThreads, (m + kGeluRows - 1) / kGeluRows);
  if (t == DType::F32)
    bias_gelu_kernel<float><<<grid, kGeluThreads, 0, stream>>>((float*)out, (const float*)bias, m, cpr, rows_dev);
  else
    bias_gelu_kernel<_Float16><<<grid, kGeluThreads, 0, stream>>>((_Float16*)out, (const _Float16*)bias, m, cpr,
                                                                  rows_dev);
}

bool layernorm_row_in_registers(DType t, int n) {
  int vec, iters;
  if (n <= 0) return false;
  return t == DType::F32 ? ln_pick<float>(n, vec, iters) : ln_pick<_Float16>(n, vec, iters);
}

bool bias_residual_layernorm_supported(DType t, int n) {
  (void)t;
  return n > 0;
}

void WarmList::add(const void* region, size_t bytes) {
  // whole lines of a 128-byte aligned region; a list that is full or a region that is not aligned is left out
  const size_t n = bytes / 128;
  int slot = 0;
  while (slot < kMax && lines[slot] != 0) ++slot;
  if (region == nullptr || n == 0 || slot == kMax || ((uintptr_t)region & 127) != 0 || n + (size_t)total > (1u << 24)) return;
  p[slot] = (const uint32_t*)region;
  lines[slot] = (int)n;
  total += (int)n;
}

void launch_bias_residual_layernorm(DType t, void* out, const void* input, const void* bias, const void* gamma,
                                    const void* beta, int m, int n, const int32_t* rows_dev, hipStream_t stream,
                                    const WarmList& warm) {
  if (!layernorm_row_in_registers(t, n)) {      // odd or very long rows: three passes over memory
    launch_layernorm_generic(t, out, input, bias, gamma, beta, m, n, rows_dev, 1e-6f, stream);
    return;
  }
  if (t == DType::F32)
    ln_launch<float>(out, input, bias, gamma, beta, m, n, rows_dev, stream, warm);
  else
    ln_launch<_Float16>(out, input, bias, gamma, beta, m, n, rows_dev, stream, warm);
}

}  // namespace et
