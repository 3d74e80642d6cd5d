// Element-wise kernels for the shapes the tuned kernels are not built for: rows and head rows that are no whole number
// of 16-byte pieces, GEMMs whose k or n the MFMA tiles cannot take.  The reference's op accepts any size_per_head
// (tf_op/bert_transformer_op.cc:53-57) and its kernels index by element (cuda/attention.cu:190-219,
// cuda/cuda_kernels.cu:88-271); these kernels do the same arithmetic with the same rounding points as the tuned ones,
// one element per thread, and make no claim on speed.
#include "et_device.hpp"
#include "kernels.hpp"

namespace et {

namespace {

template <typename T> struct Scalar;
template <> struct Scalar<float> {
  static __device__ __forceinline__ float bias_gelu(float v, float b) {
    const float x = v + b;
    return x * gelu_cdf(x, x * x * x);
  }
};
template <> struct Scalar<_Float16> {
  // the half rounding points of bias_gelu_half, one element at a time
  static __device__ __forceinline__ _Float16 bias_gelu(_Float16 v, _Float16 b) {
    const _Float16 x = v + b;
    const _Float16 x3 = x * (x * x);
    const _Float16 cdf = f2h(gelu_cdf(h2f(x), h2f(x3)));
    return x * cdf;
  }
};

// ---- C = A . B (+ bias) (gelu): 16 x 16 outputs per workgroup, operands staged through LDS, float accumulation in
// ascending k ----------------------------------------------------------------------------------------------------
struct GenericGemmArgs {
  const void* A[3];
  const void* B[3];
  const void* bias[3];
  void* C;
  const int32_t* rows_dev;
  int ldc, m_bound, n, k, b_transposed, gelu;
};

template <typename T>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GenericGemmArgs a) {
  __shared__ float As[16][17], Bs[16][17];
  const int rows = a.rows_dev ? min(*a.rows_dev, a.m_bound) : a.m_bound;
  const int grp = blockIdx.z;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int row0 = blockIdx.y * 16, col0 = blockIdx.x * 16;
  if (row0 >= rows) return;
  const T* A = (const T*)a.A[grp];
  const T* B = (const T*)a.B[grp];
  const int N = a.n, K = a.k;
  float acc = 0.f;
  for (int k0 = 0; k0 < K; k0 += 16) {
    // A tile: row row0 + ty, k k0 + tx;  B tile: k k0 + ty, column col0 + tx
    const int ar = row0 + ty, ak = k0 + tx;
    As[ty][tx] = (ar < rows && ak < K) ? (float)A[(size_t)ar * K + ak] : 0.f;
    const int bk = k0 + ty, bc = col0 + tx;
    float bv = 0.f;
    if (bk < K && bc < N) bv = (float)(a.b_transposed ? B[(size_t)bc * K + bk] : B[(size_t)bk * N + bc]);
    Bs[ty][tx] = bv;
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) acc += As[ty][kk] * Bs[kk][tx];
    __syncthreads();
  }
  const int row = row0 + ty, col = col0 + tx;
  if (row >= rows || col >= N) return;
  T o = (T)acc;
  const T* bias = (const T*)a.bias[grp];
  if (a.gelu) o = Scalar<T>::bias_gelu(o, bias[col]);
  else if (bias != nullptr) o = o + bias[col];      // in the element type, on the rounded product
  ((T*)a.C)[(size_t)row * a.ldc + (size_t)grp * N + col] = o;
}

// ---- out = gelu(out + bias), one element per thread -----------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bias_gelu_generic_kernel(T* __restrict__ out, const T* __restrict__ bias, int m,
                                                                int n, const int32_t* __restrict__ rows_dev) {
  const int rows = rows_dev ? min(*rows_dev, m) : m;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)rows * n) return;
  const int c = (int)(i % n);
  out[i] = Scalar<T>::bias_gelu(out[i], bias[c]);
}

// ---- out = LayerNorm((out + input) + bias) * gamma + beta: one wavefront per row, three passes over the row ----
template <typename T>
__global__ __launch_bounds__(256) void layernorm_generic_kernel(T* __restrict__ out, const T* __restrict__ input,
                                                                const T* __restrict__ bias, const T* __restrict__ gamma,
                                                                const T* __restrict__ beta, int m, int n,
                                                                const int32_t* __restrict__ rows_dev, float eps) {
  const int rows = rows_dev ? min(*rows_dev, m) : m;
  const int lane = threadIdx.x & (kWave - 1);
  const int r = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  if (r >= rows) return;                         // wave-uniform
  T* o = out + (size_t)r * n;
  const T* in = input + (size_t)r * n;
  auto value = [&](int c) { return (float)((o[c] + in[c]) + bias[c]); };      // the adds in the element type
  float sum = 0.f;
  for (int c = lane; c < n; c += kWave) sum += value(c);
  const float mean = wave_sum(sum) / (float)n;
  float sq = 0.f;
  for (int c = lane; c < n; c += kWave) {
    const float dlt = value(c) - mean;
    sq += dlt * dlt;
  }
  const float rstd = __builtin_amdgcn_rsqf(wave_sum(sq) / (float)n + eps);
  for (int c = lane; c < n; c += kWave) o[c] = (T)(((value(c) - mean) * rstd) * (float)gamma[c] + (float)beta[c]);
}

// ---- [T,H] + bias -> zero-padded [B,heads,S,d], and back -------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void qkv_bias_pad_generic_kernel(
    const T* __restrict__ Q, const T* __restrict__ bQ, const T* __restrict__ K, const T* __restrict__ bK,
    const T* __restrict__ V, const T* __restrict__ bV, T* __restrict__ q_buf, T* __restrict__ k_buf,
    T* __restrict__ v_buf, const int32_t* __restrict__ seq_start, const int32_t* __restrict__ word_idx, int seq_len,
    int heads, int d) {
  __shared__ int tok_of_pos[1024];
  const int b = blockIdx.x, mat = blockIdx.y;
  const T* src = mat == 0 ? Q : (mat == 1 ? K : V);
  const T* bias = mat == 0 ? bQ : (mat == 1 ? bK : bV);
  T* dst = mat == 0 ? q_buf : (mat == 1 ? k_buf : v_buf);
  for (int s = threadIdx.x; s < seq_len; s += 256) tok_of_pos[s] = -1;
  __syncthreads();
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  for (int t = t0 + threadIdx.x; t < t1; t += 256) {
    const int s = word_idx[t];
    if (s >= 0 && s < seq_len) tok_of_pos[s] = t;
  }
  __syncthreads();
  const int H = heads * d, total = heads * seq_len * d;
  T* out = dst + (size_t)b * total;
  for (int i = threadIdx.x; i < total; i += 256) {
    const int j = i % d, s = (i / d) % seq_len, head = i / (d * seq_len);
    const int t = tok_of_pos[s];
    out[i] = t >= 0 ? src[(size_t)t * H + head * d + j] + bias[head * d + j] : (T)0;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void transpose_rm_padding_generic_kernel(
    const T* __restrict__ src, T* __restrict__ dst, const int32_t* __restrict__ rows_dev, int rows_bound, int seq_len,
    int heads, int d, const int32_t* __restrict__ batch_idx, const int32_t* __restrict__ word_idx) {
  const int rows = rows_dev ? min(*rows_dev, rows_bound) : rows_bound;
  const int H = heads * d;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)rows * H) return;
  const int t = (int)(i / H), c = (int)(i - (long)t * H);
  const int head = c / d, j = c - head * d;
  const int b = batch_idx[t], s = word_idx[t];
  dst[i] = src[(((size_t)b * heads + head) * seq_len + s) * d + j];
}

}  // namespace

void launch_gemm_generic(DType t, const GemmGroups& g, void* C, int ldc, int m_bound, int n, int k,
                         const int32_t* rows_dev, hipStream_t stream) {
  GenericGemmArgs a;
  for (int i = 0; i < 3; ++i) {
    a.A[i] = i < g.groups ? g.A[i] : nullptr;
    a.B[i] = i < g.groups ? g.B[i] : nullptr;
    a.bias[i] = i < g.groups ? g.bias[i] : nullptr;
  }
  a.C = C;
  a.rows_dev = rows_dev;
  a.ldc = ldc;
  a.m_bound = m_bound;
  a.n = n;
  a.k = k;
  a.b_transposed = g.b_transposed ? 1 : 0;
  a.gelu = g.gelu ? 1 : 0;
  dim3 grid((n + 15) / 16, (m_bound + 15) / 16, g.groups);
  if (t == DType::F32) gemm_generic_kernel<float><<<grid, 256, 0, stream>>>(a);
  else gemm_generic_kernel<_Float16><<<grid, 256, 0, stream>>>(a);
}

void launch_bias_gelu_generic(DType t, void* out, const void* bias, int m, int n, const int32_t* rows_dev,
                              hipStream_t stream) {
  const long total = (long)m * n;
  const int grid = (int)((total + 255) / 256);
  if (grid == 0) return;
  if (t == DType::F32)
    bias_gelu_generic_kernel<float><<<grid, 256, 0, stream>>>((float*)out, (const float*)bias, m, n, rows_dev);
  else
    bias_gelu_generic_kernel<_Float16><<<grid, 256, 0, stream>>>((_Float16*)out, (const _Float16*)bias, m, n, rows_dev);
}

void launch_layernorm_generic(DType t, void* out, const void* input, const void* bias, const void* gamma,
                              const void* beta, int m, int n, const int32_t* rows_dev, float eps, hipStream_t stream) {
  const int grid = (m + 3) / 4;
  if (grid == 0) return;
  if (t == DType::F32)
    layernorm_generic_kernel<float><<<grid, 256, 0, stream>>>((float*)out, (const float*)input, (const float*)bias,
                                                             (const float*)gamma, (const float*)beta, m, n, rows_dev, eps);
  else
    layernorm_generic_kernel<_Float16><<<grid, 256, 0, stream>>>((_Float16*)out, (const _Float16*)input,
                                                                (const _Float16*)bias, (const _Float16*)gamma,
                                                                (const _Float16*)beta, m, n, rows_dev, eps);
}

void launch_qkv_bias_pad_generic(DType t, const void* Q, const void* bQ, const void* K, const void* bK, const void* V,
                                 const void* bV, void* q_buf, void* k_buf, void* v_buf, const int32_t* seq_start,
                                 const int32_t* word_idx, int batch, int seq_len, int heads, int d, hipStream_t stream) {
  dim3 grid(batch, 3);
  if (t == DType::F32)
    qkv_bias_pad_generic_kernel<float><<<grid, 256, 0, stream>>>(
        (const float*)Q, (const float*)bQ, (const float*)K, (const float*)bK, (const float*)V, (const float*)bV,
        (float*)q_buf, (float*)k_buf, (float*)v_buf, seq_start, word_idx, seq_len, heads, d);
  else
    qkv_bias_pad_generic_kernel<_Float16><<<grid, 256, 0, stream>>>(
        (const _Float16*)Q, (const _Float16*)bQ, (const _Float16*)K, (const _Float16*)bK, (const _Float16*)V,
        (const _Float16*)bV, (_Float16*)q_buf, (_Float16*)k_buf, (_Float16*)v_buf, seq_start, word_idx, seq_len, heads, d);
}

void launch_transpose_rm_padding_generic(DType t, const void* src, void* dst, const int32_t* rows_dev, int rows_bound,
                                         int seq_len, int heads, int d, const int32_t* batch_idx,
                                         const int32_t* word_idx, hipStream_t stream) {
  const long total = (long)rows_bound * heads * d;
  const int grid = (int)((total + 255) / 256);
  if (grid == 0) return;
  if (t == DType::F32)
    transpose_rm_padding_generic_kernel<float><<<grid, 256, 0, stream>>>((const float*)src, (float*)dst, rows_dev,
                                                                        rows_bound, seq_len, heads, d, batch_idx, word_idx);
  else
    transpose_rm_padding_generic_kernel<_Float16><<<grid, 256, 0, stream>>>((const _Float16*)src, (_Float16*)dst,
                                                                           rows_dev, rows_bound, seq_len, heads, d,
                                                                           batch_idx, word_idx);
}

}  // namespace et
