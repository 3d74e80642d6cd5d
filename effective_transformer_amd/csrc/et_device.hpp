// Device-side building blocks shared by the gfx950 kernels: 64-lane wavefront reductions
// and scans on DPP, 128-bit vector types, exact integer division by a launch constant.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace et {

constexpr int kWave = 64;

// ---- 128-bit / 64-bit movers -----------------------------------------------------------
struct alignas(16) u32x4 { uint32_t x, y, z, w; };
struct alignas(8) u32x2 { uint32_t x, y; };

template <int BYTES> struct vec_bytes;
template <> struct vec_bytes<16> { using type = u32x4; };
template <> struct vec_bytes<8> { using type = u32x2; };
template <> struct vec_bytes<4> { using type = uint32_t; };

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float2v __attribute__((ext_vector_type(2)));

// ---- DPP cross-lane helpers --------------------------------------------------------------
// update_dpp(old, src, ctrl, row_mask, bank_mask, bound_ctrl): lanes whose source is
// disabled keep `old`.
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_f32(float old, float src) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old),
                                                               __builtin_bit_cast(int, src), CTRL, ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ int dpp_i32(int old, int src) {
  return __builtin_amdgcn_update_dpp(old, src, CTRL, ROW_MASK, 0xf, false);
}

constexpr int kDppQuadXor1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;
constexpr int kDppRowBcast15 = 0x142;
constexpr int kDppRowBcast31 = 0x143;

// Sum over the 64 lanes of a wavefront; every lane receives the total.
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_f32<kDppQuadXor1>(0.f, v);
  v += dpp_f32<kDppQuadXor2>(0.f, v);
  v += dpp_f32<kDppRowHalfMirror>(0.f, v);
  v += dpp_f32<kDppRowMirror>(0.f, v);
  v += dpp_f32<kDppRowBcast15, 0xa>(0.f, v);
  v += dpp_f32<kDppRowBcast31, 0xc>(0.f, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f32<kDppQuadXor1>(v, v));
  v = fmaxf(v, dpp_f32<kDppQuadXor2>(v, v));
  v = fmaxf(v, dpp_f32<kDppRowHalfMirror>(v, v));
  v = fmaxf(v, dpp_f32<kDppRowMirror>(v, v));
  v = fmaxf(v, dpp_f32<kDppRowBcast15, 0xa>(v, v));
  v = fmaxf(v, dpp_f32<kDppRowBcast31, 0xc>(v, v));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ int wave_sum_i32(int v) {
  v += dpp_i32<kDppQuadXor1>(0, v);
  v += dpp_i32<kDppQuadXor2>(0, v);
  v += dpp_i32<kDppRowHalfMirror>(0, v);
  v += dpp_i32<kDppRowMirror>(0, v);
  v += dpp_i32<kDppRowBcast15, 0xa>(0, v);
  v += dpp_i32<kDppRowBcast31, 0xc>(0, v);
  return __builtin_amdgcn_readlane(v, 63);
}

// Inclusive prefix sum over the 64 lanes (row_shr steps inside each row of 16, then the
// row totals are carried across rows with two broadcasts).
__device__ __forceinline__ int wave_inclusive_scan_i32(int v) {
  v += dpp_i32<0x111>(0, v);                 // row_shr:1
  v += dpp_i32<0x112>(0, v);                 // row_shr:2
  v += dpp_i32<0x114>(0, v);                 // row_shr:4
  v += dpp_i32<0x118>(0, v);                 // row_shr:8
  v += dpp_i32<kDppRowBcast15, 0xa>(0, v);   // rows 1,3 += last lane of rows 0,2
  v += dpp_i32<kDppRowBcast31, 0xc>(0, v);   // rows 2,3 += lane 31
  return v;
}

__device__ __forceinline__ int lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// ---- exact division of a 32-bit unsigned by a launch-time constant ------------------------
struct fastdiv {
  uint32_t d, magic, shift;
};
inline fastdiv make_fastdiv(uint32_t d) {
  fastdiv f;
  f.d = d;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  f.shift = s;
  f.magic = (uint32_t)(((1ull << 32) * ((1ull << s) - d)) / d + 1);
  return f;
}
__device__ __forceinline__ uint32_t div_by(uint32_t n, const fastdiv& f) {
  uint32_t t = __umulhi(n, f.magic);
  return (t + n) >> f.shift;         // valid while t + n < 2^32, i.e. n < 2^31
}

// ---- half helpers ------------------------------------------------------------------------
__device__ __forceinline__ float h2f(_Float16 h) { return (float)h; }
__device__ __forceinline__ _Float16 f2h(float f) { return (_Float16)f; }   // v_cvt_f16_f32, round-to-nearest-even

// ---- bias + GELU arithmetic (reference: cuda/cuda_kernels.cu:29-51) -------------------------
// 0.5*(1+tanh(u)) is evaluated as 1/(1+exp(-2u)), which is the same function without the cancellation of 1+tanh for
// negative u.
__device__ __forceinline__ float gelu_cdf(float x, float x3) {
  // exp(-2u) = 2^(-2u*log2(e)) with u = 0.7978845608028654 * (x + 0.044715 * x3): both factors in one constant
  const float e = __builtin_amdgcn_exp2f((x + 0.044715f * x3) * (-2.8853900817779268f * 0.7978845608028654f));
  return __builtin_amdgcn_rcpf(1.0f + e);
}
// fp16 rounding points of the reference: __hadd2 for the bias, two __hmul2 for the cube, the CDF in float rounded to
// half, __hmul2.  HV is a vector of halves (half4, half8).
template <typename HV, int N>
__device__ __forceinline__ HV bias_gelu_half(HV v, HV bias) {
  const HV x = v + bias;
  const HV x3 = x * (x * x);
  HV cdf;
#pragma unroll
  for (int i = 0; i < N; ++i) cdf[i] = f2h(gelu_cdf(h2f(x[i]), h2f(x3[i])));
  return x * cdf;
}

// seq_start[b] = first packed row of sequence b (b in [0, batch]; seq_start[batch] = T), written by the thread that
// owns packed row t in [0, T]: it covers the sequences that begin at t (token-less sequences included).
__device__ __forceinline__ void seq_start_for_row(const int32_t* __restrict__ batch_idx, int T, int t, int batch,
                                                  int32_t* __restrict__ seq_start) {
  if (t > T) return;
  const int prev = t == 0 ? -1 : batch_idx[t - 1];
  const int cur = t == T ? batch : min(batch_idx[t], batch - 1);
  const int last = t == T ? batch : cur;         // entries (prev, last] start at t
  for (int b = prev + 1; b <= last; ++b) seq_start[b] = t;
}

}  // namespace et
