// MFMA GEMMs for the four dense projections of the encoder layer on gfx950 (replace the cublasGemmEx
// call sites, reference: tf_op/bert_transformer_op.cu.cc:110-141, 200-240).
//
//   C[m,n] = A[m,k] . B[k,n] (+ bias[n]),  A = packed tokens (row-major), B = TF dense kernel [in,out]
//   (row-major, used untransposed), fp32 accumulation, C in the element type.
//
// fp16: v_mfma_f32_16x16x32_f16.  B is n-contiguous in memory while the MFMA wants 8 consecutive k
// per lane, so each lane reads an 8(k) x 8(n) block of B from LDS with eight 128-bit reads and
// transposes it in registers; the eight resulting operands feed eight MFMAs whose column sets are
// {8*l + j : l = 0..15}.  A lane therefore ends up owning 8 consecutive output columns per row and
// stores C with 128-bit writes.  The k order inside a step is whatever the loads define; A and B use
// the same one.
// fp32: v_mfma_f32_32x32x2_f32, one element per lane per step.
//
// The M dimension (valid tokens) may live on the device: tiles beyond *rows_dev exit, the last tile
// is predicated.  Up to three column groups (Q/K/V) share one launch.
#include "et_device.hpp"
#include "kernels.hpp"

namespace et {

namespace {

struct GemmArgs {
  const void* A[3];
  const void* B[3];
  const void* bias[3];
  void* C;
  const int32_t* rows_dev;
  int ldc, m_bound, n, k, groups;
  int tiles_m, tiles_n;      // tiles_n per group
  int per_xcd;               // workgroups per XCD slot of the launch
};

typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

constexpr int kXcds = 8;

// Workgroups are dealt round-robin to the 8 XCDs; give every XCD a contiguous band of tiles so that
// the A rows a band shares stay in that XCD's L2.
__device__ __forceinline__ int remap_tile(int pid, int per_xcd) { return (pid % kXcds) * per_xcd + pid / kXcds; }

// ------------------------------------------------------------------------------------------
// fp16
// ------------------------------------------------------------------------------------------
constexpr int kHThreads = 256;
constexpr int kHBK = 64;                  // k per LDS stage (two MFMA steps of 32)
constexpr int kHAStride = kHBK + 8;       // halves; 144-byte rows: 16-byte reads of 8 consecutive rows hit distinct banks

template <int MI, int WAVES_M, int WAVES_N>
struct HTile {
  static constexpr int BM = WAVES_M * 16 * MI;
  static constexpr int BN = WAVES_N * 128;
  static constexpr int A_CHUNKS = BM * (kHBK / 8) / kHThreads;    // 16-byte chunks per thread per stage
  static constexpr int B_CHUNKS = kHBK * (BN / 8) / kHThreads;
  static constexpr size_t A_BYTES = (size_t)BM * kHAStride * 2;
  static constexpr size_t B_BYTES = (size_t)kHBK * BN * 2;
  static constexpr size_t STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr size_t SMEM_BYTES = 2 * STAGE_BYTES;
  static_assert(WAVES_M * WAVES_N * kWave == kHThreads, "4 wavefronts");
};

__device__ __forceinline__ uint32_t pack_lo(uint32_t x, uint32_t y) { return (x & 0xffffu) | (y << 16); }
__device__ __forceinline__ uint32_t pack_hi(uint32_t x, uint32_t y) { return (x >> 16) | (y & 0xffff0000u); }

template <int MI, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(kHThreads) void gemm_f16_kernel(GemmArgs args) {
  using Tile = HTile<MI, WAVES_M, WAVES_N>;
  constexpr int BM = Tile::BM, BN = Tile::BN;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tile = remap_tile(blockIdx.x, args.per_xcd);
  const int tiles_n_all = args.tiles_n * args.groups;
  if (tile >= args.tiles_m * tiles_n_all) return;
  const int tm = tile / tiles_n_all;
  const int tn_all = tile - tm * tiles_n_all;
  const int grp = tn_all / args.tiles_n;
  const int tn = tn_all - grp * args.tiles_n;
  const int rows = args.rows_dev ? min(*args.rows_dev, args.m_bound) : args.m_bound;
  const int m0 = tm * BM;
  if (m0 >= rows) return;
  const int n0 = tn * BN;
  const int N = args.n, K = args.k;

  const _Float16* __restrict__ A = (const _Float16*)args.A[grp];
  const _Float16* __restrict__ B = (const _Float16*)args.B[grp];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int l16 = lane & 15, g = lane >> 4;

  // global -> register staging
  u32x4 ra[Tile::A_CHUNKS], rb[Tile::B_CHUNKS];
  const int a_kc = tid & 7, a_row = tid >> 3;                 // + u*32
  const int b_nc = tid % (BN / 8), b_krow = tid / (BN / 8);   // + u*(256/(BN/8))
  constexpr int B_ROWS_PER_PASS = kHThreads / (BN / 8);
  const bool b_col_ok = n0 + b_nc * 8 < N;

  auto load_global = [&](int k0) {
#pragma unroll
    for (int u = 0; u < Tile::A_CHUNKS; ++u) {
      const int row = m0 + a_row + u * 32;
      ra[u] = u32x4{0u, 0u, 0u, 0u};
      if (row < rows) ra[u] = *reinterpret_cast<const u32x4*>(A + (size_t)row * K + k0 + a_kc * 8);
    }
#pragma unroll
    for (int u = 0; u < Tile::B_CHUNKS; ++u) {
      const int kr = k0 + b_krow + u * B_ROWS_PER_PASS;
      rb[u] = u32x4{0u, 0u, 0u, 0u};
      if (b_col_ok) rb[u] = *reinterpret_cast<const u32x4*>(B + (size_t)kr * N + n0 + b_nc * 8);
    }
  };
  auto store_lds = [&](int stage) {
    _Float16* As = reinterpret_cast<_Float16*>(smem + stage * Tile::STAGE_BYTES);
    _Float16* Bs = reinterpret_cast<_Float16*>(smem + stage * Tile::STAGE_BYTES + Tile::A_BYTES);
#pragma unroll
    for (int u = 0; u < Tile::A_CHUNKS; ++u)
      *reinterpret_cast<u32x4*>(As + (a_row + u * 32) * kHAStride + a_kc * 8) = ra[u];
#pragma unroll
    for (int u = 0; u < Tile::B_CHUNKS; ++u)
      *reinterpret_cast<u32x4*>(Bs + (b_krow + u * B_ROWS_PER_PASS) * BN + b_nc * 8) = rb[u];
  };

  float4v acc[MI][8];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

  const int nk = K / kHBK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    if (kt + 1 < nk) load_global((kt + 1) * kHBK);
    const _Float16* As = reinterpret_cast<const _Float16*>(smem + (kt & 1) * Tile::STAGE_BYTES);
    const _Float16* Bs = reinterpret_cast<const _Float16*>(smem + (kt & 1) * Tile::STAGE_BYTES + Tile::A_BYTES);
#pragma unroll
    for (int ks = 0; ks < kHBK / 32; ++ks) {
      // B: 8(k) x 8(n) block per lane, transposed in registers into 8 operands
      uint4v raw[8];
#pragma unroll
      for (int kk = 0; kk < 8; ++kk)
        raw[kk] = *reinterpret_cast<const uint4v*>(Bs + (ks * 32 + g * 8 + kk) * BN + wn * 128 + l16 * 8);
      half8 bop[8];
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {        // dword jj of a raw row holds columns 2jj, 2jj+1
        uint4v lo, hi;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          lo[p] = pack_lo(raw[2 * p][jj], raw[2 * p + 1][jj]);
          hi[p] = pack_hi(raw[2 * p][jj], raw[2 * p + 1][jj]);
        }
        bop[2 * jj] = __builtin_bit_cast(half8, lo);
        bop[2 * jj + 1] = __builtin_bit_cast(half8, hi);
      }
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const half8 a =
            *reinterpret_cast<const half8*>(As + (wm * 16 * MI + i * 16 + l16) * kHAStride + ks * 32 + g * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bop[j], acc[i][j], 0, 0, 0);
      }
    }
    if (kt + 1 < nk) store_lds((kt + 1) & 1);
    __syncthreads();
  }

  // epilogue: lane owns rows g*4+r of every 16-row sub-tile and 8 consecutive columns
  const int col = n0 + wn * 128 + l16 * 8;
  if (col < N) {
    _Float16* C = (_Float16*)args.C + (size_t)grp * N + col;
    half8 bias8;
    const bool has_bias = args.bias[grp] != nullptr;
    if (has_bias) bias8 = *reinterpret_cast<const half8*>((const _Float16*)args.bias[grp] + col);
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + wm * 16 * MI + i * 16 + g * 4 + r;
        if (row < rows) {
          half8 o;
#pragma unroll
          for (int j = 0; j < 8; ++j) o[j] = f2h(acc[i][j][r]);
          if (has_bias) o = o + bias8;      // half add on the rounded product, as the reference's next kernel does
          *reinterpret_cast<half8*>(C + (size_t)row * args.ldc) = o;
        }
      }
  }
}

// ------------------------------------------------------------------------------------------
// fp32: 128x128x16 tile, 4 wavefronts (2x2) of 64x64, v_mfma_f32_32x32x2_f32
// ------------------------------------------------------------------------------------------
constexpr int kFThreads = 256;
constexpr int kFBM = 128, kFBN = 128, kFBK = 16;
constexpr int kFAStride = kFBK + 4;       // floats; 80-byte rows
constexpr size_t kFABytes = (size_t)kFBM * kFAStride * 4;
constexpr size_t kFBBytes = (size_t)kFBK * kFBN * 4;
constexpr size_t kFStage = kFABytes + kFBBytes;

__global__ __launch_bounds__(kFThreads) void gemm_f32_kernel(GemmArgs args) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * kFStage];
  const int tile = remap_tile(blockIdx.x, args.per_xcd);
  const int tiles_n_all = args.tiles_n * args.groups;
  if (tile >= args.tiles_m * tiles_n_all) return;
  const int tm = tile / tiles_n_all;
  const int tn_all = tile - tm * tiles_n_all;
  const int grp = tn_all / args.tiles_n;
  const int tn = tn_all - grp * args.tiles_n;
  const int rows = args.rows_dev ? min(*args.rows_dev, args.m_bound) : args.m_bound;
  const int m0 = tm * kFBM;
  if (m0 >= rows) return;
  const int n0 = tn * kFBN;
  const int N = args.n, K = args.k;
  const float* __restrict__ A = (const float*)args.A[grp];
  const float* __restrict__ B = (const float*)args.B[grp];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, kb = lane >> 5;

  u32x4 ra[2], rb[2];
  const int a_kc = tid & 3, a_row = tid >> 2;       // + u*64
  const int b_nc = tid & 31, b_krow = tid >> 5;     // + u*8
  const bool b_col_ok = n0 + b_nc * 4 < N;

  auto load_global = [&](int k0) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int row = m0 + a_row + u * 64;
      ra[u] = u32x4{0u, 0u, 0u, 0u};
      if (row < rows) ra[u] = *reinterpret_cast<const u32x4*>(A + (size_t)row * K + k0 + a_kc * 4);
      rb[u] = u32x4{0u, 0u, 0u, 0u};
      if (b_col_ok) rb[u] = *reinterpret_cast<const u32x4*>(B + (size_t)(k0 + b_krow + u * 8) * N + n0 + b_nc * 4);
    }
  };
  auto store_lds = [&](int stage) {
    float* As = reinterpret_cast<float*>(smem + stage * kFStage);
    float* Bs = reinterpret_cast<float*>(smem + stage * kFStage + kFABytes);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      *reinterpret_cast<u32x4*>(As + (a_row + u * 64) * kFAStride + a_kc * 4) = ra[u];
      *reinterpret_cast<u32x4*>(Bs + (b_krow + u * 8) * kFBN + b_nc * 4) = rb[u];
    }
  };

  float16v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int nk = K / kFBK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    if (kt + 1 < nk) load_global((kt + 1) * kFBK);
    const float* As = reinterpret_cast<const float*>(smem + (kt & 1) * kFStage);
    const float* Bs = reinterpret_cast<const float*>(smem + (kt & 1) * kFStage + kFABytes);
    // step s of the stage contracts k = kb*8 + s (the same choice for A and B)
    float a[2][8], b[2][8];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const float* ap = As + (wm * 64 + i * 32 + l32) * kFAStride + kb * 8;
      const float4v a0 = *reinterpret_cast<const float4v*>(ap);
      const float4v a1 = *reinterpret_cast<const float4v*>(ap + 4);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        a[i][s] = a0[s];
        a[i][4 + s] = a1[s];
      }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int s = 0; s < 8; ++s) b[j][s] = Bs[(kb * 8 + s) * kFBN + wn * 64 + j * 32 + l32];
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][s], b[j][s], acc[i][j], 0, 0, 0);
    if (kt + 1 < nk) store_lds((kt + 1) & 1);
    __syncthreads();
  }

#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int col = n0 + wn * 64 + j * 32 + l32;
    if (col >= N) continue;
    const float bias = args.bias[grp] ? ((const float*)args.bias[grp])[col] : 0.f;
    float* C = (float*)args.C + (size_t)grp * N + col;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * kb + (r & 3);
        if (row < rows) C[(size_t)row * args.ldc] = acc[i][j][r] + bias;
      }
  }
}

template <int MI, int WAVES_M, int WAVES_N>
void launch_f16(GemmArgs a, hipStream_t stream) {
  using Tile = HTile<MI, WAVES_M, WAVES_N>;
  auto kern = gemm_f16_kernel<MI, WAVES_M, WAVES_N>;
  static bool attr_set = false;
  if (!attr_set) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)Tile::SMEM_BYTES);
    attr_set = true;
  }
  a.tiles_m = (a.m_bound + Tile::BM - 1) / Tile::BM;
  a.tiles_n = (a.n + Tile::BN - 1) / Tile::BN;
  const int total = a.tiles_m * a.tiles_n * a.groups;
  a.per_xcd = (total + kXcds - 1) / kXcds;
  kern<<<a.per_xcd * kXcds, kHThreads, Tile::SMEM_BYTES, stream>>>(a);
}

}  // namespace

bool gemm_supported(DType t, int n, int k, int groups) {
  if (groups < 1 || groups > 3 || n <= 0 || k <= 0) return false;
  if (t == DType::F16) return k % kHBK == 0 && n % 8 == 0;
  return k % kFBK == 0 && n % 4 == 0;
}

void launch_gemm(DType t, const GemmGroups& g, void* C, int ldc, int m_bound, int n, int k, const int32_t* rows_dev,
                 hipStream_t stream) {
  if (m_bound <= 0) return;
  GemmArgs a;
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
  a.groups = g.groups;
  if (t == DType::F16) {
    // few big tiles would leave most of the 256 CUs idle: fall back to 128-row tiles
    const long big = (long)((m_bound + 255) / 256) * ((n + 255) / 256) * g.groups;
    if (big >= 512)
      launch_f16<8, 2, 2>(a, stream);
    else
      launch_f16<4, 2, 2>(a, stream);
  } else {
    a.tiles_m = (m_bound + kFBM - 1) / kFBM;
    a.tiles_n = (n + kFBN - 1) / kFBN;
    const int total = a.tiles_m * a.tiles_n * a.groups;
    a.per_xcd = (total + kXcds - 1) / kXcds;
    gemm_f32_kernel<<<a.per_xcd * kXcds, kFThreads, 0, stream>>>(a);
  }
}

}  // namespace et
