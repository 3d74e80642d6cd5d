// MFMA GEMMs for the four dense projections of the encoder layer on gfx950 (replace the cublasGemmEx
// call sites, reference: tf_op/bert_transformer_op.cu.cc:110-141, 200-240).
//
//   C[m,n] = A[m,k] . B[k,n] (+ bias[n]),  A = packed tokens (row-major), B = TF dense kernel [in,out]
//   (row-major, used untransposed), fp32 accumulation, C in the element type.
//
// fp16: v_mfma_f32_16x16x32_f16.  B is n-contiguous in memory while the MFMA wants 8 consecutive k
// per lane, so each lane reads an 8(k) x 8(n) block of B from LDS with eight 128-bit reads and
// transposes it in registers (v_perm_b32); the eight resulting operands feed eight MFMAs whose column
// sets are {8*l + j : l = 0..15}.  A lane therefore ends up owning 8 consecutive output columns per
// row and stores C with 128-bit writes.  The k order inside a step is whatever the loads define; A and
// B use the same one.
// fp32: v_mfma_f32_32x32x2_f32, one element per lane per step.
//
// The M dimension (valid tokens) may live on the device: tiles beyond *rows_dev exit, the last tile
// is predicated.  Up to three column groups (Q/K/V) share one launch.
#include <algorithm>
#include <atomic>

#include <type_traits>

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
  int reverse_walk = 0;      // persistent kernel: walk the tiles from the last one
  int gelu = 0;              // C = gelu(A.B + bias) instead of A.B + bias (bias must be set)
  int a_blocked = 0;         // pair kernel: A / C hold every tile of 256 rows as blocks of [256 rows][64 columns]
  int c_blocked = 0;         //   (see GemmGroups)
  int c_cached = 0;          // persistent k-contiguous kernel: plain stores for C instead of non-temporal ones
  int col_groups = 1;        // persistent k-contiguous kernel: the tile order takes the column tiles in this many groups
};

typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

constexpr int kXcds = 8;

// Workgroups are dealt round-robin to the 8 XCDs; give every XCD a contiguous band of tiles so that
// the A rows a band shares stay in that XCD's L2.
// The banding runs over the tiles that hold valid rows only (`valid_tiles`, a prefix of the tile order): with the row
// count known on the device alone the launch covers every possible tile, and bands cut from all of them would leave
// the last XCDs nothing but empty tiles.  Returns -1 for a workgroup without a tile.
__device__ __forceinline__ int remap_valid_tile(int pid, int valid_tiles) {
  const int per_xcd = (valid_tiles + kXcds - 1) / kXcds;
  const int slot = pid / kXcds;
  const int tile = (pid % kXcds) * per_xcd + slot;
  return slot < per_xcd && tile < valid_tiles ? tile : -1;
}

// ------------------------------------------------------------------------------------------
// fp16: (32*MI) x 256 tile, 4 wavefronts (2x2), k-step 32 = one v_mfma_f32_16x16x32_f16 depth.
//
// Global -> LDS goes through buffer_load_dwordx4 ... lds (no register staging): one instruction moves
// 64 lanes x 16 bytes into 1 KB of contiguous LDS, the lane chooses which 16-byte chunk of the tile it
// fetches (32-bit lane offset + scalar k offset against a buffer descriptor that bounds the rows).  A rows are 64 bytes (4 chunks) per k-step; the chunk position inside a row is XOR-swizzled
// with bits 1-2 of the row so that the MFMA operand reads (16 rows x one chunk per 16 lanes) spread
// over the banks.  B keeps its natural [k][n] order.  A ring of kStages k-steps lives in LDS; the DMA
// runs kStages-1 k-steps ahead of the MFMAs and is tracked with explicit vmcnt waits, the only
// synchronisation per k-step is one s_barrier.  Operands of k-step t+1 are read from LDS and
// transposed while the 8*MI MFMAs of k-step t issue.
// ------------------------------------------------------------------------------------------
constexpr int kHThreads = 256;
constexpr int kHBK = 32;
constexpr int kStages = 4;

// MI: 16-row blocks per wavefront (2 wavefronts along m); NJ: 16-column blocks per wavefront (2 wavefronts along n).
// NJ = 8 is the 256-column tile; NJ = 4 halves the B bytes a workgroup moves per k-step and doubles the number of
// workgroups, which is what counts when there are fewer 256-column tiles than CUs.
template <int MI, int NJ>
struct HTile {
  static constexpr int BM = 32 * MI;
  static constexpr int BN = 32 * NJ;
  static constexpr int A_BYTES = BM * kHBK * 2;
  static constexpr int B_BYTES = kHBK * BN * 2;                // 16 KB / 8 KB
  static constexpr int B_ROW_CHUNKS = BN / 8;                  // 16-byte chunks per k-row
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int SMEM_BYTES = kStages * STAGE_BYTES;
  static constexpr int A_DMA = A_BYTES / 1024 / 4;             // DMA instructions per wavefront per stage
  static constexpr int B_DMA = B_BYTES / 1024 / 4;
  static constexpr int DMA = A_DMA + B_DMA;
};

#define ET_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// gfx9 s_waitcnt immediate: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]
template <int VM>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((VM & 15) | (7 << 4) | (15 << 8) | ((VM >> 4) << 14));
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(15 | (7 << 4) | (0 << 8) | (3 << 14)); }
// Barrier without the fence __syncthreads() carries: the fence would wait for every outstanding DMA.
__device__ __forceinline__ void barrier_only() { asm volatile("s_barrier" ::: "memory"); }

__device__ __forceinline__ int a_swizzle(int row) { return (row >> 1) & 3; }
// 128-column B stages: a wavefront reads 8 bytes per lane, 32 lanes per LDS pass, i.e. two groups of 16 lanes whose
// k-rows are 2 KB apart.  Swapping the two 128-byte halves of every second group of 8 k-rows puts them on different banks.
template <int NJ>
__device__ __forceinline__ int b_swizzle(int chunk, int k_row) {
  return NJ == 8 ? chunk : chunk ^ (((k_row >> 3) & 1) << 3);
}

typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

// raw[kk]: NJ consecutive columns of k-row kk -> bop[j]: the 8 k values of column j
template <typename Raw, int NJ>
__device__ __forceinline__ void transpose8x8(const Raw (&raw)[8], half8 (&bop)[NJ]) {
#pragma unroll
  for (int jj = 0; jj < NJ / 2; ++jj) {       // dword jj of a raw k-row holds columns 2jj, 2jj+1
    uint4v lo, hi;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      lo[p] = __builtin_amdgcn_perm(raw[2 * p + 1][jj], raw[2 * p][jj], 0x05040100u);   // low halves
      hi[p] = __builtin_amdgcn_perm(raw[2 * p + 1][jj], raw[2 * p][jj], 0x07060302u);   // high halves
    }
    bop[2 * jj] = __builtin_bit_cast(half8, lo);
    bop[2 * jj + 1] = __builtin_bit_cast(half8, hi);
  }
}

template <int MI, int NJ>
__global__ __launch_bounds__(kHThreads) __attribute__((amdgpu_waves_per_eu(2))) void gemm_f16_kernel(GemmArgs args) {
#if defined(__HIP_DEVICE_COMPILE__)   // the body uses device-only types (buffer descriptors); the host pass only needs the stub
  using Tile = HTile<MI, NJ>;
  using Raw = typename std::conditional<NJ == 8, uint4v, uint2v>::type;     // NJ halves of one k-row
  using HalfN = typename std::conditional<NJ == 8, half8, half4>::type;
  constexpr int BM = Tile::BM, BN = Tile::BN;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int rows = args.rows_dev ? min(*args.rows_dev, args.m_bound) : args.m_bound;
  const int tiles_n_all = args.tiles_n * args.groups;
  const int tile = remap_valid_tile(blockIdx.x, ((rows + BM - 1) / BM) * tiles_n_all);
  if (tile < 0) return;
  const int tm = tile / tiles_n_all;
  const int tn_all = tile - tm * tiles_n_all;
  const int grp = tn_all / args.tiles_n;
  const int tn = tn_all - grp * args.tiles_n;
  const int m0 = tm * BM;
  const int n0 = tn * BN;
  const int N = args.n, K = args.k;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);   // scalar: LDS targets of the DMA are SALU values
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, g = lane >> 4;

  // Buffer descriptors bound the DMA: A rows at or beyond the valid-token count read as zero.
  __amdgpu_buffer_rsrc_t rsrc_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(args.A[grp]), 0, (int)((uint32_t)rows * K * 2u), 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_b =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(args.B[grp]), 0, (int)((uint32_t)K * N * 2u), 0x00020000);

  // Per-lane byte offsets of the chunks this lane moves every stage (the k offset is a scalar).
  // Columns beyond N are clamped to a valid column; what they load is never stored.
  uint32_t a_off[Tile::A_DMA], b_off[Tile::B_DMA];
#pragma unroll
  for (int j = 0; j < Tile::A_DMA; ++j) {
    const int q = wave * Tile::A_DMA + j;              // 1 KB slot of the A stage: 16 rows x 4 chunks
    const int row = q * 16 + (lane >> 2);
    const int c = (lane & 3) ^ a_swizzle(row);
    a_off[j] = ((uint32_t)(m0 + row) * (uint32_t)K + (uint32_t)c * 8u) * 2u;
  }
#pragma unroll
  for (int j = 0; j < Tile::B_DMA; ++j) {
    const int q = wave * Tile::B_DMA + j;              // 1 KB slot of the B stage: 2 k-rows x 32 chunks (4 x 16)
    constexpr int RC = Tile::B_ROW_CHUNKS;
    const int kr = q * (64 / RC) + lane / RC;
    const int col = min(n0 + b_swizzle<NJ>(lane % RC, kr) * 8, N - 8);
    b_off[j] = ((uint32_t)kr * (uint32_t)N + (uint32_t)col) * 2u;
  }
  const int nk = K / kHBK;

  auto issue = [&](int kt) {
    unsigned char* st = smem + (kt % kStages) * Tile::STAGE_BYTES;
    const int ktc = min(kt, nk - 1);       // past the end: re-load the last k-step (keeps the DMA count uniform)
#pragma unroll
    for (int j = 0; j < Tile::A_DMA; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, ET_LDS_PTR(st + (wave * Tile::A_DMA + j) * 1024), 16, a_off[j],
                                               ktc * kHBK * 2, 0, 0);
#pragma unroll
    for (int j = 0; j < Tile::B_DMA; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, ET_LDS_PTR(st + Tile::A_BYTES + (wave * Tile::B_DMA + j) * 1024),
                                               16, b_off[j], ktc * kHBK * N * 2, 0, 0);
  };

  float4v acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

  // LDS read offsets in bytes: A row (wm*16*MI + i*16 + l16), chunk g (swizzled); B k-row g*8+kk, NJ columns
  const int a_rd = ((wm * 16 * MI + l16) * 4 + (g ^ a_swizzle(l16))) * 16;
  const int b_rd = NJ == 8 ? ((g * 8) * BN + wn * 128 + l16 * 8) * 2
                           : (g * 8) * BN * 2 + b_swizzle<NJ>(wn * 8 + (l16 >> 1), g * 8) * 16 + (l16 & 1) * 8;

#pragma unroll
  for (int q = 0; q < kStages; ++q) issue(q);
  wait_vmcnt<Tile::DMA * (kStages - 1)>();
  barrier_only();
  // Two operand register sets: a k-step multiplies out of one while it fills the other, and the k loop below is
  // unrolled by two so that neither set is ever copied.
  half8 a_reg[2][MI], b_reg[2][NJ];
  {
    Raw raw[8];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) raw[kk] = *reinterpret_cast<const Raw*>(smem + Tile::A_BYTES + b_rd + kk * BN * 2);
#pragma unroll
    for (int i = 0; i < MI; ++i) a_reg[0][i] = *reinterpret_cast<const half8*>(smem + a_rd + i * 16 * 64);
    transpose8x8(raw, b_reg[0]);
  }

  auto step = [&](int kt, const half8 (&a_cur)[MI], const half8 (&bop_cur)[NJ], half8 (&a_n)[MI], half8 (&bop_n)[NJ]) {
    wait_vmcnt<Tile::DMA * (kStages - 2)>();   // k-step kt+1 has landed; kt+2 and kt+3 may still be in flight
    wait_lgkmcnt0();                           // this wavefront's reads of k-step kt's buffer are complete
    barrier_only();
    issue(kt + kStages);                       // into the buffer of k-step kt, free now for every wavefront
    const unsigned char* st = smem + ((kt + 1) % kStages) * Tile::STAGE_BYTES;
    Raw raw[8];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) raw[kk] = *reinterpret_cast<const Raw*>(st + Tile::A_BYTES + b_rd + kk * BN * 2);
#pragma unroll
    for (int i = 0; i < MI; ++i) a_n[i] = *reinterpret_cast<const half8*>(st + a_rd + i * 16 * 64);
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_cur[i], bop_cur[j], acc[i][j], 0, 0, 0);
    transpose8x8(raw, bop_n);
    // issue order: the MFMAs start right behind the barrier; the LDS reads and this wave's DMA instructions go between
    // the first of them, the transposes (which wait for the reads) between the rest
    constexpr int kReads = 8 + MI, kMfma = NJ * MI, kPerms = 4 * NJ;
    constexpr int kEarly = kReads < kMfma / 2 ? kReads : kMfma / 2, kLate = kMfma - kEarly;
#pragma unroll
    for (int r = 0; r < kEarly; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                     // 1 MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, (kReads + kEarly - 1) / kEarly, 0);        // its share of the LDS reads
      __builtin_amdgcn_sched_group_barrier(0x020, (Tile::DMA + kEarly - 1) / kEarly, 0);     // and of the DMA instructions
    }
#pragma unroll
    for (int r = 0; r < kLate; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                            // 1 MFMA
      __builtin_amdgcn_sched_group_barrier(0x002, (kPerms + kLate - 1) / kLate, 0);   // its share of the transposes
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  int kt = 0;
#pragma unroll 1
  for (; kt + 1 < nk; kt += 2) {
    step(kt, a_reg[0], b_reg[0], a_reg[1], b_reg[1]);
    step(kt + 1, a_reg[1], b_reg[1], a_reg[0], b_reg[0]);
  }
  if (kt < nk) step(kt, a_reg[0], b_reg[0], a_reg[1], b_reg[1]);
  wait_vmcnt<0>();        // no DMA may still target this workgroup's LDS when it ends

  // epilogue: lane owns rows g*4+r of every 16-row sub-tile and NJ consecutive columns
  const int col = n0 + wn * (BN / 2) + l16 * NJ;
  if (col < N) {
    _Float16* C = (_Float16*)args.C + (size_t)grp * N + col;
    HalfN bias8;
    const bool has_bias = args.bias[grp] != nullptr;
    if (has_bias) bias8 = *reinterpret_cast<const HalfN*>((const _Float16*)args.bias[grp] + col);
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + wm * 16 * MI + i * 16 + g * 4 + r;
        if (row < rows) {
          HalfN o;
#pragma unroll
          for (int j = 0; j < NJ; ++j) o[j] = f2h(acc[i][j][r]);
          // half add on the rounded product, as the reference's next kernel does; optionally that kernel's GELU too
          if (args.gelu) o = bias_gelu_half<HalfN, NJ>(o, bias8);
          else if (has_bias) o = o + bias8;
          __builtin_nontemporal_store(o, reinterpret_cast<HalfN*>(C + (size_t)row * args.ldc));
        }
      }
  }
#else
  (void)args;
#endif
}

// ------------------------------------------------------------------------------------------
// fp16, large problems, B in its [k][n] storage order: persistent 256 x 256 tiles, 8 wavefronts (two per SIMD) in
// opposite phases.
//
// Wave tile 128 x 64 (32 MFMAs per k-step, 128 accumulator registers), so two wavefronts fit one SIMD.
// Waves 0-3 and 4-7 alternate: while one group issues its 32 MFMAs (raised priority) the other does
// its fetch half of the k-step -- its share of the DMA for the k-step three ahead, the LDS operand
// reads of the current k-step and the 8x4 B transpose -- and a barrier swaps the roles.  The MFMA pipe
// of a SIMD therefore always has one wave feeding it and no wave needs a second operand register set.
//
// A workgroup walks its tiles (XCD-banded order) with ONE continuous DMA stream: the last k-steps of a
// tile already fetch the first k-steps of the next one.  At a tile boundary a wave confirms every DMA
// it has issued (vmcnt 0), then issues its C stores and carries on; the vmcnt waits that follow count
// loads only (loads complete in order among themselves), so stores still in flight can delay such a
// wait but never let it pass early.
// ------------------------------------------------------------------------------------------
constexpr int kPThreads = 512;
constexpr int kPBM = 256, kPBN = 256;
constexpr int kPStage = (kPBM * kHBK + kHBK * kPBN) * 2;      // 32 KB per k-step
constexpr int kPSmem = kStages * kPStage;                     // 128 KB
[[maybe_unused]] constexpr int kPABytes = kPBM * kHBK * 2;     // A part of a k-step slot, B follows


struct PTile {
  int m0, n0, grp;
};

__global__ __launch_bounds__(kPThreads) void gemm_f16_persistent_kernel(GemmArgs args) {
#if defined(__HIP_DEVICE_COMPILE__)   // device-only types in the body; the host pass only needs the stub
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);   // 0..7, scalar
  const int phase_group = wave >> 2;
  const int wm = wave & 1, wn = (wave >> 1) & 3;                  // 128-row half, 64-column quarter of the tile
  const int l16 = lane & 15, g = lane >> 4;
  const int N = args.n, K = args.k;
  const int nk = K / kHBK;

  const int rows = args.rows_dev ? min(*args.rows_dev, args.m_bound) : args.m_bound;
  const int tiles_n_all = args.tiles_n * args.groups;
  const int total = ((rows + kPBM - 1) / kPBM) * tiles_n_all;     // tiles that hold valid rows (a prefix in tile order)
  const int per_xcd = (total + kXcds - 1) / kXcds;
  const int xcd = blockIdx.x % kXcds;
  const int G = gridDim.x;                                        // multiple of 8

  // tile number `idx` of this workgroup's walk -> tile; every XCD owns a contiguous band of tiles
  auto tile_id = [&](int idx) { return xcd * per_xcd + idx / kXcds; };
  auto valid = [&](int idx) { return idx / kXcds < per_xcd && tile_id(idx) < total; };
  auto locate = [&](int tile) {
    PTile t;
    if (args.reverse_walk) tile = total - 1 - tile;
    const int tm = tile / tiles_n_all;
    const int tn_all = tile - tm * tiles_n_all;
    t.grp = tn_all / args.tiles_n;
    t.m0 = tm * kPBM;
    t.n0 = (tn_all - t.grp * args.tiles_n) * kPBN;
    return t;
  };

  struct Src {
    __amdgpu_buffer_rsrc_t a, b;
    uint32_t off[4];        // 0,1: A chunks, 2,3: B chunks of this lane per k-step
  };
  auto make_src = [&](const PTile& t) {
    Src s;
    // descriptors bound the DMA: A rows at or beyond the valid-token count read as zero
    s.a = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(args.A[t.grp]), 0, (int)((uint32_t)rows * K * 2u), 0x00020000);
    s.b = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(args.B[t.grp]), 0, (int)((uint32_t)K * N * 2u), 0x00020000);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int q = wave * 2 + j;                      // 1 KB slot: A 16 rows x 4 chunks, B 2 k-rows x 32 chunks
      const int row = q * 16 + (lane >> 2);
      const int c = (lane & 3) ^ a_swizzle(row);
      s.off[j] = ((uint32_t)(t.m0 + row) * (uint32_t)K + (uint32_t)c * 8u) * 2u;
      const int kr = q * 2 + (lane >> 5);
      const int pc = ((lane & 31) - 8 * ((kr >> 3) & 1)) & 31;   // B rows 8..15, 24..31 are rotated by 128 bytes in LDS
      const int col = min(t.n0 + pc * 8, N - 8);                 // columns beyond N: a valid column, never stored
      s.off[2 + j] = ((uint32_t)kr * (uint32_t)N + (uint32_t)col) * 2u;
    }
    return s;
  };
  // this wave's share (4 of 32 instructions) of the DMA for k-step kt of a tile into ring slot `slot`
  auto issue = [&](int slot, int kt, const Src& s) {
    unsigned char* st = smem + slot * kPStage;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(s.a, ET_LDS_PTR(st + (wave * 2 + j) * 1024), 16, s.off[j], kt * kHBK * 2,
                                               0, 0);
#pragma unroll
    for (int j = 0; j < 2; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(s.b, ET_LDS_PTR(st + kPABytes + (wave * 2 + j) * 1024), 16, s.off[2 + j],
                                               kt * kHBK * N * 2, 0, 0);
  };

  // LDS operand addresses: A row (wm*128 + i*16 + l16), chunk g (swizzled); B k-row g*8+kk, 4 columns
  const int a_rd = ((wm * 128 + l16) * 4 + (g ^ a_swizzle(l16))) * 16;
  int b_rd[8];
#pragma unroll
  for (int kk = 0; kk < 8; ++kk) {
    const int row = g * 8 + kk;
    b_rd[kk] = row * 512 + (((wn * 64 + l16 * 4) * 2 + 128 * ((row >> 3) & 1)) & 511);
  }

  int idx = blockIdx.x;
  if (!valid(idx)) return;
  PTile tile = locate(tile_id(idx));
  Src cur = make_src(tile), nxt = cur;

  float4v acc[8][4];
  half8 a[8], bop[4];
  int u = 0;                                   // k-steps done by this workgroup: ring slot of k-step = u & 3

  auto fetch_phase = [&](int kt_issue, const Src& s, bool check) {
    issue((u + 3) & 3, kt_issue, s);
    const unsigned char* st = smem + (u & 3) * kPStage;
    uint2v raw[8];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) raw[kk] = *reinterpret_cast<const uint2v*>(st + kPABytes + b_rd[kk]);
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = *reinterpret_cast<const half8*>(st + a_rd + i * 16 * 64);
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {             // 8(k) x 4(n) block -> 4 operands
      uint4v lo, hi;
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        lo[p] = __builtin_amdgcn_perm(raw[2 * p + 1][jj], raw[2 * p][jj], 0x05040100u);
        hi[p] = __builtin_amdgcn_perm(raw[2 * p + 1][jj], raw[2 * p][jj], 0x07060302u);
      }
      bop[2 * jj] = __builtin_bit_cast(half8, lo);
      bop[2 * jj + 1] = __builtin_bit_cast(half8, hi);
    }
    if (check) wait_vmcnt<8>();                // this wave's share of k-step u+1 has landed (u+2, u+3 may fly)
    wait_lgkmcnt0();
  };
  auto mfma_phase = [&](bool first) {
    __builtin_amdgcn_s_setprio(1);
    if (first) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], bop[j], float4v{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], bop[j], acc[i][j], 0, 0, 0);
    }
    __builtin_amdgcn_s_setprio(0);
  };

  // k-steps beyond the tile (K < 96) re-load the last one; the data is never used
  issue(0, 0, cur);
  issue(1, min(1, nk - 1), cur);
  issue(2, min(2, nk - 1), cur);
  wait_vmcnt<8>();
  barrier_only();
  if (phase_group == 1) barrier_only();        // the second group runs one phase behind the first
  bool first_tile = true;
  while (true) {
    const int nidx = idx + G;
    const bool has_next = valid(nidx);
    PTile ntile = tile;
    if (has_next) {
      ntile = locate(tile_id(nidx));
      nxt = make_src(ntile);
    } else {
      nxt = cur;                               // re-loads of this tile keep the DMA count per k-step uniform
    }
    for (int t = 0; t < nk; ++t) {
      // right after a tile boundary the first two k-steps were confirmed before the C stores went out
      const bool check = first_tile || t >= 2;
      if (t + 3 < nk) fetch_phase(t + 3, cur, check);
      else fetch_phase(min(t + 3 - nk, nk - 1), nxt, check);
      barrier_only();
      mfma_phase(t == 0);
      barrier_only();
      ++u;
    }
    wait_vmcnt<0>();
    {
      // C goes out through a buffer descriptor that ends at the last valid row: rows beyond it are dropped by
      // the bounds check, and the only per-store address arithmetic is one add on the running byte offset
      const int col = tile.n0 + wn * 64 + l16 * 4;
      if (col < N) {
        const __amdgpu_buffer_rsrc_t rc =
            __builtin_amdgcn_make_buffer_rsrc(args.C, 0, (int)((uint32_t)rows * (uint32_t)args.ldc * 2u), 0x00020000);
        const uint32_t row_bytes = (uint32_t)args.ldc * 2u;
        uint32_t voff = ((uint32_t)(tile.m0 + wm * 128 + g * 4) * (uint32_t)args.ldc + (uint32_t)(tile.grp * N + col)) * 2u;
        auto store_all = [&](auto mode, half4 bias4) {     // mode 0: product, 1: + bias, 2: gelu(+ bias)
#pragma unroll
          for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              half4 o;
#pragma unroll
              for (int j = 0; j < 4; ++j) o[j] = f2h(acc[i][j][r]);
              // half add on the rounded product, as the reference's next kernel does (mode 2: and its GELU)
              if (decltype(mode)::value == 2) o = bias_gelu_half<half4, 4>(o, bias4);
              else if (decltype(mode)::value == 1) o = o + bias4;
              __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(uint2v, o), rc, voff, 0, 2 /* nt */);
              voff += row_bytes;
            }
            voff += 12u * row_bytes;
          }
        };
        if (args.bias[tile.grp] != nullptr)
          if (args.gelu)
            store_all(std::integral_constant<int, 2>{}, *reinterpret_cast<const half4*>((const _Float16*)args.bias[tile.grp] + col));
          else
            store_all(std::integral_constant<int, 1>{}, *reinterpret_cast<const half4*>((const _Float16*)args.bias[tile.grp] + col));
        else
          store_all(std::integral_constant<int, 0>{}, half4{});
      }
    }
    if (!has_next) break;
    idx = nidx;
    tile = ntile;
    cur = nxt;
    first_tile = false;
  }
  if (phase_group == 0) barrier_only();        // matches the extra barrier the second group started with
  wait_vmcnt<0>();                             // no DMA may still target this workgroup's LDS when it ends
#else
  (void)args;
#endif
}

// ------------------------------------------------------------------------------------------
// fp16, large problems, B k-contiguous ([n][k], see launch_transpose_weights): persistent 256 x 256 tiles, 8 wavefronts
// that each pipeline their own work, LDS slots of two k-steps.
//
// Both operands are fetched in rows of 64 k = 128 bytes, one full cache line per row: eight lanes of a DMA instruction
// cover a line, where rows of 32 k leave every second half-line request to the next k-step.  Two such slots (2 x 64 KB)
// make the ring.  A wave (tile 128 x 64, two operand register sets) reads the operands of k-step t+1 from LDS and
// issues its share of the DMA for the pair after next between the MFMAs of k-step t, so no wave ever stops for a fetch
// phase, and the only synchronisation is one barrier per pair of k-steps: after the even step every wave has read its
// slot for the last time (the slot becomes the DMA target during the odd step) and this wave's share of the other slot
// has landed.  The 16-byte chunks of a 128-byte LDS row are XOR-swizzled with row bits 1-3, which spreads the 16 rows
// x one chunk of an MFMA operand read over all 64 banks.
// A, B^T and C are addressed through per-tile buffer descriptors (base at the tile, records = what the matrix has
// left there), so lane offsets are tile-independent, rows beyond the valid-token count read as zero and are dropped
// on the way out, and no offset grows with the size of the matrices.
// ------------------------------------------------------------------------------------------
constexpr int kQAPair = kPBM * 128;                            // 32 KB: 256 rows x two k-steps
constexpr int kQPair = kQAPair + kPBN * 128;                   // 64 KB: A rows, then B^T rows
constexpr int kQSmem = 2 * kQPair;
constexpr int kQSmemA3 = 3 * kQAPair + 2 * (kQPair - kQAPair);   // 160 KB: three A slots, two B^T slots

__device__ __forceinline__ int pair_swizzle(int row) { return (row >> 1) & 7; }

// MI: 16-row blocks per wave, i.e. tiles of 32 MI rows (256, 224, 192 or 160).  The tile count of a launch rarely
// fills whole rounds of the chip; a lower tile can turn "one round and a bit" into one round (launch_f16_persistent
// chooses).  The A part of an LDS slot keeps its 256 rows; the rows beyond the tile lie outside the tile's buffer
// descriptor and cost no traffic.
// NT: C leaves through non-temporal stores (a matrix too big to be found in the last-level cache by its reader);
// plain stores otherwise.
// A3: three LDS slots for A instead of two, all of the 160 KB: the A rows of a pair are requested three pairs ahead
// of their first use instead of two (B^T as before).  For the projection whose A is the big matrix and comes from
// HBM (k >= 2048: FFN-down), where a pair's time does not cover that latency.  Same instructions on the same data in
// the same order: same bits.
template <bool GELU, int MI, bool NT, bool A3 = false>
__global__ __launch_bounds__(kPThreads) void gemm_f16_pair_kernel(GemmArgs args) {
#if defined(__HIP_DEVICE_COMPILE__)   // device-only types in the body; the host pass only needs the stub
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);   // 0..7, scalar
  constexpr int BM = 32 * MI;                                     // rows of a tile
  const int wm = wave & 1, wn = (wave >> 1) & 3;                  // (16 MI)-row half, 64-column quarter of the tile
  const int l16 = lane & 15, g = lane >> 4;
  const int N = args.n, K = args.k;
  const int np = K / 64;                                          // pairs of k-steps per tile, >= 2

  const int rows = args.rows_dev ? min(*args.rows_dev, args.m_bound) : args.m_bound;
  const int tiles_n_all = args.tiles_n * args.groups;
  const int total = ((rows + BM - 1) / BM) * tiles_n_all;     // tiles that hold valid rows (a prefix in tile order)
  const int per_xcd = (total + kXcds - 1) / kXcds;
  const int xcd = blockIdx.x % kXcds;
  const int G = gridDim.x;                                        // multiple of 8

  // This XCD's band holds n_loc tiles for wgs workgroups: `full` of them fill whole rounds.  When the rest would keep at
  // most half of the workgroups busy for a last round, each of those tiles is shared by two workgroups, one per
  // 128-column half: the waves of the other half only keep the operand stream going, a SIMD then has one MFMA wave
  // instead of two, and the last round takes about half a tile time.  Every element is still accumulated by one wave in
  // the same k order, so the bits do not depend on the split.
  const int wgs = G / kXcds, local = blockIdx.x / kXcds;
  const int n_loc = max(0, min(per_xcd, total - xcd * per_xcd));
  const int full = (n_loc / wgs) * wgs, rem = n_loc - full;
  const bool split = rem > 0 && 2 * rem <= wgs;
  // slot s (= local + round * wgs) of the band -> tile and half (-1: the whole tile)
  auto valid = [&](int s) { return s < full || (split ? s - full < 2 * rem : s < n_loc); };

  struct Src {
    __amdgpu_buffer_rsrc_t a, b;
    int m0, n0, grp, half;
  };
  auto locate = [&](int s) {
    Src t;
    t.half = -1;
    int tile = xcd * per_xcd + s;
    if (s >= full && split) {
      t.half = (s - full) & 1;
      tile = xcd * per_xcd + full + ((s - full) >> 1);
    }
    if (args.reverse_walk) tile = total - 1 - tile;
    // column groups: the tile order runs through all row tiles of the first tiles_n_all / col_groups column tiles,
    // then through those of the next group
    const int cpg = tiles_n_all / args.col_groups;
    const int per_group = (total / tiles_n_all) * cpg;
    const int cg = tile / per_group;
    const int r = tile - cg * per_group;
    const int tm = r / cpg;
    const int tn_all = cg * cpg + (r - tm * cpg);
    t.grp = tn_all / args.tiles_n;
    t.m0 = tm * BM;
    t.n0 = (tn_all - t.grp * args.tiles_n) * kPBN;
    // a blocked A holds whole tiles: rows beyond the valid count are there (written by the producer from zero rows)
    t.a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16*>((const _Float16*)args.A[t.grp] + (size_t)t.m0 * K), 0,
        (args.a_blocked ? BM : min(rows - t.m0, BM)) * K * 2, 0x00020000);
    t.b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16*>((const _Float16*)args.B[t.grp] + (size_t)t.n0 * K), 0, min(N - t.n0, kPBN) * K * 2, 0x00020000);
    return t;
  };

  // DMA: one instruction fills 1 KB of LDS = 8 rows x 128 bytes.  This wave owns rows wave*32 .. wave*32+31 of the A
  // part and of the B^T part of a slot (4 + 4 instructions per pair).  LDS row j*16+l of a 64-column group holds
  // column 4*l+j of the tile, so that the operand reads of B^T look like A's and a lane owns 4 consecutive columns of C.
  uint32_t voff_a[4], voff_b[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = wave * 32 + j * 8 + (lane >> 3);
    const int c = (lane & 7) ^ pair_swizzle(row);
    // blocked A: the 128 bytes of a row and pair lie 128 bytes from the next row's, a pair is one block of 32 KB
    voff_a[j] = args.a_blocked ? (uint32_t)row * 128u + (uint32_t)c * 16u
                               : ((uint32_t)row * (uint32_t)K + (uint32_t)c * 8u) * 2u;
    const int col = (row & ~63) + (row & 15) * 4 + ((row >> 4) & 3);
    voff_b[j] = ((uint32_t)col * (uint32_t)K + (uint32_t)c * 8u) * 2u;
  }
  const int a_pair_bytes = args.a_blocked ? kQAPair : 128;       // from one pair of k-steps of A to the next
  // LDS: slot s = A rows, then B^T rows of a pair (two slots); with A3 a ring of three A slots, then two B^T slots
  auto a_slot = [&](int sa) -> unsigned char* { return smem + sa * (A3 ? kQAPair : kQPair); };
  auto b_slot = [&](int sb) -> unsigned char* {
    return A3 ? smem + 3 * kQAPair + sb * (kQPair - kQAPair) : smem + sb * kQPair + kQAPair;
  };
  // instruction q (0..3) of this wave's share of the A rows / B^T rows of pair `pr` of a tile into slot sa / sb
  auto issue_a = [&](int sa, int pr, const __amdgpu_buffer_rsrc_t& ra, int q) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, ET_LDS_PTR(a_slot(sa) + (wave * 4 + q) * 1024), 16, voff_a[q],
                                             pr * a_pair_bytes, 0, 0);
  };
  auto issue_b = [&](int sb, int pr, const __amdgpu_buffer_rsrc_t& rb, int q) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, ET_LDS_PTR(b_slot(sb) + (wave * 4 + q) * 1024), 16, voff_b[q], pr * 128,
                                             0, 0);
  };
  // instruction q (0..7) of a whole pair: A first, then B^T; with A3 the other way round, and the A rows are those
  // of the pair one further ahead, so that they are the newest requests and may stay in flight at the next wait
  auto issue1 = [&](int sa, int sb, int pr_a, int pr_b, const __amdgpu_buffer_rsrc_t& ra,
                    const __amdgpu_buffer_rsrc_t& rb, int q) {
    if (A3) {
      if (q < 4) issue_b(sb, pr_b, rb, q);
      else issue_a(sa, pr_a, ra, q - 4);
    } else {
      if (q < 4) issue_a(sa, pr_a, ra, q);
      else issue_b(sb, pr_b, rb, q - 4);
    }
  };

  // operand reads: row (wm*128 + i*16 + l16) resp. (wn*64 + j*16 + l16), chunk (4*half + g), swizzled
  const int sw = pair_swizzle(l16);
  const int a_rd[2] = {(wm * 16 * MI + l16) * 128 + ((g ^ sw) * 16), (wm * 16 * MI + l16) * 128 + (((4 + g) ^ sw) * 16)};
  const int b_rd[2] = {(wn * 64 + l16) * 128 + ((g ^ sw) * 16), (wn * 64 + l16) * 128 + (((4 + g) ^ sw) * 16)};

  int idx = local;
  if (!valid(idx)) return;
  {
    // The workgroups of an XCD run their tiles in lockstep, so all of them stream operands and store C at the same
    // moments.  Those that walk one tile less than the others have a tile time to spare: they start late, spread over
    // about a quarter of a tile time (960 cycles per pair of k-steps), which takes their traffic out of step with the
    // rest at no cost to the last round (measured: -1.3 % on the encoder step, nothing gained beyond that spread).
    const int max_tiles = (n_loc + wgs - 1) / wgs;
    // first workgroup of this XCD with max_tiles - 1 tiles
    const int first_short = split ? 2 * rem : n_loc - (max_tiles - 1) * wgs;
    if (local >= first_short && first_short < wgs) {
      const int units = (np * 15 + 90) * (local - first_short + 1) / (wgs - first_short + 1);   // of 64 cycles
      for (int u = 0; u < units; u += 16) __builtin_amdgcn_s_sleep(16);
    }
  }
  Src cur = locate(idx), nxt = cur;

  float4v acc[MI][4];
  half8 a[2][MI], b[2][4];
  int pairs_done = 0;                            // by this workgroup: slot of a pair = pairs_done & 1

  // One k-step: MFMAs on operand set P; half `rh` of the slots rsa / rsb is read into the other set; with DMA set, this
  // wave's eight DMA instructions (A rows of pair dpa into slot dsa, B^T rows of pair dpb into slot dsb; descriptors
  // da, db) go out, one after each group of four MFMAs.
  auto step = [&](auto Pc, auto FIRSTc, auto DMAc, int rsa, int rsb, int dsa, int dsb, int dpa, int dpb,
                  const __amdgpu_buffer_rsrc_t& da, const __amdgpu_buffer_rsrc_t& db) {
    constexpr int P = decltype(Pc)::value;
    constexpr bool FIRST = decltype(FIRSTc)::value;
    constexpr bool DMA = decltype(DMAc)::value;
    constexpr int rh = 1 - P;                    // the even step reads half 1 of its own pair, the odd step half 0 of the next
    const unsigned char* nsa = a_slot(rsa);
    const unsigned char* nsb = b_slot(rsb);
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      // two of the 4 + MI operand reads of the next step in front of each group of four MFMAs (B^T blocks first)
#pragma unroll
      for (int r = 2 * i; r < 2 * i + 2 && r < 4 + MI; ++r) {
        if (r < 4) b[1 - P][r] = *reinterpret_cast<const half8*>(nsb + b_rd[rh] + r * 2048);
        else a[1 - P][r - 4] = *reinterpret_cast<const half8*>(nsa + a_rd[rh] + (r - 4) * 2048);
      }
      // the column blocks back and forth: between two MFMAs only one operand changes, which costs measurably less
      // power than the row-major order (the part runs the same stream 1 - 2 % faster on random operands)
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int j = (i & 1) ? 3 - jj : jj;
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[P][i], b[P][j],
                                                           FIRST ? float4v{0.f, 0.f, 0.f, 0.f} : acc[i][j], 0, 0, 0);
      }
      if (DMA) {
#pragma unroll
        for (int q = 0; q < 8; ++q)
          if (q * MI / 8 == i) issue1(dsa, dsb, dpa, dpb, da, db, q);      // the eight DMA instructions spread over the MI groups
      }
      __builtin_amdgcn_sched_barrier(0);         // keeps the reads and the DMA where they are between the MFMA groups
    }
  };
  using Even = std::integral_constant<int, 0>;
  using Odd = std::integral_constant<int, 1>;

  // pairs 0 and 1 of the first tile (with A3 also the A rows of pair 2), operands of k-step 0
#pragma unroll
  for (int q = 0; q < 4; ++q) issue_a(0, 0, cur.a, q);
#pragma unroll
  for (int q = 0; q < 4; ++q) issue_b(0, 0, cur.b, q);
#pragma unroll
  for (int q = 0; q < 4; ++q) issue_a(1, 1, cur.a, q);
#pragma unroll
  for (int q = 0; q < 4; ++q) issue_b(1, 1, cur.b, q);
  if (A3) {
#pragma unroll
    for (int q = 0; q < 4; ++q) issue_a(2, 2, cur.a, q);
    wait_vmcnt<12>();
  } else {
    wait_vmcnt<8>();
  }
  barrier_only();
#pragma unroll
  for (int j = 0; j < 4; ++j) b[0][j] = *reinterpret_cast<const half8*>(b_slot(0) + b_rd[0] + j * 2048);
#pragma unroll
  for (int i = 0; i < MI; ++i) a[0][i] = *reinterpret_cast<const half8*>(a_slot(0) + a_rd[0] + i * 2048);
  int sa = 0;                                    // A slot of the current pair = pairs_done % 3 (A3)
  auto next3 = [](int v) { return v == 2 ? 0 : v + 1; };

  bool first_tile = true;
  while (true) {
    const int nidx = idx + wgs;
    const bool has_next = valid(nidx);
    if (has_next) nxt = locate(nidx);            // otherwise the stream re-loads this tile; the data is never used
    // a shared tile: this wave computes only when its columns lie in the workgroup's half
    const bool computes = cur.half < 0 || (wn >> 1) == cur.half;
    if (computes) {
      for (int p = 0; p < np; ++p) {
        const int s = pairs_done & 1;
        const int ra = A3 ? sa : s;                // this pair's A slot
        if (p == 0) step(Even{}, std::true_type{}, std::false_type{}, ra, s, 0, 0, 0, 0, cur.a, cur.b);
        else step(Even{}, std::false_type{}, std::false_type{}, ra, s, 0, 0, 0, 0, cur.a, cur.b);
        // this wave's share of the next pair has landed (right after a tile boundary that was confirmed before the C
        // stores went out) and its last reads of slot s, which feed the odd step, are complete; with A3 the four
        // newest requests, the A rows of the pair after the next, may still be on their way
        if (first_tile || p >= 1) {
          if (A3) wait_vmcnt<4>();
          else wait_vmcnt<0>();
        }
        wait_lgkmcnt0();
        barrier_only();
        // B^T of pair p+2 (A of pair p+2, with A3 of pair p+3) of this tile, or the matching pair of the next one,
        // replaces what this pair held
        const int pa = A3 ? p + 3 : p + 2, pb = p + 2;
        const __amdgpu_buffer_rsrc_t da = pa < np ? cur.a : nxt.a;
        const __amdgpu_buffer_rsrc_t db = pb < np ? cur.b : nxt.b;
        step(Odd{}, std::false_type{}, std::true_type{}, A3 ? next3(sa) : s ^ 1, s ^ 1, ra, s, pa < np ? pa : pa - np,
             pb < np ? pb : pb - np, da, db);
        ++pairs_done;
        sa = next3(sa);
      }
    } else {
      // the other half's waves: same barriers, same share of the DMA, no operand reads and no MFMAs
      for (int p = 0; p < np; ++p) {
        const int s = pairs_done & 1;
        if (first_tile || p >= 1) {
          if (A3) wait_vmcnt<4>();
          else wait_vmcnt<0>();
        }
        barrier_only();
        const int pa = A3 ? p + 3 : p + 2, pb = p + 2;
        const __amdgpu_buffer_rsrc_t da = pa < np ? cur.a : nxt.a;
        const __amdgpu_buffer_rsrc_t db = pb < np ? cur.b : nxt.b;
#pragma unroll
        for (int q = 0; q < 8; ++q)
          issue1(A3 ? sa : s, s, pa < np ? pa : pa - np, pb < np ? pb : pb - np, da, db, q);
        ++pairs_done;
        sa = next3(sa);
      }
    }
    wait_vmcnt<0>();
    if (computes) {
      // C leaves through a descriptor that covers the tile's valid rows only: rows beyond them are dropped by the
      // bounds check, and the only per-store address arithmetic is one add on the running byte offset
      const int col = cur.n0 + wn * 64 + l16 * 4;
      if (col < N) {
        const int tile_rows = min(rows - cur.m0, BM), tile_cols = min(N - cur.n0, kPBN);
        // Blocked C (one group, n a multiple of 256, whole tiles of rows allocated): the tile's four 64-column blocks
        // of [256 rows][128 bytes] follow each other; rows beyond the valid count are written too (gelu(bias) of zero
        // rows), so that a consumer may read whole tiles.
        _Float16* cbase = args.c_blocked ? (_Float16*)args.C + (size_t)cur.m0 * args.ldc + (size_t)cur.n0 * kPBM
                                         : (_Float16*)args.C + (size_t)cur.m0 * args.ldc + (size_t)cur.grp * N + cur.n0;
        const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(
            cbase, 0, args.c_blocked ? kPBM * kPBN * 2 : ((tile_rows - 1) * args.ldc + tile_cols) * 2, 0x00020000);
        const uint32_t row_bytes = args.c_blocked ? 128u : (uint32_t)args.ldc * 2u;
        uint32_t voff = args.c_blocked
                            ? (uint32_t)wn * (uint32_t)kQAPair + (uint32_t)(wm * 16 * MI + g * 4) * 128u + (uint32_t)l16 * 8u
                            : ((uint32_t)(wm * 16 * MI + g * 4) * (uint32_t)args.ldc + (uint32_t)(wn * 64 + l16 * 4)) * 2u;
        // the offset is the same for every tile; the empty asm keeps the compiler from computing all 32 store offsets
        // once and holding them in registers across the k loop
        asm volatile("" : "+v"(voff));
        // bias added in half on the rounded product, as the reference's next kernel does; without a bias the addend is
        // -0, which leaves every value (and the sign of a zero) as it is
        half4 bias4 = {(_Float16)-0.0f, (_Float16)-0.0f, (_Float16)-0.0f, (_Float16)-0.0f};
        if (args.bias[cur.grp] != nullptr) bias4 = *reinterpret_cast<const half4*>((const _Float16*)args.bias[cur.grp] + col);
#pragma unroll
        for (int i = 0; i < MI; ++i) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            half4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = f2h(acc[i][j][r]);
            // GELU here costs no pass over C: its arithmetic runs while the stores of the tile drain
            o = GELU ? bias_gelu_half<half4, 4>(o, bias4) : o + bias4;
            __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(uint2v, o), rc, voff, 0, NT ? 2 /* nt */ : 0);
            voff += row_bytes;
          }
          voff += 12u * row_bytes;
        }
      }
    }
    if (!has_next) break;
    idx = nidx;
    cur = nxt;
    first_tile = false;
  }
  wait_vmcnt<0>();                               // no DMA may still target this workgroup's LDS when it ends
#else
  (void)args;
#endif
}

// ------------------------------------------------------------------------------------------
// fp16, problems below the persistent regime, B k-contiguous ([n][k]): one (32 MI) x (32 NJ) tile per workgroup,
// 4 wavefronts (2 x 2), LDS slots of two k-steps like the persistent kernel above.  MI = 1 .. 4 blocks of 32 rows,
// NJ = 2, 4, 6 or 8 blocks of 32 columns.
//
// With the weights in TF's [k][n] order a small tile reads its B operands with 8-byte LDS reads (half the rate of
// 16-byte ones) and transposes them in registers, and its A rows arrive in 64-byte pieces; a 64 x 128 tile then spends
// about three times as long on LDS traffic, transposes and DMA issue as on its 8 MFMAs per k-step, with one wavefront
// per SIMD and nothing to overlap them with.  Here both operands are rows of 64 k = 128 bytes (full cache lines for the
// DMA), every operand read is one 16-byte read per 16 x 32 block, and there are no transposes.  The ring holds ST slots;
// the schedule is the persistent kernel's: even k-step, barrier, odd k-step with this wave's DMA for the pair ST ahead.
// ------------------------------------------------------------------------------------------
template <int MI, int NJ, int ST>
struct BtTile {
  static constexpr int BM = 32 * MI, BN = 32 * NJ;
  static constexpr int A_BYTES = BM * 128;
  static constexpr int SLOT_BYTES = (BM + BN) * 128;
  static constexpr int SMEM_BYTES = ST * SLOT_BYTES;
  static constexpr int DMA = MI + NJ;                         // instructions per wavefront and pair: MI for A, NJ for B^T
};

template <int MI, int NJ, int ST>
__global__ __launch_bounds__(kHThreads) __attribute__((amdgpu_waves_per_eu(2))) void gemm_f16_bt_kernel(GemmArgs args) {
#if defined(__HIP_DEVICE_COMPILE__)   // device-only types in the body; the host pass only needs the stub
  using Tile = BtTile<MI, NJ, ST>;
  static_assert(Tile::DMA * (ST - 1) < 64, "the DMA instructions in flight must fit the 6-bit vmcnt");
  using HalfN = typename std::conditional<NJ == 8, half8, typename std::conditional<NJ == 4, half4, half2v>::type>::type;
  constexpr int BM = Tile::BM, BN = Tile::BN, WC = 16 * NJ;       // WC: columns of a wave tile
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int rows = args.rows_dev ? min(*args.rows_dev, args.m_bound) : args.m_bound;
  const int tiles_n_all = args.tiles_n * args.groups;
  const int tile = remap_valid_tile(blockIdx.x, ((rows + BM - 1) / BM) * tiles_n_all);
  if (tile < 0) return;
  const int tm = tile / tiles_n_all;
  const int tn_all = tile - tm * tiles_n_all;
  const int grp = tn_all / args.tiles_n;
  const int m0 = tm * BM;
  const int n0 = (tn_all - grp * args.tiles_n) * BN;
  const int N = args.n, K = args.k;
  const int np = K / 64;                                          // pairs of k-steps

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);   // scalar: LDS targets of the DMA are SALU values
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, g = lane >> 4;

  // descriptors start at the tile and end with the matrix: rows at or beyond the valid-token count and columns at or
  // beyond n read as zero, and lane offsets do not grow with the matrices
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16*>((const _Float16*)args.A[grp] + (size_t)m0 * K), 0, min(rows - m0, BM) * K * 2, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16*>((const _Float16*)args.B[grp] + (size_t)n0 * K), 0, min(N - n0, BN) * K * 2, 0x00020000);

  // DMA: one instruction fills 1 KB of LDS = 8 rows x 128 bytes; the lane picks the 16-byte chunk that belongs at its
  // (XOR-swizzled) position.  LDS row j*16+l of a wave's column group holds column NJ*l+j of the group, so that the
  // operand reads of B^T look like A's and a lane owns NJ consecutive columns of C (NJ = 6: four consecutive columns
  // among the first 64 of the group and two among the last 32, for aligned 8- and 4-byte stores).
  uint32_t voff_a[MI], voff_b[NJ];
#pragma unroll
  for (int j = 0; j < MI; ++j) {
    const int row = wave * (8 * MI) + j * 8 + (lane >> 3);
    voff_a[j] = ((uint32_t)row * (uint32_t)K + (uint32_t)((lane & 7) ^ pair_swizzle(row)) * 8u) * 2u;
  }
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int row = wave * (8 * NJ) + j * 8 + (lane >> 3);
    const int jb = (row % WC) >> 4;                                 // 16-row block of the wave's column group
    const int col = (row / WC) * WC + (NJ != 6 ? (row & 15) * NJ + jb : jb < 4 ? (row & 15) * 4 + jb : 64 + (row & 15) * 2 + jb - 4);
    voff_b[j] = ((uint32_t)col * (uint32_t)K + (uint32_t)((lane & 7) ^ pair_swizzle(row)) * 8u) * 2u;
  }
  // instruction q (0..MI-1: A, MI..: B^T) of this wave's share of pair `pr` into slot `slot`; pairs past the end
  // re-load the last one (never used; keeps the DMA count uniform)
  auto issue1 = [&](int slot, int pr, int q) {
    unsigned char* st = smem + slot * Tile::SLOT_BYTES;
    const int koff = min(pr, np - 1) * 128;
    if (q < MI)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, ET_LDS_PTR(st + (wave * MI + q) * 1024), 16, voff_a[q], koff, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, ET_LDS_PTR(st + Tile::A_BYTES + (wave * NJ + q - MI) * 1024), 16,
                                               voff_b[q - MI], koff, 0, 0);
  };

  // operand reads: row (wm*16*MI + i*16 + l16) resp. (wn*WC + j*16 + l16), chunk (4*half + g), swizzled
  const int sw = pair_swizzle(l16);
  const int a_rd[2] = {(wm * 16 * MI + l16) * 128 + ((g ^ sw) * 16), (wm * 16 * MI + l16) * 128 + (((4 + g) ^ sw) * 16)};
  const int b_rd[2] = {Tile::A_BYTES + (wn * WC + l16) * 128 + ((g ^ sw) * 16),
                       Tile::A_BYTES + (wn * WC + l16) * 128 + (((4 + g) ^ sw) * 16)};

  float4v acc[MI][NJ];
  half8 a[2][MI], b[2][NJ];

  // One k-step: MFMAs on operand set P; half 1-P of slot `rs` is read into the other set (B^T blocks first: the first
  // MFMAs of the next step need all of them); with DMA set, this wave's instructions for pair `dpr` go into slot `ds`.
  auto step = [&](auto Pc, auto FIRSTc, auto DMAc, int rs, int ds, int dpr) {
    constexpr int P = decltype(Pc)::value;
    constexpr bool FIRST = decltype(FIRSTc)::value;
    constexpr bool DMA = decltype(DMAc)::value;
    constexpr int rh = 1 - P;                    // the even step reads half 1 of its own pair, the odd step half 0 of the next
    constexpr int kRpg = (MI + NJ + MI - 1) / MI, kDpg = (Tile::DMA + MI - 1) / MI;
    const unsigned char* ns = smem + rs * Tile::SLOT_BYTES;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
      for (int r = i * kRpg; r < (i + 1) * kRpg && r < MI + NJ; ++r) {
        if (r < NJ) b[1 - P][r] = *reinterpret_cast<const half8*>(ns + b_rd[rh] + r * 2048);
        else a[1 - P][r - NJ] = *reinterpret_cast<const half8*>(ns + a_rd[rh] + (r - NJ) * 2048);
      }
#pragma unroll
      for (int j = 0; j < NJ; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[P][i], b[P][j],
                                                           FIRST ? float4v{0.f, 0.f, 0.f, 0.f} : acc[i][j], 0, 0, 0);
      if (DMA) {
#pragma unroll
        for (int q = i * kDpg; q < (i + 1) * kDpg && q < Tile::DMA; ++q) issue1(ds, dpr, q);
      }
      __builtin_amdgcn_sched_barrier(0);         // keeps the reads and the DMA where they are between the MFMA groups
    }
  };
  using Even = std::integral_constant<int, 0>;
  using Odd = std::integral_constant<int, 1>;

#pragma unroll
  for (int s = 0; s < ST; ++s)
#pragma unroll
    for (int q = 0; q < Tile::DMA; ++q) issue1(s, s, q);
  wait_vmcnt<Tile::DMA * (ST - 1)>();
  barrier_only();
#pragma unroll
  for (int j = 0; j < NJ; ++j) b[0][j] = *reinterpret_cast<const half8*>(smem + b_rd[0] + j * 2048);
#pragma unroll
  for (int i = 0; i < MI; ++i) a[0][i] = *reinterpret_cast<const half8*>(smem + a_rd[0] + i * 2048);

  int s = 0;                                     // slot of pair p
  for (int p = 0; p < np; ++p) {
    if (p == 0) step(Even{}, std::true_type{}, std::false_type{}, s, 0, 0);
    else step(Even{}, std::false_type{}, std::false_type{}, s, 0, 0);
    wait_vmcnt<Tile::DMA * (ST - 2)>();          // this wave's share of pair p+1 has landed; the ST - 2 behind it may fly
    wait_lgkmcnt0();                             // its last reads of slot s, which feed the odd step, are complete
    barrier_only();
    const int s1 = s + 1 == ST ? 0 : s + 1;
    step(Odd{}, std::false_type{}, std::true_type{}, s1, s, p + ST);      // pair p+ST replaces slot s
    s = s1;
  }
  wait_vmcnt<0>();                               // no DMA may still target this workgroup's LDS when it ends

  // epilogue: lane owns rows g*4+r of every 16-row block and NJ consecutive columns.  Plain stores, not the
  // non-temporal ones of the persistent kernel: the output of a launch this small is still in the caches when the
  // next kernel reads it (12 layers on 2000 tokens: 0.905 -> 0.843 ms; no difference from about 4000 tokens on).
  const int col = n0 + wn * WC + l16 * (NJ == 6 ? 4 : NJ);
  if (col < N) {
    _Float16* C = (_Float16*)args.C + (size_t)grp * N + col;
    if constexpr (NJ == 2 || NJ == 4 || NJ == 8) {
      // bias added in half on the rounded product, as the reference's next kernel does; without a bias the addend is
      // -0, which leaves every value (and the sign of a zero) as it is
      HalfN biasv;
#pragma unroll
      for (int j = 0; j < NJ; ++j) biasv[j] = (_Float16)-0.0f;
      if (args.bias[grp] != nullptr) biasv = *reinterpret_cast<const HalfN*>((const _Float16*)args.bias[grp] + col);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = m0 + wm * 16 * MI + i * 16 + g * 4 + r;
          if (row < rows) {
            HalfN o;
#pragma unroll
            for (int j = 0; j < NJ; ++j) o[j] = f2h(acc[i][j][r]);
            o = args.gelu ? bias_gelu_half<HalfN, NJ>(o, biasv) : o + biasv;
            *reinterpret_cast<HalfN*>(C + (size_t)row * args.ldc) = o;
          }
        }
    } else {
      // 6 columns per lane: 4 consecutive ones in the first 64 columns of the wave tile, 2 in the last 32
      static_assert(NJ == 6, "wave tiles are 32, 64, 96 or 128 columns wide");
      _Float16* C2 = C - col + n0 + wn * WC + 64 + l16 * 2;
      half4 bias4 = {(_Float16)-0.0f, (_Float16)-0.0f, (_Float16)-0.0f, (_Float16)-0.0f};
      half2v bias2 = {(_Float16)-0.0f, (_Float16)-0.0f};
      const bool ok2 = n0 + wn * WC + 64 + l16 * 2 < N;
      if (args.bias[grp] != nullptr) {
        bias4 = *reinterpret_cast<const half4*>((const _Float16*)args.bias[grp] + col);
        if (ok2) bias2 = *reinterpret_cast<const half2v*>((const _Float16*)args.bias[grp] + n0 + wn * WC + 64 + l16 * 2);
      }
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = m0 + wm * 16 * MI + i * 16 + g * 4 + r;
          if (row < rows) {
            half4 o4 = {f2h(acc[i][0][r]), f2h(acc[i][1][r]), f2h(acc[i][2][r]), f2h(acc[i][3][r])};
            half2v o2 = {f2h(acc[i][4][r]), f2h(acc[i][5][r])};
            o4 = args.gelu ? bias_gelu_half<half4, 4>(o4, bias4) : o4 + bias4;
            o2 = args.gelu ? bias_gelu_half<half2v, 2>(o2, bias2) : o2 + bias2;
            *reinterpret_cast<half4*>(C + (size_t)row * args.ldc) = o4;
            if (ok2) *reinterpret_cast<half2v*>(C2 + (size_t)row * args.ldc) = o2;
          }
        }
    }
  }
#else
  (void)args;
#endif
}

// ------------------------------------------------------------------------------------------
// fp32: 128x128x16 tile, 4 wavefronts (2x2) of 64x64, v_mfma_f32_32x32x2_f32
// ------------------------------------------------------------------------------------------
constexpr int kFThreads = 256;
constexpr int kFBK = 16;
[[maybe_unused]] constexpr int kFAStride = kFBK + 4;       // floats; 80-byte rows

// WB = 32x32 MFMA blocks per wavefront and dimension: 2 -> 128x128 tile, 1 -> 64x64 tile (problems of less than a
// round of 128x128 tiles, where the time is the k loop of one tile: a quarter of the MFMAs per k-step)
template <int WB>
__global__ __launch_bounds__(kFThreads, 4) void gemm_f32_kernel(GemmArgs args) {
#if defined(__HIP_DEVICE_COMPILE__)   // device-only types in the body; the host pass only needs the stub
  constexpr int kFBM = 64 * WB, kFBN = 64 * WB;
  constexpr size_t kFABytes = (size_t)kFBM * kFAStride * 4;
  constexpr size_t kFBBytes = (size_t)kFBK * kFBN * 4;
  constexpr size_t kFStage = kFABytes + kFBBytes;
  constexpr int kBc4 = kFBN / 4;            // 16-byte pieces per k-row of the B tile
  constexpr int kBRows = kFThreads / kBc4;  // k-rows one pass of the workgroup covers
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * kFStage];
  const int rows = args.rows_dev ? min(*args.rows_dev, args.m_bound) : args.m_bound;
  const int tiles_n_all = args.tiles_n * args.groups;
  const int tile = remap_valid_tile(blockIdx.x, ((rows + kFBM - 1) / kFBM) * tiles_n_all);
  if (tile < 0) return;
  const int tm = tile / tiles_n_all;
  const int tn_all = tile - tm * tiles_n_all;
  const int grp = tn_all / args.tiles_n;
  const int tn = tn_all - grp * args.tiles_n;
  const int m0 = tm * kFBM;
  const int n0 = tn * kFBN;
  const int N = args.n, K = args.k;
  // Loads go through buffer descriptors: rows at or beyond the valid count and columns at or beyond n read as zero
  // without a branch, so every k-step issues the same number of loads and the waits can count them.
  __amdgpu_buffer_rsrc_t rsrc_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(args.A[grp]), 0, (int)((uint32_t)rows * K * 4u), 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_b =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(args.B[grp]), 0, (int)((uint32_t)K * N * 4u), 0x00020000);

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, kb = lane >> 5;

  // Global -> registers -> LDS.  The 64 x 64 tile runs where few workgroups are resident and nothing else hides the
  // latency of a global load, so its k-steps are requested kDepth steps ahead (a ring of register sets); the big tile
  // has three wavefronts per SIMD for that and keeps one set.
  constexpr int kDepth = WB == 1 ? 4 : 2;
  u32x4 ring_a[kDepth][WB], ring_b[kDepth][WB];
  const int a_kc = tid & 3, a_row = tid >> 2;                // + u*64
  const int b_nc = tid % kBc4, b_krow = tid / kBc4;          // + u*kBRows
  const bool b_col_ok = n0 + b_nc * 4 < N;
  // offset of a lane whose columns do not exist: beyond any B this kernel accepts (k*n*4 < 2 GB) and far enough from
  // 2^32 that offset + access size cannot wrap, so the range check zero-fills it
  constexpr uint32_t kBeyondB = 0x80000000u;
  uint32_t a_off[WB], b_off[WB];      // byte offsets of this thread's pieces at k = 0; the range check looks at these
#pragma unroll
  for (int u = 0; u < WB; ++u) {
    a_off[u] = ((uint32_t)(m0 + a_row + u * 64) * (uint32_t)K + (uint32_t)a_kc * 4u) * 4u;
    b_off[u] = ((uint32_t)(b_krow + u * kBRows) * (uint32_t)N + (uint32_t)(n0 + b_nc * 4)) * 4u;
  }
  const int nk = K / kFBK;

  auto load_global = [&](int kt, u32x4 (&ra)[WB], u32x4 (&rb)[WB]) {
    const int k0 = min(kt, nk - 1) * kFBK;    // past the end: the last k-step again (never used; keeps the load count uniform)
#pragma unroll
    for (int u = 0; u < WB; ++u) {
      ra[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, a_off[u], k0 * 4, 0));
      const uint32_t off = b_col_ok ? b_off[u] + (uint32_t)k0 * (uint32_t)N * 4u : kBeyondB;
      rb[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, off, 0, 0));
    }
  };
  auto store_lds = [&](int stage, const u32x4 (&ra)[WB], const u32x4 (&rb)[WB]) {
    float* As = reinterpret_cast<float*>(smem + stage * kFStage);
    float* Bs = reinterpret_cast<float*>(smem + stage * kFStage + kFABytes);
#pragma unroll
    for (int u = 0; u < WB; ++u) {
      *reinterpret_cast<u32x4*>(As + (a_row + u * 64) * kFAStride + a_kc * 4) = ra[u];
      *reinterpret_cast<u32x4*>(Bs + (b_krow + u * kBRows) * kFBN + b_nc * 4) = rb[u];
    }
  };

  float16v acc[WB][WB];
#pragma unroll
  for (int i = 0; i < WB; ++i)
#pragma unroll
    for (int j = 0; j < WB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

#pragma unroll
  for (int d = 0; d < kDepth; ++d) load_global(d, ring_a[d], ring_b[d]);
  store_lds(0, ring_a[0], ring_b[0]);
  load_global(kDepth, ring_a[0], ring_b[0]);
  __syncthreads();
  for (int kt0 = 0; kt0 < nk; kt0 += kDepth) {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      const int kt = kt0 + d;
      if (kt >= nk) break;
      const float* As = reinterpret_cast<const float*>(smem + (kt & 1) * kFStage);
      const float* Bs = reinterpret_cast<const float*>(smem + (kt & 1) * kFStage + kFABytes);
      // step s of the stage contracts k = kb*8 + s (the same choice for A and B)
      float a[WB][8], b[WB][8];
#pragma unroll
      for (int i = 0; i < WB; ++i) {
        const float* ap = As + (wm * 32 * WB + i * 32 + l32) * kFAStride + kb * 8;
        const float4v a0 = *reinterpret_cast<const float4v*>(ap);
        const float4v a1 = *reinterpret_cast<const float4v*>(ap + 4);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          a[i][s] = a0[s];
          a[i][4 + s] = a1[s];
        }
      }
#pragma unroll
      for (int j = 0; j < WB; ++j)
#pragma unroll
        for (int s = 0; s < 8; ++s) b[j][s] = Bs[(kb * 8 + s) * kFBN + wn * 32 * WB + j * 32 + l32];
#pragma unroll
      for (int s = 0; s < 8; ++s)
#pragma unroll
        for (int i = 0; i < WB; ++i)
#pragma unroll
          for (int j = 0; j < WB; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][s], b[j][s], acc[i][j], 0, 0, 0);
      // k-step kt+1 sits in ring slot (kt+1) % kDepth = (d+1) % kDepth; once it is in LDS the slot takes k-step kt+1+kDepth
      store_lds((kt + 1) & 1, ring_a[(d + 1) % kDepth], ring_b[(d + 1) % kDepth]);
      load_global(kt + 1 + kDepth, ring_a[(d + 1) % kDepth], ring_b[(d + 1) % kDepth]);
      __syncthreads();
    }
  }

#pragma unroll
  for (int j = 0; j < WB; ++j) {
    const int col = n0 + wn * 32 * WB + j * 32 + l32;
    if (col >= N) continue;
    const float bias = args.bias[grp] ? ((const float*)args.bias[grp])[col] : 0.f;
    float* C = (float*)args.C + (size_t)grp * N + col;
#pragma unroll
    for (int i = 0; i < WB; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 32 * WB + i * 32 + 8 * (r >> 2) + 4 * kb + (r & 3);
        if (row < rows) {
          const float x = acc[i][j][r] + bias;
          C[(size_t)row * args.ldc] = args.gelu ? x * gelu_cdf(x, x * x * x) : x;
        }
      }
  }
#else
  (void)args;
#endif
}

template <int MI, int NJ>
void launch_f16(GemmArgs a, hipStream_t stream) {
  using Tile = HTile<MI, NJ>;
  auto kern = gemm_f16_kernel<MI, NJ>;
  allow_dynamic_lds(reinterpret_cast<const void*>(kern), (int)Tile::SMEM_BYTES);
  a.tiles_m = (a.m_bound + Tile::BM - 1) / Tile::BM;
  a.tiles_n = (a.n + Tile::BN - 1) / Tile::BN;
  const int total = a.tiles_m * a.tiles_n * a.groups;
  a.per_xcd = (total + kXcds - 1) / kXcds;
  kern<<<a.per_xcd * kXcds, kHThreads, Tile::SMEM_BYTES, stream>>>(a);
}

template <int MI, int NJ, int ST>
void launch_f16_bt(GemmArgs a, hipStream_t stream) {
  using Tile = BtTile<MI, NJ, ST>;
  auto kern = gemm_f16_bt_kernel<MI, NJ, ST>;
  allow_dynamic_lds(reinterpret_cast<const void*>(kern), (int)Tile::SMEM_BYTES);
  a.tiles_m = (a.m_bound + Tile::BM - 1) / Tile::BM;
  a.tiles_n = (a.n + Tile::BN - 1) / Tile::BN;
  const int total = a.tiles_m * a.tiles_n * a.groups;
  a.per_xcd = (total + kXcds - 1) / kXcds;
  kern<<<a.per_xcd * kXcds, kHThreads, Tile::SMEM_BYTES, stream>>>(a);
}

int device_cu_count() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cus[kMaxDevices] = {};      // handles on several GPUs may launch from different threads
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int n = cus[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    hipDeviceProp_t prop;
    n = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Rows per tile of the k-contiguous persistent kernel, as the count MI of 16-row blocks per wave (tile = 32 MI rows).
// A launch takes rounds x tile time, and the last round of a band of tiles (one XCD, cus / 8 workgroups) is often far
// from full; a lower tile can then do with fewer rounds, or with a shorter single round: 13097 rows x 768 columns are
// 156 tiles of 256 rows, one round on 61 % of the CUs, or 246 tiles of 160 rows, one round on 96 % of them.  The time
// of a tile falls much more slowly than its height (the B^T half of the operand stream, the DMA and the LDS traffic
// stay): measured about 1.45 us per pair of k-steps at 256 rows and 1.3 us at 160, i.e. proportional to MI + 21.  A
// lower tile must win 3 % by that estimate (measured: FFN-down of 13097 rows 75 -> 64 us, of 15866 rows 76 -> 70 us,
// attention-out 26 -> 24 us; the 13097 x 1024 one of BERT-large 35 -> 31.5 us; all with the same bits).
int pair_kernel_row_blocks(int m_bound, int n, int groups) {
  const int cus = device_cu_count();
  const int wgs = std::max(1, cus / kXcds);
  const int tiles_n = (n + kPBN - 1) / kPBN * groups;
  auto cost = [&](int mi) {
    const long tiles = (long)((m_bound + 32 * mi - 1) / (32 * mi)) * tiles_n;
    const long n_loc = (tiles + kXcds - 1) / kXcds;
    const long full = n_loc / wgs, rem = n_loc % wgs;
    // a rest of at most half the workgroups is shared, two workgroups per tile
    const double rounds = (double)full + (rem == 0 ? 0.0 : (2 * rem <= wgs ? 0.55 : 1.0));
    return rounds * (mi + 21);
  };
  const double cost8 = cost(8);
  double best = cost8;
  int best_mi = 8;
  for (int mi = 7; mi >= 5; --mi) {
    const double c = cost(mi);
    if (c < 0.97 * cost8 && c < best) {
      best = c;
      best_mi = mi;
    }
  }
  return best_mi;
}

template <bool GELU, int MI, bool NT, bool A3 = false>
void launch_pair(const GemmArgs& a, int grid, hipStream_t stream) {
  auto kern = gemm_f16_pair_kernel<GELU, MI, NT, A3>;
  constexpr int lds = A3 ? kQSmemA3 : kQSmem;
  allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds);
  kern<<<grid, kPThreads, lds, stream>>>(a);
}

void launch_f16_persistent(GemmArgs a, hipStream_t stream, bool b_transposed) {
  // the blocked hand-over is laid out for tiles of 256 rows
  const int mi = !b_transposed || a.a_blocked || a.c_blocked ? 8 : pair_kernel_row_blocks(a.m_bound, a.n, a.groups);
  const int bm = 32 * mi;
  a.tiles_m = (a.m_bound + bm - 1) / bm;
  a.tiles_n = (a.n + kPBN - 1) / kPBN;
  const int total = a.tiles_m * a.tiles_n * a.groups;
  int grid = std::min(device_cu_count(), total);
  grid = (grid + kXcds - 1) / kXcds * kXcds;
  a.per_xcd = 0;     // derived on the device from the valid row count
  // k > n: A is the big operand and was written front to back by the kernel before this one, so its last rows are the
  // ones most likely still in the last-level cache: walk the tiles from the end
  a.reverse_walk = a.k > a.n ? 1 : 0;
  // A weight matrix that does not fit an XCD's 4 MB L2 beside the A rows passing through is streamed from the
  // last-level cache again for every few row tiles of every band (FFN-up of BERT-base: 373 MiB read per launch for 64
  // MiB of operands).  Where the output is wide (n >= 2 k: A is the small operand), the tile order therefore runs
  // through the column tiles in groups whose weight slice stays in the L2 (at most 2.5 MB, at least 3 column tiles), at
  // the price of reading A once per group: 241 MiB per launch there, 290 -> 170 MiB for BERT-large's FFN-up; the
  // launches themselves gain about 1 %.
  a.col_groups = 1;
  {
    const int tn = a.tiles_n * a.groups;
    const double w_bytes = (double)a.n * a.groups * a.k * 2.0;
    if (b_transposed && (long)a.n * a.groups >= 2L * a.k && w_bytes > 4.0 * 1048576.0)
      for (int cg = 2; cg <= tn / 3; ++cg)
        if (tn % cg == 0 && w_bytes / cg <= 2.5 * 1048576.0) {
          a.col_groups = cg;
          break;
        }
  }
  if (!b_transposed) {
    allow_dynamic_lds(reinterpret_cast<const void*>(gemm_f16_persistent_kernel), kPSmem);
    gemm_f16_persistent_kernel<<<grid, kPThreads, kPSmem, stream>>>(a);
    return;
  }
  // A from HBM, few long tiles per workgroup: the A rows are requested a pair earlier (three LDS slots for A)
  if (!a.gelu && a.k >= 2048 && mi >= 7) {
    if (mi == 8 && !a.c_cached) launch_pair<false, 8, true, true>(a, grid, stream);
    else if (mi == 8) launch_pair<false, 8, false, true>(a, grid, stream);
    else if (!a.c_cached) launch_pair<false, 7, true, true>(a, grid, stream);
    else launch_pair<false, 7, false, true>(a, grid, stream);
    return;
  }
#define ET_PAIR_CASE(M)                                                      \
  case M:                                                                    \
    if (a.gelu && a.c_cached) launch_pair<true, M, false>(a, grid, stream);  \
    else if (a.gelu) launch_pair<true, M, true>(a, grid, stream);            \
    else if (a.c_cached) launch_pair<false, M, false>(a, grid, stream);      \
    else launch_pair<false, M, true>(a, grid, stream);                       \
    break;
  switch (mi) {
    ET_PAIR_CASE(8)
    ET_PAIR_CASE(7)
    ET_PAIR_CASE(6)
    ET_PAIR_CASE(5)
  }
#undef ET_PAIR_CASE
}

// Tile of the one-tile-per-workgroup k-contiguous kernel.  A workgroup's k loop runs at the rate its CU's load path
// delivers operand rows, MI + NJ units of 4 KB per pair of k-steps, so the launch takes about as long as the busiest
// CU's units: the smallest tile that still gives every workgroup a CU to itself ("solo", ring of 3 to 5 slots), or
// two workgroups per CU ("duo", rings that fit twice into the LDS) where 2 (MI + NJ) / 1.3 is less: two resident
// workgroups draw 1.3 times the rows of one.  A 96-column wave tile stores in two pieces and counts one unit more.
// Ties go to the tile whose XCD bands touch fewer distinct operand rows.  (Timed for n = 768 .. 4096, k = 768 .. 4096,
// 250 .. 16000 rows with the weights of twelve layers taking turns: within 2 % of the best tile on average.)
struct BtPick {
  int mi = 0, nj = 0;      // mi == 0: no tile keeps the launch within two workgroups per CU
  bool duo = false;
};

BtPick pick_bt_tile(int m_bound, int n, int groups, int cus, bool proven_only) {
  BtPick best;
  float best_cost = 0.f;
  long best_band = 0;
  // (the other combinations of 1 .. 4 row blocks and 2 .. 8 column blocks never come out ahead of these)
  static constexpr struct { int mi, nj; bool duo; } kTiles[] = {{1, 2, true}, {2, 2, true}, {2, 4, true}, {3, 2, true},
                                                                 {3, 4, true}, {3, 6, true}, {4, 2, true}, {4, 4, true},
                                                                 {4, 6, true}, {4, 8, false}};
  for (const auto& tile : kTiles) {
    const int mi = tile.mi, nj = tile.nj;
    const long tiles_n = (long)((n + 32 * nj - 1) / (32 * nj)) * groups;
    const long wgs = (long)((m_bound + 32 * mi - 1) / (32 * mi)) * tiles_n;
    const float units = (float)(mi + nj + (nj == 6 ? 1 : 0));
    float cost;
    bool duo = false;
    if (wgs <= cus) {
      cost = units;
    } else if (wgs <= 2L * cus && tile.duo && !(proven_only && nj > 4)) {
      cost = 2.f * units / 1.3f;
      duo = true;
    } else {
      continue;
    }
    // distinct operand rows (of A and of B^T) that the tiles of one XCD's band touch: what its L2 has to fetch
    const long per_band = (wgs + kXcds - 1) / kXcds;
    const long band = (per_band >= tiles_n ? (per_band + tiles_n - 1) / tiles_n : 1) * 32 * mi +
                      std::min(per_band, tiles_n) * 32 * nj;
    if (best.mi == 0 || cost < best_cost || (cost == best_cost && band < best_band)) {
      best.mi = mi;
      best.nj = nj;
      best.duo = duo;
      best_cost = cost;
      best_band = band;
    }
  }
  return best;
}

void launch_bt_tile(BtPick p, const GemmArgs& a, hipStream_t stream) {
  switch (p.mi * 100 + p.nj * 10 + (p.duo ? 1 : 0)) {
    case 120: return launch_f16_bt<1, 2, 5>(a, stream);
    case 121: return launch_f16_bt<1, 2, 3>(a, stream);
    case 220: return launch_f16_bt<2, 2, 4>(a, stream);
    case 221: return launch_f16_bt<2, 2, 3>(a, stream);
    case 240: return launch_f16_bt<2, 4, 4>(a, stream);
    case 241: return launch_f16_bt<2, 4, 3>(a, stream);
    case 320: return launch_f16_bt<3, 2, 4>(a, stream);
    case 321: return launch_f16_bt<3, 2, 3>(a, stream);
    case 340: return launch_f16_bt<3, 4, 4>(a, stream);
    case 341: return launch_f16_bt<3, 4, 2>(a, stream);
    case 360: return launch_f16_bt<3, 6, 3>(a, stream);
    case 361: return launch_f16_bt<3, 6, 2>(a, stream);
    case 420: return launch_f16_bt<4, 2, 4>(a, stream);
    case 421: return launch_f16_bt<4, 2, 3>(a, stream);
    case 440: return launch_f16_bt<4, 4, 4>(a, stream);
    case 460: return launch_f16_bt<4, 6, 3>(a, stream);
    case 461: return launch_f16_bt<4, 6, 2>(a, stream);
    case 480: return launch_f16_bt<4, 8, 3>(a, stream);
    default: return launch_f16_bt<4, 4, 2>(a, stream);     // 128 x 128 in rounds of two workgroups per CU
  }
}

// few big tiles would leave most of the 256 CUs idle: the persistent 256x256 kernel only runs when there is work
// for at least half of them; C is addressed with 32-bit byte offsets there
bool use_persistent(int m_bound, int ldc, int n, int k, int groups) {
  const long big = (long)((m_bound + 255) / 256) * ((n + 255) / 256) * groups;
  return big >= 128 && k >= 4 * kHBK && (uint64_t)m_bound * (uint64_t)ldc * 2u <= 0xffffffffull;
}

// With B k-contiguous, the one-tile-per-workgroup kernel is still the faster one where the launch fits a round of
// 128 x 256 tiles or two workgroups of 128 x 128 per CU (2000 rows at n = 4096, k = 1024: 21 us against 27; 8000 rows
// at n = 1024, k = 4096: 59 against 73); narrower duo tiles only tie with the persistent kernel there.
bool use_persistent_bt(int m_bound, int ldc, int n, int k, int groups) {
  return use_persistent(m_bound, ldc, n, k, groups) && pick_bt_tile(m_bound, n, groups, device_cu_count(), true).mi == 0;
}

// ------------------------------------------------------------------------------------------
// [k][n] -> [n][k] for fp16 weights: 64x64 tiles through LDS, 16-byte accesses on both sides.
// ------------------------------------------------------------------------------------------
struct TransposeArgs {
  TransposeJobs jobs;
  int tile_begin[TransposeJobs::kMax + 1];
  SeqStartJob seq;             // blocks from tile_begin[kMax] on build the sequence start table (seq_start != null)
};
constexpr int kTrTile = 64;
constexpr int kTrStride = kTrTile + 8;    // halves; 144-byte rows keep the 16-byte row reads aligned

__global__ __launch_bounds__(256) void layer_prologue_kernel(TransposeArgs args) {
  __shared__ __attribute__((aligned(16))) _Float16 tile[kTrTile * kTrStride];
  if ((int)blockIdx.x >= args.tile_begin[TransposeJobs::kMax]) {
    const int T = args.seq.rows_dev ? min(*args.seq.rows_dev, args.seq.rows_bound) : args.seq.rows_bound;
    seq_start_for_row(args.seq.batch_idx, T, ((int)blockIdx.x - args.tile_begin[TransposeJobs::kMax]) * 256 + threadIdx.x,
                      args.seq.batch, args.seq.seq_start);
    return;
  }
  int job = 0;
  while (job + 1 < args.jobs.count && (int)blockIdx.x >= args.tile_begin[job + 1]) ++job;
  const int K = args.jobs.k[job], N = args.jobs.n[job];
  const int tiles_n = (N + kTrTile - 1) / kTrTile;
  const int t = blockIdx.x - args.tile_begin[job];
  const int k0 = (t / tiles_n) * kTrTile, n0 = (t % tiles_n) * kTrTile;
  const _Float16* __restrict__ src = (const _Float16*)args.jobs.src[job];
  _Float16* __restrict__ dst = (_Float16*)args.jobs.dst[job];
  // 64 rows x 8 chunks of 8 halves: two chunks per thread
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int i = threadIdx.x + u * 256;
    const int r = i >> 3, c = i & 7;                  // source row k0+r, columns n0 + 8c ..
    half8 v = {};
    if (k0 + r < K && n0 + c * 8 < N) v = *reinterpret_cast<const half8*>(src + (size_t)(k0 + r) * N + n0 + c * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) tile[(c * 8 + j) * kTrStride + r] = v[j];
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int i = threadIdx.x + u * 256;
    const int r = i >> 3, c = i & 7;                  // destination row n0+r, columns k0 + 8c ..
    if (n0 + r < N && k0 + c * 8 < K)
      *reinterpret_cast<half8*>(dst + (size_t)(n0 + r) * K + k0 + c * 8) =
          *reinterpret_cast<const half8*>(tile + r * kTrStride + c * 8);
  }
}

}  // namespace

namespace {
// what the MFMA kernels take
bool gemm_tiled(DType t, int n, int k) {
  if (t == DType::F16) return k % kHBK == 0 && n % 8 == 0 && n >= 8;
  return k % kFBK == 0 && n % 4 == 0 && (uint64_t)k * (uint64_t)n * 4u < 0x80000000ull;
}
}  // namespace

bool gemm_takes_transposed_b(DType t, int m_bound, int ldc, int n, int k, int groups) {
  (void)m_bound; (void)ldc;
  return t == DType::F16 && gemm_supported(t, n, k, groups) && gemm_tiled(t, n, k) && k % 64 == 0 &&
         (uint64_t)k * 256u * 2u < 0x80000000ull;
}

bool gemm_blocked_handover(DType t, int m_bound, int wide, int narrow) {
  // ... and both would run on tiles of 256 rows anyway (a lower tile for one of them is worth more than the hand-over)
  return gemm_takes_transposed_b(t, m_bound, wide, wide, narrow, 1) && use_persistent_bt(m_bound, wide, wide, narrow, 1) &&
         gemm_takes_transposed_b(t, m_bound, narrow, narrow, wide, 1) && use_persistent_bt(m_bound, narrow, narrow, wide, 1) &&
         pair_kernel_row_blocks(m_bound, wide, 1) == 8 && pair_kernel_row_blocks(m_bound, narrow, 1) == 8 &&
         wide % kPBN == 0 && (uint64_t)((m_bound + kPBM - 1) / kPBM * kPBM) * (uint64_t)wide * 2u <= 0xffffffffull;
}

// Inside the layer a k-contiguous copy pays for itself at every batch size: copying all six kernels of a layer takes
// 5 .. 9 us in the launch that builds the sequence table anyway, and the kernels that read the copies (tile heights,
// ten small tiles, blocked hand-over, cached C) save more than that (12 layers of BERT-base on caller-owned weights:
// -6 % at 2000 tokens, -7 % at 12000, -2 % at 40000 against copying only Q, K, V and FFN-up for large batches).
bool gemm_prefers_transposed_b(DType t, int m_bound, int ldc, int n, int k, int groups) {
  return gemm_takes_transposed_b(t, m_bound, ldc, n, k, groups);
}

void launch_transpose_weights(const TransposeJobs& jobs, hipStream_t stream, const SeqStartJob* seq) {
  if (jobs.count == 0 && seq == nullptr) return;
  TransposeArgs a;
  a.jobs = jobs;
  int total = 0;
  for (int j = 0; j < jobs.count; ++j) {
    a.tile_begin[j] = total;
    total += ((jobs.k[j] + kTrTile - 1) / kTrTile) * ((jobs.n[j] + kTrTile - 1) / kTrTile);
  }
  for (int j = jobs.count; j <= TransposeJobs::kMax; ++j) a.tile_begin[j] = total;
  a.seq = seq ? *seq : SeqStartJob{nullptr, nullptr, 0, 0, nullptr};
  if (seq) total += (seq->rows_bound + 1 + 255) / 256;
  layer_prologue_kernel<<<total, 256, 0, stream>>>(a);
  if (seq) launch_seq_order(seq->seq_start, seq->batch, stream);
}

bool gemm_supported(DType t, int n, int k, int groups) {
  (void)t;
  return groups >= 1 && groups <= 3 && n > 0 && k > 0;
}

void launch_gemm(DType t, const GemmGroups& g, void* C, int ldc, int m_bound, int n, int k, const int32_t* rows_dev,
                 hipStream_t stream) {
  if (m_bound <= 0) return;
  if (!gemm_tiled(t, n, k)) {
    launch_gemm_generic(t, g, C, ldc, m_bound, n, k, rows_dev, stream);
    return;
  }
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
  a.gelu = g.gelu ? 1 : 0;
  a.a_blocked = g.a_blocked ? 1 : 0;
  a.c_blocked = g.c_blocked ? 1 : 0;
  a.c_cached = g.c_cached ? 1 : 0;
  if (t == DType::F16) {
    if (g.b_transposed ? use_persistent_bt(m_bound, ldc, n, k, g.groups)
                       : use_persistent(m_bound, ldc, n, k, g.groups)) {     // one workgroup per CU walks the tiles
      launch_f16_persistent(a, stream, g.b_transposed);
    } else if (g.b_transposed) {
      // one tile per workgroup, the tile chosen for the launch's shape (pick_bt_tile)
      const int cus = device_cu_count();
      launch_bt_tile(pick_bt_tile(m_bound, n, g.groups, cus, false), a, stream);
    } else {
      // Below a round of the chip the time of a launch is the k loop of one tile.  With fewer 64 x 256 tiles than CUs
      // that loop runs at the rate one CU's DMA fills its LDS: the 64 x 128 tile halves the B bytes per workgroup and
      // doubles the workgroups.  From there on the 128 x 256 tile is the faster one (measured at n = 768 .. 3072,
      // k = 768 and 3072; a 64 x 256 tile never won between the two).
      const long small = (long)((m_bound + 63) / 64) * ((n + 255) / 256) * g.groups;
      if (small <= device_cu_count()) launch_f16<2, 4>(a, stream);
      else launch_f16<4, 8>(a, stream);
    }
  } else {
    // less than a round of 128x128 tiles: 64x64 tiles finish their k loop four times sooner
    const long big = (long)((m_bound + 127) / 128) * ((n + 127) / 128) * g.groups;
    const int bt = big <= device_cu_count() ? 64 : 128;
    a.tiles_m = (m_bound + bt - 1) / bt;
    a.tiles_n = (n + bt - 1) / bt;
    const int total = a.tiles_m * a.tiles_n * a.groups;
    a.per_xcd = (total + kXcds - 1) / kXcds;
    if (bt == 64) gemm_f32_kernel<1><<<a.per_xcd * kXcds, kFThreads, 0, stream>>>(a);
    else gemm_f32_kernel<2><<<a.per_xcd * kXcds, kFThreads, 0, stream>>>(a);
  }
}

}  // namespace et
