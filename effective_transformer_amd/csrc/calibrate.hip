// Measurement aid, no part of the encoder path and no counterpart in the reference: the MFMA rate this GPU sustains
// under the instruction mix of the large fp16 GEMM's inner loop, with operands that are all zero or random halves.
//
// Every CU runs 8 wavefronts that repeat one k-step of a 128 x 64 wave tile: 32 v_mfma_f32_16x16x32_f16 on one operand
// register set while 12 ds_read_b128 refill the other set from LDS, as gemm_f16_pair_kernel does, with no global
// memory traffic, no barrier and nothing to wait for but the LDS.  The rate with zero operands is what instruction
// issue allows at the clock the part holds under that load; the rate with random operands is lower, because the
// switching activity of real data costs power and the part answers with a lower clock.  The second figure, not the
// data-sheet peak, is the ceiling a GEMM on real data runs under.
#include "et_device.hpp"
#include "kernels.hpp"

namespace et {

namespace {

constexpr int kCalThreads = 512;
constexpr int kCalLds = 32768 + 256;      // four 8 KB windows + room for the shifted reads of the last row

template <bool RANDOM>
__global__ __launch_bounds__(kCalThreads) void mfma_ceiling_kernel(float* __restrict__ sink, int iters) {
  __shared__ __attribute__((aligned(1024))) unsigned char smem[kCalLds];
  const int tid = threadIdx.x, lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  for (int i = tid; i < kCalLds / 4; i += kCalThreads) {
    uint32_t word = 0;
    if (RANDOM) {
      // two halves uniform in (-0.02, 0.02): small enough that 2^20 accumulated products stay finite
      const uint32_t h = (uint32_t)i * 2654435761u;
      const _Float16 lo = (_Float16)(((int)(h & 0xffff) - 32768) * (0.02f / 32768.f));
      const _Float16 hi = (_Float16)(((int)(h >> 16) - 32768) * (0.02f / 32768.f));
      word = (uint32_t)__builtin_bit_cast(unsigned short, lo) | ((uint32_t)__builtin_bit_cast(unsigned short, hi) << 16);
    }
    reinterpret_cast<uint32_t*>(smem)[i] = word;
  }
  __syncthreads();
  // operand rows of 128 bytes, 16-byte chunks XOR-swizzled by the row as in the GEMM (conflict-free reads); the eight
  // waves read four different 8 KB windows
  const int l16 = lane & 15, g = lane >> 4;
  const unsigned char* base = smem + (wave & 3) * 8192 + l16 * 128 + ((g ^ ((l16 >> 1) & 7)) * 16);
  half8 a[2][8], b[2][4];
  float4v acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[0][i] = *reinterpret_cast<const half8*>(base + (i & 3) * 2048);
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) b[0][j] = *reinterpret_cast<const half8*>(base + j * 2048 + 64);
#pragma unroll 1
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int P = 0; P < 2; ++P) {
      // the window moves with the step so that consecutive steps multiply different data
      const unsigned char* src = base + ((2 * it + P) & 1) * 64;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (i < 2) {
          b[1 - P][2 * i] = *reinterpret_cast<const half8*>(src + (2 * i) * 2048);
          b[1 - P][2 * i + 1] = *reinterpret_cast<const half8*>(src + (2 * i + 1) * 2048);
        } else if (i < 6) {
          a[1 - P][2 * (i - 2)] = *reinterpret_cast<const half8*>(src + ((2 * (i - 2)) & 3) * 2048 + 32);
          a[1 - P][2 * (i - 2) + 1] = *reinterpret_cast<const half8*>(src + ((2 * (i - 2) + 1) & 3) * 2048 + 32);
        }
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int j = (i & 1) ? 3 - jj : jj;       // back and forth, as in the GEMM: one operand changes per MFMA
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[P][i], b[P][j], acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) s += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  sink[(size_t)blockIdx.x * kCalThreads + tid] = s;
}

}  // namespace

size_t mfma_ceiling_sink_bytes(int cus) { return (size_t)cus * kCalThreads * sizeof(float); }

double launch_mfma_ceiling(bool random_operands, int cus, int iters, float* sink, hipStream_t stream) {
  if (random_operands) mfma_ceiling_kernel<true><<<cus, kCalThreads, 0, stream>>>(sink, iters);
  else mfma_ceiling_kernel<false><<<cus, kCalThreads, 0, stream>>>(sink, iters);
  // floating-point operations of the launch: workgroups x 8 waves x iters x 64 MFMAs x 2 * 16 * 16 * 32
  return (double)cus * 8.0 * (double)iters * 64.0 * 16384.0;
}

}  // namespace et
