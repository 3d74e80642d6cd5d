// Input / output side of the padding-free encoder on gfx950:
//   mask prefix sum + packed-token index build   (reference: cuda/cuda_kernels.cu:472-718,
//                                                 tf_op/bert_transformer_op.cu.cc:266-331)
//   compress [B,S,H] -> [T,H]                    (cuda/cuda_kernels.cu:278-384)
//   restore  [T,H]  -> [B,S,H] with zero fill    (cuda/cuda_kernels.cu:389-468,
//                                                 tf_op/bert_transformer_op.cu.cc:351-360)
// All of it is HBM-bound byte and integer work: the scan runs on 64-lane DPP prefix sums, the
// row movers use one 128-bit access per lane on a flattened (row, 16-byte chunk) index space so
// that every lane of every wavefront carries data.
#include <type_traits>

#include "et_device.hpp"
#include "kernels.hpp"

namespace et {

namespace {

constexpr int kScanThreads = 1024;     // one element per thread and tile step; 16 wavefronts share the front sum
constexpr int kScanWaves = kScanThreads / kWave;

inline int scan_tile_for(int length) {
  // at most 1024 tiles, so that one workgroup can reduce the tile totals in front of it
  int tile = 1024;
  long need = ((long)length + 1023) / 1024;
  if (need > tile) tile = (int)((need + kScanThreads - 1) / kScanThreads) * kScanThreads;
  return tile;
}

__device__ __forceinline__ int block_sum_i32(int v, int* lds /* >= kScanWaves ints */) {
  int w = wave_sum_i32(v);
  const int wave = threadIdx.x / kWave;
  __syncthreads();                       // protect lds from a previous use
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = w;
  __syncthreads();
  int total = 0;
#pragma unroll
  for (int i = 0; i < kScanWaves; ++i) total += lds[i];
  return total;
}

__global__ __launch_bounds__(kScanThreads) void scan_tile_sums_kernel(const int32_t* __restrict__ in, int n, int tile,
                                                                       int32_t* __restrict__ sums) {
  __shared__ int lds[kScanWaves];
  const int begin = blockIdx.x * tile;
  const int end = min(n, begin + tile);
  int acc = 0;
  for (int i = begin + threadIdx.x; i < end; i += kScanThreads) acc += in[i];
  int total = block_sum_i32(acc, lds);
  if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// One workgroup per tile: adds up the totals of the tiles in front of it, then walks its tile
// in steps of 256 elements with a DPP scan per wavefront.
__global__ __launch_bounds__(kScanThreads) void scan_index_kernel(const int32_t* __restrict__ in, int n, int tile,
                                                                   const int32_t* __restrict__ sums,
                                                                   int32_t* __restrict__ prefix_out,
                                                                   int32_t* __restrict__ batch_idx,
                                                                   int32_t* __restrict__ word_idx,
                                                                   int32_t* __restrict__ valid_word_num, int seq_len) {
  __shared__ int lds[kScanWaves];
  __shared__ int wave_tot[kScanWaves];
  int part = 0;
  if (sums) {
    for (int i = threadIdx.x; i < (int)blockIdx.x; i += kScanThreads) part += sums[i];
  } else {
    // few tiles: add up everything in front of this tile straight from the input (it sits in L2), saving a launch
    const int n4 = blockIdx.x * tile / 4;             // int4 words in front of this tile (tile is a multiple of 4)
    const int4* in4 = reinterpret_cast<const int4*>(in);
    // 16 unpredicated loads in flight per thread (indices past the end are clamped and their values dropped): the
    // longest front (252 KB at 64K positions) is one round trip to L2
    constexpr int kU = 16;
    for (int base = 0; base < n4; base += kU * kScanThreads) {
      int4 v[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) v[u] = in4[min(base + u * kScanThreads + (int)threadIdx.x, n4 - 1)];
#pragma unroll
      for (int u = 0; u < kU; ++u)
        part += base + u * kScanThreads + (int)threadIdx.x < n4 ? v[u].x + v[u].y + v[u].z + v[u].w : 0;
    }
  }
  int carry = block_sum_i32(part, lds);

  const int begin = blockIdx.x * tile;
  const int end = min(n, begin + tile);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  for (int c0 = begin; c0 < end; c0 += kScanThreads) {
    const int idx = c0 + threadIdx.x;
    const int v = idx < end ? in[idx] : 0;
    const int inc = wave_inclusive_scan_i32(v);
    if (lane == kWave - 1) wave_tot[wave] = inc;
    __syncthreads();
    int before = 0, chunk = 0;
#pragma unroll
    for (int w = 0; w < kScanWaves; ++w) {
      const int t = wave_tot[w];
      before += (w < wave) ? t : 0;
      chunk += t;
    }
    const int excl = carry + before + inc - v;
    if (idx < end) {
      if (prefix_out) prefix_out[idx] = excl;
      if (seq_len > 0) {
        // the reference tests mask > 0.5 (cuda_kernels.cu:292); a mask with entries above 1 would push the prefix sum
        // past the arrays, which have n slots
        if (v > 0 && excl < n) {
          const int b = idx / seq_len;
          batch_idx[excl] = b;
          word_idx[excl] = idx - b * seq_len;
        }
        // T = prefix[last] + (mask[last] == 1)   (bert_transformer_op.cu.cc:306-315)
        if (idx == n - 1) *valid_word_num = excl + (v == 1 ? 1 : 0);
      }
    }
    carry += chunk;
    __syncthreads();
  }
}

__global__ __launch_bounds__(256) void index_from_prefix_kernel(const int32_t* __restrict__ mask,
                                                                const int32_t* __restrict__ prefix,
                                                                int32_t* __restrict__ batch_idx,
                                                                int32_t* __restrict__ word_idx, int n, int seq_len) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  if (mask[idx] > 0) {
    const int t = prefix[idx];
    const int b = idx / seq_len;
    batch_idx[t] = b;
    word_idx[t] = idx - b * seq_len;
  }
}

constexpr int kMoveThreads = 256;
constexpr int kMoveUnroll = 8;

// Gather of packed rows: flattened over (packed row, chunk).  CH = the widest piece the row is a whole number of: 16
// bytes for every hidden size a BERT model has; 4 or 2 bytes for the others (the reference moves single elements,
// cuda/cuda_kernels.cu:278-384).
template <typename CH>
__global__ __launch_bounds__(kMoveThreads) void compress_rows_kernel(
    const CH* __restrict__ from, CH* __restrict__ to, const int32_t* __restrict__ batch_idx,
    const int32_t* __restrict__ word_idx, const int32_t* __restrict__ rows_dev, const int32_t* __restrict__ prefix,
    const int32_t* __restrict__ mask, int n_pos, int seq_len, fastdiv cpr) {
  int T;
  if (rows_dev) {
    T = *rows_dev;
  } else {
    T = prefix[n_pos - 1] + (mask[n_pos - 1] == 1 ? 1 : 0);
  }
  T = min(T, n_pos);
  const uint32_t total = (uint32_t)T * cpr.d;
  const uint32_t base = blockIdx.x * (kMoveThreads * kMoveUnroll) + threadIdx.x;
  if (blockIdx.x * (kMoveThreads * kMoveUnroll) >= total) return;
  // No predication at all: lanes past the end repeat the last chunk (load and store of identical data), so that
  // all index loads, then all data loads, then all stores are issued back to back.
  const uint32_t last = total - 1;
  uint32_t row[kMoveUnroll], chunk[kMoveUnroll], idx[kMoveUnroll];
  int bi[kMoveUnroll], wi[kMoveUnroll];
#pragma unroll
  for (int u = 0; u < kMoveUnroll; ++u) {
    const uint32_t i = min(base + u * kMoveThreads, last);
    idx[u] = i;
    row[u] = div_by(i, cpr);
    chunk[u] = i - row[u] * cpr.d;
    bi[u] = batch_idx[row[u]];
    wi[u] = word_idx[row[u]];
  }
  CH val[kMoveUnroll];
#pragma unroll
  for (int u = 0; u < kMoveUnroll; ++u) {
    const uint32_t src_row = (uint32_t)bi[u] * (uint32_t)seq_len + (uint32_t)wi[u];
    val[u] = from[(size_t)src_row * cpr.d + chunk[u]];
  }
#pragma unroll
  for (int u = 0; u < kMoveUnroll; ++u) to[idx[u]] = val[u];
}

constexpr int kRestorePos = 32;   // padded positions per workgroup

// One pass over the padded output: every 16-byte chunk of [B*S, row] is written exactly once,
// either from its packed row or with zeros.  The packed row of a padded position is found
// without scratch memory: keys b*S+s are ascending in t, so a 64-way search by one wavefront
// locates the first packed row at or after the workgroup's first position and the next
// kRestorePos keys cover everything that can land in the workgroup's window.
template <typename CH>
__global__ __launch_bounds__(kMoveThreads) void restore_rows_kernel(
    CH* __restrict__ to, const CH* __restrict__ from, const int32_t* __restrict__ batch_idx,
    const int32_t* __restrict__ word_idx, const int32_t* __restrict__ rows_dev, int n_pos, int seq_len, int cpr) {
  __shared__ int inv[kRestorePos];
  __shared__ int t0_sh;
  const int p0 = blockIdx.x * kRestorePos;
  const int T = min(*rows_dev, n_pos);
  if (threadIdx.x < kRestorePos) inv[threadIdx.x] = -1;
  if (threadIdx.x < kWave) {
    const int lane = threadIdx.x;
    int lo = 0, hi = T;                 // first t with key(t) >= p0 lies in [lo, hi]
    while (hi > lo) {
      const int len = hi - lo;
      const int step = (len + kWave - 1) / kWave;
      const int probe = lo + lane * step;
      bool below = false;
      if (probe < hi) below = (batch_idx[probe] * seq_len + word_idx[probe]) < p0;
      const int c = __popcll(__ballot(below));
      if (c == 0) {
        hi = lo;
      } else {
        const int nlo = lo + (c - 1) * step + 1;
        const int nhi = min(lo + c * step, hi);
        lo = nlo;
        hi = nhi;
      }
    }
    if (lane == 0) t0_sh = lo;
  }
  __syncthreads();
  const int t0 = t0_sh;
  if (threadIdx.x < kRestorePos) {
    const int t = t0 + threadIdx.x;
    if (t < T) {
      const int key = batch_idx[t] * seq_len + word_idx[t];
      if (key >= p0 && key < p0 + kRestorePos) inv[key - p0] = t;
    }
  }
  __syncthreads();
  const int npos = min(kRestorePos, n_pos - p0);
  const int total = npos * cpr;
  for (int i0 = 0; i0 < total; i0 += kMoveThreads * kMoveUnroll) {
    CH val[kMoveUnroll];
#pragma unroll
    for (int u = 0; u < kMoveUnroll; ++u) {
      const int i = i0 + u * kMoveThreads + threadIdx.x;
      val[u] = CH{};
      if (i < total) {
        const int r = i / cpr;
        const int c = i - r * cpr;
        const int t = inv[r];
        if (t >= 0) val[u] = from[(size_t)t * cpr + c];
      }
    }
#pragma unroll
    for (int u = 0; u < kMoveUnroll; ++u) {
      const int i = i0 + u * kMoveThreads + threadIdx.x;
      if (i < total) to[(size_t)p0 * cpr + i] = val[u];
    }
  }
}

__global__ __launch_bounds__(256) void seq_start_kernel(const int32_t* __restrict__ batch_idx,
                                                        const int32_t* __restrict__ rows_dev, int rows_bound,
                                                        int batch, int32_t* __restrict__ seq_start) {
  const int T = rows_dev ? min(*rows_dev, rows_bound) : rows_bound;
  seq_start_for_row(batch_idx, T, blockIdx.x * 256 + threadIdx.x, batch, seq_start);
}

// order[0..batch) = the sequences sorted by length, longest first (buckets of 16 tokens; the order inside a bucket is
// whatever the atomics give: it only decides which workgroup of the attention kernel starts first).  One workgroup.
constexpr int kOrderBuckets = 65;             // lengths up to 1024
__global__ __launch_bounds__(1024) void seq_order_kernel(const int32_t* __restrict__ seq_start, int batch,
                                                         int32_t* __restrict__ order) {
  __shared__ int hist[kOrderBuckets], base[kOrderBuckets];
  for (int i = threadIdx.x; i < kOrderBuckets; i += 1024) hist[i] = 0;
  __syncthreads();
  auto bucket_of = [&](int b) {
    const int len = seq_start[b + 1] - seq_start[b];
    return kOrderBuckets - 1 - min(max(len, 0) >> 4, kOrderBuckets - 1);      // longest first
  };
  for (int b = threadIdx.x; b < batch; b += 1024) atomicAdd(&hist[bucket_of(b)], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int i = 0; i < kOrderBuckets; ++i) {
      base[i] = run;
      run += hist[i];
    }
  }
  __syncthreads();
  for (int b = threadIdx.x; b < batch; b += 1024) order[atomicAdd(&base[bucket_of(b)], 1)] = b;
}

// to[b,:] = row of the packed matrix that sits at position 0 of sequence b, zeros where sequence b has no token
// there.  One wavefront per packed row (plus one past the end): the row that opens a sequence serves that sequence
// and zeroes the token-less sequences in front of it, like seq_start_kernel walks the batch.
template <typename CH>
__global__ __launch_bounds__(256) void first_token_kernel(CH* __restrict__ to, const CH* __restrict__ from,
                                                          const int32_t* __restrict__ batch_idx,
                                                          const int32_t* __restrict__ word_idx,
                                                          const int32_t* __restrict__ rows_dev, int rows_bound,
                                                          int batch, int cpr) {
  const int T = rows_dev ? min(*rows_dev, rows_bound) : rows_bound;
  const int t = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (t > T) return;
  const int prev = t == 0 ? -1 : min(batch_idx[t - 1], batch - 1);
  const int cur = t == T ? batch : min(batch_idx[t], batch - 1);
  if (cur == prev) return;                          // not the first row of its sequence
  const CH zero = {};
  for (int b = prev + 1; b < min(cur, batch); ++b)
    for (int c = lane; c < cpr; c += kWave) to[(size_t)b * cpr + c] = zero;
  if (t < T) {
    const bool at0 = word_idx[t] == 0;
    for (int c = lane; c < cpr; c += kWave) to[(size_t)cur * cpr + c] = at0 ? from[(size_t)t * cpr + c] : zero;
  }
}

}  // namespace

void launch_first_token(void* to, const void* from, const int32_t* batch_idx, const int32_t* word_idx,
                        const int32_t* rows_dev, int rows_bound, int batch, int row_bytes, hipStream_t stream) {
  const int n = rows_bound + 1;
  const int per_wg = 256 / kWave;
  const int grid = (n + per_wg - 1) / per_wg;
  const int cb = row_bytes % 16 == 0 ? 16 : (row_bytes % 4 == 0 ? 4 : 2);      // as the row movers below
  if (cb == 16)
    first_token_kernel<u32x4><<<grid, 256, 0, stream>>>((u32x4*)to, (const u32x4*)from, batch_idx, word_idx, rows_dev,
                                                        rows_bound, batch, row_bytes / 16);
  else if (cb == 4)
    first_token_kernel<uint32_t><<<grid, 256, 0, stream>>>((uint32_t*)to, (const uint32_t*)from, batch_idx, word_idx,
                                                           rows_dev, rows_bound, batch, row_bytes / 4);
  else
    first_token_kernel<uint16_t><<<grid, 256, 0, stream>>>((uint16_t*)to, (const uint16_t*)from, batch_idx, word_idx,
                                                           rows_dev, rows_bound, batch, row_bytes / 2);
}

size_t scan_scratch_words(int length) {
  const int tile = scan_tile_for(length);
  return (size_t)((length + tile - 1) / tile);
}

void launch_scan_index(const int32_t* in, int length, int32_t* prefix_out, int32_t* batch_idx, int32_t* word_idx,
                       int32_t* valid_word_num, int seq_len, int32_t* scratch, hipStream_t stream) {
  const int tile = scan_tile_for(length);
  const int tiles = (length + tile - 1) / tile;
  // up to 128 tiles every workgroup re-adds the elements in front of its tile itself (at most 508 KB of L2 reads);
  // beyond that a first kernel leaves the tile totals in the scratch
  const bool direct = tiles <= 128 && (reinterpret_cast<uintptr_t>(in) & 15) == 0;
  if (!direct) scan_tile_sums_kernel<<<tiles, kScanThreads, 0, stream>>>(in, length, tile, scratch);
  scan_index_kernel<<<tiles, kScanThreads, 0, stream>>>(in, length, tile, direct ? nullptr : scratch, prefix_out,
                                                         batch_idx, word_idx, valid_word_num, seq_len);
}

void launch_index_from_prefix(const int32_t* mask, const int32_t* prefix, int32_t* batch_idx, int32_t* word_idx,
                              int batch, int seq_len, hipStream_t stream) {
  const int n = batch * seq_len;
  index_from_prefix_kernel<<<(n + 255) / 256, 256, 0, stream>>>(mask, prefix, batch_idx, word_idx, n, seq_len);
}

namespace {
// the widest chunk a row of row_bytes bytes is a whole number of
inline int move_chunk_bytes(int row_bytes) { return row_bytes % 16 == 0 ? 16 : (row_bytes % 4 == 0 ? 4 : 2); }
}  // namespace

size_t move_chunks(int n_pos, int row_bytes) { return (size_t)n_pos * (size_t)(row_bytes / move_chunk_bytes(row_bytes)); }

void launch_compress_rows(const void* from, void* to, const int32_t* batch_idx, const int32_t* word_idx,
                          const int32_t* rows_dev, const int32_t* prefix, const int32_t* mask, int batch, int seq_len,
                          int row_bytes, hipStream_t stream) {
  const int n_pos = batch * seq_len;
  const int cb = move_chunk_bytes(row_bytes);
  const uint32_t cpr = (uint32_t)row_bytes / (uint32_t)cb;
  const uint64_t chunks = (uint64_t)n_pos * cpr;
  const uint32_t per_wg = kMoveThreads * kMoveUnroll;
  const uint32_t grid = (uint32_t)((chunks + per_wg - 1) / per_wg);
  if (cb == 16)
    compress_rows_kernel<u32x4><<<grid, kMoveThreads, 0, stream>>>((const u32x4*)from, (u32x4*)to, batch_idx, word_idx,
                                                                   rows_dev, prefix, mask, n_pos, seq_len, make_fastdiv(cpr));
  else if (cb == 4)
    compress_rows_kernel<uint32_t><<<grid, kMoveThreads, 0, stream>>>((const uint32_t*)from, (uint32_t*)to, batch_idx,
                                                                      word_idx, rows_dev, prefix, mask, n_pos, seq_len,
                                                                      make_fastdiv(cpr));
  else
    compress_rows_kernel<uint16_t><<<grid, kMoveThreads, 0, stream>>>((const uint16_t*)from, (uint16_t*)to, batch_idx,
                                                                      word_idx, rows_dev, prefix, mask, n_pos, seq_len,
                                                                      make_fastdiv(cpr));
}

void launch_restore_rows(void* to, const void* from, const int32_t* batch_idx, const int32_t* word_idx,
                         const int32_t* rows_dev, int batch, int seq_len, int row_bytes, hipStream_t stream) {
  const int n_pos = batch * seq_len;
  const int grid = (n_pos + kRestorePos - 1) / kRestorePos;
  const int cb = move_chunk_bytes(row_bytes);
  const int cpr = row_bytes / cb;
  if (cb == 16)
    restore_rows_kernel<u32x4><<<grid, kMoveThreads, 0, stream>>>((u32x4*)to, (const u32x4*)from, batch_idx, word_idx,
                                                                  rows_dev, n_pos, seq_len, cpr);
  else if (cb == 4)
    restore_rows_kernel<uint32_t><<<grid, kMoveThreads, 0, stream>>>((uint32_t*)to, (const uint32_t*)from, batch_idx,
                                                                     word_idx, rows_dev, n_pos, seq_len, cpr);
  else
    restore_rows_kernel<uint16_t><<<grid, kMoveThreads, 0, stream>>>((uint16_t*)to, (const uint16_t*)from, batch_idx,
                                                                     word_idx, rows_dev, n_pos, seq_len, cpr);
}

void launch_seq_order(int32_t* seq_table, int batch, hipStream_t stream) {
  seq_order_kernel<<<1, 1024, 0, stream>>>(seq_table, batch, seq_table + batch + 1);
}

void launch_seq_start(const int32_t* batch_idx, const int32_t* rows_dev, int rows_bound, int batch,
                      int32_t* seq_start, hipStream_t stream) {
  const int n = rows_bound + 1;
  seq_start_kernel<<<(n + 255) / 256, 256, 0, stream>>>(batch_idx, rows_dev, rows_bound, batch, seq_start);
  launch_seq_order(seq_start, batch, stream);
}

}  // namespace et
