// Routing metadata on the device: top-k expert ids -> the per-expert tensors the grouped operators
// consume, plus the row permutation that packs token rows expert by expert.
//
// The reference builds these on the host with torch/Python in its tests and benchmark
// (counts -> expert_offsets prefix sum: benchmark/benchmark_es_fp8_blockwise_moe.py:44-56,72-88;
// blockscale_offsets = prefix sum of the counts rounded up to 128:
// test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:42-60).  Here the same integers come out of
// three small kernels, so a caller never synchronises with the host between routing and the GEMMs.
//
//   pair p = (token p / topk, choice p % topk), id = topk_ids[p] - first_expert; local if 0 <= id < E
//   counts[e]             = number of local pairs with id == e
//   expert_offsets[e]     = sum of counts[0..e)            (E + 1 entries, the last is the total)
//   blockscale_offsets[e] = sum of align128(counts[0..e))  (E + 1 entries)
//   problem_sizes[e]      = (counts[e], n, k)
//   dst_row[p]            = expert_offsets[id] + (number of local pairs q < p with the same id), or -1
// The rank is by pair index, so the permutation is stable and the result is deterministic.
//
// Pairs are cut into chunks of kChunk; one wavefront owns a chunk.  Pass 1 counts ids per chunk, pass 2
// (one workgroup, thread = expert) scans the chunk counts of each expert and then the experts, pass 3
// ranks the pairs of a chunk 64 at a time with running per-expert counters in LDS.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace esmoe {

constexpr int kChunk = 1024;       // pairs per wavefront
constexpr int kMaxRouteExperts = 1024;

// Lanes of the wavefront that hold the same id as this lane: one ballot per bit of the id instead of one round per
// distinct id (64 pairs over 32 experts are ~25 distinct ids, and a round costs as much as all the ballots together).
// `bits` covers num_experts - 1; lanes with id < 0 get a meaningless mask.
__device__ __forceinline__ unsigned long long lanes_with_same_id(int id, int bits) {
  unsigned long long same = __ballot(id >= 0);
  for (int b = 0; b < bits; b++) {
    const bool bit = (id >> b) & 1;
    const unsigned long long m = __ballot(bit);
    same &= bit ? m : ~m;
  }
  return same;
}
__device__ __forceinline__ int id_bits(int num_experts) { return num_experts > 1 ? 32 - __builtin_clz(num_experts - 1) : 0; }

__global__ void __launch_bounds__(64) route_count_kernel(const int* __restrict__ ids, long num_pairs, int first_expert,
                                                         int num_experts, int* __restrict__ chunk_counts) {
  __shared__ int s_cnt[kMaxRouteExperts];
  const int lane = threadIdx.x;
  for (int e = lane; e < num_experts; e += 64) s_cnt[e] = 0;
  __syncthreads();
  const long base = (long)blockIdx.x * kChunk;
  for (int i = lane; i < kChunk; i += 64) {
    const long p = base + i;
    if (p < num_pairs) {
      const int id = ids[p] - first_expert;
      if (id >= 0 && id < num_experts) atomicAdd(&s_cnt[id], 1);
    }
  }
  __syncthreads();
  for (int e = lane; e < num_experts; e += 64) chunk_counts[(long)blockIdx.x * num_experts + e] = s_cnt[e];
}

__global__ void __launch_bounds__(1024) route_scan_kernel(int* __restrict__ chunk_counts, int num_chunks, int num_experts,
                                                          int n, int k, int* __restrict__ problem_sizes,
                                                          int* __restrict__ expert_offsets,
                                                          int* __restrict__ blockscale_offsets) {
  __shared__ int s_cnt[kMaxRouteExperts];
  const int e = threadIdx.x;
  int total = 0;
  if (e < num_experts) {
    // exclusive scan over the chunks, in place: chunk_counts[c][e] becomes the rank base of chunk c.  Sixteen chunks
    // are read before any is written back, so that a thread waits for memory once per sixteen chunks, not per chunk.
    constexpr int kBatch = 16;
    for (int c0 = 0; c0 < num_chunks; c0 += kBatch) {
      int v[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; u++) v[u] = c0 + u < num_chunks ? chunk_counts[(long)(c0 + u) * num_experts + e] : 0;
#pragma unroll
      for (int u = 0; u < kBatch; u++) {
        if (c0 + u < num_chunks) chunk_counts[(long)(c0 + u) * num_experts + e] = total;
        total += v[u];
      }
    }
    s_cnt[e] = total;
  }
  __syncthreads();
  if (e < num_experts) {
    int off = 0, boff = 0;
    for (int j = 0; j < e; j++) {
      const int c = s_cnt[j];
      off += c;
      boff += (c + 127) & ~127;
    }
    expert_offsets[e] = off;
    blockscale_offsets[e] = boff;
    problem_sizes[e * 3 + 0] = total;
    problem_sizes[e * 3 + 1] = n;
    problem_sizes[e * 3 + 2] = k;
    if (e == num_experts - 1) {
      expert_offsets[num_experts] = off + total;
      blockscale_offsets[num_experts] = boff + ((total + 127) & ~127);
    }
  }
}

__global__ void __launch_bounds__(64) route_rank_kernel(const int* __restrict__ ids, long num_pairs, int first_expert,
                                                        int num_experts, const int* __restrict__ chunk_base,
                                                        const int* __restrict__ expert_offsets,
                                                        int* __restrict__ dst_row) {
  __shared__ int s_run[kMaxRouteExperts];   // next free row of every expert for this chunk
  const int lane = threadIdx.x;
  for (int e = lane; e < num_experts; e += 64) s_run[e] = expert_offsets[e] + chunk_base[(long)blockIdx.x * num_experts + e];
  __syncthreads();
  const long base = (long)blockIdx.x * kChunk;
  const int bits = id_bits(num_experts);
  for (int step = 0; step < kChunk / 64; step++) {
    const long p = base + step * 64 + lane;
    if (base + step * 64 >= num_pairs) break;   // wave-uniform
    int id = -1;
    if (p < num_pairs) {
      id = ids[p] - first_expert;
      if (id < 0 || id >= num_experts) id = -1;
    }
    // lanes with the same id take consecutive rows in lane order; the first of them moves the expert's counter on
    int row = -1;
    const unsigned long long same = lanes_with_same_id(id, bits);
    const int before = __builtin_popcountll(same & ((1ull << lane) - 1ull));
    if (id >= 0) row = s_run[id] + before;
    __builtin_amdgcn_wave_barrier();
    if (id >= 0 && before == 0) s_run[id] += __builtin_popcountll(same);
    __builtin_amdgcn_wave_barrier();
    if (p < num_pairs) dst_row[p] = row;
  }
}

// Small inputs (at most kSmallChunks chunks, at most kSmallExperts experts): the three passes in one workgroup of
// kSmallChunks wavefronts, wavefront w owning chunk w, with the per-chunk counters in LDS instead of the workspace.
// Same integers as the three-kernel route; saves two launches, which is most of the time at decode sizes.
constexpr int kSmallChunks = 16;
constexpr int kSmallExperts = 256;

__global__ void __launch_bounds__(kSmallChunks * 64) route_small_kernel(const int* __restrict__ ids, long num_pairs,
                                                                       int first_expert, int num_experts, int n, int k,
                                                                       int* __restrict__ problem_sizes,
                                                                       int* __restrict__ expert_offsets,
                                                                       int* __restrict__ blockscale_offsets,
                                                                       int* __restrict__ dst_row) {
  __shared__ int s_cnt[kSmallChunks][kSmallExperts];   // per-chunk counts, then each chunk's next free row per expert
  __shared__ int s_tot[kSmallExperts];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  for (int i = tid; i < kSmallChunks * kSmallExperts; i += kSmallChunks * 64) (&s_cnt[0][0])[i] = 0;
  __syncthreads();
  const long base = (long)w * kChunk;
  for (int i = lane; i < kChunk; i += 64) {
    const long p = base + i;
    if (p < num_pairs) {
      const int id = ids[p] - first_expert;
      if (id >= 0 && id < num_experts) atomicAdd(&s_cnt[w][id], 1);
    }
  }
  __syncthreads();
  if (tid < num_experts) {
    int total = 0;
    for (int c = 0; c < kSmallChunks; c++) {
      const int v = s_cnt[c][tid];
      s_cnt[c][tid] = total;
      total += v;
    }
    s_tot[tid] = total;
  }
  __syncthreads();
  if (tid < num_experts) {
    int off = 0, boff = 0;
    for (int j = 0; j < tid; j++) {
      const int c = s_tot[j];
      off += c;
      boff += (c + 127) & ~127;
    }
    const int total = s_tot[tid];
    expert_offsets[tid] = off;
    blockscale_offsets[tid] = boff;
    problem_sizes[tid * 3 + 0] = total;
    problem_sizes[tid * 3 + 1] = n;
    problem_sizes[tid * 3 + 2] = k;
    if (tid == num_experts - 1) {
      expert_offsets[num_experts] = off + total;
      blockscale_offsets[num_experts] = boff + ((total + 127) & ~127);
    }
    for (int c = 0; c < kSmallChunks; c++) s_cnt[c][tid] += off;
  }
  __syncthreads();
  const int bits = id_bits(num_experts);
  for (int step = 0; step < kChunk / 64; step++) {
    const long p = base + step * 64 + lane;
    if (base + step * 64 >= num_pairs) break;   // wave-uniform
    int id = -1;
    if (p < num_pairs) {
      id = ids[p] - first_expert;
      if (id < 0 || id >= num_experts) id = -1;
    }
    int row = -1;
    const unsigned long long same = lanes_with_same_id(id, bits);
    const int before = __builtin_popcountll(same & ((1ull << lane) - 1ull));
    if (id >= 0) row = s_cnt[w][id] + before;
    __builtin_amdgcn_wave_barrier();
    if (id >= 0 && before == 0) s_cnt[w][id] += __builtin_popcountll(same);
    __builtin_amdgcn_wave_barrier();
    if (p < num_pairs) dst_row[p] = row;
  }
}

// Packs rows for the grouped operators: out[dst_row[p], :] = in[p / topk, :] for every local pair
// (2-byte elements, row_bytes a multiple of 16).  One wavefront moves one row in 1 KB steps.
__global__ void __launch_bounds__(256) permute_rows_kernel(const uint8_t* __restrict__ in, const int* __restrict__ dst_row,
                                                           long num_pairs, int topk, long row_bytes,
                                                           uint8_t* __restrict__ out) {
  typedef int v4i __attribute__((ext_vector_type(4)));
  const long p = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (p >= num_pairs) return;
  const int dst = dst_row[p];
  if (dst < 0) return;
  const uint8_t* src = in + (p / topk) * row_bytes;
  uint8_t* d = out + (long)dst * row_bytes;
  for (long off = (threadIdx.x & 63) * 16; off < row_bytes; off += 4096) {
    v4i v[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (off + u * 1024 < row_bytes) v[u] = __builtin_nontemporal_load((const v4i*)(src + off + u * 1024));
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (off + u * 1024 < row_bytes) __builtin_nontemporal_store(v[u], (v4i*)(d + off + u * 1024));
  }
}

// The same packing for topk > 1 (at most 64): one wavefront per token reads the row once and writes it to every
// local destination of the token's pairs, where one wavefront per pair would read it topk times.
__global__ void __launch_bounds__(256) permute_rows_by_token_kernel(const uint8_t* __restrict__ in,
                                                                    const int* __restrict__ dst_row, long num_tokens,
                                                                    int topk, long row_bytes, uint8_t* __restrict__ out) {
  typedef int v4i __attribute__((ext_vector_type(4)));
  const long t = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= num_tokens) return;
  const int lane = threadIdx.x & 63;
  const int mine = lane < topk ? dst_row[t * topk + lane] : -1;   // lane j: destination of the token's pair j
  if (__ballot(mine >= 0) == 0) return;                           // no local pair
  const uint8_t* src = in + t * row_bytes;
  for (long off = lane * 16; off < row_bytes; off += 4096) {
    v4i v[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (off + u * 1024 < row_bytes) v[u] = __builtin_nontemporal_load((const v4i*)(src + off + u * 1024));
    for (int j = 0; j < topk; j++) {
      const int dst = __builtin_amdgcn_readlane(mine, j);
      if (dst < 0) continue;
      uint8_t* d = out + (long)dst * row_bytes;
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (off + u * 1024 < row_bytes) __builtin_nontemporal_store(v[u], (v4i*)(d + off + u * 1024));
    }
  }
}

}  // namespace esmoe

extern "C" int esmoe_launch_route_metadata(const int* ids, long num_pairs, int first_expert, int num_experts, int n, int k,
                                           int* problem_sizes, int* expert_offsets, int* blockscale_offsets, int* dst_row,
                                           int* chunk_counts, hipStream_t stream) {
  using namespace esmoe;
  const int chunks = (int)((num_pairs + kChunk - 1) / kChunk);
  if (chunks <= kSmallChunks && num_experts <= kSmallExperts) {
    hipLaunchKernelGGL(route_small_kernel, dim3(1), dim3(kSmallChunks * 64), 0, stream, ids, num_pairs, first_expert,
                       num_experts, n, k, problem_sizes, expert_offsets, blockscale_offsets, dst_row);
    return (int)hipGetLastError();
  }
  if (chunks > 0)
    hipLaunchKernelGGL(route_count_kernel, dim3(chunks), dim3(64), 0, stream, ids, num_pairs, first_expert, num_experts,
                       chunk_counts);
  hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3((num_experts + 63) & ~63), 0, stream, chunk_counts, chunks,
                     num_experts, n, k, problem_sizes, expert_offsets, blockscale_offsets);
  if (chunks > 0)
    hipLaunchKernelGGL(route_rank_kernel, dim3(chunks), dim3(64), 0, stream, ids, num_pairs, first_expert, num_experts,
                       chunk_counts, expert_offsets, dst_row);
  return (int)hipGetLastError();
}

extern "C" int esmoe_launch_permute_rows(const void* in, const int* dst_row, long num_pairs, int topk, long row_bytes,
                                         void* out, hipStream_t stream) {
  using namespace esmoe;
  if (num_pairs == 0) return 0;
  if (topk > 1 && topk <= 64 && num_pairs % topk == 0) {
    const long tokens = num_pairs / topk;
    hipLaunchKernelGGL(permute_rows_by_token_kernel, dim3((unsigned)((tokens + 3) / 4)), dim3(256), 0, stream,
                       (const uint8_t*)in, dst_row, tokens, topk, row_bytes, (uint8_t*)out);
    return (int)hipGetLastError();
  }
  hipLaunchKernelGGL(permute_rows_kernel, dim3((unsigned)((num_pairs + 3) / 4)), dim3(256), 0, stream, (const uint8_t*)in,
                     dst_row, num_pairs, topk, row_bytes, (uint8_t*)out);
  return (int)hipGetLastError();
}
