// Token alignment in front of the grouped (MoE) GEMM: sort the (token, slot)
// entries of a top-k routing table by expert, keep their original order inside
// an expert, pad every expert's run to a multiple of the block size.  Integer
// work on a few thousand to a few hundred thousand entries: one workgroup of
// sixteen waves does it in one launch (count, scan, place), everything but the
// ids themselves in LDS.
#include "mxfp4_common.h"
#include "mxfp4_group_table.h"

namespace wave_mxfp4 {

namespace {

constexpr int kAlignWaves = 16;
constexpr int kAlignThreads = kAlignWaves * 64;
constexpr int kFewExperts = 16;

template <typename IdT>
__global__ void __launch_bounds__(kAlignThreads) moe_align_kernel(const IdT *__restrict__ topk_ids, int n, int num_experts,
                                                                  int block_size, int32_t *__restrict__ sorted_ids,
                                                                  int sorted_len, int32_t *__restrict__ expert_ids,
                                                                  int expert_ids_len, int32_t *__restrict__ total_out,
                                                                  int32_t *__restrict__ offsets_out) {
  extern __shared__ int lds[];
  int *cnt = lds;                                // [kAlignWaves][E]: entries of expert e in wave w's segment, later
                                                 // the next free position for them
  int *wave_sums = lds + kAlignWaves * num_experts;  // [kAlignWaves]
  int *starts = wave_sums + kAlignWaves;             // [E + 1]: first position of every expert's run, then the total
  int *counts = starts + num_experts + 1;            // [E]: entries of every expert
  const int E = num_experts;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;

  for (int i = t; i < kAlignWaves * E; i += kAlignThreads) cnt[i] = 0;
  __syncthreads();

  // wave w owns the contiguous segment [seg0, seg1) of the flat table
  const int per_wave = ((n + kAlignWaves - 1) / kAlignWaves + 63) & ~63;
  const int seg0 = min(n, wave * per_wave), seg1 = min(n, seg0 + per_wave);
  // (8 steps of 64 ids are fetched together: a step at a time would pay a memory round trip each; the first
  // eight steps stay in registers for the placement below: up to 8192 entries are read once)
  int64_t e_first[8];
  for (int base = seg0; base < seg1; base += 8 * 64) {
    int64_t e[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int i = base + s * 64 + lane;
      e[s] = i < seg1 ? (int64_t)topk_ids[i] : -1;
      if (base == seg0) e_first[s] = e[s];
    }
#pragma unroll
    for (int s = 0; s < 8; ++s)
      if (e[s] >= 0 && e[s] < E) atomicAdd(&cnt[wave * E + (int)e[s]], 1);
  }
  __syncthreads();

  // thread e: the expert's count, padded count and first position
  int count = 0;
  if (t < E) {
    for (int w = 0; w < kAlignWaves; ++w) count += cnt[w * E + t];
  }
  const int blocks = (count + block_size - 1) / block_size, padded = blocks * block_size;
  const int end = block_inclusive_scan(padded, wave_sums, lane, wave);  // also the total, in the last thread
  const int start = end - padded;
  if (t < E) {
    int run = start;
    for (int w = 0; w < kAlignWaves; ++w) {
      const int c = cnt[w * E + t];
      cnt[w * E + t] = run;
      run += c;
    }
    starts[t] = start;
    counts[t] = count;
    if (offsets_out) offsets_out[t] = start;
  }
  if (t == kAlignThreads - 1) starts[E] = end;
  __syncthreads();
  const int total = starts[E];
  if (t == 0) {
    total_out[0] = total;
    if (offsets_out) offsets_out[E] = total;
  }
  for (int i = total + t; i < sorted_len; i += kAlignThreads) sorted_ids[i] = n;  // past the padded total
  // every run's padding (fewer than block_size entries): one wave per expert, a lane per entry
  for (int e = wave; e < E; e += kAlignWaves) {
    const int from = starts[e] + counts[e], to = min(starts[e + 1], sorted_len);
    for (int i = from + lane; i < to; i += 64) sorted_ids[i] = n;
  }
  // the expert of every block: a wave per expert fills the blocks of its run (an empty expert has none)
  for (int e = wave; e < E; e += kAlignWaves) {
    const int from = starts[e] / block_size, to = min(starts[e + 1] / block_size, expert_ids_len);
    for (int b = from + lane; b < to; b += 64) expert_ids[b] = e;
  }

  // place: a wave walks its segment in order; the lanes of one expert take consecutive positions
  // Up to 64 experts the wave keeps "next free position of expert e" in lane e's register (a readlane per
  // look-up); beyond that in its row of cnt (an LDS round trip per look-up).
  const bool in_regs = E <= 64;
  volatile int *next = cnt + wave * E;
  int next_reg = in_regs && lane < E ? cnt[wave * E + lane] : 0;
  for (int base8 = seg0; base8 < seg1; base8 += 8 * 64) {
    int64_t e8[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int i = base8 + s * 64 + lane;
      e8[s] = base8 == seg0 ? e_first[s] : i < seg1 ? (int64_t)topk_ids[i] : -1;
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int i = base8 + s * 64 + lane;
      const bool valid = e8[s] >= 0 && e8[s] < E;
      const int e = valid ? (int)e8[s] : -1;
      if (__ballot(valid) == 0) continue;  // (a short table: most of the eight steps hold no entry at all)
      if (E <= kFewExperts) {
        // few experts: one ballot per expert, no search for the experts that occur
        int pos = -1;
#pragma unroll
        for (int x = 0; x < kFewExperts; ++x) {
          if (x < E) {
            const uint64_t same = __ballot(e == x);
            const int first = __builtin_amdgcn_readlane(next_reg, x);
            if (e == x) pos = first + __popcll(same & ((1ull << lane) - 1));
            if (lane == x) next_reg += __popcll(same);
          }
        }
        if (pos >= 0 && pos < sorted_len) sorted_ids[pos] = i;
        continue;
      }
      uint64_t todo = __ballot(valid);
      while (todo) {
        const int leader = __ffsll((unsigned long long)todo) - 1;
        const int e0 = __builtin_amdgcn_readlane(e, leader);
        const uint64_t same = __ballot(e == e0);
        const int first = in_regs ? __builtin_amdgcn_readlane(next_reg, e0) : next[e0];
        if (e == e0) {
          const int pos = first + __popcll(same & ((1ull << lane) - 1));
          if (pos < sorted_len) sorted_ids[pos] = i;
        }
        const int taken = __popcll(same);
        if (in_regs) {
          if (lane == e0) next_reg += taken;
        } else if (lane == leader) {
          next[e0] = first + taken;
        }
        todo &= ~same;
      }
    }
  }
}

// The M tile table of a grouped GEMM (mxfp4_group_table.h) by a launch of its own.
__global__ void __launch_bounds__(kAlignThreads) grouped_tile_table_kernel(const GroupTableArgs g) {
  __shared__ int wave_sums[kAlignWaves];
  __shared__ int carry[2];
  build_group_tile_table<kAlignThreads>(g, wave_sums, carry);
}

}  // namespace

hipError_t launch_grouped_tile_table(const int32_t *offsets, int num_groups, int bm, int short_rows, int64_t total_rows,
                                     int32_t *table, hipStream_t stream) {
  grouped_tile_table_kernel<<<1, kAlignThreads, 0, stream>>>(
      GroupTableArgs{offsets, num_groups, bm, short_rows, (int)total_rows, table});
  return hipGetLastError();
}

hipError_t launch_moe_align(const void *topk_ids, int ids_int64, int64_t n, int num_experts, int block_size,
                            int32_t *sorted_ids, int64_t sorted_len, int32_t *expert_ids, int64_t expert_ids_len,
                            int32_t *total, int32_t *offsets, hipStream_t stream) {
  const size_t lds = (size_t)(kAlignWaves * num_experts + kAlignWaves + 2 * num_experts + 1) * sizeof(int);
  static LdsAttrOnce once[2];
  const void *fn = ids_int64 ? (const void *)moe_align_kernel<int64_t> : (const void *)moe_align_kernel<int32_t>;
  const hipError_t e = allow_dynamic_lds(
      once[ids_int64 ? 1 : 0], fn, (int)((kAlignWaves * kMoeMaxExperts + kAlignWaves + 2 * kMoeMaxExperts + 1) * sizeof(int)));
  if (e != hipSuccess) return e;
  if (ids_int64)
    moe_align_kernel<int64_t><<<1, kAlignThreads, lds, stream>>>((const int64_t *)topk_ids, (int)n, num_experts, block_size,
                                                                 sorted_ids, (int)sorted_len, expert_ids,
                                                                 (int)expert_ids_len, total, offsets);
  else
    moe_align_kernel<int32_t><<<1, kAlignThreads, lds, stream>>>((const int32_t *)topk_ids, (int)n, num_experts, block_size,
                                                                 sorted_ids, (int)sorted_len, expert_ids,
                                                                 (int)expert_ids_len, total, offsets);
  return hipGetLastError();
}

}  // namespace wave_mxfp4
