// moe_align_block_size for gfx950: expert histogram, padded prefix sum and a stable
// (ascending slot id) counting sort, in one workgroup, with wavefront ballots and
// LDS counters and no atomics on the ranking path, so the result is deterministic.
//
// Semantics follow python/lightop/_lmslim_native/vllm_compat/moe_align_block_size.py:17-120
// and csrc/kernels/moe_align_sum_kernels.cu:1034-1115 of the reference; the order
// inside an expert is the ascending one of test/test_moe_align_block_size.py:81-88.
#include "common.h"

namespace lo {

// Lanes of the wave that hold the same key as this lane (key < 2^bits), as a mask.
__device__ __forceinline__ uint64_t match_any(int key, int bits, bool active) {
  uint64_t peers = __ballot(active);
  for (int b = 0; b < bits; ++b) {
    uint64_t set = __ballot(active && ((key >> b) & 1));
    peers &= ((key >> b) & 1) ? set : ~set;
  }
  return peers;
}

// Only the slots of the first num_local_tokens[0] tokens are aligned when that device
// counter is given (batches padded to a fixed size); the pad value stays the full numel
// (csrc/kernels/moe_align_sum_kernels.cu:32-45 of the reference).
__device__ __forceinline__ int64_t local_slots(int64_t numel, const int32_t *__restrict__ num_local_tokens,
                                               int slots_per_token) {
  if (!num_local_tokens) return numel;
  const int64_t v = static_cast<int64_t>(num_local_tokens[0]) * slots_per_token;
  return v < 0 ? 0 : (v < numel ? v : numel);
}

template <typename IdT>
__device__ __forceinline__ void moe_align_body(
    const IdT *__restrict__ ids, int64_t numel, int num_experts, int bs,
    const int32_t *__restrict__ expert_map, int ignore_invalid, int32_t *__restrict__ sorted,
    int64_t sorted_cap, int32_t *__restrict__ expert_ids, int64_t expert_ids_cap,
    int32_t *__restrict__ ntpp, int key_bits, uint8_t *__restrict__ slot_mask,
    const int32_t *__restrict__ num_local_tokens, int slots_per_token) {
  extern __shared__ int32_t lds[];
  const int64_t pad_val = numel;
  numel = local_slots(numel, num_local_tokens, slots_per_token);
  if (slot_mask) // slots of padding tokens belong to nobody
    for (int64_t f = numel + threadIdx.x; f < pad_val; f += blockDim.x) slot_mask[f] = 0;
  const int nw = blockDim.x / kWave;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int E = num_experts;
  int32_t *offs = lds;               // [E + 1] padded exclusive prefix
  int32_t *total = lds + (E + 1);    // [E] tokens per expert
  int32_t *wcnt = total + E;         // [nw][E] per-wave counts, later running bases

  for (int i = tid; i < nw * E; i += blockDim.x) wcnt[i] = 0;
  // Every entry of sorted[] starts as padding (one coalesced sweep while the ids are on their way);
  // the scatter of pass 3 then overwrites the valid ones.  The workgroup barriers in between
  // order the two stores to an entry.
  for (int64_t i = tid; i < sorted_cap; i += blockDim.x) sorted[i] = static_cast<int32_t>(pad_val);
  __syncthreads();

  // Each wave owns a contiguous range of slot ids, rounded to whole 64-id tiles.
  const int64_t tiles = (numel + kWave - 1) / kWave;
  const int64_t tiles_per_wave = (tiles + nw - 1) / nw;
  const int64_t t0 = wave * tiles_per_wave;
  const int64_t t1 = (t0 + tiles_per_wave < tiles) ? t0 + tiles_per_wave : tiles;

  // Raw ids of a batch of tiles are fetched back to back (no branch between the loads: an index
  // past the end re-reads slot 0 and is discarded), then turned into keys.
  constexpr int kBatch = 8;
  auto load_raw = [&](int64_t t, int64_t (&raw)[kBatch]) {
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int64_t f = (t + b) * kWave + lane;
      raw[b] = static_cast<int64_t>(ids[(t + b < t1 && f < numel) ? f : 0]);
    }
  };
  auto key_of = [&](int64_t raw, bool in_range, bool &ok) -> int {
    ok = in_range && raw >= 0 && raw < E;
    int e = ok ? static_cast<int>(raw) : 0;
    if (ignore_invalid && expert_map) { // keys are local expert ids
      const int m = expert_map[e];
      ok = ok && m >= 0 && m < E;
      e = ok ? m : 0;
    }
    return e;
  };

  // pass 1: per-wave histogram.  Counting does not depend on order, so LDS atomics are fine
  // here.  The keys of the wave's first batch stay in registers for pass 3 (up to 8192 slots
  // on 16 waves that is all of them).
  int ek0[kBatch];
  bool ok0[kBatch];
#pragma unroll
  for (int b = 0; b < kBatch; ++b) {
    ek0[b] = 0;
    ok0[b] = false;
  }
  for (int64_t t = t0; t < t1; t += kBatch) {
    int64_t raw[kBatch];
    load_raw(t, raw);
    int ek[kBatch];
    bool okk[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int64_t f = (t + b) * kWave + lane;
      const bool in_range = t + b < t1 && f < numel;
      ek[b] = key_of(raw[b], in_range, okk[b]);
      if (slot_mask && in_range) { // is the slot's expert held by this rank?
        bool local = okk[b];
        if (local && expert_map && !ignore_invalid) local = expert_map[ek[b]] >= 0;
        slot_mask[f] = local ? 1 : 0;
      }
    }
#pragma unroll
    for (int b = 0; b < kBatch; ++b)
      if (okk[b]) atomicAdd(&wcnt[wave * E + ek[b]], 1);
    if (t == t0) {
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        ek0[b] = ek[b];
        ok0[b] = okk[b];
      }
    }
  }
  __syncthreads();

  // pass 2: totals, padded sizes, exclusive scan over experts (one thread per
  // expert; wave-level inclusive scan, then a scan over wave sums)
  __shared__ int32_t wave_sum[16];
  for (int base = 0; base < E; base += blockDim.x) {
    int e = base + tid;
    int c = 0;
    if (e < E) {
      for (int w = 0; w < nw; ++w) {
        int v = wcnt[w * E + e];
        wcnt[w * E + e] = c; // tokens of expert e held by earlier waves
        c += v;
      }
      total[e] = c;
    }
    int padded = (e < E) ? (c + bs - 1) / bs * bs : 0;
    int incl = padded;
    for (int d = 1; d < kWave; d <<= 1) {
      int up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) wave_sum[wave] = incl;
    __syncthreads();
    int carry = (base == 0) ? 0 : offs[base];
    for (int w = 0; w < wave; ++w) carry += wave_sum[w];
    if (e < E) offs[e + 1] = carry + incl;
    if (base == 0 && tid == 0) offs[0] = 0;
    __syncthreads();
  }
  const int P = offs[E];
  if (tid == 0) ntpp[0] = P;

  // expert id of every block; -1 past the last block
  for (int e = tid; e < E; e += blockDim.x) {
    int v = (expert_map && !ignore_invalid) ? expert_map[e] : e;
    for (int b = offs[e] / bs; b < offs[e + 1] / bs; ++b) expert_ids[b] = v;
  }
  for (int64_t b = P / bs + tid; b < expert_ids_cap; b += blockDim.x) expert_ids[b] = -1;


  // pass 3: stable scatter.  wcnt[wave][e] is the running number of slots of expert
  // e that precede the current tile.  Ranks inside a tile come from a ballot match, the
  // running counters are updated by one lane per expert: no atomics, fixed order.
  for (int64_t t = t0; t < t1; t += kBatch) {
    int ek[kBatch];
    bool okk[kBatch];
    if (t == t0) {
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        ek[b] = ek0[b];
        okk[b] = ok0[b];
      }
    } else {
      int64_t raw[kBatch];
      load_raw(t, raw);
#pragma unroll
      for (int b = 0; b < kBatch; ++b)
        ek[b] = key_of(raw[b], t + b < t1 && (t + b) * kWave + lane < numel, okk[b]);
    }
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      if (t + b >= t1) break; // wave-uniform
      const int e = ek[b];
      const bool ok = okk[b];
      const int64_t f = (t + b) * kWave + lane;
      uint64_t peers = match_any(e, key_bits, ok);
      if (ok) {
        int before = __popcll(peers & ((1ull << lane) - 1ull));
        int leader = __ffsll(static_cast<unsigned long long>(peers)) - 1;
        int base = wcnt[wave * E + e];
        sorted[offs[e] + base + before] = static_cast<int32_t>(f);
        __builtin_amdgcn_wave_barrier();
        if (lane == leader) wcnt[wave * E + e] = base + __popcll(peers);
      }
      // the counters are LDS words touched by this wave only, and a wave's LDS operations
      // execute in order: the next tile sees them without waiting for the global stores
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();
    }
  }
}

template <typename IdT>
__global__ __launch_bounds__(1024) void moe_align_kernel(
    const IdT *__restrict__ ids, int64_t numel, int num_experts, int bs,
    const int32_t *__restrict__ expert_map, int ignore_invalid, int32_t *__restrict__ sorted,
    int64_t sorted_cap, int32_t *__restrict__ expert_ids, int64_t expert_ids_cap,
    int32_t *__restrict__ ntpp, int key_bits, uint8_t *__restrict__ slot_mask,
    const int32_t *__restrict__ num_local_tokens, int slots_per_token) {
  moe_align_body<IdT>(ids, numel, num_experts, bs, expert_map, ignore_invalid, sorted, sorted_cap, expert_ids,
                      expert_ids_cap, ntpp, key_bits, slot_mask, num_local_tokens, slots_per_token);
}

// Workgroup 0 aligns, the others quantise the activations: two independent stages, one launch.
template <typename IdT>
__global__ __launch_bounds__(1024) void quant_align_kernel(
    const uint16_t *__restrict__ x, int64_t groups, float eps, int8_t *__restrict__ q, float *__restrict__ qs,
    const IdT *__restrict__ ids, int64_t numel, int num_experts, int bs,
    const int32_t *__restrict__ expert_map, int32_t *__restrict__ sorted, int64_t sorted_cap,
    int32_t *__restrict__ expert_ids, int64_t expert_ids_cap, int32_t *__restrict__ ntpp, int key_bits,
    uint8_t *__restrict__ slot_mask) {
  if (blockIdx.x == 0) {
    moe_align_body<IdT>(ids, numel, num_experts, bs, expert_map, 0, sorted, sorted_cap, expert_ids, expert_ids_cap,
                        ntpp, key_bits, slot_mask, nullptr, 1);
  } else {
    const int per_block = blockDim.x >> 4; // groups a workgroup handles per pass
    group_quant_body<LO_BF16>(x, groups, eps, q, qs,
                              static_cast<int64_t>(blockIdx.x - 1) * per_block + (threadIdx.x >> 4),
                              static_cast<int64_t>(gridDim.x - 1) * per_block, threadIdx.x & 15);
  }
}

// ---- large inputs: the same algorithm spread over many workgroups ------------------
// Phase 1: every workgroup counts the experts of its chunk of slots into cnt[chunk][E].
// Phase 2: every workgroup rebuilds the padded expert offsets from cnt (a few KB from
// L2), adds the counts of the chunks before it, and scatters its chunk exactly like the
// single-workgroup kernel does; padding, expert ids and the tail are shared out by expert.
// Chunks, waves, tiles and lanes are all in slot order, so the result is the same stable
// order, bit for bit.
template <typename IdT>
__device__ __forceinline__ int align_key(const IdT *__restrict__ ids, int64_t f, int64_t numel, int E,
                                         const int32_t *__restrict__ expert_map, int ignore_invalid,
                                         bool &ok) {
  // no branch around the load (an index past the end re-reads slot 0 and is discarded), so that
  // the loads of a batch of tiles are issued back to back
  const bool in_range = f < numel;
  const int64_t raw = static_cast<int64_t>(ids[in_range ? f : 0]);
  ok = in_range && raw >= 0 && raw < E;
  int e = ok ? static_cast<int>(raw) : 0;
  if (ignore_invalid && expert_map) {
    const int m = expert_map[e];
    ok = ok && m >= 0 && m < E;
    e = ok ? m : 0;
  }
  return e;
}

// (nblocks: the workgroups that count, blockIdx.x 0 .. nblocks-1; the grid may hold others)
template <typename IdT>
__device__ __forceinline__ void moe_align_count_body(
    const IdT *__restrict__ ids, int64_t numel, int E, const int32_t *__restrict__ expert_map,
    int ignore_invalid, int64_t chunk_slots, int32_t *__restrict__ cnt, uint8_t *__restrict__ slot_mask,
    const int32_t *__restrict__ num_local_tokens, int slots_per_token, int32_t *__restrict__ sorted,
    int64_t sorted_cap, int nblocks) {
  extern __shared__ int32_t lds[];
  for (int i = threadIdx.x; i < E; i += blockDim.x) lds[i] = 0;
  __syncthreads();
  const int64_t pad_val = numel;
  // every entry of sorted[] starts as padding; the second launch overwrites the valid ones
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < sorted_cap;
       i += static_cast<int64_t>(nblocks) * blockDim.x)
    sorted[i] = static_cast<int32_t>(pad_val);
  numel = local_slots(numel, num_local_tokens, slots_per_token);
  const int64_t begin = blockIdx.x * chunk_slots;
  const int64_t end = (begin + chunk_slots < numel) ? begin + chunk_slots : numel;
  if (slot_mask) { // this chunk's slots of padding tokens belong to nobody
    const int64_t pend = (begin + chunk_slots < pad_val) ? begin + chunk_slots : pad_val;
    for (int64_t f = (begin > numel ? begin : numel) + threadIdx.x; f < pend; f += blockDim.x) slot_mask[f] = 0;
  }
  for (int64_t f0 = begin + threadIdx.x; f0 < end; f0 += 4 * blockDim.x) {
    int ek[4];
    bool okk[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int64_t f = f0 + static_cast<int64_t>(b) * blockDim.x;
      ek[b] = align_key(ids, f < end ? f : numel, numel, E, expert_map, ignore_invalid, okk[b]);
      if (slot_mask && f < end) {
        bool local = okk[b];
        if (local && expert_map && !ignore_invalid) local = expert_map[ek[b]] >= 0;
        slot_mask[f] = local ? 1 : 0;
      }
    }
#pragma unroll
    for (int b = 0; b < 4; ++b)
      if (okk[b]) atomicAdd(&lds[ek[b]], 1);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < E; i += blockDim.x) cnt[static_cast<int64_t>(blockIdx.x) * E + i] = lds[i];
}

template <typename IdT>
__global__ __launch_bounds__(256) void moe_align_count_kernel(
    const IdT *__restrict__ ids, int64_t numel, int E, const int32_t *__restrict__ expert_map,
    int ignore_invalid, int64_t chunk_slots, int32_t *__restrict__ cnt, uint8_t *__restrict__ slot_mask,
    const int32_t *__restrict__ num_local_tokens, int slots_per_token, int32_t *__restrict__ sorted,
    int64_t sorted_cap) {
  moe_align_count_body<IdT>(ids, numel, E, expert_map, ignore_invalid, chunk_slots, cnt, slot_mask, num_local_tokens,
                            slots_per_token, sorted, sorted_cap, static_cast<int>(gridDim.x));
}

template <typename IdT>
__device__ __forceinline__ void moe_align_scatter_body(
    const IdT *__restrict__ ids, int64_t numel, int E, int bs, const int32_t *__restrict__ expert_map,
    int ignore_invalid, int64_t chunk_slots, const int32_t *__restrict__ cnt,
    int32_t *__restrict__ sorted, int64_t sorted_cap, int32_t *__restrict__ expert_ids,
    int64_t expert_ids_cap, int32_t *__restrict__ ntpp, int key_bits,
    const int32_t *__restrict__ num_local_tokens, int slots_per_token, int chunk, int nchunks) {
  extern __shared__ int32_t lds[];
  numel = local_slots(numel, num_local_tokens, slots_per_token);
  constexpr int nw = 4;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int32_t *offs = lds;              // [E + 1] padded exclusive prefix
  int32_t *total = lds + (E + 1);   // [E]
  int32_t *cbase = total + E;       // [E] slots of expert e in earlier chunks
  int32_t *wcnt = cbase + E;        // [nw][E]
  __shared__ int32_t wave_sum[nw];

  for (int i = tid; i < nw * E; i += blockDim.x) wcnt[i] = 0;
  for (int i = tid; i < E; i += blockDim.x) total[i] = cbase[i] = 0;
  __syncthreads();
  // per expert: slots in all chunks and in the chunks before this one (coalesced sweep over
  // cnt[chunk][expert]; integer sums, so the order of the LDS atomics does not matter)
  constexpr int kSweep = 16; // loads in flight per thread: the sweep is a few round trips, not one per entry
  for (int idx0 = tid; idx0 < nchunks * E; idx0 += kSweep * blockDim.x) {
    int v[kSweep];
#pragma unroll
    for (int u = 0; u < kSweep; ++u) {
      const int idx = idx0 + u * blockDim.x;
      v[u] = cnt[idx < nchunks * E ? idx : 0];
    }
#pragma unroll
    for (int u = 0; u < kSweep; ++u) {
      const int idx = idx0 + u * blockDim.x;
      const int c = idx / E, e = idx - c * E;
      if (idx < nchunks * E && v[u]) {
        atomicAdd(&total[e], v[u]);
        if (c < chunk) atomicAdd(&cbase[e], v[u]);
      }
    }
  }
  __syncthreads();
  for (int base = 0; base < E; base += blockDim.x) {
    const int e = base + tid;
    const int t = (e < E) ? total[e] : 0;
    int incl = (e < E) ? (t + bs - 1) / bs * bs : 0;
    for (int d = 1; d < kWave; d <<= 1) {
      int up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) wave_sum[wave] = incl;
    __syncthreads();
    int carry = (base == 0) ? 0 : offs[base];
    for (int w = 0; w < wave; ++w) carry += wave_sum[w];
    if (e < E) offs[e + 1] = carry + incl;
    if (base == 0 && tid == 0) offs[0] = 0;
    __syncthreads();
  }
  const int P = offs[E];

  // shared-out bookkeeping: workgroup c looks after experts c, c + nchunks, ...
  if (chunk == 0 && tid == 0) ntpp[0] = P;
  for (int e = chunk + tid * nchunks; e < E; e += nchunks * blockDim.x) { // one thread per expert: the map reads overlap
    const int v = (expert_map && !ignore_invalid) ? expert_map[e] : e;
    for (int b = offs[e] / bs; b < offs[e + 1] / bs; ++b) expert_ids[b] = v;
  }
  for (int64_t b = P / bs + chunk * blockDim.x + tid; b < expert_ids_cap; b += static_cast<int64_t>(nchunks) * blockDim.x)
    expert_ids[b] = -1;

  // this chunk: contiguous sub-range per wave, whole 64-slot tiles
  const int64_t begin = chunk * chunk_slots;
  const int64_t end = (begin + chunk_slots < numel) ? begin + chunk_slots : numel;
  const int64_t tiles = (end > begin) ? (end - begin + kWave - 1) / kWave : 0;
  const int64_t tiles_per_wave = (tiles + nw - 1) / nw;
  const int64_t t0 = wave * tiles_per_wave;
  const int64_t t1 = (t0 + tiles_per_wave < tiles) ? t0 + tiles_per_wave : tiles;
  constexpr int kBatch = 4;
  int ek0[kBatch]; // keys of the wave's first batch, kept for the scatter below
  bool ok0[kBatch];
#pragma unroll
  for (int b = 0; b < kBatch; ++b) {
    ek0[b] = 0;
    ok0[b] = false;
  }
  for (int64_t t = t0; t < t1; t += kBatch) {
    int ek[kBatch];
    bool okk[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int64_t f = begin + (t + b) * kWave + lane;
      ek[b] = align_key(ids, (t + b < t1 && f < end) ? f : numel, numel, E, expert_map, ignore_invalid, okk[b]);
    }
#pragma unroll
    for (int b = 0; b < kBatch; ++b)
      if (okk[b]) atomicAdd(&wcnt[wave * E + ek[b]], 1);
    if (t == t0) {
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        ek0[b] = ek[b];
        ok0[b] = okk[b];
      }
    }
  }
  __syncthreads();
  for (int e = tid; e < E; e += blockDim.x) {
    int c = 0;
    for (int w = 0; w < nw; ++w) {
      const int v = wcnt[w * E + e];
      wcnt[w * E + e] = c;
      c += v;
    }
  }
  __syncthreads();
  for (int64_t t = t0; t < t1; t += kBatch) {
    int ek[kBatch];
    bool okk[kBatch];
    if (t == t0) {
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        ek[b] = ek0[b];
        okk[b] = ok0[b];
      }
    } else {
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        const int64_t f = begin + (t + b) * kWave + lane;
        ek[b] = align_key(ids, (t + b < t1 && f < end) ? f : numel, numel, E, expert_map, ignore_invalid, okk[b]);
      }
    }
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      if (t + b >= t1) break; // wave-uniform
      const int e = ek[b];
      const bool ok = okk[b];
      const int64_t f = begin + (t + b) * kWave + lane;
      uint64_t peers = match_any(e, key_bits, ok);
      if (ok) {
        int before = __popcll(peers & ((1ull << lane) - 1ull));
        int leader = __ffsll(static_cast<unsigned long long>(peers)) - 1;
        int run = wcnt[wave * E + e];
        sorted[offs[e] + cbase[e] + run + before] = static_cast<int32_t>(f);
        __builtin_amdgcn_wave_barrier();
        if (lane == leader) wcnt[wave * E + e] = run + __popcll(peers);
      }
      asm volatile("" ::: "memory"); // a wave's LDS operations execute in order: no wait for the global stores
      __builtin_amdgcn_wave_barrier();
    }
  }
}

template <typename IdT>
__global__ __launch_bounds__(256) void moe_align_scatter_kernel(
    const IdT *__restrict__ ids, int64_t numel, int E, int bs, const int32_t *__restrict__ expert_map,
    int ignore_invalid, int64_t chunk_slots, const int32_t *__restrict__ cnt,
    int32_t *__restrict__ sorted, int64_t sorted_cap, int32_t *__restrict__ expert_ids,
    int64_t expert_ids_cap, int32_t *__restrict__ ntpp, int key_bits,
    const int32_t *__restrict__ num_local_tokens, int slots_per_token) {
  moe_align_scatter_body<IdT>(ids, numel, E, bs, expert_map, ignore_invalid, chunk_slots, cnt, sorted, sorted_cap,
                              expert_ids, expert_ids_cap, ntpp, key_bits, num_local_tokens, slots_per_token,
                              static_cast<int>(blockIdx.x), static_cast<int>(gridDim.x));
}

// The first nchunks workgroups scatter, the others quantise the activations: the quantisation does
// not depend on the alignment, and the scatter (a chain of dependent round trips on a few compute
// units) costs nothing beside it.  The counting, which the scatter waits for, is a launch of its own
// before this one.
template <typename IdT>
__global__ __launch_bounds__(256) void quant_align_scatter_kernel(
    const uint16_t *__restrict__ x, int64_t groups, float eps, int8_t *__restrict__ q, float *__restrict__ qs,
    const IdT *__restrict__ ids, int64_t numel, int E, int bs, const int32_t *__restrict__ expert_map,
    int64_t chunk_slots, const int32_t *__restrict__ cnt, int32_t *__restrict__ sorted, int64_t sorted_cap,
    int32_t *__restrict__ expert_ids, int64_t expert_ids_cap, int32_t *__restrict__ ntpp, int key_bits,
    int nchunks) {
  if (static_cast<int>(blockIdx.x) < nchunks) {
    moe_align_scatter_body<IdT>(ids, numel, E, bs, expert_map, 0, chunk_slots, cnt, sorted, sorted_cap, expert_ids,
                                expert_ids_cap, ntpp, key_bits, nullptr, 1, static_cast<int>(blockIdx.x), nchunks);
  } else {
    group_quant_body<LO_BF16>(x, groups, eps, q, qs,
                              static_cast<int64_t>(blockIdx.x - nchunks) * 16 + (threadIdx.x >> 4),
                              static_cast<int64_t>(gridDim.x - nchunks) * 16, threadIdx.x & 15);
  }
}

// chunks for the multi-workgroup path: about 1024 slots each, at most 256 chunks
static void single_wg_shape(int64_t numel, int64_t sorted_cap, int32_t num_experts, int *nw, size_t *lds_bytes) {
  // waves per workgroup: as many as the per-wave LDS counters allow (<= 60 KB)
  int w = 16;
  while (w > 1 && (static_cast<int64_t>(w) + 2) * num_experts + 1 > 15360) w >>= 1;
  // a handful of slots need few waves - unless the padded buffer they have to fill is long
  if (numel <= 64 * 4 && sorted_cap <= 4096) w = w < 4 ? w : 4;
  *nw = w;
  *lds_bytes = (static_cast<size_t>(w + 2) * num_experts + 1) * sizeof(int32_t);
}

static void align_chunks(int64_t numel, int *nchunks, int64_t *chunk_slots) {
  int64_t n = (numel + 1023) / 1024;
  if (n > 256) n = 256;
  if (n < 1) n = 1;
  int64_t cs = (numel + n - 1) / n;
  cs = (cs + 255) / 256 * 256;
  *chunk_slots = cs;
  *nchunks = static_cast<int>((numel + cs - 1) / cs);
}

int launch_quant_align(const void *x, int64_t M, int64_t H, float eps, int8_t *q, float *qs,
                       const void *topk_ids, int ids_dtype, int64_t numel, int32_t num_experts,
                       int32_t block_size, const int32_t *expert_map, int32_t *sorted_ids, int64_t sorted_cap,
                       int32_t *expert_ids, int64_t expert_ids_cap, int32_t *num_tokens_post_pad,
                       uint8_t *slot_mask, void *scratch, int64_t scratch_bytes, hipStream_t stream) {
  const int64_t want = lo_moe_align_scratch_bytes(numel, num_experts);
  if (want > 0 && !(scratch && scratch_bytes >= want && (reinterpret_cast<uintptr_t>(scratch) & 3) == 0))
    return LO_ENOTSUP; // the multi-workgroup form needs its counters
  LO_REQUIRE(x && q && qs && topk_ids && sorted_ids && expert_ids && num_tokens_post_pad, LO_EINVAL,
             "quant_align: null pointer");
  LO_REQUIRE(H > 0 && H % kGroup == 0 && M >= 1 && numel >= 1 && num_experts >= 1 && num_experts <= 2048 &&
                 block_size >= 1,
             LO_EINVAL, "quant_align: bad shape");
  int64_t need = numel + static_cast<int64_t>(num_experts) * (block_size - 1);
  if (numel < num_experts && numel * block_size < need) need = numel * block_size;
  LO_REQUIRE(sorted_cap >= need && expert_ids_cap >= (need + block_size - 1) / block_size, LO_ENOSPC,
             "quant_align: alignment buffers too small");
  int key_bits = 1;
  while ((1 << key_bits) < num_experts) ++key_bits;
  const int64_t groups = M * (H / kGroup);
  if (want > 0) { // many slots: counting, then the scatter beside the quantisation
    int nchunks;
    int64_t cs;
    align_chunks(numel, &nchunks, &cs);
    int32_t *cnt = static_cast<int32_t *>(scratch);
    const size_t lds1 = static_cast<size_t>(num_experts) * 4;
    const size_t lds2 = (static_cast<size_t>(4 + 3) * num_experts + 1) * 4;
    int64_t qb = (groups + 15) / 16;
    if (qb > 8192) qb = 8192;
    const dim3 grid2(static_cast<unsigned>(nchunks + qb));
    if (ids_dtype == LO_I32) {
      hipLaunchKernelGGL(moe_align_count_kernel<int32_t>, dim3(nchunks), dim3(256), lds1, stream,
                         static_cast<const int32_t *>(topk_ids), numel, num_experts, expert_map, 0, cs, cnt, slot_mask,
                         nullptr, 1, sorted_ids, sorted_cap);
      hipLaunchKernelGGL(quant_align_scatter_kernel<int32_t>, grid2, dim3(256), lds2, stream,
                         static_cast<const uint16_t *>(x), groups, eps, q, qs, static_cast<const int32_t *>(topk_ids),
                         numel, num_experts, block_size, expert_map, cs, cnt, sorted_ids, sorted_cap, expert_ids,
                         expert_ids_cap, num_tokens_post_pad, key_bits, nchunks);
    } else {
      hipLaunchKernelGGL(moe_align_count_kernel<int64_t>, dim3(nchunks), dim3(256), lds1, stream,
                         static_cast<const int64_t *>(topk_ids), numel, num_experts, expert_map, 0, cs, cnt, slot_mask,
                         nullptr, 1, sorted_ids, sorted_cap);
      hipLaunchKernelGGL(quant_align_scatter_kernel<int64_t>, grid2, dim3(256), lds2, stream,
                         static_cast<const uint16_t *>(x), groups, eps, q, qs, static_cast<const int64_t *>(topk_ids),
                         numel, num_experts, block_size, expert_map, cs, cnt, sorted_ids, sorted_cap, expert_ids,
                         expert_ids_cap, num_tokens_post_pad, key_bits, nchunks);
    }
    return check_launch("quant_align(multi)");
  }
  int nw;
  size_t lds_bytes;
  single_wg_shape(numel, sorted_cap, num_experts, &nw, &lds_bytes);
  const int per_block = nw * kWave / 16;
  int64_t qblocks = (groups + per_block - 1) / per_block;
  if (qblocks > 4096) qblocks = 4096;
  const dim3 grid(static_cast<unsigned>(1 + qblocks)), block(nw * kWave);
  if (ids_dtype == LO_I32)
    hipLaunchKernelGGL(quant_align_kernel<int32_t>, grid, block, lds_bytes, stream, static_cast<const uint16_t *>(x),
                       groups, eps, q, qs, static_cast<const int32_t *>(topk_ids), numel, num_experts, block_size,
                       expert_map, sorted_ids, sorted_cap, expert_ids, expert_ids_cap, num_tokens_post_pad, key_bits,
                       slot_mask);
  else
    hipLaunchKernelGGL(quant_align_kernel<int64_t>, grid, block, lds_bytes, stream, static_cast<const uint16_t *>(x),
                       groups, eps, q, qs, static_cast<const int64_t *>(topk_ids), numel, num_experts, block_size,
                       expert_map, sorted_ids, sorted_cap, expert_ids, expert_ids_cap, num_tokens_post_pad, key_bits,
                       slot_mask);
  return check_launch("quant_align");
}

} // namespace lo

extern "C" int lo_moe_align_block_size(const void *topk_ids, int ids_dtype, int64_t numel,
                                       int32_t num_experts, int32_t block_size,
                                       const int32_t *expert_map, int ignore_invalid,
                                       int32_t *sorted_ids, int64_t sorted_cap,
                                       int32_t *expert_ids, int64_t expert_ids_cap,
                                       int32_t *num_tokens_post_pad, lo_stream_t stream) {
  return lo_moe_align_block_size_mask(topk_ids, ids_dtype, numel, num_experts, block_size, expert_map,
                                      ignore_invalid, sorted_ids, sorted_cap, expert_ids,
                                      expert_ids_cap, num_tokens_post_pad, nullptr, stream);
}

extern "C" int lo_moe_align_block_size_mask(const void *topk_ids, int ids_dtype, int64_t numel,
                                            int32_t num_experts, int32_t block_size,
                                            const int32_t *expert_map, int ignore_invalid,
                                            int32_t *sorted_ids, int64_t sorted_cap,
                                            int32_t *expert_ids, int64_t expert_ids_cap,
                                            int32_t *num_tokens_post_pad, uint8_t *slot_mask,
                                            lo_stream_t stream) {
  return lo_moe_align_block_size_ws(topk_ids, ids_dtype, numel, num_experts, block_size, expert_map,
                                    ignore_invalid, sorted_ids, sorted_cap, expert_ids, expert_ids_cap,
                                    num_tokens_post_pad, slot_mask, nullptr, 0, stream);
}

extern "C" int64_t lo_moe_align_scratch_bytes(int64_t numel, int32_t num_experts) {
  if (numel < 0 || num_experts < 1) return LO_EINVAL;
  if (numel < 8192) return 0; // one workgroup is faster below this
  int nchunks;
  int64_t cs;
  lo::align_chunks(numel, &nchunks, &cs);
  return static_cast<int64_t>(nchunks) * num_experts * 4;
}

extern "C" int lo_moe_align_block_size_ws(const void *topk_ids, int ids_dtype, int64_t numel,
                                          int32_t num_experts, int32_t block_size,
                                          const int32_t *expert_map, int ignore_invalid,
                                          int32_t *sorted_ids, int64_t sorted_cap,
                                          int32_t *expert_ids, int64_t expert_ids_cap,
                                          int32_t *num_tokens_post_pad, uint8_t *slot_mask,
                                          void *scratch, int64_t scratch_bytes, lo_stream_t stream) {
  return lo_moe_align_block_size_local(topk_ids, ids_dtype, numel, num_experts, block_size, expert_map,
                                       ignore_invalid, sorted_ids, sorted_cap, expert_ids, expert_ids_cap,
                                       num_tokens_post_pad, slot_mask, scratch, scratch_bytes, nullptr, 1,
                                       stream);
}

extern "C" int lo_moe_align_block_size_local(const void *topk_ids, int ids_dtype, int64_t numel,
                                             int32_t num_experts, int32_t block_size,
                                             const int32_t *expert_map, int ignore_invalid,
                                             int32_t *sorted_ids, int64_t sorted_cap,
                                             int32_t *expert_ids, int64_t expert_ids_cap,
                                             int32_t *num_tokens_post_pad, uint8_t *slot_mask,
                                             void *scratch, int64_t scratch_bytes,
                                             const int32_t *num_local_tokens, int32_t top_k,
                                             lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(!num_local_tokens || top_k >= 1, LO_EINVAL, "moe_align_block_size: top_k %d", top_k);
  LO_REQUIRE(topk_ids && sorted_ids && expert_ids && num_tokens_post_pad, LO_EINVAL,
             "moe_align_block_size: null pointer");
  LO_REQUIRE(ids_dtype == LO_I32 || ids_dtype == LO_I64, LO_EINVAL,
             "moe_align_block_size: topk_ids must be int32 or int64");
  LO_REQUIRE(numel >= 0 && numel < (1ll << 31) - 1, LO_EINVAL, "moe_align_block_size: bad numel %lld",
             (long long)numel);
  LO_REQUIRE(num_experts >= 1 && num_experts <= 2048, LO_EINVAL,
             "moe_align_block_size: num_experts %d outside [1, 2048]", num_experts);
  LO_REQUIRE(block_size >= 1, LO_EINVAL, "moe_align_block_size: block_size %d", block_size);
  int64_t need = numel + static_cast<int64_t>(num_experts) * (block_size - 1);
  if (numel < num_experts && numel * block_size < need) need = numel * block_size;
  LO_REQUIRE(sorted_cap >= need, LO_ENOSPC, "moe_align_block_size: sorted_ids holds %lld, needs %lld",
             (long long)sorted_cap, (long long)need);
  LO_REQUIRE(expert_ids_cap >= (need + block_size - 1) / block_size, LO_ENOSPC,
             "moe_align_block_size: expert_ids holds %lld, needs %lld", (long long)expert_ids_cap,
             (long long)((need + block_size - 1) / block_size));

  hipStream_t s = static_cast<hipStream_t>(stream);
  int key_bits = 1;
  while ((1 << key_bits) < num_experts) ++key_bits;
  const int64_t want = lo_moe_align_scratch_bytes(numel, num_experts);
  if (want > 0 && scratch && scratch_bytes >= want && (reinterpret_cast<uintptr_t>(scratch) & 3) == 0) {
    int nchunks;
    int64_t cs;
    align_chunks(numel, &nchunks, &cs);
    int32_t *cnt = static_cast<int32_t *>(scratch);
    const size_t lds1 = static_cast<size_t>(num_experts) * 4;
    const size_t lds2 = (static_cast<size_t>(4 + 3) * num_experts + 1) * 4;
    if (ids_dtype == LO_I32) {
      hipLaunchKernelGGL(moe_align_count_kernel<int32_t>, dim3(nchunks), dim3(256), lds1, s,
                         static_cast<const int32_t *>(topk_ids), numel, num_experts, expert_map,
                         ignore_invalid, cs, cnt, slot_mask, num_local_tokens, top_k, sorted_ids, sorted_cap);
      hipLaunchKernelGGL(moe_align_scatter_kernel<int32_t>, dim3(nchunks), dim3(256), lds2, s,
                         static_cast<const int32_t *>(topk_ids), numel, num_experts, block_size,
                         expert_map, ignore_invalid, cs, cnt, sorted_ids, sorted_cap, expert_ids,
                         expert_ids_cap, num_tokens_post_pad, key_bits, num_local_tokens, top_k);
    } else {
      hipLaunchKernelGGL(moe_align_count_kernel<int64_t>, dim3(nchunks), dim3(256), lds1, s,
                         static_cast<const int64_t *>(topk_ids), numel, num_experts, expert_map,
                         ignore_invalid, cs, cnt, slot_mask, num_local_tokens, top_k, sorted_ids, sorted_cap);
      hipLaunchKernelGGL(moe_align_scatter_kernel<int64_t>, dim3(nchunks), dim3(256), lds2, s,
                         static_cast<const int64_t *>(topk_ids), numel, num_experts, block_size,
                         expert_map, ignore_invalid, cs, cnt, sorted_ids, sorted_cap, expert_ids,
                         expert_ids_cap, num_tokens_post_pad, key_bits, num_local_tokens, top_k);
    }
    return check_launch("moe_align_block_size(multi)");
  }

  int nw;
  size_t lds_bytes;
  single_wg_shape(numel, sorted_cap, num_experts, &nw, &lds_bytes);
  if (ids_dtype == LO_I32)
    hipLaunchKernelGGL(moe_align_kernel<int32_t>, dim3(1), dim3(nw * kWave), lds_bytes, s,
                       static_cast<const int32_t *>(topk_ids), numel, num_experts, block_size,
                       expert_map, ignore_invalid, sorted_ids, sorted_cap, expert_ids,
                       expert_ids_cap, num_tokens_post_pad, key_bits, slot_mask, num_local_tokens, top_k);
  else
    hipLaunchKernelGGL(moe_align_kernel<int64_t>, dim3(1), dim3(nw * kWave), lds_bytes, s,
                       static_cast<const int64_t *>(topk_ids), numel, num_experts, block_size,
                       expert_map, ignore_invalid, sorted_ids, sorted_cap, expert_ids,
                       expert_ids_cap, num_tokens_post_pad, key_bits, slot_mask, num_local_tokens, top_k);
  return check_launch("moe_align_block_size");
}
