// Capacity-bounded slot assignment with Batch Priority Routing for gfx950.
//
// Replaces vmoe/moe.py:568-589 (+ :646-648): the reference sorts items by their
// first-choice gate, flattens the (K, S) choices K-major, takes a one-hot over
// experts and a cumulative sum down the K*S rows.  Here one workgroup owns a
// group and works entirely in LDS:
//   1. 64-bit keys (descending-gate order bits << 32 | item) are bitonic-sorted;
//      the item index in the low word makes the order stable by construction.
//      The keys stay in registers (R consecutive keys per thread): exchanges at
//      distances below R are register moves, below 64*R lane exchanges, and only
//      the few stages beyond that go through LDS with barriers;
//   2. every (item, choice) sets bit  k*S + rank(item)  in its expert's bitmap
//      (integer LDS atomics: order-independent result);
//   3. an exclusive prefix of per-word popcounts turns "how many set bits come
//      before mine" -- the cumsum of the one-hot column -- into one table
//      lookup plus one masked popcount.
// The kernel also emits the two maps the data-movement kernels use: item ->
// slot row (-1 when over capacity) and slot row -> item (-1 when empty).
#include <mutex>
#include "vmoe_common.h"
#include "router_metrics.h"
#include "compact_rows.h"

namespace vmoe {
namespace {

constexpr int kRouteThreads = 1024;

__host__ __device__ inline int pow2ceil(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

// One side of a compare-exchange: the smaller (take_min) or larger of two keys.
template <typename KeyT>
__device__ __forceinline__ KeyT pick(KeyT mine, KeyT other, bool take_min) {
  return ((other < mine) == take_min) ? other : mine;
}

__device__ __forceinline__ uint64_t lane_exchange(uint64_t v, int lane_xor) {
  return __shfl_xor((unsigned long long)v, lane_xor, kWave);
}
__device__ __forceinline__ uint32_t lane_exchange(uint32_t v, int lane_xor) {
  return __shfl_xor(v, lane_xor, kWave);
}

template <int R, int ST, typename KeyT>
__device__ __forceinline__ void bitonic_in_thread(KeyT (&key)[R], int size, int tid) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if ((r & ST) == 0 && r + ST < R) {
      const bool up = (((tid * R + r) & size) == 0);
      const KeyT a = key[r], b = key[r + ST];
      const bool swap = (b < a) == up;
      key[r] = swap ? b : a;
      key[r + ST] = swap ? a : b;
    }
  }
}

// Ascending bitonic sort of SP (a power of two) keys, element tid*R + r in key[r] of
// thread tid < nact = SP / R.  Every thread of the workgroup calls it (the LDS stages
// have barriers); `xch` holds SP keys.
template <int R, typename KeyT>
__device__ __forceinline__ void bitonic_sort_regs(KeyT (&key)[R], KeyT* xch, int SP, int tid,
                                                  int nact) {
  const bool act = tid < nact;
  for (int size = 2; size <= SP; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      if (stride >= 64 * R) {
        if (act) {
#pragma unroll
          for (int r = 0; r < R; ++r) xch[tid * R + r] = key[r];
        }
        __syncthreads();
        if (act) {
#pragma unroll
          for (int r = 0; r < R; ++r) {
            const int i = tid * R + r;
            key[r] = pick<KeyT>(key[r], xch[i ^ stride], ((i & stride) == 0) == ((i & size) == 0));
          }
        }
        __syncthreads();
      } else if (!act) {
        continue;
      } else if (stride >= R) {
        const int lane_xor = stride / R;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int i = tid * R + r;
          const KeyT other = lane_exchange(key[r], lane_xor);
          key[r] = pick(key[r], other, ((i & stride) == 0) == ((i & size) == 0));
        }
      } else {
        if constexpr (R > 4) { if (stride == 4) bitonic_in_thread<R, 4, KeyT>(key, size, tid); }
        if constexpr (R > 2) { if (stride == 2) bitonic_in_thread<R, 2, KeyT>(key, size, tid); }
        if constexpr (R > 1) { if (stride == 1) bitonic_in_thread<R, 1, KeyT>(key, size, tid); }
      }
    }
  }
}

// Keys per thread for a sort of SP keys: as many threads as the workgroup has take part
// (a stage costs a wave its shuffles and selects per key, so more waves with fewer keys
// are faster: eight keys on an eighth of the threads took 35 us where two keys on all
// take 25); 0 = the keys do not fit in the registers and are sorted in LDS.
inline int keys_per_thread(int SP) {
  const int r = SP <= kRouteThreads ? 1 : SP / kRouteThreads;
  return r <= 8 ? r : 0;
}

// The same sort with the keys resident in LDS (any SP).
__device__ __forceinline__ void bitonic_sort_lds(uint64_t* keys, int SP, int tid) {
  for (int size = 2; size <= SP; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int t = tid; t < (SP >> 1); t += kRouteThreads) {
        int lo = 2 * t - (t & (stride - 1));
        int hi = lo + stride;
        bool up = (lo & size) == 0;
        uint64_t a = keys[lo], b = keys[hi];
        if ((a > b) == up) { keys[lo] = b; keys[hi] = a; }
      }
      __syncthreads();
    }
  }
}

constexpr int kRankBins = 1024;    // bins of the counting rank: gates from 1 down to 2^-8

template <int R>
__device__ __forceinline__ void route_assign_group(
    const float* __restrict__ topk_val, const int32_t* __restrict__ topk_idx,
    int32_t* __restrict__ indices, int32_t* __restrict__ token_slot,
    int32_t* __restrict__ slot_token, int32_t* __restrict__ fill, int G, int S, int E, int K,
    int C, int bpr, int SP, int NK, int W, int g, unsigned char* smem) {
  // Layout: keys[NK] (u64, only with bpr) | bitmap[E*W] | prefix[E*W] | rank[S] | total[E]
  uint64_t* keys = reinterpret_cast<uint64_t*>(smem);
  uint32_t* bitmap = reinterpret_cast<uint32_t*>(smem + (bpr ? (size_t)NK * 8 : 0));
  uint32_t* prefix = bitmap + (size_t)E * W;
  int32_t* rank = reinterpret_cast<int32_t*>(prefix + (size_t)E * W);
  int32_t* total = rank + S;
  const int tid = threadIdx.x;
  const float* val = topk_val + (size_t)g * S * K;
  const int32_t* idx = topk_idx + (size_t)g * S * K;

  for (int i = tid; i < E * W; i += kRouteThreads) bitmap[i] = 0u;
  if (bpr) {
    if constexpr (R == 0) {
      for (int s = tid; s < SP; s += kRouteThreads) {
        uint64_t key = ~0ull;
        if (s < S) key = bpr_key64(__builtin_bit_cast(uint32_t, val[(size_t)s * K]), s);
        keys[s] = key;
      }
      __syncthreads();
      bitonic_sort_lds(keys, SP, tid);
      for (int r = tid; r < S; r += kRouteThreads) rank[(uint32_t)keys[r]] = r;
    } else {
      // Gates that came out of a bfloat16 router are non-negative floats whose low 16
      // bits are zero: gate and item index then fit one 32-bit key (S <= 65536), and the
      // sort's compare-exchanges, which are what bounds this kernel, cost half as much.
      const int nact = SP / R;
      uint32_t bits[R];
      bool narrow_ok = S <= 65536;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int s = tid * R + r;
        bits[r] = (tid < nact && s < S) ? __builtin_bit_cast(uint32_t, val[(size_t)s * K]) : 0u;
        narrow_ok = narrow_ok && bpr_gate_is_narrow(bits[r]);
      }
      // Narrow gates within a factor 2^8 of 1 (the largest gate of a softmax over up to 128
      // experts always is) take at most kRankBins distinct values, in descending order as
      // the bin number 0x3F80 - (bits >> 16) ascends: the rank of an item is then the number
      // of items in lower bins plus the number of items of its own bin with a lower index
      // -- a histogram, a prefix sum, a scatter into the bins' segments and a count inside
      // the item's own segment, four barriers in all, where the bitonic sort of 2 048 keys
      // takes 66 compare-exchange steps (15 of the kernel's 22 us on the headline layer).
      // Every step counts, none depends on the order in which the threads arrive, so the
      // ranks are those of the sort.  A segment as long as the group (all gates equal) costs
      // what the sort costs.
      bool count_ok = narrow_ok;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint32_t hi = bits[r] >> 16;
        if (tid < nact && tid * R + r < S) count_ok = count_ok && hi <= 0x3F80u && hi + kRankBins > 0x3F80u;
      }
      if (__syncthreads_and(count_ok)) {
        uint32_t* hist = reinterpret_cast<uint32_t*>(keys);      // items per bin, then the bins' cursors
        uint32_t* start = hist + kRankBins;                      // first rank of each bin
        uint32_t* seg = start + kRankBins;                       // S items, bin by bin
        for (int i = tid; i < kRankBins; i += kRouteThreads) hist[i] = 0u;
        __syncthreads();
        int bin[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          bin[r] = (int)(0x3F80u - (bits[r] >> 16));
          if (tid < nact && tid * R + r < S) atomicAdd(&hist[bin[r]], 1u);
        }
        __syncthreads();
        // Exclusive prefix over the bins: kRankBins == kRouteThreads, one bin per thread.
        {
          static_assert(kRankBins == kRouteThreads, "one bin per thread");
          const int lane = tid & 63, wave = tid >> 6;
          const uint32_t c = hist[tid];
          uint32_t incl = c;
#pragma unroll
          for (int d = 1; d < 64; d <<= 1) {
            const uint32_t o = __shfl_up(incl, d, kWave);
            if (lane >= d) incl += o;
          }
          __shared__ uint32_t wave_total[kRouteThreads / 64];
          if (lane == 63) wave_total[wave] = incl;
          __syncthreads();
          uint32_t before = 0;
          for (int w = 0; w < wave; ++w) before += wave_total[w];
          start[tid] = before + incl - c;
          hist[tid] = before + incl - c;                       // cursor of the scatter
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r)
          if (tid < nact && tid * R + r < S) seg[atomicAdd(&hist[bin[r]], 1u)] = (uint32_t)(tid * R + r);
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int item = tid * R + r;
          if (tid < nact && item < S) {
            const uint32_t first = start[bin[r]], end = hist[bin[r]];
            uint32_t lower = 0;
            for (uint32_t q = first; q < end; ++q) lower += seg[q] < (uint32_t)item ? 1u : 0u;
            rank[item] = (int)(first + lower);
          }
        }
      } else if (__syncthreads_and(narrow_ok)) {
        uint32_t key[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int s = tid * R + r;
          key[r] = s < S ? bpr_key32(bits[r], s) : ~0u;
        }
        bitonic_sort_regs<R, uint32_t>(key, reinterpret_cast<uint32_t*>(keys), SP, tid, nact);
#pragma unroll
        for (int r = 0; r < R; ++r)
          if (tid < nact && tid * R + r < S) rank[key[r] & 0xffffu] = tid * R + r;
      } else {
        uint64_t key[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int s = tid * R + r;
          key[r] = s < S ? bpr_key64(bits[r], s) : ~0ull;
        }
        bitonic_sort_regs<R, uint64_t>(key, keys, SP, tid, nact);
#pragma unroll
        for (int r = 0; r < R; ++r)
          if (tid < nact && tid * R + r < S) rank[(uint32_t)key[r]] = tid * R + r;
      }
    }
  } else {
    for (int s = tid; s < S; s += kRouteThreads) rank[s] = s;
  }
  __syncthreads();

  const int SK = S * K;
  for (int i = tid; i < SK; i += kRouteThreads) {
    int s = i / K, k = i - s * K;
    int e = idx[i];
    if (e >= 0 && e < E) {
      const int bit = choice_bit(k, S, rank[s]);
      atomicOr(&bitmap[(size_t)e * W + (bit >> 5)], 1u << (bit & 31));
    }
  }
  __syncthreads();
  // Exclusive prefix of popcounts per expert: one wave per expert, 64 words per step.
  {
    const int lane = tid & 63, wave = tid >> 6, nwaves = kRouteThreads >> 6;
    for (int e = wave; e < E; e += nwaves) {
      int carry = 0;
      for (int w0 = 0; w0 < W; w0 += 64) {
        int w = w0 + lane;
        int c = w < W ? __popc(bitmap[(size_t)e * W + w]) : 0;
        int incl = c;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          int o = __shfl_up(incl, d, kWave);
          if (lane >= d) incl += o;
        }
        if (w < W) prefix[(size_t)e * W + w] = (uint32_t)(carry + incl - c);
        carry += __shfl(incl, 63, kWave);
      }
      if (lane == 0) total[e] = carry;
    }
  }
  __syncthreads();

  for (int i = tid; i < SK; i += kRouteThreads) {
    int s = i / K, k = i - s * K;
    int e = idx[i];
    int pos = -1, slot = -1;
    if (e >= 0 && e < E) {
      const int bit = choice_bit(k, S, rank[s]);
      const int w = bit >> 5;
      pos = position_from_bitmap(prefix[(size_t)e * W + w], bitmap[(size_t)e * W + w], bit);
      if (pos < C) {
        slot = slot_row(e, g, pos, G, E, C);
        slot_token[slot] = g * S + s;
      }
    }
    size_t o = (size_t)g * SK + i;
    indices[2 * o] = e;
    indices[2 * o + 1] = pos;
    token_slot[o] = slot;
  }
  // Slots nobody claimed.
  for (int i = tid; i < E * C; i += kRouteThreads) {
    int e = i / C, c = i - e * C;
    if (c >= total[e]) slot_token[slot_row(e, g, c, G, E, C)] = -1;
  }
  if (fill != nullptr)
    for (int e = tid; e < E; e += kRouteThreads) fill[(size_t)g * E + e] = total[e] < C ? total[e] : C;
}

template <int R>
__global__ __launch_bounds__(kRouteThreads) void route_assign_kernel(
    const float* __restrict__ topk_val, const int32_t* __restrict__ topk_idx,
    int32_t* __restrict__ indices, int32_t* __restrict__ token_slot,
    int32_t* __restrict__ slot_token, int32_t* __restrict__ fill, int G, int S, int E, int K,
    int C, int bpr, int SP, int NK, int W) {
  extern __shared__ __align__(16) unsigned char smem[];
  route_assign_group<R>(topk_val, topk_idx, indices, token_slot, slot_token, fill, G, S, E, K, C,
                        bpr, SP, NK, W, blockIdx.x, smem);
}

// Slot assignment and the router's auxiliary losses in one launch: workgroups 0 .. G-1
// assign slots, workgroups G .. 2G-1 compute the losses of group blockIdx.x - G.  Both
// are one workgroup per group, bound by latency, and read the same top-k output, so side
// by side they take the time of the longer one.
template <int R, typename T>
__global__ __launch_bounds__(kRouteThreads) void route_assign_metrics_kernel(
    const float* __restrict__ topk_val, const int32_t* __restrict__ topk_idx,
    int32_t* __restrict__ indices, int32_t* __restrict__ token_slot,
    int32_t* __restrict__ slot_token, int32_t* __restrict__ fill, int G, int S, int E, int K,
    int C, int bpr, int SP, int NK, int W, RouterMetricsArgs m) {
  extern __shared__ __align__(16) unsigned char smem[];
  static_assert(kRouteThreads == kMetricThreads, "both roles use the launch's workgroup size");
  if ((int)blockIdx.x < G) {
    route_assign_group<R>(topk_val, topk_idx, indices, token_slot, slot_token, fill, G, S, E, K,
                          C, bpr, SP, NK, W, blockIdx.x, smem);
  } else {
    router_metrics_group<T>(static_cast<const T*>(m.gates), m.top1, m.imp_loss, m.gsh_loss,
                            m.aux_loss, m.w_gsh, m.w_imp, m.S, m.E, m.top1_stride, m.V,
                            (int)blockIdx.x - G, smem);
  }
}

// Experts-choice routing (vmoe/moe.py:655-694): every expert takes the C items
// with its largest gates (jax.lax.top_k over the transposed gates: descending,
// equal gates -> lower item index first).  One workgroup per (expert, group)
// sorts the S keys (descending-gate order bits << 32 | item) of that column in
// LDS; the rank of an item is its position, kept when rank < C.  The outputs are
// those of the slot-assignment kernel with one "choice" per expert (K = E), so
// the same dispatch / combine kernels serve both routing schemes.
template <typename T, int R>
__global__ __launch_bounds__(kRouteThreads) void top_items_kernel(
    const T* __restrict__ gates, int32_t* __restrict__ indices, int32_t* __restrict__ token_slot,
    int32_t* __restrict__ slot_token, float* __restrict__ weights, float* __restrict__ sel_minmax,
    int G, int S, int E, int C, int SP) {
  extern __shared__ __align__(16) unsigned char smem[];
  uint64_t* keys = reinterpret_cast<uint64_t*>(smem);
  const int tid = threadIdx.x;
  const int e = blockIdx.x, g = blockIdx.y;
  const T* col = gates + (size_t)g * S * E + e;
  const int last = (C < S ? C : S) - 1;
  // Rank r of the column holds item s: the outputs of that (item, expert) pair.
  auto emit = [&](int r, int s) {
    const size_t o = ((size_t)g * S + s) * E + e;
    int slot = -1;
    if (r < C) {
      slot = slot_row(e, g, r, G, E, C);
      slot_token[slot] = g * S + s;
    }
    indices[2 * o] = e;
    indices[2 * o + 1] = r;
    token_slot[o] = slot;
    const T gate = col[(size_t)s * E];
    weights[o] = Elt<T>::load(&gate);
    if (sel_minmax != nullptr) {
      if (r == last) sel_minmax[((size_t)g * E + e) * 2] = Elt<T>::load(&gate);
      if (r == 0) sel_minmax[((size_t)g * E + e) * 2 + 1] = Elt<T>::load(&gate);
    }
  };
  if constexpr (R == 0) {
    for (int s = tid; s < SP; s += kRouteThreads) {
      uint64_t key = ~0ull;
      if (s < S) key = bpr_key64(__builtin_bit_cast(uint32_t, Elt<T>::load(col + (size_t)s * E)), s);
      keys[s] = key;
    }
    __syncthreads();
    bitonic_sort_lds(keys, SP, tid);
    for (int r = tid; r < S; r += kRouteThreads) emit(r, (int)(uint32_t)keys[r]);
  } else {
    const int nact = SP / R;
    uint64_t key[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int s = tid * R + r;
      key[r] = (tid < nact && s < S)
                   ? bpr_key64(__builtin_bit_cast(uint32_t, Elt<T>::load(col + (size_t)s * E)), s)
                   : ~0ull;
    }
    bitonic_sort_regs<R, uint64_t>(key, keys, SP, tid, nact);
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (tid < nact && tid * R + r < S) emit(tid * R + r, (int)(uint32_t)key[r]);
  }
  for (int c = S + tid; c < C; c += kRouteThreads) slot_token[slot_row(e, g, c, G, E, C)] = -1;
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* p, size_t n, int32_t v) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

__global__ __launch_bounds__(256) void indices_to_slots_kernel(
    const int32_t* __restrict__ indices, int32_t* __restrict__ token_slot,
    int32_t* __restrict__ slot_token, int32_t* __restrict__ num_dup, int32_t* __restrict__ num_inv,
    int G, int S, int E, int K, int C) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t n = (size_t)G * S * K;
  if (i >= n) return;
  const size_t item = i / K;
  bool invalid;
  const int slot = slot_of_index_pair(indices[2 * i], indices[2 * i + 1], (int)(item / S), G, E, C,
                                      &invalid);
  if (invalid) atomicAdd(num_inv, 1);
  if (slot >= 0) {
    const int prev = atomicExch(&slot_token[slot], (int)item);
    if (prev >= 0) atomicAdd(num_dup, 1);
  }
  token_slot[i] = slot;
}

__global__ __launch_bounds__(256) void densify_kernel(
    const int32_t* __restrict__ indices, const float* __restrict__ weights,
    float* __restrict__ combine, uint8_t* __restrict__ dispatch, int G, int S, int E, int K, int C) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t n = (size_t)G * S * K;
  if (i >= n) return;
  int e = indices[2 * i], c = indices[2 * i + 1];
  if (e < 0 || c < 0 || e >= E || c >= C) return;
  size_t item = i / K;
  size_t o = (item * E + e) * C + c;
  if (combine != nullptr) combine[o] = weights[i];
  if (dispatch != nullptr) dispatch[o] = 1;
}


// Packed expert rows, step 1: exclusive prefix over the groups of fill[:, e], one
// workgroup per expert; the total is the expert's row count.
__global__ __launch_bounds__(256) void fill_prefix_kernel(
    const int32_t* __restrict__ fill, int32_t* __restrict__ prefix,
    int32_t* __restrict__ rows_per_expert, int G, int E) {
  __shared__ int32_t wsum[4];
  const int e = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int carry = 0;
  for (int g0 = 0; g0 < G; g0 += 256) {
    const int g = g0 + tid;
    const int v = g < G ? fill[(size_t)g * E + e] : 0;
    int x = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int y = __shfl_up(x, o, kWave);
      if (lane >= o) x += y;
    }
    if (lane == 63) wsum[wave] = x;
    __syncthreads();
    int woff = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (w < wave) woff += wsum[w];
      total += wsum[w];
    }
    if (g < G) prefix[(size_t)g * E + e] = carry + woff + x - v;
    carry += total;
    __syncthreads();
  }
  if (tid == 0) rows_per_expert[e] = carry;
}

// Step 2: token_slot = e*G*C + r(g, c)  ->  token_row = e*G*C + prefix[g][e] + c.
__global__ __launch_bounds__(256) void compact_rows_kernel(
    const int32_t* __restrict__ prefix, const int32_t* __restrict__ token_slot,
    int32_t* __restrict__ token_row, int32_t* __restrict__ row_token, int G, int E, int C,
    int per_group, int K, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int slot = token_slot[i];
  int row = -1;
  if (slot >= 0) {
    const int g = (int)(i / per_group);
    row = packed_row(slot, prefix[(size_t)g * E + slot_expert(slot, G, C)], G, C);
    if (row_token != nullptr) row_token[row] = (int)(i / K);
  }
  token_row[i] = row;
}

// Both steps in one launch, for E <= 256 and at least 256 assignments per group (a
// workgroup then touches at most two groups): the workgroup adds up the fill counts of
// the groups before its first group itself -- 256 / E threads per expert, each a strided
// share of the groups, joined in LDS -- instead of reading a prefix that another launch
// wrote.  Workgroup 0 also writes the experts' row counts.
__global__ __launch_bounds__(256) void compact_rows_fused_kernel(
    const int32_t* __restrict__ fill, const int32_t* __restrict__ token_slot,
    int32_t* __restrict__ token_row, int32_t* __restrict__ row_token,
    int32_t* __restrict__ rows_per_expert, int G, int E, int C, int per_group, int K, size_t n) {
  compact_rows_fused_block(fill, token_slot, token_row, row_token, rows_per_expert, G, E, C,
                           per_group, K, n, blockIdx.x);
}

}  // namespace
}  // namespace vmoe

using namespace vmoe;

static int check_route_shapes(int G, int S, int E, int K, int C) {
  if (G < 1 || S < 1 || E < 1 || K < 1 || C < 1 || K > E) return VMOE_E_SHAPE;
  if ((int64_t)G * S * K * 2 >= INT32_MAX || (int64_t)E * G * C >= INT32_MAX) return VMOE_E_OVERFLOW;
  return VMOE_OK;
}

static int check_route_assign(const VmoeRouteAssignParams* p) {
  if (p == nullptr || p->topk_idx == nullptr || p->indices == nullptr ||
      p->token_slot == nullptr || p->slot_token == nullptr)
    return VMOE_E_NULL;
  if (p->batch_priority && p->topk_val == nullptr) return VMOE_E_NULL;
  return check_route_shapes(p->G, p->S, p->E, p->K, p->C);
}

// Launches the slot assignment, with the router's losses as extra workgroups when m is given.
static int launch_route_assign(const VmoeRouteAssignParams* p, const VmoeRouterMetricsParams* m,
                               vmoe_stream_t stream) {
  const int SP = pow2ceil(p->S);
  const int W = (p->S * p->K + 31) / 32;
  const int R = keys_per_thread(SP);
  // (the region of the sort keys also serves the counting rank: two arrays of kRankBins
  // words and one of S)
  const int rank_words = 2 * kRankBins + p->S;
  const int NK = SP > (rank_words + 1) / 2 ? SP : (rank_words + 1) / 2;
  size_t lds = (p->batch_priority ? (size_t)NK * 8 : 0) + (size_t)p->E * W * 8 +
               (size_t)p->S * 4 + (size_t)p->E * 4;
  RouterMetricsArgs ma{};
  if (m != nullptr) {
    size_t mlds;
    int V;
    if (!router_metrics_geometry(m, &V, &mlds)) return VMOE_E_UNSUPPORTED;
    if (mlds > lds) lds = mlds;
    ma = RouterMetricsArgs{m->gates, m->top1_idx, m->importance_loss, m->gshard_loss,
                           m->auxiliary_loss, m->gshard_loss_weight, m->importance_loss_weight,
                           m->S, m->E, m->top1_stride, V};
  }
  if (lds > 160 * 1024) return VMOE_E_UNSUPPORTED;
  auto launch = [&](auto kern, auto... extra) -> int {
    hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, dim3(m != nullptr ? 2 * p->G : p->G), dim3(kRouteThreads), lds,
                       as_stream(stream), p->topk_val, p->topk_idx, p->indices, p->token_slot,
                       p->slot_token, p->fill, p->G, p->S, p->E, p->K, p->C,
                       p->batch_priority ? 1 : 0, SP, NK, W, extra...);
    return launch_status();
  };
  if (m == nullptr) {
    switch (R) {
      case 1: return launch(route_assign_kernel<1>);
      case 2: return launch(route_assign_kernel<2>);
      case 4: return launch(route_assign_kernel<4>);
      case 8: return launch(route_assign_kernel<8>);
      default: return launch(route_assign_kernel<0>);
    }
  }
  if (m->dtype == VMOE_BF16) {
    switch (R) {
      case 1: return launch(route_assign_metrics_kernel<1, bf16_t>, ma);
      case 2: return launch(route_assign_metrics_kernel<2, bf16_t>, ma);
      case 4: return launch(route_assign_metrics_kernel<4, bf16_t>, ma);
      case 8: return launch(route_assign_metrics_kernel<8, bf16_t>, ma);
      default: return launch(route_assign_metrics_kernel<0, bf16_t>, ma);
    }
  }
  switch (R) {
    case 1: return launch(route_assign_metrics_kernel<1, float>, ma);
    case 2: return launch(route_assign_metrics_kernel<2, float>, ma);
    case 4: return launch(route_assign_metrics_kernel<4, float>, ma);
    case 8: return launch(route_assign_metrics_kernel<8, float>, ma);
    default: return launch(route_assign_metrics_kernel<0, float>, ma);
  }
}

extern "C" int vmoe_route_assign(const VmoeRouteAssignParams* p, vmoe_stream_t stream) {
  int rc = check_route_assign(p);
  if (rc != VMOE_OK) return rc;
  return launch_route_assign(p, nullptr, stream);
}

extern "C" int vmoe_route_assign_metrics(const VmoeRouteAssignParams* p,
                                         const VmoeRouterMetricsParams* m, vmoe_stream_t stream) {
  int rc = check_route_assign(p);
  if (rc != VMOE_OK) return rc;
  rc = check_router_metrics(m);
  if (rc != VMOE_OK) return rc;
  if (m->G != p->G || m->S != p->S || m->E != p->E) return VMOE_E_SHAPE;
  return launch_route_assign(p, m, stream);
}

extern "C" int vmoe_indices_to_slots(const VmoeIndicesToSlotsParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->indices == nullptr || p->token_slot == nullptr ||
      p->slot_token == nullptr || p->num_duplicates == nullptr || p->num_invalid == nullptr)
    return VMOE_E_NULL;
  if (p->G < 1 || p->S < 1 || p->E < 1 || p->K < 1 || p->C < 1) return VMOE_E_SHAPE;
  if ((int64_t)p->G * p->S * p->K * 2 >= INT32_MAX || (int64_t)p->E * p->G * p->C >= INT32_MAX)
    return VMOE_E_OVERFLOW;
  const size_t ns = (size_t)p->E * p->G * p->C;
  const size_t n = (size_t)p->G * p->S * p->K;
  hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)((ns + 255) / 256)), dim3(256), 0,
                     as_stream(stream), p->slot_token, ns, -1);
  hipLaunchKernelGGL(indices_to_slots_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     as_stream(stream), p->indices, p->token_slot, p->slot_token,
                     p->num_duplicates, p->num_invalid, p->G, p->S, p->E, p->K, p->C);
  return launch_status();
}

extern "C" int vmoe_densify(const VmoeDensifyParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->indices == nullptr) return VMOE_E_NULL;
  if (p->combine != nullptr && p->weights == nullptr) return VMOE_E_NULL;
  if (p->G < 1 || p->S < 1 || p->E < 1 || p->K < 1 || p->C < 1) return VMOE_E_SHAPE;
  const size_t n = (size_t)p->G * p->S * p->K;
  hipLaunchKernelGGL(densify_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     as_stream(stream), p->indices, p->weights, p->combine, p->dispatch, p->G,
                     p->S, p->E, p->K, p->C);
  return launch_status();
}

extern "C" int vmoe_top_items_per_expert(const VmoeTopItemsParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->gates == nullptr || p->indices == nullptr || p->token_slot == nullptr ||
      p->slot_token == nullptr || p->weights == nullptr)
    return VMOE_E_NULL;
  if (p->G < 1 || p->S < 1 || p->E < 1 || p->C < 1) return VMOE_E_SHAPE;
  if (p->dtype != VMOE_F32 && p->dtype != VMOE_BF16) return VMOE_E_DTYPE;
  if (p->G > 65535) return VMOE_E_UNSUPPORTED;
  if ((int64_t)p->E * p->G * p->C >= INT32_MAX || (int64_t)p->G * p->S * p->E >= INT32_MAX)
    return VMOE_E_OVERFLOW;
  const int SP = pow2ceil(p->S < 2 ? 2 : p->S);
  const int R = keys_per_thread(SP);
  const size_t lds = (size_t)SP * 8;
  if (lds > 160 * 1024) return VMOE_E_UNSUPPORTED;
  dim3 grid(p->E, p->G);
  auto launch = [&](auto kern, auto* gates) -> int {
    hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, grid, dim3(kRouteThreads), lds, as_stream(stream), gates, p->indices,
                       p->token_slot, p->slot_token, p->weights, p->sel_minmax, p->G, p->S, p->E,
                       p->C, SP);
    return launch_status();
  };
  if (p->dtype == VMOE_BF16) {
    const bf16_t* gates = (const bf16_t*)p->gates;
    switch (R) {
      case 1: return launch(top_items_kernel<bf16_t, 1>, gates);
      case 2: return launch(top_items_kernel<bf16_t, 2>, gates);
      case 4: return launch(top_items_kernel<bf16_t, 4>, gates);
      case 8: return launch(top_items_kernel<bf16_t, 8>, gates);
      default: return launch(top_items_kernel<bf16_t, 0>, gates);
    }
  }
  const float* gates = (const float*)p->gates;
  switch (R) {
    case 1: return launch(top_items_kernel<float, 1>, gates);
    case 2: return launch(top_items_kernel<float, 2>, gates);
    case 4: return launch(top_items_kernel<float, 4>, gates);
    case 8: return launch(top_items_kernel<float, 8>, gates);
    default: return launch(top_items_kernel<float, 0>, gates);
  }
}

// Launches the row compaction with `prefix` as the (G, E) scratch of its two-launch form.
static int launch_compact_rows(const VmoeCompactRowsParams* p, int32_t* prefix,
                               vmoe_stream_t stream) {
  const size_t n = (size_t)p->G * p->S * p->K;
  if (compact_rows_fused_ok(p->G, p->S, p->E, p->K)) {
    hipLaunchKernelGGL(compact_rows_fused_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       as_stream(stream), p->fill, p->token_slot, p->token_row, p->row_token,
                       p->rows_per_expert, p->G, p->E, p->C, p->S * p->K, p->K, n);
    return launch_status();
  }
  hipLaunchKernelGGL(fill_prefix_kernel, dim3(p->E), dim3(256), 0, as_stream(stream), p->fill,
                     prefix, p->rows_per_expert, p->G, p->E);
  hipLaunchKernelGGL(compact_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     as_stream(stream), prefix, p->token_slot, p->token_row, p->row_token, p->G,
                     p->E, p->C, p->S * p->K, p->K, n);
  return launch_status();
}

static int check_compact_rows(const VmoeCompactRowsParams* p) {
  if (p == nullptr || p->fill == nullptr || p->token_slot == nullptr || p->token_row == nullptr ||
      p->rows_per_expert == nullptr)
    return VMOE_E_NULL;
  return check_route_shapes(p->G, p->S, p->E, p->K, p->C);
}

extern "C" int vmoe_compact_rows(const VmoeCompactRowsParams* p, vmoe_stream_t stream) {
  int rc = check_compact_rows(p);
  if (rc != VMOE_OK) return rc;
  if (p->prefix == nullptr) return VMOE_E_NULL;
  return launch_compact_rows(p, p->prefix, stream);
}

// ---------------------------------------------------------------- no allocation
// vmoe_compact_rows for callers that cannot allocate: the (G, E) scratch is a file-scope
// device array.  Its name is only a host-side handle; the device address is asked for once
// per device (each device holds its own copy) and only that address is given to kernels.
static __device__ __align__(256) int32_t scratch[VMOE_COMPACT_ROWS_STATIC_MAX_GE];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
int32_t* scratch_ptr[kMaxDevices];   // device address of `scratch` on each device, null until asked
}  // namespace

// Device address of this device's copy of `scratch` (the current device), or null with *err set.
static int32_t* scratch_address(int* err) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { *err = (int)e; return nullptr; }
  if (dev < 0 || dev >= kMaxDevices) { *err = VMOE_E_UNSUPPORTED; return nullptr; }
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      *err = e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
      return nullptr;
    }
    scratch_ptr[dev] = static_cast<int32_t*>(ptr);
  }
  return scratch_ptr[dev];
}

extern "C" int vmoe_compact_rows_static(const VmoeCompactRowsParams* p, vmoe_stream_t stream) {
  int rc = check_compact_rows(p);
  if (rc != VMOE_OK) return rc;
  if ((int64_t)p->G * p->E > VMOE_COMPACT_ROWS_STATIC_MAX_GE) return VMOE_E_WORKSPACE;
  int err = VMOE_OK;
  int32_t* prefix = scratch_address(&err);
  if (prefix == nullptr) return err;
  // Every entry of the scratch that the second launch reads (g < G, e < E) is written by the
  // first one: nothing has to start at zero, whatever an earlier call left behind.
  return launch_compact_rows(p, prefix, stream);
}
