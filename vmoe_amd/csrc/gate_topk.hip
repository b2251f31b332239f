// Fused router gating for gfx950: logits = x @ W on the matrix cores, softmax
// over experts and top-K selection in registers with cross-lane reductions.
//
// Replaces vmoe/nn/routing.py:73-80 and the jax.lax.top_k of vmoe/moe.py:567.
//
// Work split: a wave owns a tile of 32 items.  The router kernel W (D x E) is
// staged once per workgroup in LDS (bf16: transposed to [expert][k] so that a
// lane's MFMA B fragment is one 16-byte read; f32: kept [k][expert]).  Item rows
// stream from HBM with 16-byte loads, 64 contiguous bytes per lane per step; in
// bf16 they pass through two register buffers that are refilled as soon as their
// MFMAs are issued, and the first loads go out before the router kernel is staged,
// so that every workgroup of the launch is resident and loading from the start.
// After the K loop the logits tile passes through a wave-private LDS tile, so
// that each lane holds half of one item's row: softmax and top-K are serial per
// lane, with one xor-32 shuffle per reduction to join the two halves.
// bfloat16 with up to 32 experts and no logits output takes gate_topk_stream_kernel,
// which fetches the item rows with coalesced DMA requests into LDS instead.
// (VMOE_GATE_DIRECT_LOADS=1 in the environment keeps the direct loads: the switch behind
// the before / after figures.)
#include <cstdlib>
#include <type_traits>

#include "vmoe_common.h"
#include "router_metrics.h"

namespace vmoe {
namespace {


__device__ __forceinline__ float inv_orderable(uint32_t u) {
  uint32_t b = (u & 0x80000000u) ? (u & 0x7fffffffu) : ~u;
  return __builtin_bit_cast(float, b);
}

template <int MASK>
__device__ __forceinline__ float xor_max(float v) {
  return fmaxf(v, __shfl_xor(v, MASK, kWave));
}

__device__ __forceinline__ float half_wave_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 1, kWave));
  v = fmaxf(v, __shfl_xor(v, 2, kWave));
  v = fmaxf(v, __shfl_xor(v, 4, kWave));
  v = fmaxf(v, __shfl_xor(v, 8, kWave));
  v = fmaxf(v, __shfl_xor(v, 16, kWave));
  return v;
}
__device__ __forceinline__ float half_wave_sum(float v) {
  v += __shfl_xor(v, 1, kWave);
  v += __shfl_xor(v, 2, kWave);
  v += __shfl_xor(v, 4, kWave);
  v += __shfl_xor(v, 8, kWave);
  v += __shfl_xor(v, 16, kWave);
  return v;
}
__device__ __forceinline__ uint64_t half_wave_max_u64(uint64_t v) {
#pragma unroll
  for (int m = 1; m < 32; m <<= 1) {
    uint32_t lo = __shfl_xor((uint32_t)v, m, kWave);
    uint32_t hi = __shfl_xor((uint32_t)(v >> 32), m, kWave);
    uint64_t o = ((uint64_t)hi << 32) | lo;
    v = o > v ? o : v;
  }
  return v;
}

// LDS row stride (in elements) of the staged router kernel.
template <typename T> __host__ __device__ constexpr int w_stride(int kc, int epad) {
  return sizeof(T) == 2 ? kc + 8 : epad;
}

template <typename T, int NT, bool LOGITS, int WAVES, bool SPLITK = false>
__global__ __launch_bounds__(WAVES * kWave) void gate_topk_kernel(
    const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ bias,
    T* __restrict__ gates, float* __restrict__ logits, float* __restrict__ topk_val,
    int32_t* __restrict__ topk_idx,
    int num_items, int D, int E, int K, int KC, int num_chunks, int num_tiles, int stage_off) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* wl = reinterpret_cast<T*>(smem);
  constexpr int kGateWaves = WAVES;
  constexpr int kGateThreads = kGateWaves * kWave;
  constexpr int EP = NT * 32;
  constexpr bool kBf16 = sizeof(T) == 2;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int m = lane & 31;
  const int h = lane >> 5;
  const int stride = w_stride<T>(KC, EP);
  // SPLITK (float32, few items): the four waves of a workgroup share one tile of 32 items and
  // a quarter of D each, and meet in the logits tiles of the epilogue: a launch of a few dozen
  // tiles is as long as its longest chain of loads and MFMAs, which this cuts in four.
  static_assert(!SPLITK || (sizeof(T) == 4 && WAVES == 4), "split-k form");
  const int tiles_per_iter = SPLITK ? gridDim.x : gridDim.x * kGateWaves;
  const int iters = (num_tiles + tiles_per_iter - 1) / tiles_per_iter;

  for (int it = 0; it < iters; ++it) {
    const int tile = SPLITK ? it * tiles_per_iter + blockIdx.x
                            : it * tiles_per_iter + blockIdx.x * kGateWaves + wave;
    const bool active = tile < num_tiles;
    const int row0 = tile * 32;
    int r = row0 + m;
    if (r >= num_items) r = num_items - 1;
    if (r < 0) r = 0;
    const T* xrow = x + (size_t)r * D;

    floatx16 acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nt][i] = 0.f;

    // bf16: the loads of the first round of router-kernel blocks and of the first
    // batch of item rows go out together, before anything waits: the blocks come back
    // first and are staged under the latency of the rows.
    constexpr int UB = 2;   // 64-k blocks per batch; two batches (16 x 16-byte loads per lane) in flight
    uint4 wraw[kBf16 ? 8 : 1];
    uint4 a[kBf16 ? 2 : 1][UB][4];
    using Buf0 = std::integral_constant<int, 0>;
    using Buf1 = std::integral_constant<int, kBf16 ? 1 : 0>;
    auto load_w_block = [&](int k0, int kb, int nb, bool in_range) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int k = k0 + kb * 8 + i;
        wraw[kBf16 ? i : 0] = (in_range && k < D && nb * 8 < E)
                                  ? *reinterpret_cast<const uint4*>(w + (size_t)k * E + nb * 8)
                                  : make_uint4(0, 0, 0, 0);
      }
    };
    auto load_rows = [&](auto buf, int k0, int kb0, int nkb) {
#pragma unroll
      for (int u = 0; u < UB; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int kg = k0 + (kb0 + u) * 64 + h * 32 + j * 8;
          a[decltype(buf)::value][u][j] = (kb0 + u < nkb && kg + 8 <= D)
                                              ? *reinterpret_cast<const uint4*>(xrow + kg)
                                              : make_uint4(0, 0, 0, 0);
        }
    };
    auto mma_rows = [&](auto buf, int kb0, int nkb) {
#pragma unroll
      for (int u = 0; u < UB; ++u) {
        if (kb0 + u >= nkb) break;
        const int kl = (kb0 + u) * 64 + h * 32;  // this lane's 32 k's inside the chunk
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          bf16x8 af = __builtin_bit_cast(bf16x8, a[decltype(buf)::value][u][j]);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            uint4 b = *reinterpret_cast<const uint4*>(wl + (nt * 32 + m) * stride + kl + j * 8);
            acc[nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, __builtin_bit_cast(bf16x8, b),
                                                              acc[nt], 0, 0, 0);
          }
        }
      }
    };
    if constexpr (kBf16) {
      if (it == 0 && E % 8 == 0 && (reinterpret_cast<uintptr_t>(w) & 15u) == 0) {
        const int nbn = EP / 8;
        load_w_block(0, tid / nbn, tid % nbn, tid < (KC / 8) * nbn);
      }
      if (active) {
        load_rows(Buf0{}, 0, 0, KC / 64);
        load_rows(Buf1{}, 0, UB, KC / 64);
      }
    }

    // float32: the item rows are loaded four 16-wide k steps at a time, two such batches in
    // flight (a batch is refilled as soon as its MFMAs are issued); the first two go out before
    // the router kernel is staged.
    constexpr int FB = 4;
    float4 va[kBf16 ? 1 : 2][kBf16 ? 1 : FB][2];
    int kb_lo = 0, kb_hi = KC / 16;
    if (SPLITK) {
      kb_lo = wave * (KC / 16 / kGateWaves);
      kb_hi = kb_lo + KC / 16 / kGateWaves;
    }
    auto load_f = [&](const int u, int k0, int kb0) {
#pragma unroll
      for (int t = 0; t < (kBf16 ? 1 : FB); ++t)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int kg = k0 + (kb0 + t) * 16 + h * 8 + j * 4;
          va[u][t][j] = (kb0 + t < kb_hi && kg + 4 <= D)
                            ? *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(xrow) + kg)
                            : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    if constexpr (!kBf16) {
      if (active) {
        load_f(0, 0, kb_lo);
        load_f(1, 0, kb_lo + FB);
      }
    }

    for (int c = 0; c < num_chunks; ++c) {
      const int k0 = c * KC;
      if (num_chunks > 1 || it == 0) {
        __syncthreads();
        // Stage W[k0 : k0+KC, :] into LDS, zero padded in both directions.  When
        // a row of W is a whole number of 16-byte vectors the loads are vector
        // loads, all independent, so the staging costs one memory round trip.
        constexpr int VW = 16 / (int)sizeof(T);
        if (kBf16 && E % VW == 0 && (reinterpret_cast<uintptr_t>(w) & 15u) == 0) {
          // bf16: a thread loads an 8(k) x 8(expert) block with eight 16-byte loads,
          // transposes it in registers and writes each expert's eight consecutive k
          // as one 16-byte chunk (2-byte LDS writes made this the longest phase of
          // the kernel).  The first round of loads was issued before the item rows.
          const int nbn = EP / 8, nblk = (KC / 8) * nbn;
          for (int b0 = 0; b0 < nblk; b0 += kGateThreads) {
            const int b = b0 + tid;
            const int kb = b / nbn, nb = b - kb * nbn;
            if (!(b0 == 0 && c == 0 && it == 0)) load_w_block(k0, kb, nb, b < nblk);
            if (b < nblk) {
#pragma unroll
              for (int j = 0; j < 8; ++j) {
                const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
                uint32_t o[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                  const uint32_t hi = reinterpret_cast<const uint32_t*>(&wraw[2 * q + 1])[j >> 1];
                  const uint32_t lo = reinterpret_cast<const uint32_t*>(&wraw[2 * q])[j >> 1];
                  o[q] = __builtin_amdgcn_perm(hi, lo, sel);
                }
                *reinterpret_cast<uint4*>(wl + (size_t)(nb * 8 + j) * stride + kb * 8) =
                    make_uint4(o[0], o[1], o[2], o[3]);
              }
            }
          }
        } else if (E % VW == 0 && (reinterpret_cast<uintptr_t>(w) & 15u) == 0) {
          const int vec_per_row = EP / VW;
          constexpr int kBatch = 6;   // independent loads in flight per thread
          for (int idx0 = tid; idx0 < KC * vec_per_row; idx0 += kBatch * kGateThreads) {
            uint4 raw[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
              const int idx = idx0 + u * kGateThreads;
              const int k = idx / vec_per_row, n0 = (idx - k * vec_per_row) * VW;
              raw[u] = make_uint4(0, 0, 0, 0);
              if (idx < KC * vec_per_row && k0 + k < D && n0 < E)
                raw[u] = *reinterpret_cast<const uint4*>(w + (size_t)(k0 + k) * E + n0);
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
              const int idx = idx0 + u * kGateThreads;
              if (idx >= KC * vec_per_row) continue;
              const int k = idx / vec_per_row, n0 = (idx - k * vec_per_row) * VW;
              const T* v = reinterpret_cast<const T*>(&raw[u]);
#pragma unroll
              for (int t = 0; t < VW; ++t) {
                if (kBf16) wl[(n0 + t) * stride + k] = v[t]; else wl[k * stride + n0 + t] = v[t];
              }
            }
          }
        } else {
          for (int idx = tid; idx < KC * EP; idx += kGateThreads) {
            int k = idx / EP, n = idx - k * EP;
            T v = 0;
            if (k0 + k < D && n < E) v = w[(size_t)(k0 + k) * E + n];
            if (kBf16) wl[n * stride + k] = v; else wl[k * stride + n] = v;
          }
        }
        __syncthreads();
      }
      if (!active) continue;
      if constexpr (kBf16) {
        const int nkb = KC / 64;
        if (c > 0) {
          load_rows(Buf0{}, k0, 0, nkb);
          load_rows(Buf1{}, k0, UB, nkb);
        }
        // A buffer is refilled as soon as its MFMAs are issued, so two batches stay in flight.
        for (int kb0 = 0; kb0 < nkb; kb0 += 2 * UB) {
          mma_rows(Buf0{}, kb0, nkb);
          load_rows(Buf0{}, k0, kb0 + 2 * UB, nkb);
          mma_rows(Buf1{}, kb0 + UB, nkb);
          load_rows(Buf1{}, k0, kb0 + 3 * UB, nkb);
          mfma_result_fence();
        }
      } else {
        auto mma_f = [&](const int u, int kb0) {
#pragma unroll
          for (int t = 0; t < FB; ++t) {
            if (kb0 + t >= kb_hi) break;
            const int kl = (kb0 + t) * 16 + h * 8;
            const float a[8] = {va[u][t][0].x, va[u][t][0].y, va[u][t][0].z, va[u][t][0].w,
                                va[u][t][1].x, va[u][t][1].y, va[u][t][1].z, va[u][t][1].w};
#pragma unroll
            for (int i = 0; i < 8; ++i) {
#pragma unroll
              for (int nt = 0; nt < NT; ++nt) {
                float b = wl[(kl + i) * stride + nt * 32 + m];
                acc[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b, acc[nt], 0, 0, 0);
              }
            }
          }
        };
        if (c > 0) {
          load_f(0, k0, kb_lo);
          load_f(1, k0, kb_lo + FB);
        }
        for (int kb0 = kb_lo; kb0 < kb_hi; kb0 += 2 * FB) {
          mma_f(0, kb0);
          load_f(0, k0, kb0 + 2 * FB);
          mma_f(1, kb0 + FB);
          load_f(1, k0, kb0 + 3 * FB);
          mfma_result_fence();
        }
      }
    }
    if (!active) continue;

    // Epilogue.  The 32 x EP tile of (rounded, biased) logits goes through a
    // wave-private LDS tile so that a lane ends up with half of one item's row in
    // registers (lane = item r, half h of the experts): softmax and top-K are then
    // serial per lane, and the two halves of a row meet with a single xor-32
    // shuffle per reduction instead of a five-step butterfly per row.
    float* st = reinterpret_cast<float*>(smem + stage_off) + (size_t)wave * 32 * (EP + 1);
    {
      float bn[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        int n = nt * 32 + m;
        bn[nt] = (bias != nullptr && n < E) ? bias[n] : 0.f;
      }
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int rl = (i >> 2) * 8 + h * 4 + (i & 3);
          float v = acc[nt][i];
          if (!SPLITK) {
            v = Elt<T>::round(v);
            if (bias != nullptr) v = Elt<T>::round(v + bn[nt]);
          }
          st[rl * (EP + 1) + nt * 32 + m] = v;
        }
    }
    constexpr int CNT = EP / 2;          // experts per lane
    const int row = row0 + m;
    const int n0 = h * CNT;
    float g[CNT];
    float mx = -INFINITY;
    if (SPLITK) {
      // the four waves' partial logits meet here, added in wave order; wave 0 finishes the tile
      __syncthreads();
      if (wave != 0) {
        __syncthreads();          // the tiles are free again once wave 0 has read them
        continue;
      }
    }
#pragma unroll
    for (int j = 0; j < CNT; ++j) {
      float v = st[m * (EP + 1) + n0 + j];
      if (SPLITK) {
#pragma unroll
        for (int ww = 1; ww < kGateWaves; ++ww) v += st[(ww * 32 + m) * (EP + 1) + n0 + j];
        if (bias != nullptr && n0 + j < E) v += bias[n0 + j];
      }
      g[j] = (n0 + j < E) ? v : -INFINITY;
      mx = fmaxf(mx, g[j]);
    }
    if (SPLITK) __syncthreads();
    if (LOGITS && row < num_items) {
#pragma unroll
      for (int j = 0; j < CNT; ++j)
        if (n0 + j < E) logits[(size_t)row * E + n0 + j] = g[j];
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < CNT; ++j) {
      g[j] = (n0 + j < E) ? expf(g[j] - mx) : 0.f;
      sum += g[j];
    }
    sum += __shfl_xor(sum, 32, kWave);
#pragma unroll
    for (int j = 0; j < CNT; ++j) g[j] = Elt<T>::round(g[j] / sum);
    const bool row_ok = row < num_items;
    if (gates != nullptr && row_ok) {
      T* grow = gates + (size_t)row * E + n0;
      if (kBf16 && (E & 7) == 0 && (reinterpret_cast<uintptr_t>(gates) & 15u) == 0) {
#pragma unroll
        for (int j = 0; j < CNT; j += 8) {
          if (n0 + j < E) {
            uint32_t pk[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) pk[t] = pack_bf16x2(g[j + 2 * t], g[j + 2 * t + 1]);
            *reinterpret_cast<uint4*>(grow + j) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < CNT; ++j)
          if (n0 + j < E) Elt<T>::store(grow + j, g[j]);
      }
    }
    uint64_t taken = 0;
    for (int kk = 0; kk < K; ++kk) {
      uint64_t best = 0;
#pragma unroll
      for (int j = 0; j < CNT; ++j) {
        const int n = n0 + j;
        if (n < E && !(taken >> j & 1ull)) {
          uint64_t key = ((uint64_t)orderable(g[j]) << 32) | (uint32_t)(0xFFFFFFFFu - (uint32_t)n);
          best = key > best ? key : best;
        }
      }
      const uint32_t olo = __shfl_xor((uint32_t)best, 32, kWave);
      const uint32_t ohi = __shfl_xor((uint32_t)(best >> 32), 32, kWave);
      const uint64_t other = ((uint64_t)ohi << 32) | olo;
      best = other > best ? other : best;
      const int n_star = (int)(0xFFFFFFFFu - (uint32_t)best);
      if (n_star >= n0 && n_star < n0 + CNT) taken |= 1ull << (n_star - n0);
      if (h == 0 && row_ok) {
        topk_val[(size_t)row * K + kk] = inv_orderable((uint32_t)(best >> 32));
        topk_idx[(size_t)row * K + kk] = n_star;
      }
    }
  }
}

// Streaming form of the bfloat16 kernel for up to 32 experts (the routers' common case).
// The item rows are the whole traffic (77 MB on the headline layer, 0.05 MB of router
// kernel), so they are fetched the way a copy kernel fetches: every DMA request of a wave
// covers 8 rows x 128 contiguous bytes (a 64-wide k chunk of the wave's 32-row tile is four
// requests) and lands in a wave-private ring of LDS slots, from which the MFMA A fragments
// are read; the direct loads of gate_topk_kernel fetch 16 bytes per lane from 32 different
// rows per request and reach half the rate.  Eight waves per workgroup share one staged
// copy of the router kernel; a wave runs SLOTS - 1 chunks ahead of its MFMAs.  The chunk's
// 16-byte pieces are XOR-swizzled by row on their way in (the lane picks the global piece
// that belongs in its LDS position), so that the fragment reads spread over the banks.
// Epilogue as in gate_topk_kernel, its tile staged in the wave's own ring.  Headline layer
// (50 176 items x 768, 77 MB): 21.9 us against 29.5 - 31.3 with direct loads (kernel trace);
// two or three slots, seven or eight waves per workgroup make no difference.
constexpr int kStreamWaves = 8;
constexpr int kStreamChunkBytes = 32 * 128;      // 32 rows x 64 bfloat16

typedef __attribute__((address_space(3))) void* gate_lds_ptr_t;

template <int SLOTS, int WAVES>
__global__ __launch_bounds__(WAVES * kWave, 1) void gate_topk_stream_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    bf16_t* __restrict__ gates, float* __restrict__ topk_val, int32_t* __restrict__ topk_idx,
    int num_items, int D, int E, int K, int num_tiles, int w_bytes) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-resource builtins exist in the device pass only
  extern __shared__ __align__(1024) unsigned char smem[];
  bf16_t* wl = reinterpret_cast<bf16_t*>(smem);
  constexpr int kThreads = WAVES * kWave;
  constexpr int EP = 32;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = lane & 31;
  const int h = lane >> 5;
  const int stride = D + 8;                        // elements per expert row of the staged router kernel
  unsigned char* ring = smem + w_bytes + wave * (SLOTS * kStreamChunkBytes);

  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(x), 0, -1, 0x00020000);
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  const uint32_t ring_addr = (uint32_t)reinterpret_cast<uintptr_t>((gate_lds_ptr_t)ring);
  const uint32_t wl_addr = (uint32_t)reinterpret_cast<uintptr_t>((gate_lds_ptr_t)wl);
  const int nchunks = D / 64;
  const int lrow = lane >> 3;                      // row of this lane inside a request (8 rows x 8 pieces)
  const int swz = m & 7;
  const int tile0 = blockIdx.x * WAVES + wave;
  // Request i of a chunk fills LDS rows 8 i .. 8 i + 7; lane L lands in row 8 i + L / 8,
  // position L % 8, and therefore fetches piece (L % 8) ^ (row & 7) of that row.
  uint32_t goff[4];
  auto tile_offsets = [&](int tile) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int rl = i * 8 + lrow;
      const int r = min(tile * 32 + rl, num_items - 1);
      goff[i] = (uint32_t)r * (uint32_t)D * 2u + (uint32_t)(((lane & 7) ^ (rl & 7)) * 16);
    }
  };
  auto request = [&](int c) {
    unsigned char* s = ring + (c % SLOTS) * kStreamChunkBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (gate_lds_ptr_t)(s + i * 1024), 16, goff[i],
                                               c * 128, 0, 0);
  };
  // The first requests of the wave's first tile go out before the router kernel is staged:
  // every wave of the launch is loading from its first instruction on.
  if (tile0 < num_tiles) {
    tile_offsets(tile0);
#pragma unroll
    for (int c = 0; c < SLOTS - 1; ++c)
      if (c < nchunks) request(c);
  }

  // Router kernel -> LDS as [expert][k]: a thread loads an 8 (k) x 8 (expert) block with
  // eight 16-byte loads, transposes it in registers and writes each expert's eight
  // consecutive k as one 16-byte piece (E % 8 == 0 and a 16-byte aligned w: the launcher
  // checks); experts E .. 31 are zero.  The LDS writes are written as instructions, like the
  // fragment reads below: a write the compiler can see would wait for the requests above.
  {
    const int nbn = EP / 8, nblk = (D / 8) * nbn;
    for (int b0 = 0; b0 < nblk; b0 += kThreads) {
      const int b = b0 + tid;
      const int kb = b / nbn, nb = b - kb * nbn;
      uint4 wraw[8];
#pragma unroll
      for (int i = 0; i < 8; ++i)
        wraw[i] = (b < nblk && nb * 8 < E)
                      ? *reinterpret_cast<const uint4*>(w + (size_t)(kb * 8 + i) * E + nb * 8)
                      : make_uint4(0, 0, 0, 0);
      if (b < nblk) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
          u32x4_t o;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint32_t hi = reinterpret_cast<const uint32_t*>(&wraw[2 * q + 1])[j >> 1];
            const uint32_t lo = reinterpret_cast<const uint32_t*>(&wraw[2 * q])[j >> 1];
            o[q] = __builtin_amdgcn_perm(hi, lo, sel);
          }
          asm volatile("ds_write_b128 %0, %1" ::"v"(wl_addr + (uint32_t)(((nb * 8 + j) * stride + kb * 8) * 2)), "v"(o)
                       : "memory");
        }
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __syncthreads();

  for (int tile = tile0; tile < num_tiles; tile += gridDim.x * WAVES) {
    const int row0 = tile * 32;
    floatx16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    if (tile != tile0) {         // (the first tile's were issued before the router kernel was staged)
      tile_offsets(tile);
#pragma unroll
      for (int c = 0; c < SLOTS - 1; ++c)
        if (c < nchunks) request(c);
    }
    // The fragment reads are written as instructions: the compiler drains every DMA request
    // in front of an LDS read it can see (it cannot tell that the requests in flight fill
    // other slots), which would leave a wave with one chunk in flight.
    auto multiply = [&](int c) {
      const uint32_t sa = ring_addr + (uint32_t)((c % SLOTS) * kStreamChunkBytes + m * 128);
      const uint32_t sw = wl_addr + (uint32_t)((m * stride + c * 64 + h * 8) * 2);
      u32x4_t a[4], b[4];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        asm volatile("ds_read_b128 %0, %1" : "=v"(a[ks]) : "v"(sa + (uint32_t)(((2 * ks + h) ^ swz) * 16)));
        asm volatile("ds_read_b128 %0, %1" : "=v"(b[ks]) : "v"(sw + (uint32_t)(ks * 32)));
      }
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[ks]),
                                                      __builtin_bit_cast(bf16x8, b[ks]), acc, 0, 0, 0);
    };
    int c = 0;
    for (; c + SLOTS - 1 < nchunks; ++c) {       // chunk c + SLOTS - 1 goes into the slot chunk c - 1 has left
      request(c + SLOTS - 1);
      wait_vmcnt<(SLOTS - 1) * 4>();
      multiply(c);
    }
    wait_vmcnt<0>();
    for (; c < nchunks; ++c) multiply(c);
    mfma_result_fence();

    // Epilogue (gate_topk_kernel's, for one tile of experts): logits through a wave-private
    // LDS tile so that a lane ends up with half of one item's row.
    float* st = reinterpret_cast<float*>(ring);
    {
      const float bn = (bias != nullptr && m < E) ? bias[m] : 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int rl = (i >> 2) * 8 + h * 4 + (i & 3);
        float v = bf16r(acc[i]);
        if (bias != nullptr) v = bf16r(v + bn);
        st[rl * (EP + 1) + m] = v;
      }
    }
    constexpr int CNT = EP / 2;
    const int row = row0 + m;
    const int n0 = h * CNT;
    float g[CNT];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < CNT; ++j) {
      const float v = st[m * (EP + 1) + n0 + j];
      g[j] = (n0 + j < E) ? v : -INFINITY;
      mx = fmaxf(mx, g[j]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < CNT; ++j) {
      g[j] = (n0 + j < E) ? expf(g[j] - mx) : 0.f;
      sum += g[j];
    }
    sum += __shfl_xor(sum, 32, kWave);
#pragma unroll
    for (int j = 0; j < CNT; ++j) g[j] = bf16r(g[j] / sum);
    const bool row_ok = row < num_items;
    if (gates != nullptr && row_ok) {
      bf16_t* grow = gates + (size_t)row * E + n0;
      if ((reinterpret_cast<uintptr_t>(gates) & 15u) == 0) {
#pragma unroll
        for (int j = 0; j < CNT; j += 8) {
          if (n0 + j < E) {
            uint32_t pk[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) pk[t] = pack_bf16x2(g[j + 2 * t], g[j + 2 * t + 1]);
            *reinterpret_cast<uint4*>(grow + j) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < CNT; ++j)
          if (n0 + j < E) Elt<bf16_t>::store(grow + j, g[j]);
      }
    }
    uint64_t taken = 0;
    for (int kk = 0; kk < K; ++kk) {
      uint64_t best = 0;
#pragma unroll
      for (int j = 0; j < CNT; ++j) {
        const int n = n0 + j;
        if (n < E && !(taken >> j & 1ull)) {
          uint64_t key = ((uint64_t)orderable(g[j]) << 32) | (uint32_t)(0xFFFFFFFFu - (uint32_t)n);
          best = key > best ? key : best;
        }
      }
      const uint32_t olo = __shfl_xor((uint32_t)best, 32, kWave);
      const uint32_t ohi = __shfl_xor((uint32_t)(best >> 32), 32, kWave);
      const uint64_t other = ((uint64_t)ohi << 32) | olo;
      best = other > best ? other : best;
      const int n_star = (int)(0xFFFFFFFFu - (uint32_t)best);
      if (n_star >= n0 && n_star < n0 + CNT) taken |= 1ull << (n_star - n0);
      if (h == 0 && row_ok) {
        topk_val[(size_t)row * K + kk] = inv_orderable((uint32_t)(best >> 32));
        topk_idx[(size_t)row * K + kk] = n_star;
      }
    }
  }
#endif
}

// Top-K of given float32 gates, one wave per item, E <= 1024.
__global__ __launch_bounds__(256) void topk_kernel(const float* __restrict__ gates,
                                                   float* __restrict__ topk_val,
                                                   int32_t* __restrict__ topk_idx,
                                                   int num_items, int E, int K) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= num_items) return;
  const float* g = gates + (size_t)item * E;
  float v[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    int n = j * 64 + lane;
    v[j] = n < E ? g[n] : 0.f;
  }
  uint32_t taken = 0;
  for (int kk = 0; kk < K; ++kk) {
    uint64_t best = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      int n = j * 64 + lane;
      if (n < E && !(taken >> j & 1u)) {
        uint64_t key = ((uint64_t)orderable(v[j]) << 32) | (uint32_t)(0xFFFFFFFFu - (uint32_t)n);
        best = key > best ? key : best;
      }
    }
#pragma unroll
    for (int msk = 1; msk < 64; msk <<= 1) {
      uint32_t lo = __shfl_xor((uint32_t)best, msk, kWave);
      uint32_t hi = __shfl_xor((uint32_t)(best >> 32), msk, kWave);
      uint64_t o = ((uint64_t)hi << 32) | lo;
      best = o > best ? o : best;
    }
    const int n_star = (int)(0xFFFFFFFFu - (uint32_t)best);
    if ((n_star & 63) == lane) taken |= 1u << (n_star >> 6);
    if (lane == 0) {
      // Return the stored bits of the winner (keeps -0.0 / payloads intact).
      topk_val[(size_t)item * K + kk] = g[n_star];
      topk_idx[(size_t)item * K + kk] = n_star;
    }
  }
}

// Per-group auxiliary losses: one workgroup of 1024 threads per group (router_metrics.h).
template <typename T>
__global__ __launch_bounds__(kMetricThreads) void router_metrics_kernel(
    const T* __restrict__ gates, const int32_t* __restrict__ top1, float* __restrict__ imp_loss,
    float* __restrict__ gsh_loss, float* __restrict__ aux_loss, float w_gsh, float w_imp,
    int S, int E, int top1_stride, int V) {
  extern __shared__ __align__(16) unsigned char smem[];
  router_metrics_group<T>(gates, top1, imp_loss, gsh_loss, aux_loss, w_gsh, w_imp, S, E,
                          top1_stride, V, blockIdx.x, smem);
}

template <typename T>
int launch_gate(const VmoeGateTopkParams* p, hipStream_t stream) {
  const int nt = (p->E + 31) / 32;
  const int ep = (nt == 3 ? 4 : nt) * 32;
  const int gran = sizeof(T) == 2 ? 64 : 16;
  const int dpad = (p->D + gran - 1) / gran * gran;
  // LDS: the staged router kernel (split along D when it would not fit) and,
  // behind it, a 32 x (ep + 1) float32 logits tile per wave for the epilogue.
  const size_t budget = 88 * 1024;
  int kc = dpad;
  while ((size_t)(sizeof(T) == 2 ? ep * (kc + 8) : kc * ep) * sizeof(T) > budget && kc > gran)
    kc = ((kc / 2) + gran - 1) / gran * gran;
  const int num_chunks = (dpad + kc - 1) / kc;
  const size_t w_bytes = ((size_t)(sizeof(T) == 2 ? ep * (kc + 8) : kc * ep) * sizeof(T) + 15) / 16 * 16;
  // Two workgroups of four waves per CU, each with its own staged copy of the router
  // kernel, where both copies fit in LDS; one workgroup of eight waves sharing a copy
  // where they do not (D = 1024 in bf16), the registers allow it (up to 32 experts) and
  // four-wave workgroups would not all be resident at once anyway.
  const size_t tile_bytes = (size_t)32 * (ep + 1) * sizeof(float);
  const size_t lds_cu = 160 * 1024;
  const int num_tiles = (p->num_items + 31) / 32;
  const int waves = (nt == 1 && 2 * (w_bytes + 4 * tile_bytes) > lds_cu &&
                     w_bytes + 8 * tile_bytes <= lds_cu && num_tiles > 4 * 256) ? 8 : 4;
  const size_t stage_bytes = waves * tile_bytes;
  const size_t lds = w_bytes + stage_bytes;
  int blocks = (num_tiles + waves - 1) / waves;
  if (blocks > 1024) blocks = 1024;
  // bfloat16, up to 32 experts, no logits output, enough items to fill the chip: the
  // streaming kernel (coalesced DMA requests into wave-private LDS rings).
  if constexpr (sizeof(T) == 2) {
    const size_t stream_w = ((size_t)32 * (p->D + 8) * 2 + 1023) / 1024 * 1024;
    const size_t ring3 = (size_t)kStreamWaves * 3 * kStreamChunkBytes, ring2 = (size_t)kStreamWaves * 2 * kStreamChunkBytes;
    const bool stream_ok = nt == 1 && p->logits == nullptr && p->E % 8 == 0 && aligned16(p->w) &&
                           p->D % 64 == 0 && (int64_t)p->num_items * p->D * 2 < ((int64_t)1 << 32) &&
                           num_tiles >= 256 && stream_w + ring2 <= lds_cu &&
                           getenv("VMOE_GATE_DIRECT_LOADS") == nullptr;
    if (stream_ok) {
      const bool three = stream_w + ring3 <= lds_cu;
      const size_t stream_lds = stream_w + (three ? ring3 : ring2);
      constexpr int swaves = kStreamWaves;
      int sblocks = (num_tiles + swaves - 1) / swaves;
      if (sblocks > 256) sblocks = 256;
      auto srun = [&](auto kern) {
        hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), stream_lds);
        if (e != hipSuccess) return (int)e;
        hipLaunchKernelGGL(kern, dim3(sblocks), dim3(swaves * kWave), stream_lds, stream,
                           (const bf16_t*)p->x, (const bf16_t*)p->w, p->logit_bias, (bf16_t*)p->gates,
                           p->topk_val, p->topk_idx, p->num_items, p->D, p->E, p->K, num_tiles,
                           (int)stream_w);
        return launch_status();
      };
      return three ? srun(gate_topk_stream_kernel<3, 8>) : srun(gate_topk_stream_kernel<2, 8>);
    }
  }
  // float32, up to 32 experts, at most two tiles of items per CU: a tile per workgroup, its k
  // range dealt to the four waves.
  const bool split_k = sizeof(T) == 4 && nt == 1 && waves == 4 && num_tiles <= 512 && kc % 64 == 0 &&
                       getenv("VMOE_GATE_NO_SPLIT_K") == nullptr;
  if (split_k) blocks = num_tiles;
  auto run = [&](auto kern) {
    hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(waves * kWave), lds, stream,
                       (const T*)p->x, (const T*)p->w, p->logit_bias, (T*)p->gates, p->logits,
                       p->topk_val, p->topk_idx, p->num_items, p->D, p->E, p->K, kc, num_chunks, num_tiles,
                       (int)w_bytes);
    return launch_status();
  };
  // The logits output is a separate instantiation: its extra live pointer costs
  // the common one a wave of occupancy.
  if constexpr (sizeof(T) == 4) {
    if (split_k)
      return p->logits != nullptr ? run(gate_topk_kernel<T, 1, true, 4, true>)
                                  : run(gate_topk_kernel<T, 1, false, 4, true>);
  }
  if (p->logits != nullptr) {
    switch (nt) {
      case 1: return waves == 8 ? run(gate_topk_kernel<T, 1, true, 8>) : run(gate_topk_kernel<T, 1, true, 4>);
      case 2: return run(gate_topk_kernel<T, 2, true, 4>);
      default: return run(gate_topk_kernel<T, 4, true, 4>);
    }
  }
  switch (nt) {
    case 1: return waves == 8 ? run(gate_topk_kernel<T, 1, false, 8>) : run(gate_topk_kernel<T, 1, false, 4>);
    case 2: return run(gate_topk_kernel<T, 2, false, 4>);
    default: return run(gate_topk_kernel<T, 4, false, 4>);
  }
}


// Noisy branch of the routers (vmoe/nn/routing.py:92-114): softmax of the noisy
// logits and, per group, the load loss (vmoe/nn/routing.py:159-183).  One
// workgroup per group, a wave per item, a lane per expert (two for E > 64).
constexpr int kNoisyWaves = 8;

__device__ __forceinline__ float wave_max_f(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}
__device__ __forceinline__ float wave_sum_f(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint32_t lo = __shfl_xor((uint32_t)v, o, kWave);
    const uint32_t hi = __shfl_xor((uint32_t)(v >> 32), o, kWave);
    const uint64_t other = ((uint64_t)hi << 32) | lo;
    v = other > v ? other : v;
  }
  return v;
}

__global__ __launch_bounds__(kNoisyWaves * 64) void noisy_gates_kernel(
    const float* __restrict__ logits, const float* __restrict__ noise,
    float* __restrict__ gates, float* __restrict__ load_loss, int S, int E, int K,
    float noise_std) {
  __shared__ float psum[kNoisyWaves][128];
  const int g = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool has0 = lane < E, has1 = lane + 64 < E;
  const float inv = 1.0f / (noise_std * 1.41421356237309515f);
  float acc0 = 0.f, acc1 = 0.f;
  for (int s = wave; s < S; s += kNoisyWaves) {
    const size_t base = ((size_t)g * S + s) * E;
    const float l0 = has0 ? logits[base + lane] : 0.f;
    const float l1 = has1 ? logits[base + lane + 64] : 0.f;
    const float v0 = has0 ? l0 + noise_std * noise[base + lane] : -INFINITY;
    const float v1 = has1 ? l1 + noise_std * noise[base + lane + 64] : -INFINITY;
    const float mx = wave_max_f(fmaxf(v0, v1));
    const float e0 = has0 ? expf(v0 - mx) : 0.f;
    const float e1 = has1 ? expf(v1 - mx) : 0.f;
    const float sum = wave_sum_f(e0 + e1);
    if (has0) gates[base + lane] = e0 / sum;
    if (has1) gates[base + lane + 64] = e1 / sum;
    if (load_loss == nullptr) continue;
    // Value of the K-th largest noisy logit (lax.top_k order: equal values, lower index first).
    uint64_t k0 = has0 ? (((uint64_t)orderable(v0) << 32) | (0xFFFFFFFFu - (uint32_t)lane)) : 0;
    uint64_t k1 = has1 ? (((uint64_t)orderable(v1) << 32) | (0xFFFFFFFFu - (uint32_t)(lane + 64))) : 0;
    uint64_t best = 0;
    for (int kk = 0; kk < K; ++kk) {
      best = wave_max_u64(k0 > k1 ? k0 : k1);
      if (best == k0) k0 = 0;
      else if (best == k1) k1 = 0;
    }
    const float thr = inv_orderable((uint32_t)(best >> 32));
    // p = 1 - Phi(z) = erfc(z / sqrt(2)) / 2,  z = (thr - logit) / noise_std.
    if (has0) acc0 += 0.5f * erfcf((thr - l0) * inv);
    if (has1) acc1 += 0.5f * erfcf((thr - l1) * inv);
  }
  if (load_loss == nullptr) return;
  psum[wave][lane] = acc0;
  psum[wave][lane + 64] = acc1;
  __syncthreads();
  if (wave == 0) {
    float p0 = 0.f, p1 = 0.f;
#pragma unroll
    for (int w = 0; w < kNoisyWaves; ++w) {
      p0 += psum[w][lane];
      p1 += psum[w][lane + 64];
    }
    p0 = has0 ? p0 / (float)S : 0.f;
    p1 = has1 ? p1 / (float)S : 0.f;
    const float mean = wave_sum_f(p0 + p1) / (float)E;
    const float d0 = has0 ? p0 - mean : 0.f, d1 = has1 ? p1 - mean : 0.f;
    const float var = wave_sum_f(d0 * d0 + d1 * d1) / (float)E;
    if (lane == 0) load_loss[g] = var / (mean * mean);
  }
}

}  // namespace
}  // namespace vmoe

using namespace vmoe;

extern "C" int vmoe_gate_topk(const VmoeGateTopkParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->x == nullptr || p->w == nullptr || p->topk_val == nullptr ||
      p->topk_idx == nullptr)
    return VMOE_E_NULL;
  if (p->num_items < 1 || p->D < 1 || p->E < 1 || p->K < 1 || p->K > p->E) return VMOE_E_SHAPE;
  if (p->dtype != VMOE_F32 && p->dtype != VMOE_BF16) return VMOE_E_DTYPE;
  if (p->E > 128) return VMOE_E_UNSUPPORTED;
  const int vec = p->dtype == VMOE_BF16 ? 8 : 4;
  if (p->D % vec != 0 || !aligned16(p->x)) return VMOE_E_ALIGN;
  if ((int64_t)p->num_items * (p->D > p->E * p->K ? p->D : p->E * p->K) >= (int64_t)1 << 40)
    return VMOE_E_OVERFLOW;
  return p->dtype == VMOE_BF16 ? launch_gate<bf16_t>(p, as_stream(stream))
                               : launch_gate<float>(p, as_stream(stream));
}

extern "C" int vmoe_topk(const VmoeTopkParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->gates == nullptr || p->topk_val == nullptr || p->topk_idx == nullptr)
    return VMOE_E_NULL;
  if (p->num_items < 1 || p->E < 1 || p->K < 1 || p->K > p->E) return VMOE_E_SHAPE;
  if (p->E > 1024) return VMOE_E_UNSUPPORTED;
  const int blocks = (p->num_items + 3) / 4;
  hipLaunchKernelGGL(topk_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), p->gates,
                     p->topk_val, p->topk_idx, p->num_items, p->E, p->K);
  return launch_status();
}

extern "C" int vmoe_router_metrics(const VmoeRouterMetricsParams* p, vmoe_stream_t stream) {
  int rc = check_router_metrics(p);
  if (rc != VMOE_OK) return rc;
  int V;
  size_t lds;
  if (!router_metrics_geometry(p, &V, &lds)) return VMOE_E_UNSUPPORTED;
  if (p->dtype == VMOE_BF16)
    hipLaunchKernelGGL(router_metrics_kernel<bf16_t>, dim3(p->G), dim3(kMetricThreads), lds,
                       as_stream(stream), (const bf16_t*)p->gates, p->top1_idx, p->importance_loss,
                       p->gshard_loss, p->auxiliary_loss, p->gshard_loss_weight,
                       p->importance_loss_weight, p->S, p->E, p->top1_stride, V);
  else
    hipLaunchKernelGGL(router_metrics_kernel<float>, dim3(p->G), dim3(kMetricThreads), lds,
                       as_stream(stream), (const float*)p->gates, p->top1_idx, p->importance_loss,
                       p->gshard_loss, p->auxiliary_loss, p->gshard_loss_weight,
                       p->importance_loss_weight, p->S, p->E, p->top1_stride, V);
  return launch_status();
}

extern "C" int vmoe_noisy_gates(const VmoeNoisyGatesParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->logits == nullptr || p->noise == nullptr || p->gates_noisy == nullptr)
    return VMOE_E_NULL;
  if (p->G < 1 || p->S < 1 || p->E < 1 || p->K < 1 || p->K > p->E || !(p->noise_std > 0.f))
    return VMOE_E_SHAPE;
  if (p->E > 128) return VMOE_E_UNSUPPORTED;
  hipLaunchKernelGGL(noisy_gates_kernel, dim3(p->G), dim3(kNoisyWaves * 64), 0, as_stream(stream),
                     p->logits, p->noise, p->gates_noisy, p->load_loss, p->S, p->E, p->K,
                     p->noise_std);
  return launch_status();
}
