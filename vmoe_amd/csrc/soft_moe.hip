// Soft MoE routing and dense (einsum) dispatch / combine for gfx950.
//
// soft_route replaces vmoe/projects/soft_moe/router.py:57-96: one workgroup per
// group normalises the item rows, multiplies them with the unit-norm slot
// parameters on the matrix cores, keeps the (S x N) logits of the group in LDS
// and takes both softmaxes (over items for the dispatch weights, over slots for
// the combine weights) from that one copy.  The bfloat16 kernel for the model
// widths up to 768 splits the waves of a workgroup into two roles
// (soft_route_roles_kernel).
//
// einsum_dispatch / einsum_combine replace EinsumDispatcher.dispatch/.combine
// (vmoe/moe.py:148-161) for dense weights, including the expert-buffer row
// order of _dispatch/_receive (moe.py:488-519).  They run on
// v_mfma_f32_32x32x2_f32: the weights keep full float32 precision (the
// reference promotes bf16 data to the weights' dtype), and a lane's operands
// are single scalars, so neither the (S, N) weights nor the (rows, D) data need
// a transposed copy.
#include <algorithm>

#include "vmoe_common.h"
#include "einsum_bf16.h"

namespace vmoe {
namespace {

constexpr float kNormEps = 1e-6f;

__device__ __forceinline__ float load_any(const void* p, size_t i, int dtype) {
  return dtype == VMOE_F32 ? reinterpret_cast<const float*>(p)[i]
                           : bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ float load_w(const void* p, size_t i, int wdtype) {
  if (wdtype == VMOE_W_F32) return reinterpret_cast<const float*>(p)[i];
  if (wdtype == VMOE_W_BF16) return bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
  return reinterpret_cast<const uint8_t*>(p)[i] ? 1.f : 0.f;
}
__device__ __forceinline__ void store_any(void* p, size_t i, float v, int dtype) {
  if (dtype == VMOE_F32) reinterpret_cast<float*>(p)[i] = v;
  else reinterpret_cast<bf16_t*>(p)[i] = f2bf(v);
}

// Unit-normalise the columns of mu (D, N) and apply the scale when it belongs to
// mu.  bf16: writes muT (N, D) so that a column's k run is contiguous;
// f32: writes (D, N).
// frag_ksw > 0 (bf16, D = 32 * frag_ksw): the order in which soft_route_roles_kernel's
// consumer waves hold the parameters, [slot / 32][slot % 32 / 16][d / 32][lane][d % 8]
// with lane = (d % 32 / 8) * 16 + slot % 16, so that every fragment load of a wave is
// 1 KB of consecutive memory; the grid then covers the slots up to a multiple of 32 and
// the ones past N are zeros.
template <typename T>
__global__ __launch_bounds__(256) void soft_prep_mu_kernel(const T* __restrict__ mu,
                                                           T* __restrict__ out, float scale,
                                                           int scale_mu, int D, int N,
                                                           int frag_ksw = 0) {
  __shared__ float red[256];
  const int n = blockIdx.x, tid = threadIdx.x;
  auto frag_index = [&](int d) -> size_t {
    const int lane = ((d & 31) >> 3) * 16 + (n & 15);
    return ((((size_t)(n >> 5) * 2 + ((n & 31) >> 4)) * frag_ksw + (d >> 5)) * 64 + lane) * 8 + (d & 7);
  };
  if (n >= N) {     // padding slots of the fragment order
    for (int d = tid; d < D; d += 256) Elt<T>::store(out + frag_index(d), 0.f);
    return;
  }
  float s = 0.f;
  for (int d = tid; d < D; d += 256) {
    float v = Elt<T>::load(mu + (size_t)d * N + n);
    s += v * v;
  }
  red[tid] = s;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (tid < o) red[tid] += red[tid + o];
    __syncthreads();
  }
  const float inv = 1.0f / sqrtf(red[0] + kNormEps);
  const float sc = Elt<T>::round(scale);
  for (int d = tid; d < D; d += 256) {
    float v = Elt<T>::round(Elt<T>::load(mu + (size_t)d * N + n) * inv);
    if (scale_mu) v = Elt<T>::round(v * sc);
    if (frag_ksw > 0) Elt<T>::store(out + frag_index(d), v);
    else if (sizeof(T) == 2) Elt<T>::store(out + (size_t)n * D + d, v);
    else Elt<T>::store(out + (size_t)d * N + n, v);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void soft_route_kernel(
    const T* __restrict__ x, const T* __restrict__ muw, T* __restrict__ dispatch_w,
    T* __restrict__ combine_w, T* __restrict__ logits_out, float scale, int scale_x, int S, int D,
    int N, int SP, int NP) {
  extern __shared__ __align__(16) unsigned char smem[];
  float* inv_norm = reinterpret_cast<float*>(smem);                  // SP
  T* lg = reinterpret_cast<T*>(smem + (size_t)SP * 4);               // SP x LDW
  const int LDW = NP + (sizeof(T) == 2 ? 2 : 1);
  constexpr bool kBf16 = sizeof(T) == 2;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, h = lane >> 5;
  const int g = blockIdx.x;
  const T* xg = x + (size_t)g * S * D;
  const float sc = Elt<T>::round(scale);

  // Phase 1: 1/sqrt(sum x^2 + eps) per item row.
  for (int s = wave; s < SP; s += 4) {
    float acc = 0.f;
    if (s < S)
      for (int d = lane; d < D; d += 64) {
        float v = Elt<T>::load(xg + (size_t)s * D + d);
        acc += v * v;
      }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, kWave);
    if (lane == 0) inv_norm[s] = s < S ? 1.0f / sqrtf(acc + kNormEps) : 0.f;
  }
  __syncthreads();

  // Phase 2: logits tile by tile (32 items x 32 slots per MFMA accumulator).
  const int row_tiles = SP / 32, col_tiles = NP / 32;
  for (int rt = wave; rt < row_tiles; rt += 4) {
    int r = rt * 32 + m;
    const float inv = inv_norm[r];
    if (r >= S) r = S - 1;
    const T* xrow = xg + (size_t)r * D;
    for (int ct0 = 0; ct0 < col_tiles; ct0 += 4) {
      floatx16 acc[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;
      if constexpr (kBf16) {
        for (int k0 = 0; k0 < D; k0 += 16) {
          const int k = k0 + h * 8;
          bf16x8 af;
          if (k + 8 <= D) {
            uint4 raw = *reinterpret_cast<const uint4*>(xrow + k);
            const uint32_t w4[4] = {raw.x, raw.y, raw.z, raw.w};
            uint32_t o4[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              float lo = bf16r(__builtin_bit_cast(float, w4[i] << 16) * inv);
              float hi = bf16r(__builtin_bit_cast(float, w4[i] & 0xffff0000u) * inv);
              if (scale_x) { lo = bf16r(lo * sc); hi = bf16r(hi * sc); }
              o4[i] = (uint32_t)f2bf(lo) | ((uint32_t)f2bf(hi) << 16);
            }
            af = __builtin_bit_cast(bf16x8, make_uint4(o4[0], o4[1], o4[2], o4[3]));
          } else {
            af = __builtin_bit_cast(bf16x8, make_uint4(0, 0, 0, 0));
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int n = (ct0 + j) * 32 + m;
            uint4 braw = make_uint4(0, 0, 0, 0);
            if (ct0 + j < col_tiles && n < N && k + 8 <= D)
              braw = *reinterpret_cast<const uint4*>(muw + (size_t)n * D + k);
            acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, __builtin_bit_cast(bf16x8, braw),
                                                             acc[j], 0, 0, 0);
          }
        }
      } else {
        for (int k0 = 0; k0 < D; k0 += 2) {
          const int k = k0 + h;
          float a = 0.f;
          if (k < D) {
            a = Elt<T>::load(xrow + k) * inv;
            if (scale_x) a = a * sc;
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int n = (ct0 + j) * 32 + m;
            float bv = 0.f;
            if (ct0 + j < col_tiles && n < N && k < D) bv = Elt<T>::load(muw + (size_t)k * N + n);
            acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bv, acc[j], 0, 0, 0);
          }
        }
      }
      mfma_result_fence();
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (ct0 + j >= col_tiles) continue;
        const int col = (ct0 + j) * 32 + m;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = rt * 32 + (v >> 2) * 8 + h * 4 + (v & 3);
          Elt<T>::store(lg + (size_t)row * LDW + col, acc[j][v]);
        }
      }
    }
  }
  __syncthreads();

  // Phase 3: combine weights = softmax over the N slots of each item (wave per row).
  for (int s = wave; s < S; s += 4) {
    const T* row = lg + (size_t)s * LDW;
    float mx = -INFINITY;
    for (int n = lane; n < N; n += 64) mx = fmaxf(mx, Elt<T>::load(row + n));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, kWave));
    float sum = 0.f;
    for (int n = lane; n < N; n += 64) sum += expf(Elt<T>::load(row + n) - mx);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, kWave);
    const size_t base = ((size_t)g * S + s) * N;
    for (int n = lane; n < N; n += 64) {
      float l = Elt<T>::load(row + n);
      Elt<T>::store(combine_w + base + n, expf(l - mx) / sum);
      if (logits_out != nullptr) Elt<T>::store(logits_out + base + n, l);
    }
  }
  // Phase 4: dispatch weights = softmax over the S items of each slot (thread per column).
  for (int n = tid; n < N; n += 256) {
    float mx = -INFINITY;
    for (int s = 0; s < S; ++s) mx = fmaxf(mx, Elt<T>::load(lg + (size_t)s * LDW + n));
    float sum = 0.f;
    for (int s = 0; s < S; ++s) sum += expf(Elt<T>::load(lg + (size_t)s * LDW + n) - mx);
    for (int s = 0; s < S; ++s) {
      float l = Elt<T>::load(lg + (size_t)s * LDW + n);
      Elt<T>::store(dispatch_w + ((size_t)g * S + s) * N + n, expf(l - mx) / sum);
    }
  }
}

// bfloat16 soft routing, fast path (N <= 128 slots, D <= 32 * 2 * KSW).
//
// One workgroup of eight waves per group, with the unit-norm slot parameters held
// in registers for the whole kernel: wave w keeps the B fragments of 16 slots for
// the whole contraction (v_mfma_f32_16x16x32_bf16).  The item rows then stream
// through once, 32 at a time: each wave loads four whole rows (coalesced), takes
// their norms from its registers, and writes the normalised rows into an LDS tile
// while the loads of the next 64 rows are already in flight; every wave multiplies
// the tile with its slots, and the logits of the group collect in LDS as
// bfloat16.  Both softmaxes (over slots for the combine weights, over items for
// the dispatch weights) are taken from that one copy, so memory sees the items
// once and each weight once.
constexpr int kSrThreads = 512;
constexpr int kSrRows = 32;

// Model widths the register-resident fast path is instantiated for.
inline bool soft_fast_width(int D) { return D == 256 || D == 384 || D == 512 || D == 768 || D == 1024; }

struct SoftLds {
  size_t xs, part, red, cmx, csum, lg, total;
};
inline SoftLds soft_lds_layout(int D, int SP, int NP) {
  SoftLds l;
  l.xs = 0;
  l.part = l.xs + (size_t)kSrRows * (D + 8) * 2;
  l.red = l.part;
  l.cmx = l.red + kSrThreads * sizeof(float);
  l.csum = l.cmx + 128 * sizeof(float);
  l.lg = l.csum + 128 * sizeof(float);
  l.total = l.lg + (size_t)SP * (NP + 8) * 2;
  return l;
}

// exp(l - mx) / sum as exp2(l * log2e - mx * log2e) * (1 / sum) with the hardware
// exp2 and reciprocal: relative error ~1e-6, against 4e-3 for the bfloat16 result.
constexpr float kLog2e = 1.4426950408889634f;

template <int KSW>
__global__ __launch_bounds__(kSrThreads) void soft_route_bf16_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ muw, bf16_t* __restrict__ dispatch_w,
    bf16_t* __restrict__ combine_w, bf16_t* __restrict__ logits_out, float scale, int scale_x, int S,
    int D, int N, int SP, int NP, SoftLds L) {
  constexpr int CP = (KSW + 7) / 8;   // 16-byte pieces of an item row per lane of a half wave
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem + L.xs);
  float* red = reinterpret_cast<float*>(smem + L.red);
  float* cmx = reinterpret_cast<float*>(smem + L.cmx);
  float* csum = reinterpret_cast<float*>(smem + L.csum);
  bf16_t* lg = reinterpret_cast<bf16_t*>(smem + L.lg);
  const int LDX = D + 8, LDW = NP + 8;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, h = lane >> 5;
  const int g = blockIdx.x;
  const bf16_t* xg = x + (size_t)g * S * D;
  const float sc = bf16r(scale);
  const int row_chunks = D / 8, row_tiles = SP / kSrRows;
  const int r16 = lane & 15, kq = lane >> 4;   // 16x16x32 fragment: row / column, k quarter
  const bool mma_on = wave * 16 < NP;

  // Slot parameters of this wave: slots wave*16 .. +16, every k step (D == 32 * KSW).
  bf16x8 bfr[KSW];
  {
    const bf16_t* brow = muw + (size_t)min(wave * 16 + r16, N - 1) * D + kq * 8;
#pragma unroll
    for (int i = 0; i < KSW; ++i)
      bfr[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(brow + i * 32));
  }

  // Combine weights of the item rows [s_begin, s_end): softmax over the N slots.
  // Half wave = one row, lane = four consecutive slots; two rows per half wave at a
  // time so that the two shuffle chains overlap.
  auto combine_rows = [&](int s_begin, int s_end) {
    for (int s0 = s_begin + wave * 4; s0 < s_end; s0 += 32) {
      const int c = m * 4;
      float l[2][4], mx[2];
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int s = s0 + 2 * r + h;
#pragma unroll
        for (int u = 0; u < 4; ++u) l[r][u] = -INFINITY;
        if (s < s_end && c < N) {
          const uint2 pr = *reinterpret_cast<const uint2*>(lg + (size_t)s * LDW + c);
          l[r][0] = bf_lo(pr.x); l[r][1] = bf_hi(pr.x); l[r][2] = bf_lo(pr.y); l[r][3] = bf_hi(pr.y);
        }
        mx[r] = fmaxf(fmaxf(l[r][0], l[r][1]), fmaxf(l[r][2], l[r][3]));
      }
#pragma unroll
      for (int o = 16; o > 0; o >>= 1)
#pragma unroll
        for (int r = 0; r < 2; ++r) mx[r] = fmaxf(mx[r], __shfl_xor(mx[r], o, kWave));
      float e[2][4], sum[2];
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const float mb = mx[r] * kLog2e;
        sum[r] = 0.f;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          e[r][u] = __builtin_amdgcn_exp2f(fmaf(l[r][u], kLog2e, -mb));   // exp2(-inf) = 0 past N
          sum[r] += e[r][u];
        }
      }
#pragma unroll
      for (int o = 16; o > 0; o >>= 1)
#pragma unroll
        for (int r = 0; r < 2; ++r) sum[r] += __shfl_xor(sum[r], o, kWave);
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int s = s0 + 2 * r + h;
        const float rs = __builtin_amdgcn_rcpf(sum[r]);
        if (s < s_end && c < N)
          *reinterpret_cast<uint2*>(combine_w + ((size_t)g * S + s) * N + c) = make_uint2(
              pack_bf16x2(e[r][0] * rs, e[r][1] * rs), pack_bf16x2(e[r][2] * rs, e[r][3] * rs));
      }
    }
  };

  // Four item rows per wave and tile, one row per half wave at a time (rows
  // wave*4 + 2*i + h); rows past S re-read row S-1 and are written as zeros.
  auto load_rows = [&](uint4 (&raw)[2][CP], int t) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int r = min(t * kSrRows + wave * 4 + 2 * i + h, S - 1);
#pragma unroll
      for (int ps = 0; ps < CP; ++ps) {
        const int c = min(ps * 32 + m, row_chunks - 1);
        raw[i][ps] = *reinterpret_cast<const uint4*>(xg + (size_t)r * D + c * 8);
      }
    }
  };

  // One tile of 32 item rows, held in raw; its registers then take the tile after next.
  auto tile = [&](uint4 (&raw)[2][CP], int t) {
    // norms from the registers, normalised rows into the LDS tile
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      float sq = 0.f;
#pragma unroll
      for (int ps = 0; ps < CP; ++ps) {
        const uint32_t w4[4] = {raw[i][ps].x, raw[i][ps].y, raw[i][ps].z, raw[i][ps].w};
        float tsum = 0.f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float lo = bf_lo(w4[q]), hi = bf_hi(w4[q]);
          tsum = fmaf(lo, lo, tsum);
          tsum = fmaf(hi, hi, tsum);
        }
        if (ps * 32 + m < row_chunks) sq += tsum;
      }
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) sq += __shfl_xor(sq, o, kWave);
      const int lrow = wave * 4 + 2 * i + h;
      const float inv = t * kSrRows + lrow < S ? 1.0f / sqrtf(sq + kNormEps) : 0.f;
#pragma unroll
      for (int ps = 0; ps < CP; ++ps) {
        const int c = ps * 32 + m;
        const uint32_t w4[4] = {raw[i][ps].x, raw[i][ps].y, raw[i][ps].z, raw[i][ps].w};
        uint32_t o4[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float lo = bf_lo(w4[q]) * inv, hi = bf_hi(w4[q]) * inv;
          if (scale_x) { lo = bf16r(lo) * sc; hi = bf16r(hi) * sc; }
          o4[q] = pack_bf16x2(lo, hi);
        }
        if (c < row_chunks)
          *reinterpret_cast<uint4*>(xs + (size_t)lrow * LDX + c * 8) = make_uint4(o4[0], o4[1], o4[2], o4[3]);
      }
    }
    wait_lgkmcnt0();
    raw_barrier();
    if (t + 2 < row_tiles) load_rows(raw, t + 2);
    // the logits of the previous tile are complete: their combine weights fill the
    // time the loads are in flight
    if (t > 0) combine_rows((t - 1) * kSrRows, min(t * kSrRows, S));

    if (mma_on) {
      floatx4 acc[2];
#pragma unroll
      for (int rh = 0; rh < 2; ++rh)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[rh][v] = 0.f;
      const bf16_t* arow = xs + (size_t)r16 * LDX + kq * 8;
#pragma unroll
      for (int i = 0; i < KSW; ++i) {
        const int ko = i * 32;
#pragma unroll
        for (int rh = 0; rh < 2; ++rh) {
          const bf16x8 af = __builtin_bit_cast(
              bf16x8, *reinterpret_cast<const uint4*>(arow + (size_t)rh * 16 * LDX + ko));
          acc[rh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, bfr[i], acc[rh], 0, 0, 0);
        }
        // bound how many fragment reads the scheduler hoists (register pressure)
        if ((i & 3) == 3) __builtin_amdgcn_sched_barrier(0);
      }
      mfma_result_fence();
      const int col = wave * 16 + r16;
#pragma unroll
      for (int rh = 0; rh < 2; ++rh)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int row = t * kSrRows + rh * 16 + kq * 4 + v;
          lg[(size_t)row * LDW + col] = f2bf(acc[rh][v]);
        }
    }
    wait_lgkmcnt0();
    raw_barrier();
  };

  uint4 raw0[2][CP], raw1[2][CP];
  load_rows(raw0, 0);
  if (row_tiles > 1) load_rows(raw1, 1);
  for (int t = 0; t < row_tiles; t += 2) {
    tile(raw0, t);
    if (t + 1 < row_tiles) tile(raw1, t + 1);
  }
  __syncthreads();
  combine_rows((row_tiles - 1) * kSrRows, S);

  // Thread -> (16-byte piece c of a weights row, rows s = sr, sr + rpp, ...).
  const int lchunks = N / 8, rpp = kSrThreads / lchunks;
  const int sr = tid / lchunks, pc = tid - sr * lchunks;
  if (logits_out != nullptr && sr < rpp) {
    for (int s = sr; s < S; s += rpp)
      *reinterpret_cast<uint4*>(logits_out + ((size_t)g * S + s) * N + pc * 8) =
          *reinterpret_cast<const uint4*>(lg + (size_t)s * LDW + pc * 8);
  }

  // Dispatch weights: softmax over the S items of each slot.  For the maxima and
  // sums a column is shared by RG threads that take every RG-th row and meet in LDS.
  {
    const int RG = kSrThreads / NP;
    const int n = tid % NP, rg = tid / NP;
    const bool act = rg < RG;
    float mx = -INFINITY;
    if (act)
#pragma unroll 8
      for (int s = rg; s < S; s += RG) mx = fmaxf(mx, bf2f(lg[(size_t)s * LDW + n]));
    red[tid] = mx;
    __syncthreads();
    if (act) {
      mx = -INFINITY;
      for (int q = 0; q < RG; ++q) mx = fmaxf(mx, red[q * NP + n]);
    }
    __syncthreads();
    const float mb = mx * kLog2e;
    float sum = 0.f;
    if (act)
#pragma unroll 8
      for (int s = rg; s < S; s += RG)
        sum += __builtin_amdgcn_exp2f(fmaf(bf2f(lg[(size_t)s * LDW + n]), kLog2e, -mb));
    red[tid] = sum;
    __syncthreads();
    if (act && rg == 0) {
      sum = 0.f;
      for (int q = 0; q < RG; ++q) sum += red[q * NP + n];
      cmx[n] = mb;
      csum[n] = __builtin_amdgcn_rcpf(sum);
    }
    __syncthreads();
    if (sr < rpp) {
      float cm[8], cr[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        cm[u] = cmx[pc * 8 + u];
        cr[u] = csum[pc * 8 + u];
      }
#pragma unroll 4
      for (int s = sr; s < S; s += rpp) {
        const uint4 rawl = *reinterpret_cast<const uint4*>(lg + (size_t)s * LDW + pc * 8);
        const uint32_t w4[4] = {rawl.x, rawl.y, rawl.z, rawl.w};
        uint32_t o4[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float lo = __builtin_amdgcn_exp2f(fmaf(bf_lo(w4[u]), kLog2e, -cm[2 * u])) * cr[2 * u];
          const float hi = __builtin_amdgcn_exp2f(fmaf(bf_hi(w4[u]), kLog2e, -cm[2 * u + 1])) * cr[2 * u + 1];
          o4[u] = pack_bf16x2(lo, hi);
        }
        *reinterpret_cast<uint4*>(dispatch_w + ((size_t)g * S + s) * N + pc * 8) =
            make_uint4(o4[0], o4[1], o4[2], o4[3]);
      }
    }
  }
}

// Reductions over the 32 lanes of a half wave: four DPP steps inside a row of 16 lanes
// (quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror), then one exchange
// between the two rows.  Every lane ends with the result.
template <int CTRL>
__device__ __forceinline__ float dpp_lane(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float half_wave_sum(float v) {
  v += dpp_lane<0xB1>(v);
  v += dpp_lane<0x4E>(v);
  v += dpp_lane<0x141>(v);
  v += dpp_lane<0x140>(v);
  return v + __shfl_xor(v, 16, kWave);
}
// The same where only the upper 16 lanes of the half wave need the result: the last step is
// a DPP broadcast of lane 15 of the lower row into the upper one (row_bcast15 on rows 1
// and 3), no lane exchange through the LDS unit.
__device__ __forceinline__ float row_bcast15(float v) {
  const int x = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(x, x, 0x142, 0xa, 0xf, false));
}
__device__ __forceinline__ float half_wave_min_upper(float v) {
  v = fminf(v, dpp_lane<0xB1>(v));
  v = fminf(v, dpp_lane<0x4E>(v));
  v = fminf(v, dpp_lane<0x141>(v));
  v = fminf(v, dpp_lane<0x140>(v));
  return fminf(v, row_bcast15(v));
}
__device__ __forceinline__ float half_wave_max_upper(float v) {
  v = fmaxf(v, dpp_lane<0xB1>(v));
  v = fmaxf(v, dpp_lane<0x4E>(v));
  v = fmaxf(v, dpp_lane<0x141>(v));
  v = fmaxf(v, dpp_lane<0x140>(v));
  return fmaxf(v, row_bcast15(v));
}
__device__ __forceinline__ float half_wave_max(float v) {
  v = fmaxf(v, dpp_lane<0xB1>(v));
  v = fmaxf(v, dpp_lane<0x4E>(v));
  v = fmaxf(v, dpp_lane<0x141>(v));
  v = fmaxf(v, dpp_lane<0x140>(v));
  return fmaxf(v, __shfl_xor(v, 16, kWave));
}

// soft_route_bf16_kernel with the waves of a workgroup in two roles (N <= 128 slots,
// D = 32 * KSW <= 768).  In the single-role kernel every wave normalises rows (VALU), then
// every wave multiplies (LDS reads and matrix cores), then every wave takes the row
// softmax (VALU): the units take turns.  Here waves 0..3 only fetch and normalise item rows
// (tile t + 1 into one of two LDS tiles) while waves 4..7, each with the unit-norm
// parameters of 32 slots in registers, multiply tile t and take the combine weights of
// tile t - 1; one barrier per tile hands the tiles over.  A consumer wave reads an item
// tile once for 32 slots (the single-role kernel: once per 16), so the LDS reads halve as
// well.  The arithmetic per element is that of soft_route_bf16_kernel.
struct SoftPipeLds {
  size_t xs, red, cmx, csum, lg, total;
};
inline SoftPipeLds soft_pipe_lds_layout(int D, int SP, int NP, int rows) {
  SoftPipeLds l;
  l.xs = 0;                                           // two tiles of `rows` normalised rows
  l.red = 0;                                          // (the column reductions reuse them)
  l.cmx = l.xs + (size_t)2 * rows * (D + 16) * 2;
  l.csum = l.cmx + 128 * sizeof(float);
  l.lg = l.csum + 128 * sizeof(float);
  l.total = l.lg + (size_t)SP * (NP + 8) * 2;
  return l;
}

constexpr int kTailRows = 8;   // rows per thread of the register-resident dispatch softmax
template <int KSW, int ROWS, bool SCALE_X>
__global__ __launch_bounds__(kSrThreads) void soft_route_roles_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ muw, bf16_t* __restrict__ dispatch_w,
    bf16_t* __restrict__ combine_w, bf16_t* __restrict__ logits_out, float scale, int S, int D,
    int N, int SP, int NP, SoftPipeLds L, float* __restrict__ stats_partial) {
  constexpr int CP = (KSW + 7) / 8;   // 16-byte pieces of an item row per lane of a half wave
  constexpr int RPW = ROWS / 4;       // rows of a tile per producer wave
  constexpr int PAIRS = RPW / 2;      // a half wave takes one row at a time
  constexpr int RB = ROWS / 16;       // 16-row blocks of a tile
  static_assert(ROWS == 16 || ROWS == 32, "tile height");
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem + L.xs);
  float* red = reinterpret_cast<float*>(smem + L.red);
  float* cmx = reinterpret_cast<float*>(smem + L.cmx);
  float* csum = reinterpret_cast<float*>(smem + L.csum);
  bf16_t* lg = reinterpret_cast<bf16_t*>(smem + L.lg);
  const int LDX = D + 16, LDW = NP + 8;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = lane & 31, h = lane >> 5;
  const int g = blockIdx.x;
  const bf16_t* xg = x + (size_t)g * S * D;
  const float sc = bf16r(scale);
  const int row_chunks = D / 8, row_tiles = SP / ROWS;
  bf16_t* const xtile[2] = {xs, xs + (size_t)ROWS * LDX};

  // Combine weights of the item rows [s_begin, s_end) of one tile: softmax over the N slots.
  // Each role takes half of the tile's rows (tile t - 1 while tile t is multiplied, which
  // keeps the two roles' iterations about equally long), its four waves a quarter of those;
  // half wave = one row, lane = four consecutive slots.
  constexpr int CR = ROWS / 16;   // rows of a tile per half wave: their chains overlap
  // With `stats_partial` (only where the register-resident dispatch softmax applies) the
  // launch also leaves the group's partial sums of the router's monitoring scalars: the
  // sums over the items of the smallest / largest combine weight, and over the slots of the
  // smallest / largest dispatch weight, taken from the rounded values that are stored.
  float row_min_sum = 0.f, row_max_sum = 0.f;
  float* const st_rows = cmx;                         // 8 waves x 2 half waves x 2
  auto combine_rows = [&](int s_begin, int s_end) {
    {
      const int s0 = s_begin + (wave >> 2) * (ROWS / 2) + (wave & 3) * (ROWS / 8);
      const int c = m * 4;
      float l[CR][4], mx[CR];
#pragma unroll
      for (int r = 0; r < CR; ++r) {
        const int s = s0 + 2 * r + h;
#pragma unroll
        for (int u = 0; u < 4; ++u) l[r][u] = -INFINITY;
        if (s < s_end && c < N) {
          const uint2 pr = *reinterpret_cast<const uint2*>(lg + (size_t)s * LDW + c);
          l[r][0] = bf_lo(pr.x); l[r][1] = bf_hi(pr.x); l[r][2] = bf_lo(pr.y); l[r][3] = bf_hi(pr.y);
        }
        mx[r] = fmaxf(fmaxf(l[r][0], l[r][1]), fmaxf(l[r][2], l[r][3]));
      }
#pragma unroll
      for (int r = 0; r < CR; ++r) mx[r] = half_wave_max(mx[r]);
      float e[CR][4], sum[CR];
#pragma unroll
      for (int r = 0; r < CR; ++r) {
        const float mb = mx[r] * kLog2e;
        sum[r] = 0.f;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          e[r][u] = __builtin_amdgcn_exp2f(fmaf(l[r][u], kLog2e, -mb));   // exp2(-inf) = 0 past N
          sum[r] += e[r][u];
        }
      }
#pragma unroll
      for (int r = 0; r < CR; ++r) sum[r] = half_wave_sum(sum[r]);
#pragma unroll
      for (int r = 0; r < CR; ++r) {
        const int s = s0 + 2 * r + h;
        const float rs = __builtin_amdgcn_rcpf(sum[r]);
        const uint32_t p0 = pack_bf16x2(e[r][0] * rs, e[r][1] * rs);
        const uint32_t p1 = pack_bf16x2(e[r][2] * rs, e[r][3] * rs);
        if (s < s_end && c < N)
          *reinterpret_cast<uint2*>(combine_w + ((size_t)g * S + s) * N + c) = make_uint2(p0, p1);
        if (stats_partial != nullptr) {    // smallest and largest stored weight of the row
          float lo = fminf(fminf(bf_lo(p0), bf_hi(p0)), fminf(bf_lo(p1), bf_hi(p1)));
          float hi = fmaxf(fmaxf(bf_lo(p0), bf_hi(p0)), fmaxf(bf_lo(p1), bf_hi(p1)));
          if (c >= N) { lo = INFINITY; hi = -INFINITY; }
          lo = half_wave_min_upper(lo);     // (lanes 16..31 of the half wave hold the result)
          hi = half_wave_max_upper(hi);
          if (s < s_end) { row_min_sum += lo; row_max_sum += hi; }
        }
      }
    }
  };
  if (wave < 4) {
    // ---- producers: item rows wave * RPW .. + RPW of every tile
    auto load_rows = [&](uint4 (&raw)[PAIRS][CP], int t) {
#pragma unroll
      for (int i = 0; i < PAIRS; ++i) {
        const int r = min(t * ROWS + wave * RPW + 2 * i + h, S - 1);   // rows past S: zeros below
#pragma unroll
        for (int ps = 0; ps < CP; ++ps) {
          const int c = min(ps * 32 + m, row_chunks - 1);
          raw[i][ps] = *reinterpret_cast<const uint4*>(xg + (size_t)r * D + c * 8);
        }
      }
    };
    auto norm_rows = [&](uint4 (&raw)[PAIRS][CP], int t, bf16_t* xt) {
#pragma unroll
      for (int i = 0; i < PAIRS; ++i) {
        float sq = 0.f;
#pragma unroll
        for (int ps = 0; ps < CP; ++ps) {
          const uint32_t w4[4] = {raw[i][ps].x, raw[i][ps].y, raw[i][ps].z, raw[i][ps].w};
          float tsum = 0.f;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float lo = bf_lo(w4[q]), hi = bf_hi(w4[q]);
            tsum = fmaf(lo, lo, tsum);
            tsum = fmaf(hi, hi, tsum);
          }
          if (KSW % 8 == 0 || ps * 32 + m < row_chunks) sq += tsum;
        }
        sq = half_wave_sum(sq);
        const int lrow = wave * RPW + 2 * i + h;
        const float inv = t * ROWS + lrow < S ? 1.0f / sqrtf(sq + kNormEps) : 0.f;
#pragma unroll
        for (int ps = 0; ps < CP; ++ps) {
          const int c = ps * 32 + m;
          const uint32_t w4[4] = {raw[i][ps].x, raw[i][ps].y, raw[i][ps].z, raw[i][ps].w};
          uint32_t o4[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float lo = bf_lo(w4[q]) * inv, hi = bf_hi(w4[q]) * inv;
            if (SCALE_X) { lo = bf16r(lo) * sc; hi = bf16r(hi) * sc; }
            o4[q] = pack_bf16x2(lo, hi);
          }
          if (KSW % 8 == 0 || c < row_chunks)
            *reinterpret_cast<uint4*>(xt + (size_t)lrow * LDX + c * 8) = make_uint4(o4[0], o4[1], o4[2], o4[3]);
        }
      }
    };
    // Tile t + 1 is normalised while tile t is multiplied; its registers then fetch tile
    // t + 3, so the rows of two tiles are always on their way.
    uint4 raw0[PAIRS][CP], raw1[PAIRS][CP];
    load_rows(raw0, 0);
    if (row_tiles > 1) load_rows(raw1, 1);
    norm_rows(raw0, 0, xtile[0]);
    if (row_tiles > 2) load_rows(raw0, 2);
    wait_lgkmcnt0();
    raw_barrier();
    for (int t = 0; t < row_tiles; t += 2) {
      if (t + 1 < row_tiles) {
        norm_rows(raw1, t + 1, xtile[1]);
        if (t + 3 < row_tiles) load_rows(raw1, t + 3);
      }
      // (the logits of tile t - 1 were complete at the last barrier)
      if (t > 0) combine_rows((t - 1) * ROWS, min(t * ROWS, S));
      wait_lgkmcnt0();
      raw_barrier();
      if (t + 1 < row_tiles) {
        if (t + 2 < row_tiles) {
          norm_rows(raw0, t + 2, xtile[0]);
          if (t + 4 < row_tiles) load_rows(raw0, t + 4);
        }
        combine_rows(t * ROWS, min((t + 1) * ROWS, S));
        wait_lgkmcnt0();
        raw_barrier();
      }
    }
    combine_rows((row_tiles - 1) * ROWS, S);
  } else {
    // ---- consumers: slots cw * 32 .. + 32 of every tile, and the combine weights
    const int cw = wave - 4;
    const int r16 = lane & 15, kq = lane >> 4;   // 16x16x32 fragment: row / column, k quarter
    const bool mma_on = cw * 32 < NP;
    bf16x8 bfr[2][KSW];   // (soft_prep_mu_kernel wrote them in this order: 1 KB per load)
    if (mma_on) {
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
        const bf16_t* frag = muw + ((size_t)(cw * 2 + cb) * KSW * 64 + lane) * 8;
#pragma unroll
        for (int i = 0; i < KSW; ++i)
          bfr[cb][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(frag + (size_t)i * 512));
      }
    }
    auto multiply = [&](int t, const bf16_t* xt) {
      if (!mma_on) return;
      floatx4 acc[RB][2];
#pragma unroll
      for (int rh = 0; rh < RB; ++rh)
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[rh][cb][v] = 0.f;
      const bf16_t* arow = xt + (size_t)r16 * LDX + kq * 8;
      // The item fragments of k step i + kAhead are requested before the MFMAs of step i
      // (a ring of kAhead + 1 register sets; the scheduling barriers keep that order).
      constexpr int kAhead = 2;
      bf16x8 af[kAhead + 1][RB];
      auto read_step = [&](int i, bf16x8 (&dst)[RB]) {
#pragma unroll
        for (int rh = 0; rh < RB; ++rh)
          dst[rh] = __builtin_bit_cast(
              bf16x8, *reinterpret_cast<const uint4*>(arow + (size_t)rh * 16 * LDX + i * 32));
      };
#pragma unroll
      for (int i = 0; i < kAhead && i < KSW; ++i) read_step(i, af[i]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < KSW; ++i) {
        if (i + kAhead < KSW) read_step(i + kAhead, af[(i + kAhead) % (kAhead + 1)]);
#pragma unroll
        for (int rh = 0; rh < RB; ++rh)
#pragma unroll
          for (int cb = 0; cb < 2; ++cb)
            acc[rh][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i % (kAhead + 1)][rh], bfr[cb][i],
                                                                 acc[rh][cb], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      mfma_result_fence();
#pragma unroll
      for (int rh = 0; rh < RB; ++rh)
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int row = t * ROWS + rh * 16 + kq * 4 + v;
            lg[(size_t)row * LDW + cw * 32 + cb * 16 + r16] = f2bf(acc[rh][cb][v]);
          }
    };
    raw_barrier();
    for (int t = 0; t < row_tiles; ++t) {
      multiply(t, xtile[t & 1]);
      // (the logits of tile t - 1 were complete at the last barrier)
      if (t > 0) combine_rows((t - 1) * ROWS, min(t * ROWS, S));
      wait_lgkmcnt0();
      raw_barrier();
    }
    combine_rows((row_tiles - 1) * ROWS, S);
  }
  if (stats_partial != nullptr && m == 31) {
    st_rows[(wave * 2 + h) * 2] = row_min_sum;
    st_rows[(wave * 2 + h) * 2 + 1] = row_max_sum;
  }

  // Thread -> (16-byte piece c of a weights row, rows s = sr, sr + rpp, ...).
  const int lchunks = N / 8, rpp = kSrThreads / lchunks;
  const int sr = tid / lchunks, pc = tid - sr * lchunks;
  if (logits_out != nullptr && sr < rpp) {
    for (int s = sr; s < S; s += rpp)
      *reinterpret_cast<uint4*>(logits_out + ((size_t)g * S + s) * N + pc * 8) =
          *reinterpret_cast<const uint4*>(lg + (size_t)s * LDW + pc * 8);
  }

  // Dispatch weights: softmax over the S items of each slot.
  if (SP <= 32 * kTailRows) {
    // Up to 256 items: a thread keeps one 16-byte piece (8 slots) of every 32nd row in
    // registers, so the logits are read from LDS once and every exponential is taken once.
    // Maxima and sums of a column meet across the lanes of a wave (rows 16 and 32 lanes
    // apart), then across the waves in LDS (the item tiles, which nobody reads any more).
    const int tc = tid & 15, tr = tid >> 4;
    const bool col_on = tc * 8 < NP;
    float* red_max = red;
    float* red_sum = red + 8 * 128;
    uint32_t lw[kTailRows][4];
    float cm[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) cm[u] = -INFINITY;
#pragma unroll
    for (int j = 0; j < kTailRows; ++j) {
      const int s_ = tr + 32 * j;
      uint4 q = make_uint4(0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u);   // -inf pairs
      if (s_ < S && col_on) q = *reinterpret_cast<const uint4*>(lg + (size_t)s_ * LDW + tc * 8);
      lw[j][0] = q.x; lw[j][1] = q.y; lw[j][2] = q.z; lw[j][3] = q.w;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        cm[2 * u] = fmaxf(cm[2 * u], bf_lo(lw[j][u]));
        cm[2 * u + 1] = fmaxf(cm[2 * u + 1], bf_hi(lw[j][u]));
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      cm[u] = fmaxf(cm[u], __shfl_xor(cm[u], 16, kWave));
      cm[u] = fmaxf(cm[u], __shfl_xor(cm[u], 32, kWave));
    }
    if (lane < 16) {
      *reinterpret_cast<float4*>(red_max + wave * 128 + tc * 8) = make_float4(cm[0], cm[1], cm[2], cm[3]);
      *reinterpret_cast<float4*>(red_max + wave * 128 + tc * 8 + 4) = make_float4(cm[4], cm[5], cm[6], cm[7]);
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const float4 a = *reinterpret_cast<const float4*>(red_max + w * 128 + tc * 8);
      const float4 b = *reinterpret_cast<const float4*>(red_max + w * 128 + tc * 8 + 4);
      const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int u = 0; u < 8; ++u) cm[u] = w == 0 ? v[u] : fmaxf(cm[u], v[u]);
    }
    float ev[kTailRows][8], cs[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      cm[u] *= kLog2e;
      cs[u] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < kTailRows; ++j)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        ev[j][2 * u] = __builtin_amdgcn_exp2f(fmaf(bf_lo(lw[j][u]), kLog2e, -cm[2 * u]));   // exp2(-inf) = 0
        ev[j][2 * u + 1] = __builtin_amdgcn_exp2f(fmaf(bf_hi(lw[j][u]), kLog2e, -cm[2 * u + 1]));
        cs[2 * u] += ev[j][2 * u];
        cs[2 * u + 1] += ev[j][2 * u + 1];
      }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      cs[u] += __shfl_xor(cs[u], 16, kWave);
      cs[u] += __shfl_xor(cs[u], 32, kWave);
    }
    if (lane < 16) {
      *reinterpret_cast<float4*>(red_sum + wave * 128 + tc * 8) = make_float4(cs[0], cs[1], cs[2], cs[3]);
      *reinterpret_cast<float4*>(red_sum + wave * 128 + tc * 8 + 4) = make_float4(cs[4], cs[5], cs[6], cs[7]);
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const float4 a = *reinterpret_cast<const float4*>(red_sum + w * 128 + tc * 8);
      const float4 b = *reinterpret_cast<const float4*>(red_sum + w * 128 + tc * 8 + 4);
      const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int u = 0; u < 8; ++u) cs[u] = w == 0 ? v[u] : cs[u] + v[u];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) cs[u] = __builtin_amdgcn_rcpf(cs[u]);
    float dmin[8], dmax[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      dmin[u] = INFINITY;
      dmax[u] = -INFINITY;
    }
#pragma unroll
    for (int j = 0; j < kTailRows; ++j) {
      const int s_ = tr + 32 * j;
      uint32_t o[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) o[u] = pack_bf16x2(ev[j][2 * u] * cs[2 * u], ev[j][2 * u + 1] * cs[2 * u + 1]);
      if (s_ < S && tc * 8 < N)
        *reinterpret_cast<uint4*>(dispatch_w + ((size_t)g * S + s_) * N + tc * 8) =
            make_uint4(o[0], o[1], o[2], o[3]);
      if (stats_partial != nullptr && s_ < S) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          dmin[2 * u] = fminf(dmin[2 * u], bf_lo(o[u]));
          dmax[2 * u] = fmaxf(dmax[2 * u], bf_lo(o[u]));
          dmin[2 * u + 1] = fminf(dmin[2 * u + 1], bf_hi(o[u]));
          dmax[2 * u + 1] = fmaxf(dmax[2 * u + 1], bf_hi(o[u]));
        }
      }
    }
    if (stats_partial != nullptr) {
      // Smallest / largest stored weight of every slot: across the lanes of a wave, across
      // the waves in LDS, then wave 0 adds up the slots and the producers' row sums.
      float* st_min = red + 16 * 128;
      float* st_max = red + 24 * 128;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        dmin[u] = fminf(dmin[u], __shfl_xor(dmin[u], 16, kWave));
        dmin[u] = fminf(dmin[u], __shfl_xor(dmin[u], 32, kWave));
        dmax[u] = fmaxf(dmax[u], __shfl_xor(dmax[u], 16, kWave));
        dmax[u] = fmaxf(dmax[u], __shfl_xor(dmax[u], 32, kWave));
      }
      if (lane < 16) {
        *reinterpret_cast<float4*>(st_min + wave * 128 + tc * 8) = make_float4(dmin[0], dmin[1], dmin[2], dmin[3]);
        *reinterpret_cast<float4*>(st_min + wave * 128 + tc * 8 + 4) = make_float4(dmin[4], dmin[5], dmin[6], dmin[7]);
        *reinterpret_cast<float4*>(st_max + wave * 128 + tc * 8) = make_float4(dmax[0], dmax[1], dmax[2], dmax[3]);
        *reinterpret_cast<float4*>(st_max + wave * 128 + tc * 8 + 4) = make_float4(dmax[4], dmax[5], dmax[6], dmax[7]);
      }
      __syncthreads();
      if (wave == 0) {
        float smin = 0.f, smax = 0.f;
        if (lane < 16) {
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            float lo = INFINITY, hi = -INFINITY;
            for (int w = 0; w < 8; ++w) {
              lo = fminf(lo, st_min[w * 128 + lane * 8 + u]);
              hi = fmaxf(hi, st_max[w * 128 + lane * 8 + u]);
            }
            if (lane * 8 + u < N) {
              smin += lo;
              smax += hi;
            }
          }
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) {
          smin += __shfl_xor(smin, o, kWave);
          smax += __shfl_xor(smax, o, kWave);
        }
        if (lane == 0) {
          float rmin = 0.f, rmax = 0.f;
          for (int q = 0; q < 16; ++q) {
            rmin += st_rows[2 * q];
            rmax += st_rows[2 * q + 1];
          }
          stats_partial[(size_t)g * 4 + 0] = rmin;
          stats_partial[(size_t)g * 4 + 1] = rmax;
          stats_partial[(size_t)g * 4 + 2] = smin;
          stats_partial[(size_t)g * 4 + 3] = smax;
        }
      }
    }
  } else {
    // More items: three passes over the logits in LDS.  For the maxima and sums a column
    // is shared by RG threads that take every RG-th row and meet in LDS.
    const int RG = kSrThreads / NP;
    const int n = tid % NP, rg = tid / NP;
    const bool act = rg < RG;
    float mx = -INFINITY;
    if (act)
#pragma unroll 8
      for (int s = rg; s < S; s += RG) mx = fmaxf(mx, bf2f(lg[(size_t)s * LDW + n]));
    red[tid] = mx;
    __syncthreads();
    if (act) {
      mx = -INFINITY;
      for (int q = 0; q < RG; ++q) mx = fmaxf(mx, red[q * NP + n]);
    }
    __syncthreads();
    const float mb = mx * kLog2e;
    float sum = 0.f;
    if (act)
#pragma unroll 8
      for (int s = rg; s < S; s += RG)
        sum += __builtin_amdgcn_exp2f(fmaf(bf2f(lg[(size_t)s * LDW + n]), kLog2e, -mb));
    red[tid] = sum;
    __syncthreads();
    if (act && rg == 0) {
      sum = 0.f;
      for (int q = 0; q < RG; ++q) sum += red[q * NP + n];
      cmx[n] = mb;
      csum[n] = __builtin_amdgcn_rcpf(sum);
    }
    __syncthreads();
    if (sr < rpp) {
      float cm[8], cr[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        cm[u] = cmx[pc * 8 + u];
        cr[u] = csum[pc * 8 + u];
      }
#pragma unroll 4
      for (int s = sr; s < S; s += rpp) {
        const uint4 rawl = *reinterpret_cast<const uint4*>(lg + (size_t)s * LDW + pc * 8);
        const uint32_t w4[4] = {rawl.x, rawl.y, rawl.z, rawl.w};
        uint32_t o4[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float lo = __builtin_amdgcn_exp2f(fmaf(bf_lo(w4[u]), kLog2e, -cm[2 * u])) * cr[2 * u];
          const float hi = __builtin_amdgcn_exp2f(fmaf(bf_hi(w4[u]), kLog2e, -cm[2 * u + 1])) * cr[2 * u + 1];
          o4[u] = pack_bf16x2(lo, hi);
        }
        *reinterpret_cast<uint4*>(dispatch_w + ((size_t)g * S + s) * N + pc * 8) =
            make_uint4(o4[0], o4[1], o4[2], o4[3]);
      }
    }
  }
}

// Dense einsum between per-group weights and data on the float32 matrix cores.
//   DISPATCH: out[slot(g,mm)] = sum_s w[g,s,mm] * data[g,s,:]      (M = E*C, Kd = S)
//   COMBINE:  out[g,mm,:]     = sum_n w[g,mm,n] * data[slot(g,n)]  (M = S,   Kd = E*C)
template <bool DISPATCH>
__global__ __launch_bounds__(256) void einsum_kernel(const void* __restrict__ w,
                                                     const void* __restrict__ data,
                                                     void* __restrict__ out, int G, int S, int E,
                                                     int C, int D, int wdt, int ddt, int odt) {
  __shared__ float sa[64][16 + 1];
  __shared__ float sb[16][64 + 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m = lane & 31, h = lane >> 5;
  const int g = blockIdx.z;
  const int N = E * C;
  const int M = DISPATCH ? N : S;
  const int Kd = DISPATCH ? S : N;
  const int row0 = blockIdx.y * 64, col0 = blockIdx.x * 64;
  const size_t wbase = (size_t)g * S * N;
  floatx16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  for (int k0 = 0; k0 < Kd; k0 += 16) {
    float va[4], vb[4];
    if (DISPATCH) {
      const int kk = k0 + (tid >> 4), m4 = row0 + (tid & 15) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        va[i] = (kk < Kd && m4 + i < M) ? load_w(w, wbase + (size_t)kk * N + m4 + i, wdt) : 0.f;
    } else {
      const int mm = row0 + (tid >> 2), k4 = k0 + (tid & 3) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        va[i] = (mm < M && k4 + i < Kd) ? load_w(w, wbase + (size_t)mm * N + k4 + i, wdt) : 0.f;
    }
    {
      const int kk = k0 + (tid >> 4), n4 = col0 + (tid & 15) * 4;
      size_t rowi = 0;
      if (kk < Kd) rowi = DISPATCH ? (size_t)g * S + kk : (size_t)slot_row(kk / C, g, kk % C, G, E, C);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        vb[i] = (kk < Kd && n4 + i < D) ? load_any(data, rowi * D + n4 + i, ddt) : 0.f;
    }
    __syncthreads();
    if (DISPATCH) {
#pragma unroll
      for (int i = 0; i < 4; ++i) sa[(tid & 15) * 4 + i][tid >> 4] = va[i];
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) sa[tid >> 2][(tid & 3) * 4 + i] = va[i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) sb[tid >> 4][(tid & 15) * 4 + i] = vb[i];
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(sa[wm * 32 + m][ks * 2 + h],
                                                 sb[ks * 2 + h][wn * 32 + m], acc, 0, 0, 0);
  }
  mfma_result_fence();
  const int col = col0 + wn * 32 + m;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int mm = row0 + wm * 32 + (v >> 2) * 8 + h * 4 + (v & 3);
    if (mm < M && col < D) {
      size_t orow = DISPATCH ? (size_t)slot_row(mm / C, g, mm % C, G, E, C) : (size_t)g * S + mm;
      store_any(out, orow * D + col, acc[v], odt);
    }
  }
}

int check_einsum(const VmoeEinsumParams* p, bool dispatch) {
  if (p == nullptr || p->w == nullptr || p->data == nullptr || p->out == nullptr) return VMOE_E_NULL;
  if (p->G < 1 || p->S < 1 || p->E < 1 || p->C < 1 || p->D < 1) return VMOE_E_SHAPE;
  if (p->G > 65535) return VMOE_E_UNSUPPORTED;
  if (p->w_dtype < VMOE_W_F32 || p->w_dtype > VMOE_W_BOOL) return VMOE_E_DTYPE;
  if (!dispatch && p->w_dtype == VMOE_W_BOOL) return VMOE_E_DTYPE;
  if ((p->data_dtype != VMOE_F32 && p->data_dtype != VMOE_BF16) ||
      (p->out_dtype != VMOE_F32 && p->out_dtype != VMOE_BF16))
    return VMOE_E_DTYPE;
  if ((int64_t)p->E * p->G * p->C >= INT32_MAX || (int64_t)p->G * p->S >= INT32_MAX)
    return VMOE_E_OVERFLOW;
  return VMOE_OK;
}


// Monitoring scalars of the Soft MoE router (vmoe/projects/soft_moe/router.py:119-125),
// per group: sum over items of the min / max over slots of the combine weights, and
// sum over slots of the min / max over items of the dispatch weights.  The caller
// sums the (G, 4) partials and divides by the counts.
template <typename T>
__global__ __launch_bounds__(256) void soft_stats_kernel(const T* __restrict__ combine_w,
                                                         const T* __restrict__ dispatch_w,
                                                         float* __restrict__ partial, int S, int N) {
  __shared__ float red[4][4];
  const int g = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* cw = combine_w + (size_t)g * S * N;
  const T* dw = dispatch_w + (size_t)g * S * N;
  // combine weights: a wave per item row
  float cmin_sum = 0.f, cmax_sum = 0.f;
  for (int r = wave; r < S; r += 4) {
    float mn = INFINITY, mx = -INFINITY;
    for (int c = lane; c < N; c += 64) {
      const float v = Elt<T>::load(cw + (size_t)r * N + c);
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      mn = fminf(mn, __shfl_xor(mn, o, 64));
      mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    }
    cmin_sum += mn;
    cmax_sum += mx;
  }
  // dispatch weights: a thread per slot column
  float dmin_sum = 0.f, dmax_sum = 0.f;
  for (int c = tid; c < N; c += 256) {
    float mn = INFINITY, mx = -INFINITY;
    for (int r = 0; r < S; ++r) {
      const float v = Elt<T>::load(dw + (size_t)r * N + c);
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
    dmin_sum += mn;
    dmax_sum += mx;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    dmin_sum += __shfl_xor(dmin_sum, o, 64);
    dmax_sum += __shfl_xor(dmax_sum, o, 64);
  }
  if (lane == 0) {
    red[wave][0] = cmin_sum; red[wave][1] = cmax_sum;
    red[wave][2] = dmin_sum; red[wave][3] = dmax_sum;
  }
  __syncthreads();
  if (tid < 4) partial[(size_t)g * 4 + tid] = red[0][tid] + red[1][tid] + red[2][tid] + red[3][tid];
}

template <typename T> __device__ __forceinline__ void unpack16(uint4 q, float* v);
template <> __device__ __forceinline__ void unpack16<float>(uint4 q, float* v) {
  v[0] = __builtin_bit_cast(float, q.x); v[1] = __builtin_bit_cast(float, q.y);
  v[2] = __builtin_bit_cast(float, q.z); v[3] = __builtin_bit_cast(float, q.w);
}
template <> __device__ __forceinline__ void unpack16<bf16_t>(uint4 q, float* v) {
  v[0] = bf_lo(q.x); v[1] = bf_hi(q.x); v[2] = bf_lo(q.y); v[3] = bf_hi(q.y);
  v[4] = bf_lo(q.z); v[5] = bf_hi(q.z); v[6] = bf_lo(q.w); v[7] = bf_hi(q.w);
}

// The same sums with 16-byte loads when a row is a power-of-two number NC <= 64 of
// 16-byte chunks.  blockIdx.y = 0 takes the combine weights (a row's chunks sit in NC
// adjacent lanes, so the row minimum is a lane exchange), blockIdx.y = 1 the dispatch
// weights (a thread keeps one chunk column over all its rows; the 256 / NC threads of
// a column meet in LDS).
template <typename T>
__global__ __launch_bounds__(256) void soft_stats_vec_kernel(const T* __restrict__ combine_w,
                                                             const T* __restrict__ dispatch_w,
                                                             float* __restrict__ partial, int S, int N) {
  constexpr int V = 16 / sizeof(T);
  __shared__ float lds_min[256 * V];
  __shared__ float lds_max[256 * V];
  __shared__ float red[4][2];
  const int g = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int NC = N / V;
  const int total = S * NC;
  float sum_min = 0.f, sum_max = 0.f;
  if (blockIdx.y == 0) {
    const uint4* src = reinterpret_cast<const uint4*>(combine_w + (size_t)g * S * N);
    const int rounds = (total + 255) / 256;
    for (int k = 0; k < rounds; ++k) {
      const int i = k * 256 + tid;
      float mn = INFINITY, mx = -INFINITY;
      if (i < total) {
        float v[V];
        unpack16<T>(src[i], v);
#pragma unroll
        for (int j = 0; j < V; ++j) { mn = fminf(mn, v[j]); mx = fmaxf(mx, v[j]); }
      }
      for (int o = 1; o < NC; o <<= 1) {
        mn = fminf(mn, __shfl_xor(mn, o, 64));
        mx = fmaxf(mx, __shfl_xor(mx, o, 64));
      }
      if (i < total && (lane & (NC - 1)) == 0) { sum_min += mn; sum_max += mx; }
    }
  } else {
    const uint4* src = reinterpret_cast<const uint4*>(dispatch_w + (size_t)g * S * N);
    float mn[V], mx[V];
#pragma unroll
    for (int j = 0; j < V; ++j) { mn[j] = INFINITY; mx[j] = -INFINITY; }
    for (int i = tid; i < total; i += 256) {
      float v[V];
      unpack16<T>(src[i], v);
#pragma unroll
      for (int j = 0; j < V; ++j) { mn[j] = fminf(mn[j], v[j]); mx[j] = fmaxf(mx[j], v[j]); }
    }
    // thread t holds chunk column t % NC; LDS as [t / NC][column * V + j]
#pragma unroll
    for (int j = 0; j < V; ++j) {
      lds_min[(tid / NC) * N + (tid % NC) * V + j] = mn[j];
      lds_max[(tid / NC) * N + (tid % NC) * V + j] = mx[j];
    }
    __syncthreads();
    const int parts = 256 / NC;
    for (int c = tid; c < N; c += 256) {
      float a = INFINITY, b = -INFINITY;
      for (int q = 0; q < parts; ++q) { a = fminf(a, lds_min[q * N + c]); b = fmaxf(b, lds_max[q * N + c]); }
      sum_min += a;
      sum_max += b;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    sum_min += __shfl_xor(sum_min, o, 64);
    sum_max += __shfl_xor(sum_max, o, 64);
  }
  if (lane == 0) { red[wave][0] = sum_min; red[wave][1] = sum_max; }
  __syncthreads();
  if (tid < 2)
    partial[(size_t)g * 4 + blockIdx.y * 2 + tid] = red[0][tid] + red[1][tid] + red[2][tid] + red[3][tid];
}

// Sums the (G, 4) partials over the groups in index order and scales them to means;
// stats[4] is the router's auxiliary loss, which is always zero.
__global__ __launch_bounds__(256) void soft_stats_finish_kernel(const float* __restrict__ partial,
                                                                float* __restrict__ stats, int G,
                                                                float inv_items, float inv_slots) {
  __shared__ float part[64][4];
  const int tid = threadIdx.x, col = tid & 3, seg = tid >> 2;
  const int per = (G + 63) / 64;
  float s = 0.f;
  for (int g = seg * per; g < min(G, (seg + 1) * per); ++g) s += partial[(size_t)g * 4 + col];
  part[seg][col] = s;
  __syncthreads();
  if (tid < 4) {
    float t = 0.f;
    for (int q = 0; q < 64; ++q) t += part[q][tid];
    stats[tid] = t * (tid < 2 ? inv_items : inv_slots);
  }
  if (tid == 4) stats[4] = 0.f;
}

}  // namespace
}  // namespace vmoe

using namespace vmoe;

extern "C" size_t vmoe_soft_route_workspace_bytes(const VmoeSoftRouteParams* p) {
  if (p == nullptr || p->D < 1 || p->N < 1) return 0;
  // float32: (D, N) floats; bfloat16: the slots padded to a multiple of 32
  const size_t padded = (size_t)p->D * ((p->N + 31) / 32 * 32) * 2;
  return std::max((size_t)p->D * p->N * sizeof(float), padded);
}

// vmoe_soft_route; with `stats_partial` the routing launch also writes the (G, 4) partial
// sums of the monitoring scalars where it can (`*wrote_partial` says whether it did).
static int soft_route_launch(const VmoeSoftRouteParams* p, vmoe_stream_t stream_, float* stats_partial,
                             bool* wrote_partial) {
  if (p == nullptr || p->x == nullptr || p->mu == nullptr || p->dispatch_w == nullptr ||
      p->combine_w == nullptr)
    return VMOE_E_NULL;
  if (p->G < 1 || p->S < 1 || p->D < 1 || p->N < 1) return VMOE_E_SHAPE;
  if (p->dtype != VMOE_F32 && p->dtype != VMOE_BF16) return VMOE_E_DTYPE;
  if (p->N > 1024) return VMOE_E_UNSUPPORTED;
  if (p->dtype == VMOE_BF16 && (p->D % 8 != 0 || !aligned16(p->x))) return VMOE_E_ALIGN;
  if (p->workspace == nullptr || p->workspace_bytes < vmoe_soft_route_workspace_bytes(p) ||
      !aligned16(p->workspace))
    return VMOE_E_WORKSPACE;
  const size_t esz = p->dtype == VMOE_BF16 ? 2 : 4;
  const int SP = (p->S + 31) / 32 * 32, NP = (p->N + 31) / 32 * 32;
  const int LDW = NP + (esz == 2 ? 2 : 1);
  const size_t lds = (size_t)SP * 4 + (size_t)SP * LDW * esz;
  hipStream_t stream = as_stream(stream_);
  // router.py:79-82: the scale multiplies whichever of the two operands is smaller.
  const int scale_x = ((int64_t)p->G * p->S * p->D < (int64_t)p->D * p->N) ? 1 : 0;
  const SoftLds L = soft_lds_layout(p->D, SP, NP);
  if (p->dtype == VMOE_BF16 && p->N <= 128 && p->N % 8 == 0 && soft_fast_width(p->D) && L.total <= 160 * 1024 && aligned16(p->dispatch_w) && aligned16(p->combine_w) &&
      (p->logits == nullptr || aligned16(p->logits))) {
    // Two roles per workgroup where the slot parameters of 32 slots fit a wave's registers
    // (D <= 768) and two item tiles fit LDS beside the logits (tiles of 32 rows, else 16).
    // (VMOE_SOFT_ROUTE_SINGLE_ROLE=1 in the environment keeps the single-role kernel: the
    // switch behind the before / after figures)
    const int tile_rows = soft_pipe_lds_layout(p->D, SP, NP, 32).total <= 160 * 1024 ? 32 : 16;
    const SoftPipeLds PL = soft_pipe_lds_layout(p->D, SP, NP, tile_rows);
    if (p->D <= 768 && PL.total <= 160 * 1024 && getenv("VMOE_SOFT_ROUTE_SINGLE_ROLE") == nullptr) {
      using Kern = void (*)(const bf16_t*, const bf16_t*, bf16_t*, bf16_t*, bf16_t*, float, int, int,
                            int, int, int, SoftPipeLds, float*);
      // (the partial sums come out of the register-resident dispatch softmax only)
      // (VMOE_SOFT_STATS_SEPARATE=1 in the environment keeps the separate launches: the switch
      // behind the before / after figures)
      float* partial_out = SP <= 32 * kTailRows && getenv("VMOE_SOFT_STATS_SEPARATE") == nullptr
                               ? stats_partial : nullptr;
      if (wrote_partial != nullptr) *wrote_partial = partial_out != nullptr;
      auto pick = [&](auto ksw) -> Kern {
        constexpr int K = decltype(ksw)::value;
        if (tile_rows == 32)
          return scale_x ? soft_route_roles_kernel<K, 32, true> : soft_route_roles_kernel<K, 32, false>;
        return scale_x ? soft_route_roles_kernel<K, 16, true> : soft_route_roles_kernel<K, 16, false>;
      };
      Kern kern = p->D == 768   ? pick(std::integral_constant<int, 24>{})
                  : p->D == 512 ? pick(std::integral_constant<int, 16>{})
                  : p->D == 384 ? pick(std::integral_constant<int, 12>{})
                                : pick(std::integral_constant<int, 8>{});
      hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), PL.total);
      if (e != hipSuccess) return (int)e;
      if (!p->workspace_prepared)
        hipLaunchKernelGGL(soft_prep_mu_kernel<bf16_t>, dim3(NP), dim3(256), 0, stream,
                           (const bf16_t*)p->mu, (bf16_t*)p->workspace, p->scale, !scale_x, p->D, p->N,
                           p->D / 32);
      hipLaunchKernelGGL(kern, dim3(p->G), dim3(kSrThreads), PL.total, stream, (const bf16_t*)p->x,
                         (const bf16_t*)p->workspace, (bf16_t*)p->dispatch_w, (bf16_t*)p->combine_w,
                         (bf16_t*)p->logits, p->scale, p->S, p->D, p->N, SP, NP, PL, partial_out);
      return launch_status();
    }
    if (!p->workspace_prepared)
      hipLaunchKernelGGL(soft_prep_mu_kernel<bf16_t>, dim3(p->N), dim3(256), 0, stream,
                         (const bf16_t*)p->mu, (bf16_t*)p->workspace, p->scale, !scale_x, p->D, p->N);
    auto kern = p->D == 1024 ? soft_route_bf16_kernel<32>
                : p->D == 768 ? soft_route_bf16_kernel<24>
                : p->D == 512 ? soft_route_bf16_kernel<16>
                : p->D == 384 ? soft_route_bf16_kernel<12>
                              : soft_route_bf16_kernel<8>;
    hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), L.total);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, dim3(p->G), dim3(kSrThreads), L.total, stream, (const bf16_t*)p->x,
                       (const bf16_t*)p->workspace, (bf16_t*)p->dispatch_w, (bf16_t*)p->combine_w,
                       (bf16_t*)p->logits, p->scale, scale_x, p->S, p->D, p->N, SP, NP, L);
  } else if (lds > 160 * 1024) {
    return VMOE_E_UNSUPPORTED;
  } else if (p->dtype == VMOE_BF16) {
    if (!p->workspace_prepared)
      hipLaunchKernelGGL(soft_prep_mu_kernel<bf16_t>, dim3(p->N), dim3(256), 0, stream,
                         (const bf16_t*)p->mu, (bf16_t*)p->workspace, p->scale, !scale_x, p->D, p->N);
    auto kern = soft_route_kernel<bf16_t>;
    hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, dim3(p->G), dim3(256), lds, stream, (const bf16_t*)p->x,
                       (const bf16_t*)p->workspace, (bf16_t*)p->dispatch_w, (bf16_t*)p->combine_w,
                       (bf16_t*)p->logits, p->scale, scale_x, p->S, p->D, p->N, SP, NP);
  } else {
    if (!p->workspace_prepared)
      hipLaunchKernelGGL(soft_prep_mu_kernel<float>, dim3(p->N), dim3(256), 0, stream,
                         (const float*)p->mu, (float*)p->workspace, p->scale, !scale_x, p->D, p->N);
    auto kern = soft_route_kernel<float>;
    hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, dim3(p->G), dim3(256), lds, stream, (const float*)p->x,
                       (const float*)p->workspace, (float*)p->dispatch_w, (float*)p->combine_w,
                       (float*)p->logits, p->scale, scale_x, p->S, p->D, p->N, SP, NP);
  }
  return launch_status();
}

extern "C" int vmoe_soft_route(const VmoeSoftRouteParams* p, vmoe_stream_t stream) {
  return soft_route_launch(p, stream, nullptr, nullptr);
}

extern "C" int vmoe_einsum_dispatch(const VmoeEinsumParams* p, vmoe_stream_t stream) {
  int rc = check_einsum(p, true);
  if (rc != VMOE_OK) return rc;
  if (ein::dispatch_fast_ok(p)) return ein::launch_dispatch_fast(p, as_stream(stream));
  const int M = p->E * p->C;
  dim3 grid((p->D + 63) / 64, (M + 63) / 64, p->G);
  hipLaunchKernelGGL(einsum_kernel<true>, grid, dim3(256), 0, as_stream(stream), p->w, p->data,
                     p->out, p->G, p->S, p->E, p->C, p->D, p->w_dtype, p->data_dtype, p->out_dtype);
  return launch_status();
}

extern "C" int vmoe_einsum_combine(const VmoeEinsumParams* p, vmoe_stream_t stream) {
  int rc = check_einsum(p, false);
  if (rc != VMOE_OK) return rc;
  if (ein::combine_fast_ok(p)) return ein::launch_combine_fast(p, as_stream(stream));
  dim3 grid((p->D + 63) / 64, (p->S + 63) / 64, p->G);
  hipLaunchKernelGGL(einsum_kernel<false>, grid, dim3(256), 0, as_stream(stream), p->w, p->data,
                     p->out, p->G, p->S, p->E, p->C, p->D, p->w_dtype, p->data_dtype, p->out_dtype);
  return launch_status();
}

extern "C" int vmoe_soft_router_stats(const VmoeSoftStatsParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->combine_w == nullptr || p->dispatch_w == nullptr ||
      p->partial == nullptr || p->stats == nullptr)
    return VMOE_E_NULL;
  if (p->G < 1 || p->S < 1 || p->N < 1) return VMOE_E_SHAPE;
  if (p->dtype != VMOE_BF16 && p->dtype != VMOE_F32) return VMOE_E_DTYPE;
  const int vec = p->dtype == VMOE_BF16 ? 8 : 4;
  const int nc = p->N / vec;
  const bool wide = p->N % vec == 0 && nc <= 64 && (nc & (nc - 1)) == 0 &&
                    aligned16(p->combine_w) && aligned16(p->dispatch_w) && p->G <= 65535 * 32;
  hipStream_t s = as_stream(stream);
  if (wide && p->dtype == VMOE_BF16)
    hipLaunchKernelGGL(soft_stats_vec_kernel<bf16_t>, dim3(p->G, 2), dim3(256), 0, s,
                       (const bf16_t*)p->combine_w, (const bf16_t*)p->dispatch_w, p->partial, p->S,
                       p->N);
  else if (wide)
    hipLaunchKernelGGL(soft_stats_vec_kernel<float>, dim3(p->G, 2), dim3(256), 0, s,
                       (const float*)p->combine_w, (const float*)p->dispatch_w, p->partial, p->S,
                       p->N);
  else if (p->dtype == VMOE_BF16)
    hipLaunchKernelGGL(soft_stats_kernel<bf16_t>, dim3(p->G), dim3(256), 0, s,
                       (const bf16_t*)p->combine_w, (const bf16_t*)p->dispatch_w, p->partial, p->S,
                       p->N);
  else
    hipLaunchKernelGGL(soft_stats_kernel<float>, dim3(p->G), dim3(256), 0, s,
                       (const float*)p->combine_w, (const float*)p->dispatch_w, p->partial, p->S,
                       p->N);
  hipLaunchKernelGGL(soft_stats_finish_kernel, dim3(1), dim3(256), 0, s, p->partial, p->stats, p->G,
                     1.0f / ((float)p->G * (float)p->S), 1.0f / ((float)p->G * (float)p->N));
  return launch_status();
}

extern "C" int vmoe_soft_route_stats(const VmoeSoftRouteParams* route, const VmoeSoftStatsParams* st,
                                     vmoe_stream_t stream) {
  if (route == nullptr || st == nullptr || st->partial == nullptr || st->stats == nullptr) return VMOE_E_NULL;
  if (st->combine_w != route->combine_w || st->dispatch_w != route->dispatch_w || st->G != route->G ||
      st->S != route->S || st->N != route->N || st->dtype != route->dtype)
    return VMOE_E_SHAPE;
  bool wrote = false;
  const int rc = soft_route_launch(route, stream, st->partial, &wrote);
  if (rc != VMOE_OK) return rc;
  if (!wrote) return vmoe_soft_router_stats(st, stream);
  hipLaunchKernelGGL(soft_stats_finish_kernel, dim3(1), dim3(256), 0, as_stream(stream), st->partial, st->stats,
                     st->G, 1.0f / ((float)st->G * (float)st->S), 1.0f / ((float)st->G * (float)st->N));
  return launch_status();
}
