// Dispatch (item rows -> expert buffer slots) and combine (weighted sum of the
// K expert outputs of an item) for gfx950.  HBM-bound row movers.
//
// Replaces ExpertIndicesDispatcher.dispatch / .combine, vmoe/moe.py:190-209,
// including the zero-initialised buffer of _scatter_nd (moe.py:542) and the
// row order of _dispatch (moe.py:488-500), which is already folded into the
// slot rows computed by the slot-assignment kernel.
//
// dispatch is item-major: every item row is read from HBM exactly once and
// written to its <= K slots; a second set of waves in the same launch writes
// zeros to the slots no item claimed.  Every slot row has exactly one writer,
// so there are no atomics and the result is bit-deterministic.
// combine is item-major as well: <= K row reads, float32 multiply and add in k
// order (no fused multiply-add, to match a float32 einsum), one rounded store.
// One wave moves kRows rows per step with 16-byte accesses per lane, all loads
// of a step issued before the first store.
#include "vmoe_common.h"

namespace vmoe {
namespace {

constexpr int kRows = 4;          // rows per wave per step
constexpr int kZeroSlots = 16;    // slots checked per zero-fill wave
constexpr int kMoveThreads = 256;

__global__ __launch_bounds__(kMoveThreads) void dispatch_kernel(
    const uint4* __restrict__ x, const int32_t* __restrict__ token_slot,
    const int32_t* __restrict__ slot_token, uint4* __restrict__ out, int num_items, int num_slots,
    int K, int cpr, int item_waves) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(
      (int)((blockIdx.x * (unsigned)kMoveThreads + threadIdx.x) >> 6));
  if (wave < item_waves) {
    const int t0 = wave * kRows;
    for (int ch = lane; ch < cpr; ch += kWave) {
      uint4 v[kRows];
#pragma unroll
      for (int r = 0; r < kRows; ++r)
        if (t0 + r < num_items) v[r] = x[(size_t)(t0 + r) * cpr + ch];
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        if (t0 + r < num_items) {
          for (int k = 0; k < K; ++k) {
            int slot = token_slot[(size_t)(t0 + r) * K + k];
            if (slot >= 0) out[(size_t)slot * cpr + ch] = v[r];
          }
        }
      }
    }
  } else {
    const int s0 = (wave - item_waves) * kZeroSlots;
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (int i = 0; i < kZeroSlots; ++i) {
      int s = s0 + i;
      if (s < num_slots && slot_token[s] < 0)
        for (int ch = lane; ch < cpr; ch += kWave) out[(size_t)s * cpr + ch] = z;
    }
  }
}

template <typename T> struct Chunk;
template <> struct Chunk<float> {
  static constexpr int n = 4;
  __device__ static __forceinline__ void unpack(const uint4& v, float* f) {
    f[0] = __builtin_bit_cast(float, v.x); f[1] = __builtin_bit_cast(float, v.y);
    f[2] = __builtin_bit_cast(float, v.z); f[3] = __builtin_bit_cast(float, v.w);
  }
  __device__ static __forceinline__ uint4 pack(const float* f) {
    return make_uint4(__builtin_bit_cast(uint32_t, f[0]), __builtin_bit_cast(uint32_t, f[1]),
                      __builtin_bit_cast(uint32_t, f[2]), __builtin_bit_cast(uint32_t, f[3]));
  }
};
template <> struct Chunk<bf16_t> {
  static constexpr int n = 8;
  __device__ static __forceinline__ void unpack(const uint4& v, float* f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __builtin_bit_cast(float, w[i] << 16);
      f[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
    }
  }
  __device__ static __forceinline__ uint4 pack(const float* f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f2bf(f[2 * i]) | ((uint32_t)f2bf(f[2 * i + 1]) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
  }
};

constexpr int kMaxK = 8;  // register-resident fast path; larger K takes the generic loop

template <typename T>
__global__ __launch_bounds__(kMoveThreads) void combine_kernel(
    const uint4* __restrict__ y, const int32_t* __restrict__ token_slot,
    const float* __restrict__ weights, uint4* __restrict__ out, int num_items, int K, int cpr) {
  constexpr int N = Chunk<T>::n;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(
      (int)((blockIdx.x * (unsigned)kMoveThreads + threadIdx.x) >> 6));
  const int t0 = wave * kRows;
  if (t0 >= num_items) return;
  if (K == 2) {
    // The common case: both reads of all rows in flight before any arithmetic.
    for (int ch = lane; ch < cpr; ch += kWave) {
      uint4 v[kRows][2];
      int slot[kRows][2];
      float w[kRows][2];
#pragma unroll
      for (int r = 0; r < kRows; ++r)
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          bool ok = t0 + r < num_items;
          slot[r][k] = ok ? token_slot[(size_t)(t0 + r) * 2 + k] : -1;
          w[r][k] = ok ? weights[(size_t)(t0 + r) * 2 + k] : 0.f;
          v[r][k] = make_uint4(0, 0, 0, 0);
          if (slot[r][k] >= 0) v[r][k] = y[(size_t)slot[r][k] * cpr + ch];
        }
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        if (t0 + r >= num_items) continue;
        float a[N], b[N], o[N];
        Chunk<T>::unpack(v[r][0], a);
        Chunk<T>::unpack(v[r][1], b);
#pragma unroll
        for (int j = 0; j < N; ++j) {
          float p0 = slot[r][0] >= 0 ? __fmul_rn(w[r][0], a[j]) : 0.f;
          float p1 = slot[r][1] >= 0 ? __fmul_rn(w[r][1], b[j]) : 0.f;
          o[j] = __fadd_rn(p0, p1);
        }
        out[(size_t)(t0 + r) * cpr + ch] = Chunk<T>::pack(o);
      }
    }
    return;
  }
  for (int r = 0; r < kRows; ++r) {
    const int t = t0 + r;
    if (t >= num_items) break;
    for (int ch = lane; ch < cpr; ch += kWave) {
      float acc[N];
#pragma unroll
      for (int j = 0; j < N; ++j) acc[j] = 0.f;
      for (int k = 0; k < K; ++k) {
        int slot = token_slot[(size_t)t * K + k];
        if (slot < 0) continue;
        float w = weights[(size_t)t * K + k];
        float a[N];
        Chunk<T>::unpack(y[(size_t)slot * cpr + ch], a);
#pragma unroll
        for (int j = 0; j < N; ++j) acc[j] = __fadd_rn(acc[j], __fmul_rn(w, a[j]));
      }
      out[(size_t)t * cpr + ch] = Chunk<T>::pack(acc);
    }
  }
}

__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ in,
                                                   uint4* __restrict__ out, size_t n16) {
  size_t i = (size_t)blockIdx.x * 256 * 4 + threadIdx.x;
  uint4 v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
    if (i + j * 256 < n16) v[j] = in[i + j * 256];
#pragma unroll
  for (int j = 0; j < 4; ++j)
    if (i + j * 256 < n16) out[i + j * 256] = v[j];
}

__global__ __launch_bounds__(256) void cast_f32_to_bf16_kernel(const float* __restrict__ in,
                                                               bf16_t* __restrict__ out, size_t n) {
  size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i + 4 <= n) {
    float4 v = *reinterpret_cast<const float4*>(in + i);
    uint2 o;
    o.x = (uint32_t)f2bf(v.x) | ((uint32_t)f2bf(v.y) << 16);
    o.y = (uint32_t)f2bf(v.z) | ((uint32_t)f2bf(v.w) << 16);
    *reinterpret_cast<uint2*>(out + i) = o;
  } else {
    for (; i < n; ++i) out[i] = f2bf(in[i]);
  }
}
__global__ __launch_bounds__(256) void cast_bf16_to_f32_kernel(const bf16_t* __restrict__ in,
                                                               float* __restrict__ out, size_t n) {
  size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i + 4 <= n) {
    uint2 v = *reinterpret_cast<const uint2*>(in + i);
    float4 o;
    o.x = __builtin_bit_cast(float, v.x << 16); o.y = __builtin_bit_cast(float, v.x & 0xffff0000u);
    o.z = __builtin_bit_cast(float, v.y << 16); o.w = __builtin_bit_cast(float, v.y & 0xffff0000u);
    *reinterpret_cast<float4*>(out + i) = o;
  } else {
    for (; i < n; ++i) out[i] = bf2f(in[i]);
  }
}

int check_move(const void* a, const void* b, const void* c, int num_items, int num_slots, int K,
               int D, int dtype) {
  if (a == nullptr || b == nullptr || c == nullptr) return VMOE_E_NULL;
  if (num_items < 1 || num_slots < 1 || K < 1 || D < 1) return VMOE_E_SHAPE;
  if (dtype != VMOE_F32 && dtype != VMOE_BF16) return VMOE_E_DTYPE;
  const size_t row = (size_t)D * (dtype == VMOE_BF16 ? 2 : 4);
  if (row % 16 != 0 || !aligned16(a) || !aligned16(c)) return VMOE_E_ALIGN;
  if ((int64_t)num_items * K >= INT32_MAX) return VMOE_E_OVERFLOW;
  return VMOE_OK;
}

}  // namespace
}  // namespace vmoe

using namespace vmoe;

extern "C" int vmoe_dispatch(const VmoeDispatchParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->token_slot == nullptr || p->slot_token == nullptr) return VMOE_E_NULL;
  int rc = check_move(p->x, p->token_slot, p->out, p->num_items, p->num_slots, p->K, p->D, p->dtype);
  if (rc != VMOE_OK) return rc;
  const int cpr = (int)((size_t)p->D * (p->dtype == VMOE_BF16 ? 2 : 4) / 16);
  const int item_waves = (p->num_items + kRows - 1) / kRows;
  const int zero_waves = (p->num_slots + kZeroSlots - 1) / kZeroSlots;
  const int waves_per_block = kMoveThreads / kWave;
  const int blocks = (item_waves + zero_waves + waves_per_block - 1) / waves_per_block;
  hipLaunchKernelGGL(dispatch_kernel, dim3(blocks), dim3(kMoveThreads), 0, as_stream(stream),
                     (const uint4*)p->x, p->token_slot, p->slot_token, (uint4*)p->out,
                     p->num_items, p->num_slots, p->K, cpr, item_waves);
  return launch_status();
}

extern "C" int vmoe_combine(const VmoeCombineParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->weights == nullptr) return VMOE_E_NULL;
  int rc = check_move(p->y, p->token_slot, p->out, p->num_items, p->num_slots, p->K, p->D, p->dtype);
  if (rc != VMOE_OK) return rc;
  const int cpr = (int)((size_t)p->D * (p->dtype == VMOE_BF16 ? 2 : 4) / 16);
  const int waves = (p->num_items + kRows - 1) / kRows;
  const int waves_per_block = kMoveThreads / kWave;
  const int blocks = (waves + waves_per_block - 1) / waves_per_block;
  if (p->dtype == VMOE_BF16)
    hipLaunchKernelGGL(combine_kernel<bf16_t>, dim3(blocks), dim3(kMoveThreads), 0,
                       as_stream(stream), (const uint4*)p->y, p->token_slot, p->weights,
                       (uint4*)p->out, p->num_items, p->K, cpr);
  else
    hipLaunchKernelGGL(combine_kernel<float>, dim3(blocks), dim3(kMoveThreads), 0,
                       as_stream(stream), (const uint4*)p->y, p->token_slot, p->weights,
                       (uint4*)p->out, p->num_items, p->K, cpr);
  return launch_status();
}

extern "C" int vmoe_copy_bytes(const void* in, void* out, size_t n, vmoe_stream_t stream) {
  if (in == nullptr || out == nullptr) return VMOE_E_NULL;
  if (n == 0 || n % 16 != 0 || !aligned16(in) || !aligned16(out)) return VMOE_E_ALIGN;
  const size_t n16 = n / 16;
  const size_t blocks = (n16 + 1023) / 1024;
  if (blocks > 0x7fffffffull) return VMOE_E_OVERFLOW;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                     (const uint4*)in, (uint4*)out, n16);
  return launch_status();
}

extern "C" int vmoe_cast(const VmoeCastParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->in == nullptr || p->out == nullptr) return VMOE_E_NULL;
  if (p->n == 0) return VMOE_E_SHAPE;
  if (!aligned16(p->in) || !aligned16(p->out)) return VMOE_E_ALIGN;
  const size_t blocks = (p->n + 1023) / 1024;
  if (blocks > 0x7fffffffull) return VMOE_E_OVERFLOW;
  if (p->in_dtype == VMOE_F32 && p->out_dtype == VMOE_BF16)
    hipLaunchKernelGGL(cast_f32_to_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       as_stream(stream), (const float*)p->in, (bf16_t*)p->out, p->n);
  else if (p->in_dtype == VMOE_BF16 && p->out_dtype == VMOE_F32)
    hipLaunchKernelGGL(cast_bf16_to_f32_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       as_stream(stream), (const bf16_t*)p->in, (float*)p->out, p->n);
  else
    return VMOE_E_DTYPE;
  return launch_status();
}
