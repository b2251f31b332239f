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
// Work is flattened over (row, 16-byte chunk), eight rows per workgroup, so all
// lanes carry data for any row width; accesses carry the non-temporal hint.
#include "vmoe_common.h"

namespace vmoe {
namespace {

constexpr int kRowsPerBlock = 8;   // item rows (or slot rows) moved by one workgroup
constexpr int kMoveThreads = 256;
constexpr int kMaxK = 8;           // choices per item held in LDS; larger K takes the generic kernels

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Streaming accesses: every row is touched once per kernel, so loads and stores
// carry the non-temporal hint.
__device__ __forceinline__ uint4 load_stream(const uint4* p) {
  return __builtin_bit_cast(uint4, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}
__device__ __forceinline__ void store_stream(uint4* p, const uint4& v) {
  __builtin_nontemporal_store(__builtin_bit_cast(u32x4, v), reinterpret_cast<u32x4*>(p));
}

// A slot row outside [0, num_slots) counts as a dropped assignment (-1): maps that do not
// come from the slot-assignment kernels cannot make a row mover leave the buffer.
__device__ __forceinline__ int checked_slot(int slot, int num_slots) {
  return (unsigned)slot < (unsigned)num_slots ? slot : -1;
}

// idx / cpr for idx < 2^16 with magic = ceil(2^32 / cpr); magic == 0 encodes cpr == 1.
__device__ __forceinline__ int div_chunks(int idx, uint32_t magic) {
  return magic == 0 ? idx : (int)__umulhi((uint32_t)idx, magic);
}

// Work is flattened over (row, 16-byte chunk) so that every lane of every wave
// moves data whatever the row width: thread t of a workgroup handles chunks
// t, t+256, ... of the workgroup's kRowsPerBlock rows.
__global__ __launch_bounds__(kMoveThreads) void dispatch_kernel(
    const uint4* __restrict__ x, const int32_t* __restrict__ token_slot,
    const int32_t* __restrict__ slot_token, uint4* __restrict__ out, int num_items, int num_slots,
    int K, int cpr, uint32_t magic, int item_blocks) {
  __shared__ int32_t slots[kRowsPerBlock * kMaxK];
  const int tid = threadIdx.x;
  const int total = kRowsPerBlock * cpr;
  if ((int)blockIdx.x < item_blocks) {
    const int t0 = blockIdx.x * kRowsPerBlock;
    if (tid < kRowsPerBlock * K) {
      const int r = tid / K;
      slots[tid] = t0 + r < num_items ? checked_slot(token_slot[(size_t)t0 * K + tid], num_slots) : -1;
    }
    __syncthreads();
    for (int idx = tid; idx < total; idx += kMoveThreads) {
      const int r = div_chunks(idx, magic);
      const int ch = idx - r * cpr;
      if (t0 + r >= num_items) continue;
      const uint4 v = load_stream(x + (size_t)(t0 + r) * cpr + ch);
      for (int k = 0; k < K; ++k) {
        const int slot = slots[r * K + k];
        if (slot >= 0) store_stream(out + (size_t)slot * cpr + ch, v);
      }
    }
  } else {
    // Zero-fill of the slots no item claimed.
    const int s0 = (blockIdx.x - item_blocks) * kRowsPerBlock;
    if (tid < kRowsPerBlock) slots[tid] = s0 + tid < num_slots ? slot_token[s0 + tid] : 0;
    __syncthreads();
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (int idx = tid; idx < total; idx += kMoveThreads) {
      const int r = div_chunks(idx, magic);
      const int ch = idx - r * cpr;
      if (slots[r] < 0) store_stream(out + (size_t)(s0 + r) * cpr + ch, z);
    }
  }
}

// Any K (choices read from global memory), one wave per item row.
__global__ __launch_bounds__(kMoveThreads) void dispatch_generic_kernel(
    const uint4* __restrict__ x, const int32_t* __restrict__ token_slot,
    const int32_t* __restrict__ slot_token, uint4* __restrict__ out, int num_items, int num_slots,
    int K, int cpr, int item_waves) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(
      (int)((blockIdx.x * (unsigned)kMoveThreads + threadIdx.x) >> 6));
  if (wave < item_waves) {
    for (int ch = lane; ch < cpr; ch += kWave) {
      const uint4 v = x[(size_t)wave * cpr + ch];
      for (int k = 0; k < K; ++k) {
        const int slot = checked_slot(token_slot[(size_t)wave * K + k], num_slots);
        if (slot >= 0) out[(size_t)slot * cpr + ch] = v;
      }
    }
  } else {
    const int s = wave - item_waves;
    if (s < num_slots && slot_token[s] < 0)
      for (int ch = lane; ch < cpr; ch += kWave) out[(size_t)s * cpr + ch] = make_uint4(0, 0, 0, 0);
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

template <typename T>
__global__ __launch_bounds__(kMoveThreads) void combine_kernel(
    const uint4* __restrict__ y, const int32_t* __restrict__ token_slot,
    const float* __restrict__ weights, uint4* __restrict__ out, int num_items, int num_slots,
    int K, int cpr, uint32_t magic) {
  constexpr int N = Chunk<T>::n;
  __shared__ int32_t slots[kRowsPerBlock * kMaxK];
  __shared__ float wts[kRowsPerBlock * kMaxK];
  const int tid = threadIdx.x;
  const int t0 = blockIdx.x * kRowsPerBlock;
  if (tid < kRowsPerBlock * K) {
    const int r = tid / K;
    const bool ok = t0 + r < num_items;
    slots[tid] = ok ? checked_slot(token_slot[(size_t)t0 * K + tid], num_slots) : -1;
    wts[tid] = ok ? weights[(size_t)t0 * K + tid] : 0.f;
  }
  __syncthreads();
  const int total = kRowsPerBlock * cpr;
  for (int idx = tid; idx < total; idx += kMoveThreads) {
    const int r = div_chunks(idx, magic);
    const int ch = idx - r * cpr;
    if (t0 + r >= num_items) continue;
    float acc[N];
    if (K == 2) {
      // Both reads in flight before any arithmetic.
      const int s0 = slots[r * 2], s1 = slots[r * 2 + 1];
      uint4 v0 = make_uint4(0, 0, 0, 0), v1 = v0;
      if (s0 >= 0) v0 = load_stream(y + (size_t)s0 * cpr + ch);
      if (s1 >= 0) v1 = load_stream(y + (size_t)s1 * cpr + ch);
      float a[N], b[N];
      Chunk<T>::unpack(v0, a);
      Chunk<T>::unpack(v1, b);
      const float w0 = wts[r * 2], w1 = wts[r * 2 + 1];
#pragma unroll
      for (int j = 0; j < N; ++j) {
        float p0 = s0 >= 0 ? __fmul_rn(w0, a[j]) : 0.f;
        float p1 = s1 >= 0 ? __fmul_rn(w1, b[j]) : 0.f;
        acc[j] = __fadd_rn(p0, p1);
      }
    } else {
#pragma unroll
      for (int j = 0; j < N; ++j) acc[j] = 0.f;
      for (int k = 0; k < K; ++k) {
        const int slot = slots[r * K + k];
        if (slot < 0) continue;
        const float w = wts[r * K + k];
        float a[N];
        Chunk<T>::unpack(load_stream(y + (size_t)slot * cpr + ch), a);
#pragma unroll
        for (int j = 0; j < N; ++j) acc[j] = __fadd_rn(acc[j], __fmul_rn(w, a[j]));
      }
    }
    store_stream(out + (size_t)(t0 + r) * cpr + ch, Chunk<T>::pack(acc));
  }
}

// Any K, one wave per item row.
template <typename T>
__global__ __launch_bounds__(kMoveThreads) void combine_generic_kernel(
    const uint4* __restrict__ y, const int32_t* __restrict__ token_slot,
    const float* __restrict__ weights, uint4* __restrict__ out, int num_items, int num_slots,
    int K, int cpr) {
  constexpr int N = Chunk<T>::n;
  const int lane = threadIdx.x & 63;
  const int t = __builtin_amdgcn_readfirstlane(
      (int)((blockIdx.x * (unsigned)kMoveThreads + threadIdx.x) >> 6));
  if (t >= num_items) return;
  for (int ch = lane; ch < cpr; ch += kWave) {
    float acc[N];
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] = 0.f;
    for (int k = 0; k < K; ++k) {
      const int slot = checked_slot(token_slot[(size_t)t * K + k], num_slots);
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

// Grid-stride streaming copy: the bandwidth yardstick.
__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ in,
                                                   uint4* __restrict__ out, size_t n16) {
  const size_t stride = (size_t)gridDim.x * 256 * 4;
  for (size_t i = (size_t)blockIdx.x * 256 * 4 + threadIdx.x; i < n16; i += stride) {
    uint4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (i + j * 256 < n16) v[j] = load_stream(in + i + j * 256);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (i + j * 256 < n16) store_stream(out + i + j * 256, v[j]);
  }
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


// ---------------------------------------------------------------- gradients
// combine is  out[t] = sum_k w[t,k] * y[slot(t,k)].  Its duals:
//   dy[slot(t,k)] = w[t,k] * dout[t]   (a dispatch that scales; unclaimed slots get 0)
//   dw[t,k]       = <dout[t], y[slot(t,k)]>
// (dispatch's own dual, dx[t] = sum_k dbuf[slot(t,k)], is combine with unit weights.)
template <typename T>
__global__ __launch_bounds__(kMoveThreads) void scatter_scaled_kernel(
    const uint4* __restrict__ g, const int32_t* __restrict__ token_slot,
    const float* __restrict__ weights, const int32_t* __restrict__ slot_token,
    uint4* __restrict__ out, int num_items, int num_slots, int K, int cpr, int item_waves) {
  constexpr int N = Chunk<T>::n;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(
      (int)((blockIdx.x * (unsigned)kMoveThreads + threadIdx.x) >> 6));
  if (wave < item_waves) {
    for (int ch = lane; ch < cpr; ch += kWave) {
      float a[N];
      Chunk<T>::unpack(g[(size_t)wave * cpr + ch], a);
      for (int k = 0; k < K; ++k) {
        const int slot = checked_slot(token_slot[(size_t)wave * K + k], num_slots);
        if (slot < 0) continue;
        const float w = weights[(size_t)wave * K + k];
        float b[N];
#pragma unroll
        for (int j = 0; j < N; ++j) b[j] = __fmul_rn(w, a[j]);
        out[(size_t)slot * cpr + ch] = Chunk<T>::pack(b);
      }
    }
  } else {
    const int s = wave - item_waves;
    if (slot_token != nullptr && s < num_slots && slot_token[s] < 0)
      for (int ch = lane; ch < cpr; ch += kWave) out[(size_t)s * cpr + ch] = make_uint4(0, 0, 0, 0);
  }
}

template <typename T>
__global__ __launch_bounds__(kMoveThreads) void row_dots_kernel(
    const uint4* __restrict__ g, const uint4* __restrict__ y,
    const int32_t* __restrict__ token_slot, float* __restrict__ dw, int num_items, int num_slots,
    int K, int cpr) {
  constexpr int N = Chunk<T>::n;
  const int lane = threadIdx.x & 63;
  const int t = __builtin_amdgcn_readfirstlane(
      (int)((blockIdx.x * (unsigned)kMoveThreads + threadIdx.x) >> 6));
  if (t >= num_items) return;
  for (int k = 0; k < K; ++k) {
    const int slot = checked_slot(token_slot[(size_t)t * K + k], num_slots);
    float acc = 0.f;
    if (slot >= 0) {
      for (int ch = lane; ch < cpr; ch += kWave) {
        float a[N], b[N];
        Chunk<T>::unpack(g[(size_t)t * cpr + ch], a);
        Chunk<T>::unpack(y[(size_t)slot * cpr + ch], b);
#pragma unroll
        for (int j = 0; j < N; ++j) acc += a[j] * b[j];
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, kWave);
    }
    if (lane == 0) dw[(size_t)t * K + k] = acc;
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

static uint32_t chunk_magic(int cpr) {
  return cpr == 1 ? 0u : (uint32_t)(((1ull << 32) + cpr - 1) / cpr);
}

extern "C" int vmoe_dispatch(const VmoeDispatchParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->token_slot == nullptr) return VMOE_E_NULL;
  int rc = check_move(p->x, p->token_slot, p->out, p->num_items, p->num_slots, p->K, p->D, p->dtype);
  if (rc != VMOE_OK) return rc;
  const int cpr = (int)((size_t)p->D * (p->dtype == VMOE_BF16 ? 2 : 4) / 16);
  const bool zero_fill = p->slot_token != nullptr;
  if (p->K <= kMaxK && kRowsPerBlock * cpr < 65536) {
    const int item_blocks = (p->num_items + kRowsPerBlock - 1) / kRowsPerBlock;
    const int zero_blocks = zero_fill ? (p->num_slots + kRowsPerBlock - 1) / kRowsPerBlock : 0;
    hipLaunchKernelGGL(dispatch_kernel, dim3(item_blocks + zero_blocks), dim3(kMoveThreads), 0,
                       as_stream(stream), (const uint4*)p->x, p->token_slot, p->slot_token,
                       (uint4*)p->out, p->num_items, p->num_slots, p->K, cpr, chunk_magic(cpr),
                       item_blocks);
  } else {
    const long long waves = (long long)p->num_items + (zero_fill ? p->num_slots : 0);
    const long long blocks = (waves + 3) / 4;
    if (blocks > 0x7fffffffLL) return VMOE_E_OVERFLOW;
    hipLaunchKernelGGL(dispatch_generic_kernel, dim3((unsigned)blocks), dim3(kMoveThreads), 0,
                       as_stream(stream), (const uint4*)p->x, p->token_slot, p->slot_token,
                       (uint4*)p->out, p->num_items, p->num_slots, p->K, cpr, p->num_items);
  }
  return launch_status();
}

extern "C" int vmoe_combine(const VmoeCombineParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->weights == nullptr) return VMOE_E_NULL;
  int rc = check_move(p->y, p->token_slot, p->out, p->num_items, p->num_slots, p->K, p->D, p->dtype);
  if (rc != VMOE_OK) return rc;
  const int cpr = (int)((size_t)p->D * (p->dtype == VMOE_BF16 ? 2 : 4) / 16);
  const bool bf16 = p->dtype == VMOE_BF16;
  if (p->K <= kMaxK && kRowsPerBlock * cpr < 65536) {
    const int blocks = (p->num_items + kRowsPerBlock - 1) / kRowsPerBlock;
    if (bf16)
      hipLaunchKernelGGL(combine_kernel<bf16_t>, dim3(blocks), dim3(kMoveThreads), 0,
                         as_stream(stream), (const uint4*)p->y, p->token_slot, p->weights,
                         (uint4*)p->out, p->num_items, p->num_slots, p->K, cpr, chunk_magic(cpr));
    else
      hipLaunchKernelGGL(combine_kernel<float>, dim3(blocks), dim3(kMoveThreads), 0,
                         as_stream(stream), (const uint4*)p->y, p->token_slot, p->weights,
                         (uint4*)p->out, p->num_items, p->num_slots, p->K, cpr, chunk_magic(cpr));
  } else {
    const int blocks = (p->num_items + 3) / 4;
    if (bf16)
      hipLaunchKernelGGL(combine_generic_kernel<bf16_t>, dim3(blocks), dim3(kMoveThreads), 0,
                         as_stream(stream), (const uint4*)p->y, p->token_slot, p->weights,
                         (uint4*)p->out, p->num_items, p->num_slots, p->K, cpr);
    else
      hipLaunchKernelGGL(combine_generic_kernel<float>, dim3(blocks), dim3(kMoveThreads), 0,
                         as_stream(stream), (const uint4*)p->y, p->token_slot, p->weights,
                         (uint4*)p->out, p->num_items, p->num_slots, p->K, cpr);
  }
  return launch_status();
}

extern "C" int vmoe_copy_bytes(const void* in, void* out, size_t n, vmoe_stream_t stream) {
  if (in == nullptr || out == nullptr) return VMOE_E_NULL;
  if (n == 0 || n % 16 != 0 || !aligned16(in) || !aligned16(out)) return VMOE_E_ALIGN;
  const size_t n16 = n / 16;
  size_t blocks = (n16 + 1023) / 1024;
  if (blocks > 4096) blocks = 4096;
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

extern "C" int vmoe_combine_backward_data(const VmoeCombineBackwardParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->weights == nullptr || p->dy == nullptr) return VMOE_E_NULL;
  int rc = check_move(p->dout, p->token_slot, p->dy, p->num_items, p->num_slots, p->K, p->D, p->dtype);
  if (rc != VMOE_OK) return rc;
  const int cpr = (int)((size_t)p->D * (p->dtype == VMOE_BF16 ? 2 : 4) / 16);
  const long long waves = (long long)p->num_items + (p->slot_token != nullptr ? p->num_slots : 0);
  const long long blocks = (waves + 3) / 4;
  if (blocks > 0x7fffffffLL) return VMOE_E_OVERFLOW;
  if (p->dtype == VMOE_BF16)
    hipLaunchKernelGGL(scatter_scaled_kernel<bf16_t>, dim3((unsigned)blocks), dim3(kMoveThreads), 0,
                       as_stream(stream), (const uint4*)p->dout, p->token_slot, p->weights,
                       p->slot_token, (uint4*)p->dy, p->num_items, p->num_slots, p->K, cpr,
                       p->num_items);
  else
    hipLaunchKernelGGL(scatter_scaled_kernel<float>, dim3((unsigned)blocks), dim3(kMoveThreads), 0,
                       as_stream(stream), (const uint4*)p->dout, p->token_slot, p->weights,
                       p->slot_token, (uint4*)p->dy, p->num_items, p->num_slots, p->K, cpr,
                       p->num_items);
  return launch_status();
}

extern "C" int vmoe_combine_backward_weights(const VmoeCombineBackwardParams* p,
                                             vmoe_stream_t stream) {
  if (p == nullptr || p->y == nullptr || p->dweights == nullptr) return VMOE_E_NULL;
  int rc = check_move(p->dout, p->token_slot, p->y, p->num_items, p->num_slots, p->K, p->D, p->dtype);
  if (rc != VMOE_OK) return rc;
  const int cpr = (int)((size_t)p->D * (p->dtype == VMOE_BF16 ? 2 : 4) / 16);
  const int blocks = (p->num_items + 3) / 4;
  if (p->dtype == VMOE_BF16)
    hipLaunchKernelGGL(row_dots_kernel<bf16_t>, dim3(blocks), dim3(kMoveThreads), 0,
                       as_stream(stream), (const uint4*)p->dout, (const uint4*)p->y, p->token_slot,
                       p->dweights, p->num_items, p->num_slots, p->K, cpr);
  else
    hipLaunchKernelGGL(row_dots_kernel<float>, dim3(blocks), dim3(kMoveThreads), 0,
                       as_stream(stream), (const uint4*)p->dout, (const uint4*)p->y, p->token_slot,
                       p->dweights, p->num_items, p->num_slots, p->K, cpr);
  return launch_status();
}
