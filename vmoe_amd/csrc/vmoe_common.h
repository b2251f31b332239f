// Shared device helpers for the gfx950 kernels of libvmoe_hip.so.
#ifndef VMOE_COMMON_H_
#define VMOE_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <map>
#include <mutex>
#include <utility>

#include "vmoe_hip.h"
#include "route_index.h"

namespace vmoe {

constexpr int kWave = 64;

typedef uint16_t bf16_t;  // bfloat16 storage
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// float32 -> bfloat16, round to nearest even (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ bf16_t f2bf(float f) {
  __bf16 b = (__bf16)f;
  return __builtin_bit_cast(bf16_t, b);
}
__device__ __forceinline__ float bf2f(bf16_t h) {
  return __builtin_bit_cast(float, (uint32_t)h << 16);
}
// Two float32 -> two bfloat16 in one dword (lo in bits 0..15): one v_cvt_pk_bf16_f32.
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  floatx2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ float bf_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
// Round a float32 to the nearest bfloat16 value, kept as float32.
__device__ __forceinline__ float bf16r(float f) { return bf2f(f2bf(f)); }

template <typename T> struct Elt;
template <> struct Elt<float> {
  static constexpr int dtype = VMOE_F32;
  __device__ static __forceinline__ float load(const float* p) { return *p; }
  __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
  __device__ static __forceinline__ float round(float v) { return v; }
};
template <> struct Elt<bf16_t> {
  static constexpr int dtype = VMOE_BF16;
  __device__ static __forceinline__ float load(const bf16_t* p) { return bf2f(*p); }
  __device__ static __forceinline__ void store(bf16_t* p, float v) { *p = f2bf(v); }
  __device__ static __forceinline__ float round(float v) { return bf16r(v); }
};

__device__ __forceinline__ float gelu_tanh(float x) {
  const float c = 0.7978845608028654f;  // sqrt(2/pi)
  float inner = c * (x + 0.044715f * (x * x * x));
  return 0.5f * x * (1.0f + tanhf(inner));
}
__device__ __forceinline__ float gelu_erf(float x) {
  return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f));
}

// Monotone map float32 -> uint32 (larger float -> larger uint); -0.0 == +0.0.
__device__ __forceinline__ uint32_t orderable(float f) {
  return orderable_bits(__builtin_bit_cast(uint32_t, f));
}

// s_waitcnt vmcnt(N) with lgkmcnt/expcnt left at their maxima.
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xc07f); }
// Workgroup barrier without the implicit "wait for every outstanding memory
// operation" of __syncthreads(): callers wait for exactly what they need first.
// The asm clobbers keep the compiler from moving LDS accesses across it.
__device__ __forceinline__ void raw_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// Gap between the last MFMA of a loop and the first read of its accumulators.
// The matrix cores write a result over many cycles and a reader must leave
// enough wait states.  The compiler counts them within straight-line code, but
// a v_mfma_f32_32x32x16_bf16 result read a few instructions behind a loop
// back-edge came back with its last register stale (rows 27 and 31 of every
// tile wrong), so every kernel states the gap explicitly before it touches
// accumulators that a loop has just written.
__device__ __forceinline__ void mfma_result_fence() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// Gap behind a 16-byte buffer store whose data registers the next instructions overwrite.
// The store reads its data registers a few cycles after it has issued.  For a store with an
// immediate scalar offset the compiler leaves the wait states itself; for one whose scalar
// offset is a register it leaves none, and a VALU result written to a data register in the very
// next instruction reached memory in place of the stored value in a few lanes (seen with the
// register-hungry GELU epilogue, where the allocator reuses the registers at once).  Two idle
// cycles between scheduling barriers close the window.
__device__ __forceinline__ void store_data_guard() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_nop 1" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

inline hipStream_t as_stream(vmoe_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int launch_status() {
  hipError_t err = hipGetLastError();
  return err == hipSuccess ? VMOE_OK : (int)err;
}

// Raises a kernel's limit of dynamic LDS.  hipFuncSetAttribute takes a lock and walks the
// runtime's tables on the host, so it is called once per (kernel, device) and limit: a
// launch whose size the recorded limit already covers skips it.
inline hipError_t allow_dynamic_lds(const void* kern, size_t bytes) {
  static std::mutex mu;
  static std::map<std::pair<const void*, int>, size_t> limit;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  std::lock_guard<std::mutex> lock(mu);
  size_t& have = limit[std::make_pair(kern, dev)];
  if (bytes <= have) return hipSuccess;
  e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e == hipSuccess) have = bytes;
  return e;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace vmoe
#endif  // VMOE_COMMON_H_
