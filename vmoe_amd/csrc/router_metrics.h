// Per-group auxiliary losses of the top-experts routers (vmoe/nn/routing.py:133-157),
// as a device function so that it can run as a kernel of its own or as extra workgroups
// of the slot-assignment launch.
#pragma once

#include "vmoe_common.h"

namespace vmoe {

// Per-group auxiliary losses.  One workgroup of 1024 threads per group; thread
// (r, q) sums a strip of V expert columns over rows r, r+R, ... in a fixed
// order, the R partial sums per column are then added in a fixed order, so
// results are run-to-run identical.
constexpr int kMetricThreads = 1024;

template <typename T>
__device__ __forceinline__ void router_metrics_group(
    const T* __restrict__ gates, const int32_t* __restrict__ top1, float* __restrict__ imp_loss,
    float* __restrict__ gsh_loss, float* __restrict__ aux_loss, float w_gsh, float w_imp,
    int S, int E, int top1_stride, int V, int g, unsigned char* smem) {
  const int tid = threadIdx.x;
  const int strips = (E + V - 1) / V;                        // column strips per row
  const int R = kMetricThreads / strips > 0 ? kMetricThreads / strips : 1;   // row lanes
  float* part = reinterpret_cast<float*>(smem);              // (R, strips * V)
  const int EW = strips * V;
  int* count = reinterpret_cast<int*>(part + (size_t)R * EW);  // (E,)
  float* imp = reinterpret_cast<float*>(count + E);          // (E,)
  for (int e = tid; e < E; e += kMetricThreads) count[e] = 0;
  __syncthreads();
  const int r = tid / strips;
  const int q = tid - r * strips;
  const bool wave_rows = strips <= kWave && (strips & (strips - 1)) == 0;
  if (r < R) {
    float s[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) s[t] = 0.f;
    const T* base = gates + (size_t)g * S * E + q * V;
    if (V == 16 / (int)sizeof(T)) {
      // One 16-byte load per row (E is a multiple of V and rows are 16-byte aligned).
      for (int i = r; i < S; i += R) {
        const uint4 raw = *reinterpret_cast<const uint4*>(base + (size_t)i * E);
        const T* v = reinterpret_cast<const T*>(&raw);
#pragma unroll
        for (int t = 0; t < (int)(16 / sizeof(T)); ++t) s[t] += Elt<T>::load(&v[t]);
      }
    } else {
      for (int i = r; i < S; i += R)
        for (int t = 0; t < V; ++t)
          if (q * V + t < E) s[t] += Elt<T>::load(base + (size_t)i * E + t);
    }
    // A power-of-two number of strips <= 64 puts 64 / strips row lanes of every strip in
    // one wave: they are added with lane exchanges (a fixed tree) and one row of partial
    // sums per wave goes to LDS; otherwise every row lane writes its own.
    if (wave_rows) {
#pragma unroll
      for (int t = 0; t < 8; ++t)
        if (t < V)
          for (int m = strips; m < kWave; m <<= 1) s[t] += __shfl_xor(s[t], m, kWave);
      if ((tid & (kWave - 1)) < strips)
        for (int t = 0; t < V; ++t) part[(size_t)(tid >> 6) * EW + q * V + t] = s[t];
    } else {
      for (int t = 0; t < V; ++t) part[(size_t)r * EW + q * V + t] = s[t];
    }
  }
  for (int i = tid; i < S; i += kMetricThreads) {
    int t = top1[((size_t)g * S + i) * top1_stride];
    if (t >= 0 && t < E) atomicAdd(&count[t], 1);
  }
  __syncthreads();
  if (wave_rows) {
    for (int e = tid; e < E; e += kMetricThreads) {
      float total = 0.f;
      for (int w = 0; w < kMetricThreads / kWave; ++w) total += part[(size_t)w * EW + e];
      imp[e] = total;
    }
  } else {
    // Fixed-order tree over the row lanes.
    int span = 1;
    while (span < R) span <<= 1;
    for (int off = span >> 1; off > 0; off >>= 1) {
      for (int idx = tid; idx < off * EW; idx += kMetricThreads) {
        int rr = idx / EW, c = idx - rr * EW;
        if (rr + off < R) part[(size_t)rr * EW + c] += part[(size_t)(rr + off) * EW + c];
      }
      __syncthreads();
    }
    for (int e = tid; e < E; e += kMetricThreads) imp[e] = part[e];
  }
  __syncthreads();
  if (tid == 0) {
    float mean = 0.f;
    for (int e = 0; e < E; ++e) mean += imp[e];
    mean /= (float)E;
    float var = 0.f, gs = 0.f;
    for (int e = 0; e < E; ++e) {
      float d = imp[e] - mean;
      var += d * d;
      gs += ((float)count[e] / (float)S) * (imp[e] / (float)S);
    }
    var /= (float)E;
    float il = var / (mean * mean);
    float gl = gs / (float)E * (float)E * (float)E;
    imp_loss[g] = il;
    gsh_loss[g] = gl;
    float a = 0.f;
    if (w_gsh > 0.f) a += gl * w_gsh;
    if (w_imp > 0.f) a += il * w_imp;
    aux_loss[g] = a;
  }
}

// Arguments of router_metrics_group that do not depend on the element type.
struct RouterMetricsArgs {
  const void* gates;
  const int32_t* top1;
  float* imp_loss;
  float* gsh_loss;
  float* aux_loss;
  float w_gsh, w_imp;
  int S, E, top1_stride, V;
};

// Column strip width, shape of the partial sums and LDS bytes of one group.
inline bool router_metrics_geometry(const VmoeRouterMetricsParams* p, int* V, size_t* lds) {
  const int esz = p->dtype == VMOE_BF16 ? 2 : 4;
  const int vec = 16 / esz;
  const bool vec_ok = p->E % vec == 0 && aligned16(p->gates);
  *V = vec_ok ? vec : 1;
  const int strips = (p->E + *V - 1) / *V;
  const int R = kMetricThreads / strips > 0 ? kMetricThreads / strips : 1;
  *lds = ((size_t)R * strips * *V + 2 * (size_t)p->E) * 4;
  return *lds <= 64 * 1024;
}

inline int check_router_metrics(const VmoeRouterMetricsParams* p) {
  if (p == nullptr || p->gates == nullptr || p->top1_idx == nullptr ||
      p->importance_loss == nullptr || p->gshard_loss == nullptr || p->auxiliary_loss == nullptr)
    return VMOE_E_NULL;
  if (p->G < 1 || p->S < 1 || p->E < 1 || p->top1_stride < 1) return VMOE_E_SHAPE;
  if (p->dtype != VMOE_F32 && p->dtype != VMOE_BF16) return VMOE_E_DTYPE;
  if (p->E > 1024) return VMOE_E_UNSUPPORTED;
  return VMOE_OK;
}

}  // namespace vmoe
