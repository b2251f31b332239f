// Batched bf16 GEMM on the gfx950 matrix cores, float32 accumulate:
//   C[b] (R x N) = epilogue(A[b] (R x Kd) . Bt[b] (N x Kd)^T + bias[b])
// Both operands are K-contiguous, so a lane's MFMA fragment (8 consecutive k
// of one row) is a single 16-byte LDS read for A and for B alike.
//
// Tiling: a workgroup of WM x WN waves computes a BM x BN tile; each wave owns
// (BM/WM) x (BN/WN) of it as a grid of 32x32 v_mfma_f32_32x32x16_bf16 tiles held
// in accumulator registers.  K advances in steps of BK = 64 through two LDS
// stages: the global loads of step k+1 are issued into registers before the
// MFMAs of step k and written to the other stage after them, one barrier per
// step.  LDS rows are padded by 16 bytes so that the eight lanes served per
// clock hit all 32 banks.
#ifndef VMOE_GEMM_BF16_H_
#define VMOE_GEMM_BF16_H_

#include "vmoe_common.h"

namespace vmoe {

enum { kEpiBias = 0, kEpiBiasGeluTanh = 1, kEpiBiasGeluErf = 2 };

template <int BM_, int BN_, int WM_, int WN_>
struct GemmCfg {
  static constexpr int BM = BM_, BN = BN_, BK = 64, WM = WM_, WN = WN_;
  static constexpr int kThreads = 64 * WM * WN;
  static constexpr int TM = BM / WM, TN = BN / WN;   // wave tile
  static constexpr int FM = TM / 32, FN = TN / 32;   // 32x32 MFMA tiles per wave
  static constexpr int kLd = BK + 8;                 // padded LDS row, elements
  static constexpr int kStageElems = (BM + BN) * kLd;
  static constexpr size_t kLdsBytes = 2ull * kStageElems * sizeof(bf16_t);
  static constexpr int kChunksPerRow = BK / 8;
  static constexpr int kAChunks = BM * kChunksPerRow / kThreads;  // 16-byte loads per thread
  static constexpr int kBChunks = BN * kChunksPerRow / kThreads;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be 32-aligned");
  static_assert((BM * kChunksPerRow) % kThreads == 0 && (BN * kChunksPerRow) % kThreads == 0,
                "tile loads must divide evenly");
};

template <typename Cfg, int EPI>
__global__ __launch_bounds__(Cfg::kThreads) void gemm_bf16_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bt, const bf16_t* __restrict__ bias,
    bf16_t* __restrict__ C, int R, int N, int Kd, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* lds = reinterpret_cast<bf16_t*>(smem);
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, LD = Cfg::kLd;
  constexpr int FM = Cfg::FM, FN = Cfg::FN;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int m = lane & 31, h = lane >> 5;

  // Tile order: consecutive workgroups share the same weight columns (tile_n)
  // and walk down the rows, so a weight tile stays in L2 while it is reused.
  const int per_batch = tiles_m * tiles_n;
  const int b = blockIdx.x / per_batch;
  const int rem = blockIdx.x - b * per_batch;
  const int tile_n = rem / tiles_m;
  const int tile_m = rem - tile_n * tiles_m;
  const int row0 = tile_m * BM, col0 = tile_n * BN;
  const bf16_t* Ab = A + (size_t)b * R * Kd;
  const bf16_t* Bb = Bt + (size_t)b * N * Kd;

  // Per-thread global chunk coordinates (fixed over the K loop).
  const bf16_t* a_src[Cfg::kAChunks];
  const bf16_t* b_src[Cfg::kBChunks];
  int a_dst[Cfg::kAChunks], b_dst[Cfg::kBChunks], a_kc[Cfg::kAChunks], b_kc[Cfg::kBChunks];
#pragma unroll
  for (int i = 0; i < Cfg::kAChunks; ++i) {
    int c = tid + i * Cfg::kThreads;
    int r = c / Cfg::kChunksPerRow, kc = c % Cfg::kChunksPerRow;
    int gr = row0 + r;
    if (gr >= R) gr = R - 1;
    a_src[i] = Ab + (size_t)gr * Kd + kc * 8;
    a_dst[i] = r * LD + kc * 8;
    a_kc[i] = kc * 8;
  }
#pragma unroll
  for (int i = 0; i < Cfg::kBChunks; ++i) {
    int c = tid + i * Cfg::kThreads;
    int r = c / Cfg::kChunksPerRow, kc = c % Cfg::kChunksPerRow;
    int gn = col0 + r;
    if (gn >= N) gn = N - 1;
    b_src[i] = Bb + (size_t)gn * Kd + kc * 8;
    b_dst[i] = BM * LD + r * LD + kc * 8;
    b_kc[i] = kc * 8;
  }

  floatx16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  uint4 ra[Cfg::kAChunks], rb[Cfg::kBChunks];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < Cfg::kAChunks; ++i)
      ra[i] = (k0 + a_kc[i] + 8 <= Kd) ? *reinterpret_cast<const uint4*>(a_src[i] + k0)
                                       : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < Cfg::kBChunks; ++i)
      rb[i] = (k0 + b_kc[i] + 8 <= Kd) ? *reinterpret_cast<const uint4*>(b_src[i] + k0)
                                       : make_uint4(0, 0, 0, 0);
  };
  auto store_lds = [&](int stage) {
    bf16_t* s = lds + stage * Cfg::kStageElems;
#pragma unroll
    for (int i = 0; i < Cfg::kAChunks; ++i) *reinterpret_cast<uint4*>(s + a_dst[i]) = ra[i];
#pragma unroll
    for (int i = 0; i < Cfg::kBChunks; ++i) *reinterpret_cast<uint4*>(s + b_dst[i]) = rb[i];
  };

  const int nk = (Kd + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const bool more = kt + 1 < nk;
    if (more) load_global((kt + 1) * BK);
    const bf16_t* sa = lds + (kt & 1) * Cfg::kStageElems + (wm * Cfg::TM + m) * LD + h * 8;
    const bf16_t* sb = lds + (kt & 1) * Cfg::kStageElems + BM * LD + (wn * Cfg::TN + m) * LD + h * 8;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 fa[FM], fb[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i)
        fa[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(sa + i * 32 * LD + ks * 16));
#pragma unroll
      for (int j = 0; j < FN; ++j)
        fb[j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(sb + j * 32 * LD + ks * 16));
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (more) store_lds((kt + 1) & 1);
    __syncthreads();
  }

  // Epilogue: lane holds column (col0 + ... + m) for rows (v/4)*8 + h*4 + v%4.
  const bf16_t* biasb = bias != nullptr ? bias + (size_t)b * N : nullptr;
  bf16_t* Cb = C + (size_t)b * R * N;
#pragma unroll
  for (int j = 0; j < FN; ++j) {
    const int col = col0 + wn * Cfg::TN + j * 32 + m;
    const bool col_ok = col < N;
    const float bv = (biasb != nullptr && col_ok) ? bf2f(biasb[col]) : 0.f;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = row0 + wm * Cfg::TM + i * 32 + (v >> 2) * 8 + h * 4 + (v & 3);
        float o = bf16r(acc[i][j][v]);
        if (biasb != nullptr) o = bf16r(o + bv);
        if (EPI == kEpiBiasGeluTanh) o = gelu_tanh(o);
        if (EPI == kEpiBiasGeluErf) o = gelu_erf(o);
        if (row < R && col_ok) Cb[(size_t)row * N + col] = f2bf(o);
      }
    }
  }
}

template <typename Cfg, int EPI>
int launch_gemm_bf16(const bf16_t* A, const bf16_t* Bt, const bf16_t* bias, bf16_t* C, int batch,
                     int R, int N, int Kd, hipStream_t stream) {
  const int tiles_m = (R + Cfg::BM - 1) / Cfg::BM;
  const int tiles_n = (N + Cfg::BN - 1) / Cfg::BN;
  const long long blocks = (long long)batch * tiles_m * tiles_n;
  if (blocks > 0x7fffffffLL) return VMOE_E_OVERFLOW;
  auto kern = gemm_bf16_kernel<Cfg, EPI>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)Cfg::kLdsBytes);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, A,
                     Bt, bias, C, R, N, Kd, tiles_m, tiles_n);
  return launch_status();
}

}  // namespace vmoe
#endif  // VMOE_GEMM_BF16_H_
