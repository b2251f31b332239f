// Expert MLPs (Dense -> GELU -> Dense per expert) for gfx950.
//
// Replaces the expert vmap of vmoe/moe.py:434-439 over
// vit_jax.models_vit.MlpBlock (vmoe/nn/vit_moe.py:38-45): a GEMM batched over
// the expert axis with the bias add and the GELU fused into the epilogue of the
// first product and the bias add into the second.
#include <cstring>

#include "gemm_bf16_wide.h"
#include "gemm_bf16_w8.h"
#include "gemm_f32.h"
#include "compact_rows.h"

namespace vmoe {
namespace {

// ---------------------------------------------------------------- float32 path
// C[b] (R x N) = epi(A[b] (R x Kd) . B[b] (Kd x N) + bias[b]) with
// v_mfma_f32_32x32x2_f32 (IEEE float32 multiply-add).  64x64 tile, 4 waves,
// B is consumed in the reference's (in, out) order: a lane's B operand is one
// scalar B[k][n], so no transposition is needed.
constexpr int kF32Tile = 64, kF32BK = 32;

template <int EPI>
__global__ __launch_bounds__(256) void gemm_f32_kernel(
    const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ bias,
    float* __restrict__ C, int R, int N, int Kd, int tiles_m, int tiles_n,
    const int32_t* __restrict__ rows) {
  // Two LDS stages of a 32-wide k tile: the global loads of k tile t + 1 are issued before the
  // MFMAs of k tile t and written to the other stage behind them, one barrier per k tile.
  __shared__ float sa[2][kF32Tile][kF32BK + 1];
  __shared__ float sb[2][kF32BK][kF32Tile + 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m = lane & 31, h = lane >> 5;
  const int per_batch = tiles_m * tiles_n;
  const int b = blockIdx.x / per_batch;
  const int rem = blockIdx.x - b * per_batch;
  const int tile_n = rem / tiles_m, tile_m = rem - tile_n * tiles_m;
  const int row0 = tile_m * kF32Tile, col0 = tile_n * kF32Tile;
  int live = R;               // ragged batches: only rows[b] rows of batch b hold data
  if (rows != nullptr) {
    live = min(rows[b], R);
    if (row0 >= live) return;
  }
  const float* Ab = A + (size_t)b * R * Kd;
  const float* Bb = B + (size_t)b * Kd * N;
  floatx16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  // A: 64 rows x 8 float4 per k tile, B: 32 rows x 16 float4: two float4 of each per thread.
  const int ar = tid >> 3, akc = (tid & 7) * 4;    // rows ar, ar + 32
  const int bk = tid >> 4, bn = (tid & 15) * 4;    // k rows bk, bk + 16
  float4 va[2], vb[2];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      va[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      vb[u] = va[u];
      const int gr = min(row0 + ar + u * 32, R - 1);
      if (k0 + akc + 4 <= Kd) va[u] = *reinterpret_cast<const float4*>(Ab + (size_t)gr * Kd + k0 + akc);
      const int gk = k0 + bk + u * 16, gn = col0 + bn;
      if (gk < Kd && gn + 4 <= N) vb[u] = *reinterpret_cast<const float4*>(Bb + (size_t)gk * N + gn);
    }
  };
  auto stage = [&](int s_) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      float* pa = &sa[s_][ar + u * 32][akc];
      pa[0] = va[u].x; pa[1] = va[u].y; pa[2] = va[u].z; pa[3] = va[u].w;
      float* pb = &sb[s_][bk + u * 16][bn];
      pb[0] = vb[u].x; pb[1] = vb[u].y; pb[2] = vb[u].z; pb[3] = vb[u].w;
    }
  };
  fetch(0);
  stage(0);
  __syncthreads();
  int cur = 0;
  for (int k0 = 0; k0 < Kd; k0 += kF32BK) {
    const bool more = k0 + kF32BK < Kd;
    if (more) fetch(k0 + kF32BK);
#pragma unroll
    for (int ks = 0; ks < kF32BK / 2; ++ks) {
      float a = sa[cur][wm * 32 + m][ks * 2 + h];
      float bb = sb[cur][ks * 2 + h][wn * 32 + m];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bb, acc, 0, 0, 0);
    }
    if (more) stage(cur ^ 1);
    __syncthreads();
    cur ^= 1;
  }
  mfma_result_fence();
  const int col = col0 + wn * 32 + m;
  const bool col_ok = col < N;
  const float bv = (bias != nullptr && col_ok) ? bias[(size_t)b * N + col] : 0.f;
  float* Cb = C + (size_t)b * R * N;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int row = row0 + wm * 32 + (v >> 2) * 8 + h * 4 + (v & 3);
    float o = acc[v] + bv;
    if (EPI == kEpiBiasGeluTanh) o = gelu_tanh(o);
    if (EPI == kEpiBiasGeluErf) o = gelu_erf(o);
    if (row < live && col_ok) Cb[(size_t)row * N + col] = o;
  }
}

template <int EPI>
int launch_gemm_f32(const float* A, const float* B, const float* bias, float* C, int batch, int R,
                    int N, int Kd, hipStream_t stream, const int32_t* rows = nullptr,
                    const int32_t* a_rows = nullptr, int a_items = 0) {
  // The DMA kernel where its shapes allow: 64 x 128 tiles when they outnumber the CUs twice
  // over, 64 x 64 otherwise.  VMOE_F32_GEMM=plain keeps the register-staged kernel below.
  const char* which = getenv("VMOE_F32_GEMM");
  // (gathered rows are the DMA kernel's alone: check_mlp has made sure that it applies)
  if (gemm_f32_dma_ok(A, B, R, N, Kd, a_items) &&
      (a_rows != nullptr || !(which != nullptr && strcmp(which, "plain") == 0))) {
    const long long wide_tiles = (long long)batch * ((R + 63) / 64) * ((N + 127) / 128);
    if (wide_tiles >= 2 * kCusPerXcd * kNumXcd && !(which != nullptr && strcmp(which, "64") == 0))
      return launch_gemm_f32_dma<EPI, 128>(A, B, bias, C, batch, R, N, Kd, stream, rows, a_rows, a_items);
    return launch_gemm_f32_dma<EPI, 64>(A, B, bias, C, batch, R, N, Kd, stream, rows, a_rows, a_items);
  }
  if (a_rows != nullptr) return VMOE_E_UNSUPPORTED;
  const int tiles_m = (R + kF32Tile - 1) / kF32Tile, tiles_n = (N + kF32Tile - 1) / kF32Tile;
  const long long blocks = (long long)batch * tiles_m * tiles_n;
  if (blocks > 0x7fffffffLL) return VMOE_E_OVERFLOW;
  hipLaunchKernelGGL(gemm_f32_kernel<EPI>, dim3((unsigned)blocks), dim3(256), 0, stream, A, B, bias,
                     C, R, N, Kd, tiles_m, tiles_n, rows);
  return launch_status();
}

// ---------------------------------------------------------------- transpose
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ in,
                                                        T* __restrict__ out, int rows, int cols) {
  __shared__ T tile[64][64 + 2];
  const int b = blockIdx.z;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const T* src = in + (size_t)b * rows * cols;
  T* dst = out + (size_t)b * rows * cols;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    int r = r0 + i, c = c0 + tx;
    if (r < rows && c < cols) tile[i][tx] = src[(size_t)r * cols + c];
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    int c = c0 + i, r = r0 + tx;
    if (r < rows && c < cols) dst[(size_t)c * rows + r] = tile[tx][i];
  }
}

int transpose(const void* in, void* out, int batch, int rows, int cols, int dtype,
              hipStream_t stream) {
  dim3 grid((cols + 63) / 64, (rows + 63) / 64, batch);
  if (dtype == VMOE_BF16)
    hipLaunchKernelGGL(transpose_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)in,
                       (bf16_t*)out, rows, cols);
  else
    hipLaunchKernelGGL(transpose_kernel<float>, grid, dim3(256), 0, stream, (const float*)in,
                       (float*)out, rows, cols);
  return launch_status();
}

// First product (short K = D, GELU epilogue): two 128x256 workgroups per CU so one
// workgroup's epilogue overlaps the other's MFMAs.  Second product (long K = M):
// one 256x256 workgroup per CU for the highest arithmetic intensity.
using CfgUp = GemmCfg<128, 256, 2, 2, 32, 3, 2>;
using CfgDown = GemmCfg<256, 256, 2, 2, 32, 4, 1>;
// The persistent form of the second product takes k in 64-wide tiles, two stages: a DMA
// load then requests whole 128-byte lines of an operand row (64-byte halves of a line,
// requested a k tile apart, move at two thirds of the rate when the line comes from
// beyond L2).  Its A rows sit in a ring of three LDS slots, its B rows in one of two (all of
// the 160 KB); the output is staged in the A slot that the tile's last k tile has left.
// Tile shape and launch plan are CfgDown's.
using CfgDownPersistent = GemmCfg<256, 256, 2, 2, 64, 2, 1>;

// Register-resident MFMA loop: the arithmetic ceiling that the expert GEMMs are
// compared with.  Every wave keeps a 128 x 128 accumulator tile (16 MFMA tiles,
// as in the 256 x 256 GEMM) and multiplies operand fragments that it read once
// from `seed` (real data, so that operand toggling, and with it the clock the
// power management settles on, resembles the GEMM's); nothing moves but
// registers.
__global__ __launch_bounds__(256) void mfma_probe_kernel(const uint4* __restrict__ seed,
                                                         float* __restrict__ sink, int iters,
                                                         size_t seed_vecs) {
  bf16x8 fa[2][4], fb[2][4];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const size_t base = ((size_t)blockIdx.x * 256 + threadIdx.x) * 16 + u * 8 + i * 2;
      fa[u][i] = __builtin_bit_cast(bf16x8, seed[base % seed_vecs]);
      fb[u][i] = __builtin_bit_cast(bf16x8, seed[(base + 1) % seed_vecs]);
    }
  floatx16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[u][j], fa[u][i], acc[i][j], 0, 0, 0);
  }
  mfma_result_fence();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) t += acc[i][j][v];
  sink[(size_t)blockIdx.x * 256 + threadIdx.x] = t;
}

// Load-only counterpart of the 256x256 product: every workgroup issues the LDS-DMA
// loads of its tile's k tiles (same addresses, request shapes and tile order as the product
// kernels) and nothing else; no barrier, no wait except the one that keeps a stage from
// being requested again while a request for it is in flight.  PCfg = CfgDown: 32-wide k
// tiles (64-byte row segments), a ring of four stages, two k tiles in flight;
// PCfg = CfgDownPersistent: 64-wide k tiles (128-byte row segments), two stages, one to two
// k tiles in flight.  The rate at which it moves operand tiles is the ceiling of any kernel
// with requests of that shape.
template <typename PCfg>
__global__ __launch_bounds__(256, 1) void operand_delivery_probe_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bt, int R, int N, int Kd,
    int tiles_m, int tiles_n, int num_tiles, int tiles_per_xcd, int panel_rows) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-resource builtins exist in the device pass only
  extern __shared__ __align__(1024) unsigned char smem[];
  using Cfg = PCfg;
  int b, tile_m, tile_n;
  if (!map_tile(tiles_m, tiles_n, num_tiles, tiles_per_xcd, panel_rows, b, tile_m, tile_n)) return;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int CPR = Cfg::kChunksPerRow, RPL = Cfg::kRowsPerLoad, RB = Cfg::kRowBytes;
  const int lrow = lane / CPR, chunk = lane % CPR;
  uint32_t a_off[Cfg::kAIssues], b_off[Cfg::kBIssues];
#pragma unroll
  for (int i = 0; i < Cfg::kAIssues; ++i)
    a_off[i] = (uint32_t)min(tile_m * Cfg::BM + (i * Cfg::kWaves + wave) * RPL + lrow, R - 1) *
                   (uint32_t)Kd * 2u + chunk * 16;
#pragma unroll
  for (int i = 0; i < Cfg::kBIssues; ++i)
    b_off[i] = (uint32_t)min(tile_n * Cfg::BN + (i * Cfg::kWaves + wave) * RPL + lrow, N - 1) *
                   (uint32_t)Kd * 2u + chunk * 16;
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(A + (size_t)b * R * Kd), 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(Bt + (size_t)b * N * Kd), 0, -1, 0x00020000);
  const int nk = Kd / Cfg::BK;
  for (int kt = 0; kt < nk; ++kt) {
    unsigned char* s = smem + (kt % Cfg::NSTAGE) * Cfg::kStageBytes;
#pragma unroll
    for (int i = 0; i < Cfg::kAIssues; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(s + (i * Cfg::kWaves + wave) * RPL * RB),
                                               16, a_off[i], kt * Cfg::BK * 2, 0, 0);
#pragma unroll
    for (int i = 0; i < Cfg::kBIssues; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          b_rsrc, (lds_ptr_t)(s + Cfg::BM * RB + (i * Cfg::kWaves + wave) * RPL * RB), 16, b_off[i],
          kt * Cfg::BK * 2, 0, 0);
    wait_vmcnt<(Cfg::NSTAGE >= 4 ? 2 : 1) * Cfg::kLoads>();   // a stage is written again NSTAGE k tiles later
  }
  wait_vmcnt<0>();
#endif
}

// Row compaction and the launch plans of the expert MLP's ragged products in one launch:
// workgroups 0 .. compact_blocks - 1 renumber the assignments (compact_rows_fused_block),
// the others plan (plan_ragged_tiles_block, row counts from the fill counts).  Neither part
// reads what the other writes.
__global__ __launch_bounds__(256) void compact_rows_planned_kernel(
    const int32_t* __restrict__ fill, const int32_t* __restrict__ token_slot,
    int32_t* __restrict__ token_row, int32_t* __restrict__ row_token,
    int32_t* __restrict__ rows_per_expert, int G, int E, int C, int per_group, int K, size_t n,
    unsigned compact_blocks, int R, RaggedGeom ga, RaggedGeom gb) {
  extern __shared__ int32_t tile_prefix[];
  if (blockIdx.x < compact_blocks)
    compact_rows_fused_block(fill, token_slot, token_row, row_token, rows_per_expert, G, E, C,
                             per_group, K, n, blockIdx.x);
  else
    plan_ragged_tiles_block(nullptr, fill, G, E, R, ga, gb, blockIdx.x - compact_blocks, tile_prefix);
}

size_t align256(size_t v) { return (v + 255) / 256 * 256; }

// The status words of a bfloat16 call sit behind the hidden activations.
constexpr size_t kStatusBytes = 256;
static_assert(kStatusWords * sizeof(int32_t) <= kStatusBytes, "status block");

// Which kernel runs the second product (bfloat16).
//  kDownShared: 256 x 256 tiles walked by one workgroup per CU, the last, partial round of a
//    die shared along k (stream-K): its time follows the number of tiles, not of rounds.
//  kDownEightWaves: the same tiles walked by eight waves per workgroup with 16 x 16 x 32 MFMAs
//    (gemm_bf16_w8.h), the tiles of a partial round whole: ahead where a die's run is long
//    enough that a partial round is a small part of it.
//  kDownNarrow: the same kernel on 256 x 192 tiles: where that tiling fills the chip's rounds
//    better (768 output columns: four column tiles instead of three).
//  kDownWide: 384 x 256 tiles, eight waves; whole rounds of one tile per CU.
//  kDownHalf: 128 x 256 tiles, two per CU (static launches the tile-walking kernels do not
//    cover, where whole rounds of 256 x 256 tiles would waste a tenth or more).
//  kDownPlain: 256 x 256 tiles, one workgroup per tile.
enum DownKernel { kDownShared, kDownEightWaves, kDownNarrow, kDownWide, kDownHalf, kDownPlain };
using CfgDownNarrow = W8Cfg<6>;

bool down_prefers_half_tiles(int E, int R, int N) {
  constexpr int64_t kNumCu = 256;
  const int64_t tn = (N + 255) / 256;
  const int64_t full = (int64_t)E * ((R + 255) / 256) * tn;
  const int64_t half = (int64_t)E * ((R + 127) / 128) * tn;
  const double t_full = (double)((full + kNumCu - 1) / kNumCu);
  const double t_half = 0.5 * 1.05 * (double)((half + kNumCu - 1) / kNumCu);
  return t_half < 0.9 * t_full;
}

// Launch plans of the two ragged products of an MLP: geometry, bytes, one planning launch.
struct MlpPlans {
  GemmGeom up, down;
  DownKernel down_kernel = kDownPlain;
  int down_bm = CfgDown::BM;
  size_t up_bytes = 0, down_bytes = 0;   // 0: that product keeps the static tile order
  size_t streamk_bytes = 0;              // exchange memory of kDownShared
};

MlpPlans mlp_plans(int E, int R, int D, int M, bool ragged) {
  MlpPlans m;
  m.up = gemm_geometry<CfgUp>(E, R, M, D);
  // Ragged launches are planned whenever the geometry allows: with whole experts per
  // die in a static order the die that drew the fullest experts sets the time (a layer
  // with capacity factor 0.5 and a skewed router: 399 -> 267 us for the two products,
  // a third off the MoE blocks of the B/16 model with 8 experts), and on a balanced
  // layer the planned launch costs 0.3 %.
  auto bytes = [&](const GemmGeom& g) -> size_t {
    if (!ragged || !g.fast || g.ragged_slots * kNumXcd > 0x7ffffff0LL ||
        plan_ragged_tiles_lds(E) > 60000)
      return 0;
    return align256(((size_t)g.ragged_slots * kNumXcd + 1) * sizeof(int4));   // + the header entry
  };
  m.up_bytes = bytes(m.up);
  const GemmGeom square = gemm_geometry<CfgDown>(E, R, D, M);
  const GemmGeom wide = gemm_geometry<WideCfg>(E, R, D, M);
  const int4* const planned = reinterpret_cast<const int4*>(&m);   // stands for "a plan exists"
  const int32_t* const rows = ragged ? reinterpret_cast<const int32_t*>(&m) : nullptr;
  const bool shared_ok = persistent_gemm_ok<CfgDownPersistent>(
      E, R, D, M, rows, bytes(square) ? planned : nullptr) && M / CfgDownPersistent::BK % kStreamKGranule == 0;
  const bool wide_ok = wide_gemm_ok(E, R, D, M, nullptr, nullptr, nullptr, 0) && (!ragged || bytes(wide));
  constexpr double kNumCu = kCusPerXcd * kNumXcd;
  // Time in units of one 256 x 256 tile of the four-wave kernel on one CU, fitted to alternating
  // bench runs of the layer configurations (B/16 layer, Soft MoE layer, L/16 layer at capacity
  // 0.5, B/16 model): the shared kernel pays for its tiles (the padding of the last row tile
  // of a batch included) plus the exchange; the eight-wave kernel runs whole rounds at 0.95
  // per tile (two waves per SIMD, 16 x 16 x 32 MFMAs); its 192-column form whole rounds of
  // tiles three quarters the size at 0.97 of the time per flop, taken only where it wins by
  // 3 % (Soft MoE: 512 tiles = 2 rounds instead of 1.5 shared ones, 417 -> 397 us for the
  // MLP; the B/16 model's 13 rounds against 10: 0.2 ms slower); the wide kernel's tile is 1.5
  // of them at 1.04 of the time per flop, in whole rounds.
  const GemmGeom narrow = gemm_geometry<CfgDownNarrow>(E, R, D, M);
  const bool eight_ok = w8_gemm_ok<8>(E, R, D, M, rows, bytes(square) ? planned : nullptr);
  const bool narrow_ok = w8_gemm_ok<6>(E, R, D, M, rows, bytes(narrow) ? planned : nullptr);
  const double t_wide = 1.5 * 1.04 * std::ceil((double)wide.tiles / kNumCu);
  // the shared form balances a partial round but runs 32x32x16 MFMAs and exchanges sums: on the
  // L/16 half-capacity layer (0.8 tiles per CU) it measures 2 % behind eight waves
  const double t_shared = 1.12 * (double)square.tiles / kNumCu + 0.1;
  const double t_eight = 0.95 * std::ceil((double)square.tiles / kNumCu);
  const double t_narrow = 0.75 * 0.97 * std::ceil((double)narrow.tiles / kNumCu);
  double t_best = 1e300;
  m.down_kernel = !ragged && down_prefers_half_tiles(E, R, D) ? kDownHalf : kDownPlain;
  if (wide_ok) { m.down_kernel = kDownWide; t_best = t_wide; }
  if (shared_ok && t_shared <= t_best) { m.down_kernel = kDownShared; t_best = t_shared; }
  if (eight_ok && t_eight <= t_best) { m.down_kernel = kDownEightWaves; t_best = t_eight; }
  if (narrow_ok && t_narrow < 0.97 * t_best) { m.down_kernel = kDownNarrow; t_best = t_narrow; }
  // (VMOE_SECOND_PRODUCT=shared|eight|narrow|wide in the environment overrides the choice
  // where the named kernel applies: the switch behind the figures that the model above was
  // fitted to)
  if (const char* force = getenv("VMOE_SECOND_PRODUCT")) {
    if (strcmp(force, "shared") == 0 && shared_ok) m.down_kernel = kDownShared;
    if (strcmp(force, "eight") == 0 && eight_ok) m.down_kernel = kDownEightWaves;
    if (strcmp(force, "narrow") == 0 && narrow_ok) m.down_kernel = kDownNarrow;
    if (strcmp(force, "wide") == 0 && wide_ok) m.down_kernel = kDownWide;
  }
  m.down = m.down_kernel == kDownWide ? wide : m.down_kernel == kDownNarrow ? narrow : square;
  m.down_bm = m.down_kernel == kDownWide ? WideCfg::BM : CfgDown::BM;
  static_assert(CfgDownNarrow::BM == CfgDown::BM, "row tiles of the narrow kernel");
  m.down_bytes = bytes(m.down);
  if (m.down_kernel == kDownShared)
    m.streamk_bytes = align256(StreamKWorkspace<CfgDownPersistent>::kBytes);
  return m;
}

}  // namespace
}  // namespace vmoe

using namespace vmoe;

static int check_mlp(const VmoeExpertMlpParams* p) {
  if (p == nullptr || p->x == nullptr || p->out == nullptr) return VMOE_E_NULL;
  if (p->E < 1 || p->R < 1 || p->D < 1 || p->M < 1) return VMOE_E_SHAPE;
  if (p->dtype != VMOE_F32 && p->dtype != VMOE_BF16) return VMOE_E_DTYPE;
  if (p->x_rows != nullptr) {
    if (p->rows_per_expert == nullptr) return VMOE_E_NULL;
    if (p->num_items < 1) return VMOE_E_SHAPE;
    // float32: the LDS-DMA kernel gathers (whole 32-wide k tiles, 16-byte aligned operands)
    if (p->dtype != VMOE_BF16 &&
        !gemm_f32_dma_ok((const float*)p->x, (const float*)p->w0, p->R, p->M, p->D, p->num_items))
      return VMOE_E_UNSUPPORTED;
  }
  if (p->gelu != VMOE_GELU_TANH && p->gelu != VMOE_GELU_ERF) return VMOE_E_DTYPE;
  if (p->dtype == VMOE_BF16) {
    if ((p->w0 == nullptr && p->w0t == nullptr) || (p->w1 == nullptr && p->w1t == nullptr))
      return VMOE_E_NULL;
    if (p->D % 8 != 0 || p->M % 8 != 0) return VMOE_E_ALIGN;
  } else {
    if (p->w0 == nullptr || p->w1 == nullptr) return VMOE_E_NULL;
    if (p->D % 4 != 0 || p->M % 4 != 0) return VMOE_E_ALIGN;
  }
  if (!aligned16(p->x) || !aligned16(p->out)) return VMOE_E_ALIGN;
  if ((int64_t)p->E * p->R >= INT32_MAX) return VMOE_E_OVERFLOW;
  // Unpacked weights are transposed with the expert as the grid's z dimension.
  if (p->dtype == VMOE_BF16 && (p->w0t == nullptr || p->w1t == nullptr) && p->E > 65535)
    return VMOE_E_UNSUPPORTED;
  return VMOE_OK;
}

extern "C" size_t vmoe_expert_mlp_workspace_bytes(const VmoeExpertMlpParams* p) {
  if (p == nullptr || p->E < 1 || p->R < 1 || p->D < 1 || p->M < 1) return 0;
  const size_t b = p->dtype == VMOE_BF16 ? 2 : 4;
  size_t bytes = align256((size_t)p->E * p->R * p->M * b);  // hidden activations
  if (p->dtype == VMOE_BF16) {   // status words, launch plans of the ragged products, stream-K exchange
    const MlpPlans m = mlp_plans(p->E, p->R, p->D, p->M, p->rows_per_expert != nullptr);
    bytes += kStatusBytes + m.up_bytes + m.down_bytes + m.streamk_bytes;
  }
  if (p->dtype == VMOE_BF16) {
    if (p->w0t == nullptr) bytes += align256((size_t)p->E * p->D * p->M * b);
    if (p->w1t == nullptr) bytes += align256((size_t)p->E * p->D * p->M * b);
  }
  return bytes;
}

// Where the pieces of a bfloat16 MLP's workspace lie, and what the planning launch is given.
struct MlpWorkspace {
  void* hidden = nullptr;
  int32_t* status = nullptr;         // the call's status words (bfloat16 only)
  int4* plan_up = nullptr;
  int4* plan_down = nullptr;
  void* streamk = nullptr;
  unsigned char* rest = nullptr;     // transposed weights, where the caller did not pack them
  MlpPlans m;
  RaggedGeom ga{}, gb{};
  int plan_blocks = 0;               // workgroups of the planning launch (0: nothing to plan)
};

MlpWorkspace mlp_workspace(const VmoeExpertMlpParams* p) {
  MlpWorkspace w;
  unsigned char* ws = static_cast<unsigned char*>(p->workspace);
  const size_t b = p->dtype == VMOE_BF16 ? 2 : 4;
  w.hidden = ws;
  ws += align256((size_t)p->E * p->R * p->M * b);
  if (p->dtype == VMOE_BF16) {
    w.status = reinterpret_cast<int32_t*>(ws);
    ws += kStatusBytes;
    w.m = mlp_plans(p->E, p->R, p->D, p->M, p->rows_per_expert != nullptr);
    if (w.m.up_bytes) w.plan_up = reinterpret_cast<int4*>(ws);
    ws += w.m.up_bytes;
    if (w.m.down_bytes) w.plan_down = reinterpret_cast<int4*>(ws);
    ws += w.m.down_bytes;
    if (w.m.streamk_bytes) w.streamk = ws;
    ws += w.m.streamk_bytes;
    if (w.plan_up != nullptr || w.plan_down != nullptr) {
      w.ga = RaggedGeom{CfgUp::BM, w.m.up.tiles_n, w.m.up.panel_rows,
                        w.plan_up ? (int)(w.m.up.ragged_slots * kNumXcd) : 0,
                        reinterpret_cast<PlanEntry*>(w.plan_up)};
      w.gb = RaggedGeom{w.m.down_bm, w.m.down.tiles_n, w.m.down.panel_rows,
                        w.plan_down ? (int)(w.m.down.ragged_slots * kNumXcd) : 0,
                        reinterpret_cast<PlanEntry*>(w.plan_down)};
      const int n = w.ga.num_blocks > w.gb.num_blocks ? w.ga.num_blocks : w.gb.num_blocks;
      w.plan_blocks = (n + 255) / 256;
    }
  }
  w.rest = ws;
  return w;
}

// `planned`: the launch plans in the workspace have been written (vmoe_compact_rows_planned).
static int run_expert_mlp(const VmoeExpertMlpParams* p, vmoe_stream_t stream_, bool planned_already) {
  int rc = check_mlp(p);
  if (rc != VMOE_OK) return rc;
  const size_t need = vmoe_expert_mlp_workspace_bytes(p);
  if (p->workspace == nullptr || p->workspace_bytes < need || !aligned16(p->workspace))
    return VMOE_E_WORKSPACE;
  hipStream_t stream = as_stream(stream_);
  const size_t b = p->dtype == VMOE_BF16 ? 2 : 4;
  const MlpWorkspace w = mlp_workspace(p);
  void* hidden = w.hidden;
  int4* plan_up = w.plan_up;
  int4* plan_down = w.plan_down;
  void* streamk = w.streamk;
  const MlpPlans& m = w.m;
  unsigned char* ws = w.rest;
  if (planned_already && w.plan_blocks == 0) return VMOE_E_UNSUPPORTED;
  if (w.plan_blocks > 0 && !planned_already)
    hipLaunchKernelGGL(plan_ragged_tiles_kernel, dim3(w.plan_blocks), dim3(256),
                       plan_ragged_tiles_lds(p->E), stream, p->rows_per_expert, p->E, p->R, w.ga, w.gb);
  const bool tanh_gelu = p->gelu == VMOE_GELU_TANH;
  if (p->dtype == VMOE_BF16) {
    const void* w0t = p->w0t;
    const void* w1t = p->w1t;
    if (w0t == nullptr) {
      rc = transpose(p->w0, ws, p->E, p->D, p->M, VMOE_BF16, stream);
      if (rc != VMOE_OK) return rc;
      w0t = ws;
      ws += align256((size_t)p->E * p->D * p->M * b);
    }
    if (w1t == nullptr) {
      rc = transpose(p->w1, ws, p->E, p->M, p->D, VMOE_BF16, stream);
      if (rc != VMOE_OK) return rc;
      w1t = ws;
    }
    // The counters of the second product's stream-K exchange are set to zero by the first
    // product's launch, in every call: a call that finds its plans written
    // (vmoe_expert_mlp_planned) can be repeated on the same workspace.
    using SK = StreamKWorkspace<CfgDownPersistent>;
    int32_t* clear = streamk != nullptr ? SK::flags(streamk) : nullptr;
    int32_t* status = w.status;
    static_assert(std::is_same<CfgUp, GemmCfg<128, 256, 2, 2, 32, 3, 2>>::value,
                  "launch_gemm_bf16_first runs CfgUp's geometry");
    if (tanh_gelu)
      rc = launch_gemm_bf16_first<kEpiBiasGeluTanh>((const bf16_t*)p->x, (const bf16_t*)w0t,
                                                    (const bf16_t*)p->b0, (bf16_t*)hidden, p->E,
                                                    p->R, p->M, p->D, stream, p->rows_per_expert,
                                                    plan_up, p->x_rows, p->num_items, clear, SK::kFlags, status);
    else
      rc = launch_gemm_bf16_first<kEpiBiasGeluErf>((const bf16_t*)p->x, (const bf16_t*)w0t,
                                                   (const bf16_t*)p->b0, (bf16_t*)hidden, p->E,
                                                   p->R, p->M, p->D, stream, p->rows_per_expert,
                                                   plan_up, p->x_rows, p->num_items, clear, SK::kFlags, status);
    if (rc != VMOE_OK) return rc;
    switch (m.down_kernel) {
      case kDownShared:
        return launch_gemm_bf16_persistent<CfgDownPersistent, kEpiBias>(
            (const bf16_t*)hidden, (const bf16_t*)w1t, (const bf16_t*)p->b1, (bf16_t*)p->out, p->E,
            p->R, p->D, p->M, stream, plan_down, streamk, status);
      case kDownEightWaves:
        return launch_gemm_bf16_w8<kEpiBias, 8>((const bf16_t*)hidden, (const bf16_t*)w1t,
                                                (const bf16_t*)p->b1, (bf16_t*)p->out, p->E, p->R,
                                                p->D, p->M, stream, plan_down, nullptr, 0, status);
      case kDownNarrow:
        return launch_gemm_bf16_w8<kEpiBias, 6>((const bf16_t*)hidden, (const bf16_t*)w1t,
                                                 (const bf16_t*)p->b1, (bf16_t*)p->out, p->E, p->R,
                                                 p->D, p->M, stream, plan_down, nullptr, 0, status);
      case kDownWide:
        return launch_gemm_bf16_wide<kEpiBias>((const bf16_t*)hidden, (const bf16_t*)w1t,
                                               (const bf16_t*)p->b1, (bf16_t*)p->out, p->E, p->R,
                                               p->D, p->M, stream, plan_down, nullptr, 0, status);
      case kDownHalf:
        return launch_gemm_bf16<CfgUp, kEpiBias>((const bf16_t*)hidden, (const bf16_t*)w1t,
                                                (const bf16_t*)p->b1, (bf16_t*)p->out, p->E, p->R,
                                                p->D, p->M, stream, nullptr, nullptr);
      default:
        return launch_gemm_bf16<CfgDown, kEpiBias>((const bf16_t*)hidden, (const bf16_t*)w1t,
                                                  (const bf16_t*)p->b1, (bf16_t*)p->out, p->E, p->R,
                                                  p->D, p->M, stream, p->rows_per_expert, plan_down,
                                                  nullptr, 0, nullptr, 0, status);
    }
  }
  if (tanh_gelu)
    rc = launch_gemm_f32<kEpiBiasGeluTanh>((const float*)p->x, (const float*)p->w0,
                                           (const float*)p->b0, (float*)hidden, p->E, p->R, p->M,
                                           p->D, stream, p->rows_per_expert, p->x_rows, p->num_items);
  else
    rc = launch_gemm_f32<kEpiBiasGeluErf>((const float*)p->x, (const float*)p->w0,
                                          (const float*)p->b0, (float*)hidden, p->E, p->R, p->M,
                                          p->D, stream, p->rows_per_expert, p->x_rows, p->num_items);
  if (rc != VMOE_OK) return rc;
  return launch_gemm_f32<kEpiBias>((const float*)hidden, (const float*)p->w1, (const float*)p->b1,
                                   (float*)p->out, p->E, p->R, p->D, p->M, stream,
                                   p->rows_per_expert);
}

extern "C" int vmoe_expert_mlp(const VmoeExpertMlpParams* p, vmoe_stream_t stream) {
  return run_expert_mlp(p, stream, false);
}

extern "C" int vmoe_expert_mlp_planned(const VmoeExpertMlpParams* p, vmoe_stream_t stream) {
  return run_expert_mlp(p, stream, true);
}

extern "C" int vmoe_expert_mlp_status(const VmoeExpertMlpParams* p, const int32_t** status) {
  if (status == nullptr) return VMOE_E_NULL;
  *status = nullptr;
  int rc = check_mlp(p);
  if (rc != VMOE_OK) return rc;
  if (p->dtype != VMOE_BF16) return VMOE_OK;       // the float32 kernels keep no such state
  if (p->workspace == nullptr || p->workspace_bytes < vmoe_expert_mlp_workspace_bytes(p) ||
      !aligned16(p->workspace))
    return VMOE_E_WORKSPACE;
  *status = mlp_workspace(p).status;
  return VMOE_OK;
}

extern "C" int vmoe_compact_rows_planned(const VmoeCompactRowsParams* c,
                                         const VmoeExpertMlpParams* mlp, vmoe_stream_t stream) {
  if (c == nullptr || mlp == nullptr || c->fill == nullptr || c->token_slot == nullptr ||
      c->token_row == nullptr || c->rows_per_expert == nullptr)
    return VMOE_E_NULL;
  if (c->G < 1 || c->S < 1 || c->E < 1 || c->K < 1 || c->C < 1 || c->K > c->E) return VMOE_E_SHAPE;
  if ((int64_t)c->G * c->S * c->K * 2 >= INT32_MAX || (int64_t)c->E * c->G * c->C >= INT32_MAX)
    return VMOE_E_OVERFLOW;
  int rc = check_mlp(mlp);
  if (rc != VMOE_OK) return rc;
  if (mlp->E != c->E || (int64_t)mlp->R != (int64_t)c->G * c->C ||
      mlp->rows_per_expert != c->rows_per_expert)
    return VMOE_E_SHAPE;
  if (mlp->workspace == nullptr || mlp->workspace_bytes < vmoe_expert_mlp_workspace_bytes(mlp) ||
      !aligned16(mlp->workspace))
    return VMOE_E_WORKSPACE;
  // One launch needs the one-launch form of the compaction and an MLP whose products are planned.
  if (!compact_rows_fused_ok(c->G, c->S, c->E, c->K) || mlp->dtype != VMOE_BF16)
    return VMOE_E_UNSUPPORTED;
  const MlpWorkspace w = mlp_workspace(mlp);
  if (w.plan_blocks == 0) return VMOE_E_UNSUPPORTED;
  const size_t n = (size_t)c->G * c->S * c->K;
  const unsigned compact_blocks = (unsigned)((n + 255) / 256);
  hipLaunchKernelGGL(compact_rows_planned_kernel, dim3(compact_blocks + (unsigned)w.plan_blocks),
                     dim3(256), plan_ragged_tiles_lds(c->E), as_stream(stream), c->fill,
                     c->token_slot, c->token_row, c->row_token, c->rows_per_expert, c->G, c->E, c->C,
                     c->S * c->K, c->K, n, compact_blocks, mlp->R, w.ga, w.gb);
  return launch_status();
}

template <typename PCfg>
static int launch_operand_delivery_probe(const void* a, const void* bt, int32_t batch, int32_t rows,
                                         int32_t n, int32_t kd, double* bytes, vmoe_stream_t stream) {
  if (a == nullptr || bt == nullptr || bytes == nullptr) return VMOE_E_NULL;
  if (batch < 1 || rows < 1 || n < 1 || kd < 1) return VMOE_E_SHAPE;
  if (!aligned16(a) || !aligned16(bt)) return VMOE_E_ALIGN;
  const GemmGeom g = gemm_geometry<PCfg>(batch, rows, n, kd);
  if (!g.fast) return VMOE_E_UNSUPPORTED;    // kd not a multiple of the k tile, or an operand beyond 32-bit offsets
  if (g.tiles > 0x7ffffff0LL) return VMOE_E_OVERFLOW;
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(operand_delivery_probe_kernel<PCfg>), PCfg::kLdsBytes);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(operand_delivery_probe_kernel<PCfg>, dim3((unsigned)g.tiles_per_xcd * kNumXcd),
                     dim3(PCfg::kThreads), PCfg::kLdsBytes, as_stream(stream),
                     (const bf16_t*)a, (const bf16_t*)bt, rows, n, kd, g.tiles_m, g.tiles_n,
                     (int)g.tiles, g.tiles_per_xcd, g.panel_rows);
  *bytes = (double)g.tiles * (PCfg::BM + PCfg::BN) * (double)kd * 2.0;
  return launch_status();
}

extern "C" int vmoe_operand_delivery_probe(const void* a, const void* bt, int32_t batch, int32_t rows,
                                           int32_t n, int32_t kd, double* bytes,
                                           vmoe_stream_t stream) {
  return launch_operand_delivery_probe<CfgDown>(a, bt, batch, rows, n, kd, bytes, stream);
}

extern "C" int vmoe_operand_delivery_probe_k64(const void* a, const void* bt, int32_t batch,
                                               int32_t rows, int32_t n, int32_t kd, double* bytes,
                                               vmoe_stream_t stream) {
  return launch_operand_delivery_probe<CfgDownPersistent>(a, bt, batch, rows, n, kd, bytes, stream);
}

// The same requests over tiles that the workgroups share: kNumCu workgroups of 256 threads walk
// `tiles_per_workgroup` tiles each, taken round robin from the `distinct` tiles of 512 rows
// that `buf` holds (with few tiles, many workgroups per tile and hardly a miss), k tile by k
// tile of 64 KB, at most two k tiles in flight.  SEG = 128: a request is 8 rows x 128 bytes;
// SEG = 64: 16 rows x 64 bytes, two requests per row and k tile.  What it moves per time is what
// the request path delivers when latency is that of the caches: the gap to the other delivery probes
// is what misses cost at this ring depth.
template <int SEG>
__global__ __launch_bounds__(256, 1) void resident_delivery_probe_kernel(
    const unsigned char* __restrict__ buf, int distinct, int k_tiles, int tiles_per_workgroup,
    uint32_t row_bytes) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __align__(1024) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int kRowsPerRequest = 1024 / SEG, kLanesPerRow = SEG / 16;
  const uint32_t lane_off = (uint32_t)(lane / kLanesPerRow) * row_bytes + (lane % kLanesPerRow) * 16;
  for (int t = 0; t < tiles_per_workgroup; ++t) {
    const size_t tile = ((size_t)blockIdx.x * tiles_per_workgroup + t) % distinct;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<unsigned char*>(buf + tile * 512 * row_bytes), 0, -1, 0x00020000);
    for (int kt = 0; kt < k_tiles; ++kt) {
      unsigned char* s = smem + (kt & 1) * 65536;
#pragma unroll
      for (int part = 0; part < 128 / SEG; ++part)
#pragma unroll
        for (int i = 0; i < 512 / kRowsPerRequest / 4; ++i) {
          const int request = i * 4 + wave;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              rsrc, (lds_ptr_t)(s + (part * (512 / kRowsPerRequest) + request) * 1024), 16,
              lane_off + (uint32_t)request * kRowsPerRequest * row_bytes, kt * 128 + part * SEG, 0, 0);
        }
      wait_vmcnt<16>();     // the k tile before this one has landed
    }
  }
  wait_vmcnt<0>();
#endif
}

extern "C" int vmoe_resident_delivery_probe(const void* buf, size_t buf_bytes, int32_t row_bytes,
                                            int32_t k_tiles, int32_t tiles_per_workgroup,
                                            int32_t segment_bytes, double* bytes,
                                            vmoe_stream_t stream) {
  if (buf == nullptr || bytes == nullptr) return VMOE_E_NULL;
  if (row_bytes < 128 || k_tiles < 1 || tiles_per_workgroup < 1 || (int64_t)k_tiles * 128 > row_bytes)
    return VMOE_E_SHAPE;
  if (segment_bytes != 64 && segment_bytes != 128) return VMOE_E_SHAPE;
  if (!aligned16(buf) || row_bytes % 16 != 0) return VMOE_E_ALIGN;
  const size_t tile_bytes = (size_t)512 * row_bytes;
  if (tile_bytes >= ((size_t)1 << 32)) return VMOE_E_OVERFLOW;
  const size_t distinct = buf_bytes / tile_bytes;
  if (distinct < 1 || distinct > 0x7fffffff) return VMOE_E_SHAPE;
  constexpr int kLds = 2 * 65536;
  auto launch = [&](auto kern) -> int {
    hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), kLds);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, dim3(kCusPerXcd * kNumXcd), dim3(256), kLds, as_stream(stream),
                       static_cast<const unsigned char*>(buf), (int)distinct, k_tiles,
                       tiles_per_workgroup, (uint32_t)row_bytes);
    return launch_status();
  };
  *bytes = (double)(kCusPerXcd * kNumXcd) * tiles_per_workgroup * k_tiles * 65536.0;
  return segment_bytes == 128 ? launch(resident_delivery_probe_kernel<128>)
                              : launch(resident_delivery_probe_kernel<64>);
}

extern "C" int vmoe_pack_expert_weights(const VmoeTransposeParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->in == nullptr || p->out == nullptr) return VMOE_E_NULL;
  if (p->batch < 1 || p->rows < 1 || p->cols < 1 || p->batch > 65535) return VMOE_E_SHAPE;
  if (p->dtype != VMOE_F32 && p->dtype != VMOE_BF16) return VMOE_E_DTYPE;
  return transpose(p->in, p->out, p->batch, p->rows, p->cols, p->dtype, as_stream(stream));
}

extern "C" int vmoe_mfma_probe(const void* seed, size_t seed_bytes, void* sink, int32_t blocks,
                               int32_t iters, double* flops, vmoe_stream_t stream) {
  if (seed == nullptr || sink == nullptr || flops == nullptr) return VMOE_E_NULL;
  if (seed_bytes < 16 || !aligned16(seed) || blocks < 1 || iters < 1) return VMOE_E_SHAPE;
  hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                     (const uint4*)seed, (float*)sink, iters, seed_bytes / 16);
  // 4 waves x 32 MFMAs of 32 x 32 x 16 per iteration
  *flops = (double)blocks * 4.0 * iters * 32.0 * (2.0 * 32 * 32 * 16);
  return launch_status();
}
