// float32 expert products (vmoe/nn/vit_moe.py:38-45 on float32 parameters) on
// v_mfma_f32_32x32x2_f32, operands delivered by LDS-DMA.
//
// C[b] = epilogue(A[b] (R x Kd) . B[b] (Kd x N) + bias[b]); B in the reference's (in, out)
// order, so a lane's B operand is one scalar B[k][n] and nothing is transposed.
//
// The matrix cores' operand appetite is small here (a 32x32x2 MFMA takes 64 clocks for one A and
// one B scalar per lane, and a register-resident loop of them runs at 0.99 of the float32 matrix
// peak), so the design is about the traffic between L2 and the CUs and about how few, long
// tiles fall on 256 CUs:
//   * a 64 x 64 tile fetches 512 bytes per 8 192 flops, 9.8 TB/s at the float32 matrix peak; the
//     first product therefore takes 64 x 128 tiles where those still outnumber the CUs twice;
//   * the tile list is cut into eight contiguous runs, one per XCD (a workgroup's XCD is its
//     index modulo 8), batch-major and column-panel-major inside a run: with eight experts each
//     die multiplies one expert, and the tiles of a run walk k in step, so that a k slice of
//     the operands is fetched into the die's L2 once for all of them;
//   * rows beyond a ragged batch's count cost nothing: a wave skips the 32-row blocks that
//     hold none, so a tile's time follows its live blocks.
// With requests, fragment reads and barriers taken out the launches of the S/32 layer last
// nearly as long as with them: what is left between them and the peak is the 3.4 or 1.75 tiles
// per CU, and that the workgroups that share a CU, taking turns MFMA by MFMA, also reach their
// prologues and epilogues together.
// Loop: k tiles of 32 in a ring of three LDS stages, requested two iterations before their
// fragments are read, one barrier per k tile.  A rows are stored with their
// 16-byte pieces XOR-swizzled by (row / 2) % 8, B rows 16..31 with their column halves
// exchanged: both fragment reads are then free of bank conflicts.  The k values of a k tile are
// dealt to the sixteen MFMAs as {s, 16 + s} (the products of a k tile commute), so a lane's A
// operands are 64 contiguous bytes (four 16-byte LDS reads).
#pragma once
#include "gemm_bf16.h"

namespace vmoe {

typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <int BN_>
struct F32Cfg {
  static constexpr int BM = 64, BN = BN_, BK = 32, kWaves = 4, kThreads = 256, kStages = 3;
  static constexpr int WN = BN / 32 >= 4 ? 4 : BN / 32;   // waves side by side
  static constexpr int WM = kWaves / WN;                  // waves on top of each other
  static constexpr int FM = BM / WM / 32;                 // 32-row blocks per wave
  static constexpr int kABytes = BM * BK * 4, kBBytes = BK * BN * 4;
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kAIssues = kABytes / 1024 / kWaves, kBIssues = kBBytes / 1024 / kWaves;
  static constexpr int kIssues = kAIssues + kBIssues;
  static constexpr int kLds = kStages * kStageBytes;
  static constexpr int kBChunksPerRow = BN / 4, kBRowsPerIssue = 64 / kBChunksPerRow;
  static_assert(WN * 32 == BN && WM * FM * 32 == BM, "wave tiles");
};

template <int EPI, int BN_>
__global__ __launch_bounds__(256) void gemm_f32_dma_kernel(
    const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ bias,
    float* __restrict__ C, int batch, int R, int N, int Kd, int tiles_m, int tiles_n, int per_xcd,
    const int32_t* __restrict__ rows, const int32_t* __restrict__ a_rows, int a_items) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-resource builtins exist in the device pass only
  using Cfg = F32Cfg<BN_>;
  extern __shared__ __align__(1024) unsigned char smem[];
  const int slot = blockIdx.x >> 3;
  const int per_batch = tiles_m * tiles_n;
  const int id = (blockIdx.x & 7) * per_xcd + slot;
  if (slot >= per_xcd || id >= batch * per_batch) return;
  const int b = id / per_batch;
  const int rem = id - b * per_batch;
  const int tile_n = rem / tiles_m, tile_m = rem - tile_n * tiles_m;
  const int row0 = tile_m * Cfg::BM, col0 = tile_n * Cfg::BN;
  int live = R;
  if (rows != nullptr) live = min(rows[b], R);
  if (row0 >= live) return;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / Cfg::WN, wn = wave - wm * Cfg::WN;
  const int m = lane & 31, h = lane >> 5;

  // Requests.  One wave-wide request fills 1 KB of LDS in lane order, 16 bytes per lane: eight
  // A rows (128 bytes of k each) or 64 / (BN / 4) B rows (BN floats each).
  uint32_t a_goff[Cfg::kAIssues], b_goff[Cfg::kBIssues];
  {
    const int lrow = lane >> 3, pos = lane & 7;
#pragma unroll
    for (int i = 0; i < Cfg::kAIssues; ++i) {
      const int r = (i * Cfg::kWaves + wave) * 8 + lrow;
      const int piece = pos ^ ((r >> 1) & 7);
      // a_rows: A is the matrix of items (a_items x Kd) and a_rows[b][row] names the item of a
      // row (rows past the count hold no index: they read the last live row's item)
      int arow = min(row0 + r, (a_rows != nullptr ? live : R) - 1);
      if (a_rows != nullptr) {
        arow = a_rows[(size_t)b * R + arow];
        arow = (unsigned)arow < (unsigned)a_items ? arow : 0;
      }
      a_goff[i] = (uint32_t)arow * (uint32_t)Kd * 4u + piece * 16;
    }
  }
  {
    const int lrow = lane / Cfg::kBChunksPerRow, pos = lane % Cfg::kBChunksPerRow;
#pragma unroll
    for (int i = 0; i < Cfg::kBIssues; ++i) {
      const int k = (i * Cfg::kWaves + wave) * Cfg::kBRowsPerIssue + lrow;
      const int piece = pos ^ ((k & 16) >> 1);
      b_goff[i] = (uint32_t)k * (uint32_t)N * 4u + (uint32_t)(col0 * 4 + piece * 16);
    }
  }
  // Reads past the end of a batch's operand return zero (the last column tile of the last k
  // row reaches there when N is not a multiple of the tile).
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(a_rows != nullptr ? A : A + (size_t)b * R * Kd), 0,
      (int)((uint32_t)(a_rows != nullptr ? a_items : R) * (uint32_t)Kd * 4u), 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(B + (size_t)b * Kd * N), 0, (int)((uint32_t)Kd * (uint32_t)N * 4u), 0x00020000);
  auto request = [&](int stage, int kt) {
    unsigned char* s = smem + stage * Cfg::kStageBytes;
#pragma unroll
    for (int i = 0; i < Cfg::kAIssues; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(s + (i * Cfg::kWaves + wave) * 1024),
                                               16, a_goff[i], kt * (Cfg::BK * 4), 0, 0);
#pragma unroll
    for (int i = 0; i < Cfg::kBIssues; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          b_rsrc, (lds_ptr_t)(s + Cfg::kABytes + (i * Cfg::kWaves + wave) * 1024), 16, b_goff[i],
          kt * (Cfg::BK * 4) * N, 0, 0);
  };

  bool block_live[Cfg::FM];
#pragma unroll
  for (int i = 0; i < Cfg::FM; ++i) block_live[i] = row0 + (wm * Cfg::FM + i) * 32 < live;
  // the bias is fetched ahead of the loop: its latency would otherwise open the epilogue
  const int col = col0 + wn * 32 + m;
  const bool col_ok = col < N;
  const float bv = (bias != nullptr && col_ok) ? bias[(size_t)b * N + col] : 0.f;
  floatx16 acc[Cfg::FM];
#pragma unroll
  for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

  // Fragment addresses inside a stage.  The fragment reads are written as instructions: a
  // read that the compiler can see waits for every request in flight, the ones just issued
  // for two k tiles ahead included.
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>((lds_ptr_t)smem);
  uint32_t a_off[Cfg::FM];
#pragma unroll
  for (int i = 0; i < Cfg::FM; ++i) a_off[i] = lds0 + ((wm * Cfg::FM + i) * 32 + m) * 128;
  const int a_swz = (m >> 1) & 7;    // (row / 2) % 8: the block's first row is a multiple of 32
  uint32_t a_piece[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) a_piece[c] = ((h * 4 + c) ^ a_swz) * 16;
  const uint32_t b_off = lds0 + Cfg::kABytes + h * 16 * (Cfg::BN * 4) + ((wn * 32 + m) ^ (h * 32)) * 4;

  // The fragments of k tile t + 1 are read while the MFMAs of k tile t run (two register sets):
  // two waves that share a SIMD take turns MFMA by MFMA and so reach their fragment reads
  // together; with the reads one k tile ahead neither wait is exposed.  Iteration t: the
  // wave's fragments of t have arrived; its requests of t + 1 have landed; barrier (every
  // wave's requests of t + 1 have landed, every wave has read stage t % 3); requests of t + 3
  // into stage t % 3; fragment reads of t + 1; MFMAs of t.
  float bf[2][16];
  f32x4_t af[2][Cfg::FM][4];
  const int nk = Kd / Cfg::BK;
  auto read_frags = [&](const int u, int stage) {
    const uint32_t s = stage * Cfg::kStageBytes;
#pragma unroll
    for (int q = 0; q < 16; ++q)
      asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(bf[u][q]) : "v"(s + b_off), "n"(q * (Cfg::BN * 4)));
#pragma unroll
    for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c)
        asm volatile("ds_read_b128 %0, %1" : "=v"(af[u][i][c]) : "v"(s + a_off[i] + a_piece[c]));
  };
  auto step = [&](const int u, int kt, int stage) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(bf[u][0]), "+v"(bf[u][1]), "+v"(bf[u][2]), "+v"(bf[u][3]), "+v"(bf[u][4]),
                   "+v"(bf[u][5]), "+v"(bf[u][6]), "+v"(bf[u][7]), "+v"(bf[u][8]), "+v"(bf[u][9]),
                   "+v"(bf[u][10]), "+v"(bf[u][11]), "+v"(bf[u][12]), "+v"(bf[u][13]),
                   "+v"(bf[u][14]), "+v"(bf[u][15]));
#pragma unroll
    for (int i = 0; i < Cfg::FM; ++i)
      asm volatile("" : "+v"(af[u][i][0]), "+v"(af[u][i][1]), "+v"(af[u][i][2]), "+v"(af[u][i][3]));
    if (kt + 1 < nk) {
      if (kt + 2 < nk) wait_vmcnt<Cfg::kIssues>(); else wait_vmcnt<0>();
      raw_barrier();
      if (kt + 3 < nk) request(stage, kt + 3);
      read_frags(1 - u, stage == 2 ? 0 : stage + 1);
    }
#pragma unroll
    for (int i = 0; i < Cfg::FM; ++i) {
      if (!block_live[i]) continue;
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[u][i][c][t], bf[u][c * 4 + t], acc[i], 0, 0, 0);
    }
  };
  request(0, 0);
  if (nk > 1) request(1, 1);
  if (nk > 2) request(2, 2);
  if (nk > 2) wait_vmcnt<2 * Cfg::kIssues>(); else if (nk > 1) wait_vmcnt<Cfg::kIssues>(); else wait_vmcnt<0>();
  raw_barrier();
  read_frags(0, 0);
  int stage = 0;
  for (int kt = 0; kt < nk; kt += 2) {
    step(0, kt, stage);
    stage = stage == 2 ? 0 : stage + 1;
    if (kt + 1 < nk) {
      step(1, kt + 1, stage);
      stage = stage == 2 ? 0 : stage + 1;
    }
  }
  mfma_result_fence();

  float* Cb = C + (size_t)b * R * N;
#pragma unroll
  for (int i = 0; i < Cfg::FM; ++i) {
    if (!block_live[i]) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = row0 + (wm * Cfg::FM + i) * 32 + (v >> 2) * 8 + h * 4 + (v & 3);
      float o = acc[i][v] + bv;
      if (EPI == kEpiBiasGeluTanh) o = gelu_tanh_fast(o);   // hardware exp2 and reciprocal: ~1e-7 relative
      if (EPI == kEpiBiasGeluErf) o = gelu_erf(o);
      if (row < live && col_ok) Cb[(size_t)row * N + col] = o;
    }
  }
#endif
}

// Shapes the DMA kernel takes: whole 32-wide k tiles, operand rows that are whole 16-byte
// pieces at 16-byte aligned addresses, a batch's operands within reach of 32-bit offsets.
// (a_items: rows of the matrix of items when the rows are gathered, else 0)
inline bool gemm_f32_dma_ok(const float* A, const float* B, int R, int N, int Kd, int a_items = 0) {
  return Kd % 32 == 0 && N % 4 == 0 && R > 0 && (reinterpret_cast<uintptr_t>(A) & 15u) == 0 &&
         (reinterpret_cast<uintptr_t>(B) & 15u) == 0 &&
         (int64_t)(a_items > R ? a_items : R) * Kd * 4 < ((int64_t)1 << 31) &&
         (int64_t)Kd * N * 4 < ((int64_t)1 << 31);
}

template <int EPI, int BN_>
int launch_gemm_f32_dma(const float* A, const float* B, const float* bias, float* C, int batch,
                        int R, int N, int Kd, hipStream_t stream, const int32_t* rows,
                        const int32_t* a_rows = nullptr, int a_items = 0) {
  using Cfg = F32Cfg<BN_>;
  const int tiles_m = (R + Cfg::BM - 1) / Cfg::BM, tiles_n = (N + Cfg::BN - 1) / Cfg::BN;
  const long long total = (long long)batch * tiles_m * tiles_n;
  if (total > 0x0fffffffLL) return VMOE_E_OVERFLOW;
  const int per_xcd = (int)((total + 7) / 8);
  auto kern = gemm_f32_dma_kernel<EPI, BN_>;
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::kLds);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3((unsigned)per_xcd * 8), dim3(Cfg::kThreads), Cfg::kLds, stream, A, B,
                     bias, C, batch, R, N, Kd, tiles_m, tiles_n, per_xcd, rows, a_rows, a_items);
  return launch_status();
}

}  // namespace vmoe
