// Batched bf16 GEMM, wide-tile persistent form: eight waves per workgroup (two per SIMD)
// compute a 384 x 256 tile, each wave 96 x 128 of it (3 x 4 MFMA tiles, 192 accumulator
// registers, so that two waves share a SIMD's 512 registers).
//
// Why this shape.  On gfx950 a compute unit's vector-memory path moves operand tiles into
// LDS at a rate that grows with the number of waves issuing the loads (four waves: about
// 24 bytes per clock, eight: 35), while a 256 x 256 tile needs 32 bytes per clock to keep
// the matrix cores fed.  384 x 256 needs 27, and eight waves issue the loads.  With two
// waves per SIMD one wave's LDS waits and DMA issue stalls (a full address FIFO blocks the
// wave's next MFMA too: waves issue in order) are covered by the other wave's MFMAs.
//
// Per wave and 16-wide k slice: the three A fragments are resident (double buffered across
// slices), the four B fragments stream through two registers sets, each read one group
// (three MFMAs) ahead of its use.  Operand path, swizzle and ring as in gemm_bf16.h; the
// ring has three stages and a stage is read from the middle of the k tile before its own
// until the end of its own, so the DMA loads of k tile kt + 2 go out in the second half
// of k tile kt, into the stage of k tile kt - 1.
#ifndef VMOE_GEMM_BF16_WIDE_H_
#define VMOE_GEMM_BF16_WIDE_H_

#include "gemm_bf16.h"

namespace vmoe {

// NSTAGE_ = 3: the output is staged in an LDS region of its own.  NSTAGE_ = 4: the ring takes
// all 160 KB and the output is staged in the ring stage that the tile's last k tile has just
// left (the loads that would refill it only go out half a k tile into the next tile).
template <int NSTAGE_>
struct WideCfgT {
  static constexpr int BM = 384, BN = 256, BK = 32, WM = 4, WN = 2, NSTAGE = NSTAGE_;
  static constexpr int kBlocksPerCu = 1;
  static constexpr int kWaves = WM * WN, kThreads = 64 * kWaves;
  static constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32;
  static constexpr int kRowBytes = BK * 2, kChunksPerRow = BK / 8, kRowsPerLoad = 64 / kChunksPerRow;
  static constexpr int kSwzShift = 2;
  static constexpr int kStageBytes = (BM + BN) * kRowBytes;
  static constexpr int kAIssues = BM / kRowsPerLoad / kWaves, kBIssues = BN / kRowsPerLoad / kWaves;
  static constexpr int kLoads = kAIssues + kBIssues;
  static constexpr int kStageCols = 64;                 // output columns staged at a time
  static constexpr int kOutLd = kStageCols + 8;
  static constexpr size_t kRing = (size_t)NSTAGE * kStageBytes;
  static constexpr size_t kStaging = (size_t)kWaves * 32 * kOutLd * sizeof(bf16_t);
  static constexpr bool kStageInRing = NSTAGE >= 4;
  static constexpr size_t kLdsBytes = kStageInRing ? kRing : kRing + kStaging;
  static_assert(FM == 3 && FN == 4 && kAIssues == 3 && kBIssues == 2, "the k loop is written for this shape");
  static_assert(NSTAGE == 3 || NSTAGE == 4, "ring depth");
  static_assert(kStaging <= (size_t)kStageBytes, "the staged output fits one ring stage");
  static_assert(kLdsBytes <= 160 * 1024, "LDS budget");
};
using WideCfg = WideCfgT<4>;

// GATHER: A is the (items, Kd) matrix and a_rows[b * R + r] names the item in row r of batch
// b (the plan is then required).  Otherwise A is (batch, R, Kd).
template <typename Cfg, int EPI, bool HAS_BIAS, bool GATHER>
__global__ __launch_bounds__(Cfg::kThreads, 1) void gemm_bf16_wide_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bt, const bf16_t* __restrict__ bias,
    bf16_t* __restrict__ C, int R, int N, int Kd, int tiles_m, int tiles_n, int num_tiles,
    int tiles_per_xcd, int panel_rows, PlanRef plan_ref,
    const int32_t* __restrict__ a_rows, int a_items, int32_t* __restrict__ status) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-resource builtins exist in the device pass only
  extern __shared__ __align__(1024) unsigned char smem[];
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
  constexpr int RB = Cfg::kRowBytes, NS = Cfg::NSTAGE, L = Cfg::kLoads, STAGE = Cfg::kStageBytes;
  constexpr int CPR = Cfg::kChunksPerRow, RPL = Cfg::kRowsPerLoad;
  const int tid = threadIdx.x;
  const int4* plan = plan_ref.entries;
  const int plan_blocks = plan_ref.blocks;
  // (a plan whose header does not carry this launch's tag: nothing runs, the status words say so)
  if (plan != nullptr && plan[plan_blocks].y != plan_ref.tag) {
    if (blockIdx.x == 0 && tid == 0 && status != nullptr) atomicAdd(status + kStatusPlanMismatches, 1);
    return;
  }
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int m = lane & 31, h = lane >> 5;
  const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
  const int lrow = lane / CPR;
  const int chunk = (lane % CPR) ^ (((wave * RPL + lrow) >> Cfg::kSwzShift) & (CPR - 1));

  struct TileCtx {
    int b, row0, col0, live;
    uint32_t a[Cfg::kAIssues], bo[Cfg::kBIssues];
  };
  auto setup_tile = [&](int i, TileCtx& t) -> bool {
    const int s_ = slot + i * kCusPerXcd;
    int tile_m, tile_n;
    if (plan != nullptr) {
      const int vblock = s_ * kNumXcd + xcd;
      if (vblock >= plan_blocks) return false;
      const int4 mine = plan[vblock];
      if (mine.x < 0) return false;      // a die's run is dense from slot 0: nothing follows
      t.b = mine.x;
      tile_m = mine.y;
      tile_n = mine.z;
      t.live = mine.w;
    } else {
      const int logical = xcd * tiles_per_xcd + s_;
      if (s_ >= tiles_per_xcd || logical >= num_tiles) return false;
      const int per_batch = tiles_m * tiles_n;
      t.b = logical / per_batch;
      const int rem = logical - t.b * per_batch;
      const int panel = rem / (panel_rows * tiles_n);
      const int in_panel = rem - panel * panel_rows * tiles_n;
      const int rows_here = min(panel_rows, tiles_m - panel * panel_rows);
      tile_n = in_panel / rows_here;
      tile_m = panel * panel_rows + in_panel - tile_n * rows_here;
      t.live = R;
    }
    t.row0 = tile_m * BM;
    t.col0 = tile_n * BN;
#pragma unroll
    for (int u = 0; u < Cfg::kAIssues; ++u) {
      const int r = (u * Cfg::kWaves + wave) * RPL + lrow;
      int arow = t.b * R + min(t.row0 + r, (GATHER ? t.live : R) - 1);
      if (GATHER) {
        arow = a_rows[arow];
        arow = (unsigned)arow < (unsigned)a_items ? arow : 0;
      }
      t.a[u] = (uint32_t)arow * (uint32_t)Kd * 2u + chunk * 16;
    }
#pragma unroll
    for (int u = 0; u < Cfg::kBIssues; ++u) {
      const int r = (u * Cfg::kWaves + wave) * RPL + lrow;
      t.bo[u] = (uint32_t)(t.b * N + min(t.col0 + r, N - 1)) * (uint32_t)Kd * 2u + chunk * 16;
    }
    return true;
  };
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(A), 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(Bt), 0, -1, 0x00020000);
  // DMA load u (0..2: A rows, 3..4: B rows) of a k tile into ring stage `stage`.
#define VMOE_WIDE_DMA(T, STG, K0, U) do { \
    if constexpr ((U) < Cfg::kAIssues) \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, \
          (lds_ptr_t)(smem + (STG) * STAGE + ((U) * Cfg::kWaves + wave) * RPL * RB), 16, (T).a[(U)], (K0) * 2, 0, 0); \
    else \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, \
          (lds_ptr_t)(smem + (STG) * STAGE + BM * RB + (((U) - Cfg::kAIssues) * Cfg::kWaves + wave) * RPL * RB), 16, \
          (T).bo[(U) - Cfg::kAIssues], (K0) * 2, 0, 0); \
  } while (0)

  floatx16 acc[3][4];
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  bf16x8 fa[2][3], fb[2];
  const int swz = (m >> Cfg::kSwzShift) & (CPR - 1);
  const int a_lane = (wm * Cfg::TM + m) * RB;
  const int b_lane = BM * RB + (wn * Cfg::TN + m) * RB;
  const int koff0 = ((0 + h) ^ swz) * 16, koff1 = ((2 + h) ^ swz) * 16;
  auto rdA = [&](int stage, int i, int ks) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
        smem + stage * STAGE + a_lane + i * 32 * RB + (ks ? koff1 : koff0)));
  };
  auto rdB = [&](int stage, int j, int ks) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
        smem + stage * STAGE + b_lane + j * 32 * RB + (ks ? koff1 : koff0)));
  };
#define VMOE_WIDE_MFMA3(FB, BUF, J) do { \
    acc[0][J] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(FB, fa[BUF][0], acc[0][J], 0, 0, 0); \
    acc[1][J] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(FB, fa[BUF][1], acc[1][J], 0, 0, 0); \
    acc[2][J] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(FB, fa[BUF][2], acc[2][J], 0, 0, 0); \
    __builtin_amdgcn_sched_barrier(0); \
  } while (0)
  // One k tile.  On entry fa[0][*] and fb[0] hold the first slice's A fragments and first B
  // fragment of the tile in ring stage `stage`; on exit they hold those of the next k tile.
  // SRC / K0: the k tile requested in the second half (NS - 1 k tiles ahead), into the stage
  // of the k tile before this one.
#define VMOE_WIDE_K_TILE(SRC, K0) do { \
    const int s1 = stage + 1 == NS ? 0 : stage + 1; \
    const int sp = stage == 0 ? NS - 1 : stage - 1; \
    fb[1] = rdB(stage, 1, 0); fa[1][0] = rdA(stage, 0, 1); VMOE_WIDE_MFMA3(fb[0], 0, 0); \
    fb[0] = rdB(stage, 2, 0); fa[1][1] = rdA(stage, 1, 1); VMOE_WIDE_MFMA3(fb[1], 0, 1); \
    fb[1] = rdB(stage, 3, 0); fa[1][2] = rdA(stage, 2, 1); VMOE_WIDE_MFMA3(fb[0], 0, 2); \
    fb[0] = rdB(stage, 0, 1);                              VMOE_WIDE_MFMA3(fb[1], 0, 3); \
    wait_vmcnt<(NS - 3) * L>();   /* this wave's part of the next k tile has landed */ \
    raw_barrier();     /* ... and everyone's; nobody reads the k tile before this one any more */ \
    fb[1] = rdB(stage, 1, 1); fa[0][0] = rdA(s1, 0, 0); \
    VMOE_WIDE_DMA(SRC, sp, K0, 0); VMOE_WIDE_DMA(SRC, sp, K0, 1); VMOE_WIDE_MFMA3(fb[0], 1, 0); \
    fb[0] = rdB(stage, 2, 1); fa[0][1] = rdA(s1, 1, 0); \
    VMOE_WIDE_DMA(SRC, sp, K0, 2);                                VMOE_WIDE_MFMA3(fb[1], 1, 1); \
    fb[1] = rdB(stage, 3, 1); fa[0][2] = rdA(s1, 2, 0); \
    VMOE_WIDE_DMA(SRC, sp, K0, 3);                                VMOE_WIDE_MFMA3(fb[0], 1, 2); \
    fb[0] = rdB(s1, 0, 0); \
    VMOE_WIDE_DMA(SRC, sp, K0, 4);                                VMOE_WIDE_MFMA3(fb[1], 1, 3); \
    stage = s1; \
  } while (0)

  const int nk = Kd / BK;      // at least NS
  TileCtx cur, nxt;
  if (!setup_tile(0, cur)) return;
  VMOE_WIDE_DMA(cur, 0, 0, 0); VMOE_WIDE_DMA(cur, 0, 0, 1); VMOE_WIDE_DMA(cur, 0, 0, 2);
  VMOE_WIDE_DMA(cur, 0, 0, 3); VMOE_WIDE_DMA(cur, 0, 0, 4);
  VMOE_WIDE_DMA(cur, 1, BK, 0); VMOE_WIDE_DMA(cur, 1, BK, 1); VMOE_WIDE_DMA(cur, 1, BK, 2);
  VMOE_WIDE_DMA(cur, 1, BK, 3); VMOE_WIDE_DMA(cur, 1, BK, 4);
  if constexpr (NS == 4) {
    VMOE_WIDE_DMA(cur, 2, 2 * BK, 0); VMOE_WIDE_DMA(cur, 2, 2 * BK, 1); VMOE_WIDE_DMA(cur, 2, 2 * BK, 2);
    VMOE_WIDE_DMA(cur, 2, 2 * BK, 3); VMOE_WIDE_DMA(cur, 2, 2 * BK, 4);
  }
  wait_vmcnt<(NS - 2) * L>();
  raw_barrier();
  fa[0][0] = rdA(0, 0, 0); fa[0][1] = rdA(0, 1, 0); fa[0][2] = rdA(0, 2, 0); fb[0] = rdB(0, 0, 0);
  int stage = 0;
  constexpr int OLD = Cfg::kOutLd, SC = Cfg::kStageCols;
  for (int ti = 0;; ++ti) {
    const bool has_next = setup_tile(ti + 1, nxt);
    if (!has_next) nxt = cur;   // the last tile requests its own first k tiles again: in bounds, never read
    for (int kt = 0; kt < nk - (NS - 1); ++kt) VMOE_WIDE_K_TILE(cur, (kt + NS - 1) * BK);
    VMOE_WIDE_K_TILE(nxt, 0);
    VMOE_WIDE_K_TILE(nxt, BK);
    if constexpr (NS == 4) VMOE_WIDE_K_TILE(nxt, 2 * BK);
    // No load that writes LDS is pending while the output is staged.
    wait_vmcnt<0>();
    bf16_t* so;
    if constexpr (Cfg::kStageInRing) {
      // The stage of the tile's last k tile: every wave has taken its last fragments out of
      // it once all have arrived here; it is refilled only behind the next k tile's barrier.
      raw_barrier();
      const int last = stage == 0 ? NS - 1 : stage - 1;
      so = reinterpret_cast<bf16_t*>(smem + last * STAGE) + (size_t)wave * 32 * OLD;
    } else {
      so = reinterpret_cast<bf16_t*>(smem + Cfg::kRing) + (size_t)wave * 32 * OLD;
    }
    mfma_result_fence();
    bf16_t* Cb = C + (size_t)cur.b * R * N;
    const int wrow0 = cur.row0 + wm * Cfg::TM, wcol0 = cur.col0 + wn * Cfg::TN;
    constexpr int kChunksOut = SC / 8;                  // 8 lanes cover a staged row
    constexpr int kRowsPerPass = 64 / kChunksOut;
    const int oc = (lane % kChunksOut) * 8;
    const int orow = lane / kChunksOut;
#pragma unroll
    for (int i = 0; i < 3; ++i) {
#pragma unroll
      for (int c0 = 0; c0 < Cfg::TN; c0 += SC) {
        uint2 bias_pk[SC / 8];
#pragma unroll
        for (int jq = 0; jq < SC / 8; ++jq) {
          bias_pk[jq] = make_uint2(0, 0);
          if (HAS_BIAS) {
            const int col = wcol0 + c0 + jq * 8 + h * 4;
            bias_pk[jq] = *reinterpret_cast<const uint2*>(bias + (size_t)cur.b * N + min(col, N - 4));
          }
        }
#pragma unroll
        for (int j = c0 / 32; j < (c0 + SC) / 32; ++j) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int cl = j * 32 - c0 + q * 8 + h * 4;
            const uint2 bp = bias_pk[(j * 32 - c0) / 8 + q];
            const float bv[4] = {bf_lo(bp.x), bf_hi(bp.x), bf_lo(bp.y), bf_hi(bp.y)};
            const uint32_t p0 = epilogue_pair<EPI, HAS_BIAS>(acc[i][j][q * 4], acc[i][j][q * 4 + 1], bv[0], bv[1]);
            const uint32_t p1 = epilogue_pair<EPI, HAS_BIAS>(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3], bv[2], bv[3]);
            *reinterpret_cast<uint2*>(so + m * OLD + cl) = make_uint2(p0, p1);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[i][j][q * 4 + v] = 0.f;
          }
        }
        // A wave reads back only what it wrote (its LDS operations complete in order).
#pragma unroll
        for (int r0 = 0; r0 < 32; r0 += kRowsPerPass) {
          const int rl = r0 + orow;
          const int row = wrow0 + i * 32 + rl;
          const int col = wcol0 + c0 + oc;
          const uint4 v = *reinterpret_cast<const uint4*>(so + rl * OLD + oc);
          if (row < cur.live && col + 8 <= N) {
            if constexpr (EPI != kEpiBias) {   // hidden layer: streaming store
              typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
              __builtin_nontemporal_store(__builtin_bit_cast(u32x4_t, v),
                                          reinterpret_cast<u32x4_t*>(Cb + (size_t)row * N + col));
            } else {
              *reinterpret_cast<uint4*>(Cb + (size_t)row * N + col) = v;
            }
          }
        }
      }
    }
    if (!has_next) break;
    cur = nxt;
  }
  wait_vmcnt<0>();
#undef VMOE_WIDE_K_TILE
#undef VMOE_WIDE_MFMA3
#undef VMOE_WIDE_DMA
#endif
}

// Whether the wide kernel covers the product (N % 8 == 0 and N >= 4 for the packed bias
// loads, at least four k tiles, operands addressable with 32-bit byte offsets).
inline bool wide_gemm_ok(int batch, int R, int N, int Kd, const int32_t* rows, const int4* plan,
                         const int32_t* a_rows, long long a_items) {
  const GemmGeom g = gemm_geometry<WideCfg>(batch, R, N, Kd);
  const uint64_t lim = 1ull << 32;
  const uint64_t a_bytes = a_rows != nullptr ? (uint64_t)a_items * Kd * 2 : (uint64_t)batch * R * Kd * 2;
  return g.fast && Kd / WideCfg::BK >= 4 && (N & 7) == 0 && a_bytes < lim &&
         (uint64_t)batch * N * Kd * 2 < lim && g.tiles <= 0x7ffffff0LL &&
         (rows == nullptr || plan != nullptr) && (a_rows == nullptr || plan != nullptr);
}

template <int EPI, typename Cfg = WideCfg>
int launch_gemm_bf16_wide(const bf16_t* A, const bf16_t* Bt, const bf16_t* bias, bf16_t* C, int batch,
                          int R, int N, int Kd, hipStream_t stream, const int4* plan = nullptr,
                          const int32_t* a_rows = nullptr, long long a_items = 0,
                          int32_t* status = nullptr) {
  const GemmGeom g = gemm_geometry<Cfg>(batch, R, N, Kd);
  void (*kern)(const bf16_t*, const bf16_t*, const bf16_t*, bf16_t*, int, int, int, int, int, int, int,
               int, PlanRef, const int32_t*, int, int32_t*);
  if (a_rows != nullptr)
    kern = bias != nullptr ? gemm_bf16_wide_kernel<Cfg, EPI, true, true> : gemm_bf16_wide_kernel<Cfg, EPI, false, true>;
  else
    kern = bias != nullptr ? gemm_bf16_wide_kernel<Cfg, EPI, true, false> : gemm_bf16_wide_kernel<Cfg, EPI, false, false>;
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::kLdsBytes);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3(kCusPerXcd * kNumXcd), dim3(Cfg::kThreads), Cfg::kLdsBytes,
                     stream, A, Bt, bias, C, R, N, Kd, g.tiles_m, g.tiles_n, (int)g.tiles,
                     g.tiles_per_xcd, g.panel_rows, plan_ref<Cfg>(g, plan, batch, R), a_rows,
                     (int)a_items, status);
  return launch_status();
}

}  // namespace vmoe
#endif  // VMOE_GEMM_BF16_WIDE_H_
