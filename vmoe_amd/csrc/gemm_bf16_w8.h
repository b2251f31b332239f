// Batched bf16 GEMM, 256 x 256 tiles on eight waves: two waves per SIMD, each wave 64 x 128
// of the tile (2 x 4 MFMA tiles, 128 accumulator registers, so that two waves share a SIMD's
// 512 registers), 64-wide k tiles, one workgroup per compute unit walking a list of tiles.
//
// Why eight waves.  With one wave per SIMD (gemm_bf16_persistent_kernel) whatever makes that
// wave wait -- the fragments of its next slice, the tile's barrier, a DMA request that the
// address unit does not take at once -- leaves the SIMD's matrix core idle.  With two waves
// per SIMD the other wave's MFMAs fill those gaps and the epilogue is half as long per wave.
// The price: every B row is read from LDS by four waves instead of two (fragment traffic
// x 1.5).  Measured on the second product of the B/16 layer: 3 % fewer clocks per launch than
// the four-wave kernel, at a clock that the power management sets 2 % lower (the chip runs
// these products at its power limit, so clocks saved come back only in part): 12 - 14 us of
// 410 per launch.  The tiles of a die's last, partial round run whole here (no stream-K).
//
// Operand path, swizzle and ring are those of gemm_bf16_persistent_kernel: A rows in a ring
// of three 32 KB slots, B rows in one of two (all of the 160 KB), the requests of a k tile
// spread over the four slices of two iterations, never drained inside a tile, the ring kept
// full across tile boundaries.  The output leaves without LDS: the two half waves exchange
// packed pairs (v_permlane32_swap) so that a lane holds eight consecutive columns of one
// row, and stores them as 16 bytes.
#ifndef VMOE_GEMM_BF16_W8_H_
#define VMOE_GEMM_BF16_W8_H_

#include "gemm_bf16.h"

namespace vmoe {

struct W8Cfg {
  static constexpr int BM = 256, BN = 256, BK = 64;
  static constexpr int kWaves = 8, kThreads = 512, kBlocksPerCu = 1;
  static constexpr int TM = 64, TN = 128, FM = 2, FN = 4;      // wave tile, MFMA tiles per wave
  static constexpr int RB = BK * 2;                              // bytes of one row of a k tile
  static constexpr int kABytes = BM * RB, kBBytes = BN * RB;     // one slot: 32 KB
  static constexpr int kLdsBytes = 3 * kABytes + 2 * kBBytes;    // 160 KB
  static constexpr int kIssues = BM / 8 / kWaves;                // DMA requests per wave, operand and k tile: 4
  static_assert(kLdsBytes <= 160 * 1024, "LDS budget");
};

// A is (batch, R, Kd).  `clear` / `status`: begin_call.
template <int EPI, bool HAS_BIAS>
__global__ __launch_bounds__(W8Cfg::kThreads, 1) void gemm_bf16_w8_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bt, const bf16_t* __restrict__ bias,
    bf16_t* __restrict__ C, int R, int N, int Kd, int tiles_m, int tiles_n, int num_tiles,
    int tiles_per_xcd, int panel_rows, PlanRef plan_ref, int32_t* __restrict__ clear,
    int clear_count, int32_t* __restrict__ status, int active_xcds, int active_slots) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-resource builtins exist in the device pass only
  extern __shared__ __align__(1024) unsigned char smem[];
  using Cfg = W8Cfg;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, RB = Cfg::RB;
  constexpr int FM = Cfg::FM, FN = Cfg::FN;
  constexpr int kABytes = Cfg::kABytes, kBBytes = Cfg::kBBytes;
  const int tid = threadIdx.x;
  const int4* plan = plan_ref.entries;
  const int plan_blocks = plan_ref.blocks;
  if (blockIdx.x == 0) begin_call(clear, clear_count, status, tid, Cfg::kThreads);
  if (plan != nullptr && plan[plan_blocks].y != plan_ref.tag) {
    if (blockIdx.x == 0 && tid == 0 && status != nullptr) atomicAdd(status + kStatusPlanMismatches, 1);
    return;
  }
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int m = lane & 31, h = lane >> 5;
  const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
  if (xcd >= active_xcds || slot >= active_slots) return;   // (measurement only, see active_units)
  // A request fills 8 rows x 128 bytes; lane L lands in LDS position L of the request and
  // fetches the 16-byte piece that the XOR swizzle of its row puts there.
  const int lrow = lane >> 3;
  const int piece = (lane & 7) ^ (((wave * 8 + lrow) >> 1) & 7);

  const int nk = Kd / BK;      // at least 4
  int die_tiles;
  if (plan != nullptr) {
    const int total = plan[plan_blocks].x;               // live row tiles of all batches
    const int share = (total + kNumXcd - 1) / kNumXcd;
    die_tiles = max(0, min(xcd * share + share, total) - xcd * share) * tiles_n;
  } else {
    die_tiles = max(0, min(tiles_per_xcd, num_tiles - xcd * tiles_per_xcd));
  }
  die_tiles = __builtin_amdgcn_readfirstlane(die_tiles);
  const int num_items = (die_tiles - slot + kCusPerXcd - 1) / kCusPerXcd;   // tiles slot, slot + 32, ...

  struct TileCtx {
    int b, row0, col0, live;
    uint32_t a[Cfg::kIssues], bo[Cfg::kIssues];
  };
  auto setup_tile = [&](int i, TileCtx& t) -> bool {
    if (i >= num_items) return false;
    const int s_ = slot + i * kCusPerXcd;
    int tile_m, tile_n;
    if (plan != nullptr) {
      const int vblock = s_ * kNumXcd + xcd;
      if (vblock >= plan_blocks) return false;
      const int4 mine = plan[vblock];
      if (mine.x < 0) return false;
      t.b = mine.x;
      tile_m = mine.y;
      tile_n = mine.z;
      t.live = mine.w;
    } else {
      const int logical = xcd * tiles_per_xcd + s_;
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
    t.b = __builtin_amdgcn_readfirstlane(t.b);
    t.live = __builtin_amdgcn_readfirstlane(t.live);
    t.row0 = __builtin_amdgcn_readfirstlane(tile_m * BM);
    t.col0 = __builtin_amdgcn_readfirstlane(tile_n * BN);
#pragma unroll
    for (int u = 0; u < Cfg::kIssues; ++u) {
      const int r = (u * Cfg::kWaves + wave) * 8 + lrow;
      t.a[u] = (uint32_t)(t.b * R + min(t.row0 + r, R - 1)) * (uint32_t)Kd * 2u + piece * 16;
      t.bo[u] = (uint32_t)(t.b * N + min(t.col0 + r, N - 1)) * (uint32_t)Kd * 2u + piece * 16;
    }
    return true;
  };
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(A), 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(Bt), 0, -1, 0x00020000);
  // Half of the wave's requests for the A (B) rows of one k tile.
  auto load_a = [&](const TileCtx& t, int slot_a, int k0, auto half) {
    unsigned char* s = smem + slot_a * kABytes;
    constexpr int u0 = decltype(half)::value * 2;
#pragma unroll
    for (int u = u0; u < u0 + 2; ++u)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(s + (u * Cfg::kWaves + wave) * 1024), 16,
                                               t.a[u], k0 * 2, 0, 0);
  };
  auto load_b = [&](const TileCtx& t, int slot_b, int k0, auto half) {
    unsigned char* s = smem + 3 * kABytes + slot_b * kBBytes;
    constexpr int u0 = decltype(half)::value * 2;
#pragma unroll
    for (int u = u0; u < u0 + 2; ++u)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (lds_ptr_t)(s + (u * Cfg::kWaves + wave) * 1024), 16,
                                               t.bo[u], k0 * 2, 0, 0);
  };
  using Half0 = std::integral_constant<int, 0>;
  using Half1 = std::integral_constant<int, 1>;

  floatx16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  bf16x8 fa[2][FM], fb[2][FN];
  const int a_row_off = (wm * Cfg::TM + m) * RB;
  const int b_row_off = 3 * kABytes + (wn * Cfg::TN + m) * RB;
  const int swz = (m >> 1) & 7;
  auto frags = [&](int buf, int slot_a, int slot_b, int ks) {
    const int col = ((2 * ks + h) ^ swz) * 16;
    const unsigned char* pa = smem + slot_a * kABytes + a_row_off + col;
    const unsigned char* pb = smem + slot_b * kBBytes + b_row_off + col;
#pragma unroll
    for (int i = 0; i < FM; ++i)
      fa[buf][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(pa + i * 32 * RB));
#pragma unroll
    for (int j = 0; j < FN; ++j)
      fb[buf][j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(pb + j * 32 * RB));
  };
  auto mfma_slice = [&](int buf) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
  };
  // First slice of a tile: the sums start from zero in the MFMA itself.
  auto mfma_slice_first = [&](int buf) {
    const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i], zero, 0, 0, 0);
  };
  // Issue order inside a slice: a fragment read of the next slice behind each of the first six
  // MFMAs, the two DMA requests behind the last two.
  auto slice_schedule = [&]() {
#pragma unroll
    for (int g = 0; g < FM + FN; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
#pragma unroll
    for (int g = 0; g < FM * FN - (FM + FN); ++g) {
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // Iteration j multiplies k tile j out of A slot j mod 3 and B slot j mod 2; two requests
  // per wave under each of its four slices:
  //   slice 0   second half of the B rows of k tile j + 1 (into the other B slot)
  //   slice 1   first half of the A rows of k tile j + 2 (into the A slot that k tile j - 1
  //   slice 2   second half of them                       left at the last barrier)
  //   wait until only those A requests are in flight; barrier (every wave has read the last
  //   fragments of k tile j)
  //   slice 3   first half of the B rows of k tile j + 2 (into k tile j's B slot)
  // SRC, K0: k tile j + 2; PSRC, PK0: k tile j + 1.
#define VMOE_W8_ITERATION(SRC, K0, PSRC, PK0, FIRST) do { \
    const int prev_a = sa == 0 ? 2 : sa - 1, next_a = sa == 2 ? 0 : sa + 1; \
    W8_PRIO(2); \
    frags(1, sa, sb, 1); \
    load_b(PSRC, sb ^ 1, (PK0), Half1{}); \
    if constexpr (FIRST) mfma_slice_first(0); else mfma_slice(0); \
    slice_schedule(); \
    W8_PRIO(1); \
    frags(0, sa, sb, 2); \
    load_a(SRC, prev_a, (K0), Half0{}); \
    mfma_slice(1); \
    slice_schedule(); \
    W8_PRIO(0); \
    frags(1, sa, sb, 3); \
    load_a(SRC, prev_a, (K0), Half1{}); \
    mfma_slice(0); \
    slice_schedule(); \
    wait_vmcnt<Cfg::kIssues>(); \
    wait_lgkmcnt0(); \
    raw_barrier(); \
    W8_PRIO(3); \
    frags(0, next_a, sb ^ 1, 0); \
    load_b(SRC, sb, (K0), Half0{}); \
    mfma_slice(1); \
    slice_schedule(); \
    sa = next_a; \
    sb ^= 1; \
  } while (0)

  // The two waves of a SIMD run the same instruction stream, and the SIMD issues from the older
  // wave whenever it can: left alone, the older wave runs through a k tile ahead of the younger
  // one and then sits at the tile's barrier while the younger one works alone, its waits
  // unfilled.  The priority therefore falls from slice to slice between two barriers, so that
  // the wave that lags is the one served first and the two stay within a slice of each other.
#define W8_PRIO(P) __builtin_amdgcn_s_setprio(P)
  TileCtx cur, nxt;
  if (!setup_tile(0, cur)) return;
  int sa = 0, sb = 0;      // slots of the k tile that the next iteration multiplies
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    load_a(cur, t, t * BK, Half0{});
    load_a(cur, t, t * BK, Half1{});
    load_b(cur, t, t * BK, Half0{});
    if (t == 0) load_b(cur, t, t * BK, Half1{});   // (k tile 1's second half: first iteration)
  }
  wait_vmcnt<0>();
  raw_barrier();
  frags(0, 0, 0, 0);
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  for (int ti = 0;; ++ti) {
    const bool has_next = setup_tile(ti + 1, nxt);
    if (!has_next) nxt = cur;   // the last tile requests its own first k tiles again: in bounds, never read
    VMOE_W8_ITERATION(cur, 2 * BK, cur, 1 * BK, true);
    for (int kt = 1; kt < nk - 2; ++kt)
      VMOE_W8_ITERATION(cur, (kt + 2) * BK, cur, (kt + 1) * BK, false);
    VMOE_W8_ITERATION(nxt, 0, cur, (nk - 1) * BK, false);
    VMOE_W8_ITERATION(nxt, BK, nxt, 0, false);
    // Bias of the lane's columns: for column block j and pair of quads qp the lane stores
    // columns j * 32 + qp * 16 + h * 8 .. + 7, whose sums come from its own registers (four
    // columns at (2 qp + h) * 8 + h * 4) and from the other half wave's.  The bias is added
    // before the exchange, so a lane needs it for its own four columns of every quad.
    uint2 bias_pk[FN * 4];
    if constexpr (HAS_BIAS) {
      const bf16_t* src = bias + (size_t)cur.b * N;
#pragma unroll
      for (int jq = 0; jq < FN * 4; ++jq) {
        const int col = cur.col0 + wn * Cfg::TN + h * 4 + jq * 8;
        bias_pk[jq] = *reinterpret_cast<const uint2*>(src + min(col, N - 4));
      }
    }
    mfma_result_fence();
    // Rows and columns past the edge leave through the range check of a buffer store.
    bf16_t* Cb = C + (size_t)cur.b * R * N;
    const uint64_t cb_bits = reinterpret_cast<uint64_t>(Cb);
    bf16_t* cb_uniform = reinterpret_cast<bf16_t*>(
        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(cb_bits >> 32)) << 32) |
        (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)cb_bits));
    const __amdgpu_buffer_rsrc_t c_rsrc = __builtin_amdgcn_make_buffer_rsrc(cb_uniform, 0, R * N * 2, 0x00020000);
    const int wrow0 = cur.row0 + wm * Cfg::TM, wcol0 = cur.col0 + wn * Cfg::TN;
    const uint32_t lane_off = (uint32_t)(m * N + h * 8) * 2u;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const bool row_ok = m < cur.live - (wrow0 + i * 32);
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        uint32_t p[4][2];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint2 bp = bias_pk[j * 4 + q];
          const float bv[4] = {bf_lo(bp.x), bf_hi(bp.x), bf_lo(bp.y), bf_hi(bp.y)};
          p[q][0] = epilogue_pair<EPI, HAS_BIAS>(acc[i][j][q * 4], acc[i][j][q * 4 + 1], bv[0], bv[1]);
          p[q][1] = epilogue_pair<EPI, HAS_BIAS>(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3], bv[2], bv[3]);
        }
#pragma unroll
        for (int qp = 0; qp < 2; ++qp) {
          // quads 2 qp (kept by the lower half wave) and 2 qp + 1 (kept by the upper one)
          const auto x = __builtin_amdgcn_permlane32_swap(p[2 * qp][0], p[2 * qp + 1][0], false, false);
          const auto y = __builtin_amdgcn_permlane32_swap(p[2 * qp][1], p[2 * qp + 1][1], false, false);
          const u32x4_t v = {x[0], y[0], x[1], y[1]};
          const int col_s = wcol0 + j * 32 + qp * 16;
          const bool ok = row_ok && h * 8 + 8 <= N - col_s;
          __builtin_amdgcn_raw_buffer_store_b128(v, c_rsrc, ok ? lane_off : 0xfffffff0u,
                                                 ((wrow0 + i * 32) * N + col_s) * 2, EPI != kEpiBias ? 2 : 0);
          store_data_guard();
        }
      }
    }
    if (!has_next) break;
    cur = nxt;
  }
  wait_vmcnt<0>();
#undef W8_PRIO
#undef VMOE_W8_ITERATION
#endif
}

// Whether the eight-wave kernel covers the product: k a multiple of 64 and at least 256,
// operands addressable with 32-bit byte offsets from their start, N a multiple of 8, output
// of one batch below 2 GiB, and a ragged launch only with its plan.
inline bool w8_gemm_ok(int batch, int R, int N, int Kd, const int32_t* rows, const int4* plan) {
  const GemmGeom g = gemm_geometry<W8Cfg>(batch, R, N, Kd);
  const uint64_t lim = 1ull << 32;
  return g.fast && Kd / W8Cfg::BK >= 4 && (N & 7) == 0 && (uint64_t)batch * R * Kd * 2 < lim &&
         (uint64_t)batch * N * Kd * 2 < lim && (uint64_t)R * N * 2 < (1ull << 31) &&
         g.tiles <= 0x7ffffff0LL && (rows == nullptr || plan != nullptr);
}

template <int EPI>
int launch_gemm_bf16_w8(const bf16_t* A, const bf16_t* Bt, const bf16_t* bias, bf16_t* C, int batch,
                        int R, int N, int Kd, hipStream_t stream, const int4* plan = nullptr,
                        int32_t* clear = nullptr, int clear_count = 0, int32_t* status = nullptr) {
  const GemmGeom g = gemm_geometry<W8Cfg>(batch, R, N, Kd);
  auto kern = bias != nullptr ? gemm_bf16_w8_kernel<EPI, true> : gemm_bf16_w8_kernel<EPI, false>;
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), W8Cfg::kLdsBytes);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3(kCusPerXcd * kNumXcd), dim3(W8Cfg::kThreads), W8Cfg::kLdsBytes,
                     stream, A, Bt, bias, C, R, N, Kd, g.tiles_m, g.tiles_n, (int)g.tiles,
                     g.tiles_per_xcd, g.panel_rows, plan_ref<W8Cfg>(g, plan, batch, R), clear,
                     clear_count, status, active_units().xcds, active_units().slots);
  return launch_status();
}

}  // namespace vmoe
#endif  // VMOE_GEMM_BF16_W8_H_
