// Batched bf16 GEMM on eight waves with v_mfma_f32_16x16x32_bf16: tiles of 256 rows by 256
// (FN = 8) or 192 (FN = 6) columns, two waves per SIMD, each wave 64 rows x half the columns
// (4 x FN MFMA tiles of 16 x 16: 128 or 96 accumulator registers, so that two waves share a
// SIMD's 512 registers), 64-wide k tiles, one workgroup per compute unit walking a list of
// tiles.  The tiles of a die's last, partial round run whole here (no stream-K).
//
// Why eight waves.  With one wave per SIMD (gemm_bf16_persistent_kernel) whatever makes that
// wave wait -- the fragments of its next MFMAs, the k tile's barrier, a DMA request that the
// address unit does not take at once -- leaves the SIMD's matrix core idle.  With two waves
// per SIMD the other wave's MFMAs fill those gaps and the epilogue is half as long per wave.
// The price: every B row is read from LDS by four waves instead of two (fragment traffic
// x 1.5).
//
// Why this MFMA.  The chip runs these products at its power limit, and in a loop over
// registers the 16x16x32 instruction sustains about 14 % more flops at that limit than the
// 32x32x16 one (2.13 against 1.86 PFLOP/s); its fragments are also what lets a lane collect
// eight consecutive output columns with one v_permlane16_swap per pair of registers, so the
// output leaves without LDS.  Second product of the B/16 layer (32 experts x ~3010 rows x 768
// x 3072), 256-column tiles: the step went from 1.002 - 1.007 to 0.983 - 0.989 ms against the
// same kernel written with 32x32x16 MFMAs (three alternating pairs of runs), which in turn
// had gained 12 - 19 us on the four-wave kernel.
//
// Why 192 columns (FN = 6).  With 768 output columns and 12 full row tiles in each of 32
// experts, 256-column tiles make 1152 tiles, 4.5 per compute unit: five rounds for the work
// of four and a half; 192-column tiles make 1536, six apiece (392 against 424 us on that
// shape, dense).  The choice between the two is made on the host from the launch's geometry.
//
// Operand path: global memory -> LDS by DMA (buffer_load ... lds), 8 rows x 128 bytes per
// request, the 16-byte pieces of a row XOR-swizzled by row so that fragment reads are free
// of bank conflicts.  A rows sit in a ring of three 32 KB slots, B rows in one of two (24 or
// 32 KB each: up to all of the 160 KB); requests are never drained inside a tile, and the
// last two iterations of a tile request the first k tiles of the next one, so the ring stays
// full across tile boundaries.  A k tile is two steps of 32; a step is FN units, one per
// column block: four MFMAs (the wave's four row blocks times that column block).  The wave
// holds the A fragments of the current step, reads those of the next step during the step's
// last two units, and keeps the B fragments of the next kLook units in flight.
#ifndef VMOE_GEMM_BF16_W8_H_
#define VMOE_GEMM_BF16_W8_H_

#include <type_traits>
#include <utility>

#include "gemm_bf16.h"

namespace vmoe {

template <int FN_>
struct W8Cfg {
  static constexpr int FM = 4, FN = FN_;                         // 16 x 16 MFMA tiles per wave
  static constexpr int BM = 256, BN = 32 * FN, BK = 64;
  static constexpr int kWaves = 8, kThreads = 512, kBlocksPerCu = 1;
  static constexpr int TM = 64, TN = 16 * FN;                    // wave tile
  static constexpr int RB = BK * 2;                              // bytes of one row of a k tile
  static constexpr int kABytes = BM * RB, kBBytes = BN * RB;     // one slot
  static constexpr int kLdsBytes = 3 * kABytes + 2 * kBBytes;
  static constexpr int kIssuesA = BM / 8 / kWaves;               // DMA requests per wave and k tile: 4
  static constexpr int kIssuesB = BN / 8 / kWaves;               // 3 or 4
  static constexpr int kUnits = 2 * FN;                          // units per k tile
  // B fragments in flight beyond the current one.  The ring of kLook + 1 fragment sets must
  // divide the units of a k tile so that every unit names its registers at compile time.
  static constexpr int kLook = FN == 6 ? 5 : 3;
  // The barrier of a k tile stands before the first unit that reads from the next k tile.
  static constexpr int kBarrierUnit = kUnits - (kLook > 2 ? kLook : 2);
  static_assert(kUnits % (kLook + 1) == 0, "fragment ring");
  // After the barrier every fragment of the k tile's B rows has been read (kLook >= 1 units
  // ago), so the B rows of the k tile after next go into its slot from there on, one request
  // per unit; what does not fit goes under the first units of the next iteration, then the A
  // rows of the k tile after next.
  static constexpr int kPostB = kIssuesB < kUnits - kBarrierUnit ? kIssuesB : kUnits - kBarrierUnit;
  static constexpr int kRestB = kIssuesB - kPostB;
  static_assert(kRestB + kIssuesA <= kBarrierUnit, "requests of the first units come before the barrier");
  // Issue priority of unit g: falls in four stages from one barrier to the next.
  static constexpr int prio_of(int g) { return 3 - (((g - kBarrierUnit + kUnits) % kUnits) * 4) / kUnits; }
  static_assert(FN % 2 == 0 && BN % 64 == 0, "column blocks leave in pairs; 64 B rows per request");
  static_assert(kLdsBytes <= 160 * 1024, "LDS budget");
};

// A is (batch, R, Kd).  `clear` / `status`: begin_call.
template <int EPI, bool HAS_BIAS, int FN_>
__global__ __launch_bounds__(512, 1) void gemm_bf16_w8_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bt, const bf16_t* __restrict__ bias,
    bf16_t* __restrict__ C, int R, int N, int Kd, int tiles_m, int tiles_n, int num_tiles,
    int tiles_per_xcd, int panel_rows, PlanRef plan_ref, int32_t* __restrict__ clear,
    int clear_count, int32_t* __restrict__ status, int active_xcds, int active_slots) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-resource builtins exist in the device pass only
  extern __shared__ __align__(1024) unsigned char smem[];
  using Cfg = W8Cfg<FN_>;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, RB = Cfg::RB;
  constexpr int FM = Cfg::FM, FN = Cfg::FN;
  constexpr int kABytes = Cfg::kABytes, kBBytes = Cfg::kBBytes;
  constexpr int kUnits = Cfg::kUnits, kLook = Cfg::kLook, kRing = Cfg::kLook + 1;
  constexpr int kBarrierUnit = Cfg::kBarrierUnit;
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
  const int n16 = lane & 15, g4 = lane >> 4;
  const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
  if (xcd >= active_xcds || slot >= active_slots) return;   // (measurement only, see active_units)
  // A request fills 8 rows x 128 bytes; lane L lands in LDS position L of the request and
  // fetches the 16-byte piece that the XOR swizzle of its row puts there.
  const int lrow = lane >> 3;
  const int piece = (lane & 7) ^ (((wave * 8 + lrow) >> 1) & 7);
  // First B row of request u of this wave.  Request u brings column blocks 2u and 2u + 1 of
  // both halves of the tile (waves 0-3 the left half's 32 rows, waves 4-7 the right half's),
  // so that the part of a slot that request 0 overwrites is the part whose fragments every
  // wave reads first.
  const int b_wave_row = (wave >> 2) * Cfg::TN + (wave & 3) * 8;
  auto b_request_row = [&](int u) { return b_wave_row + u * 32; };

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

  // What a tile is: uniform values.  The current tile also keeps the byte offsets of the lane's
  // DMA requests; for the tile after it (requested from only in the last two iterations) they
  // are worked out at the request.
  struct TileId {
    int b, row0, col0, live;
  };
  struct TileCtx : TileId {
    uint32_t a[Cfg::kIssuesA], bo[Cfg::kIssuesB];
  };
  auto a_offset = [&](const TileId& t, int u) {
    const int r = (u * Cfg::kWaves + wave) * 8 + lrow;
    return (uint32_t)(t.b * R + min(t.row0 + r, R - 1)) * (uint32_t)Kd * 2u + piece * 16;
  };
  auto b_offset = [&](const TileId& t, int u) {
    const int rb = b_request_row(u) + lrow;
    return (uint32_t)(t.b * N + min(t.col0 + rb, N - 1)) * (uint32_t)Kd * 2u + piece * 16;
  };
  auto materialize = [&](const TileId& id, TileCtx& t) {
    static_cast<TileId&>(t) = id;
#pragma unroll
    for (int u = 0; u < Cfg::kIssuesA; ++u) t.a[u] = a_offset(id, u);
#pragma unroll
    for (int u = 0; u < Cfg::kIssuesB; ++u) t.bo[u] = b_offset(id, u);
  };
  auto setup_tile = [&](int i, TileId& t) -> bool {
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
    return true;
  };
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(A), 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(Bt), 0, -1, 0x00020000);
  // One request of the wave for the A (B) rows of a k tile.
  auto load_a = [&](const auto& t, int slot_a, int k0, int u) {
    uint32_t off;
    if constexpr (std::is_same_v<std::decay_t<decltype(t)>, TileCtx>) off = t.a[u]; else off = a_offset(t, u);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        a_rsrc, (lds_ptr_t)(smem + slot_a * kABytes + (u * Cfg::kWaves + wave) * 1024), 16, off, k0 * 2, 0, 0);
  };
  auto load_b = [&](const auto& t, int slot_b, int k0, int u) {
    uint32_t off;
    if constexpr (std::is_same_v<std::decay_t<decltype(t)>, TileCtx>) off = t.bo[u]; else off = b_offset(t, u);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        b_rsrc, (lds_ptr_t)(smem + 3 * kABytes + slot_b * kBBytes + b_request_row(u) * RB), 16, off, k0 * 2, 0, 0);
  };

  floatx4 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;
  // v_mfma_f32_16x16x32_bf16: a lane supplies 8 consecutive k of one row (row = lane % 16,
  // k = 8 * (lane / 16) of the 32-wide step).
  bf16x8 fa[2][FM], fb[kRing];
  const int a_row_off = (wm * Cfg::TM + n16) * RB;
  const int b_row_off = 3 * kABytes + (wn * Cfg::TN + n16) * RB;
  const int swz = (n16 >> 1) & 7;
  auto read_a = [&](int buf, int slot_a, int step, int i) {
    fa[buf][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
        smem + slot_a * kABytes + a_row_off + (((4 * step + g4) ^ swz) * 16) + i * 16 * RB));
  };
  auto read_b = [&](int buf, int slot_b, int step, int j) {
    fb[buf] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
        smem + slot_b * kBBytes + b_row_off + (((4 * step + g4) ^ swz) * 16) + j * 16 * RB));
  };

  // The two waves of a SIMD run the same instruction stream, and the SIMD issues from the older
  // wave whenever it can: left alone, the older wave runs through a k tile ahead of the younger
  // one and then sits at the tile's barrier while the younger one works alone, its waits
  // unfilled.  The priority therefore falls in four stages between two barriers, so that the
  // wave that lags is the one served first.

  // Iteration j multiplies k tile j out of A slot j mod 3 and B slot j mod 2, one DMA request
  // of the wave under a unit:
  //   first units        the last kRestB requests of the B rows of k tile j + 1, then the A rows
  //                      of k tile j + 2 (into the A slot that k tile j - 1 left)
  //   before unit kBarrierUnit: wait until only those A requests are in flight; barrier (k tile
  //                      j + 1 has landed; every fragment of k tile j's B rows has been read)
  //   from there         the first kPostB requests of the B rows of k tile j + 2 (into k tile
  //                      j's B slot)
  // src, k0: k tile j + 2; psrc, pk0: k tile j + 1.
  int sa = 0, sb = 0;      // slots of the k tile that the next iteration multiplies
  auto iteration = [&](const auto& src, int k0, const auto& psrc, int pk0, auto first) __attribute__((always_inline)) {
    const int prev_a = sa == 0 ? 2 : sa - 1, next_a = sa == 2 ? 0 : sa + 1;
    static_for<kUnits>([&](auto g_c) __attribute__((always_inline)) {
      constexpr int g = decltype(g_c)::value;
      constexpr int step = g / FN, j = g % FN;
      if constexpr (g == kBarrierUnit) {
        __builtin_amdgcn_sched_barrier(0);
        wait_vmcnt<Cfg::kIssuesA>();
        wait_lgkmcnt0();
        raw_barrier();
      }
      if constexpr (g == 0 || Cfg::prio_of(g) != Cfg::prio_of(g - 1)) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(Cfg::prio_of(g));
      }
      // fragment reads: the B fragment kLook units on, and during a step's last two units the A
      // fragments of the next step
      constexpr int gl = g + kLook;
      constexpr int reads = j >= FN - 2 ? 3 : 1;
      if constexpr (gl < kUnits) read_b(gl % kRing, sb, gl / FN, gl % FN);
      else read_b(gl % kRing, sb ^ 1, (gl - kUnits) / FN, (gl - kUnits) % FN);
      if constexpr (j >= FN - 2) {
        constexpr int i0 = (j - (FN - 2)) * 2;
        if constexpr (step == 0) { read_a(1, sa, 1, i0); read_a(1, sa, 1, i0 + 1); }
        else { read_a(0, next_a, 0, i0); read_a(0, next_a, 0, i0 + 1); }
      }
      // DMA request
      constexpr bool dma = g < Cfg::kRestB + Cfg::kIssuesA || (g >= kBarrierUnit && g < kBarrierUnit + Cfg::kPostB);
      if constexpr (g < Cfg::kRestB) load_b(psrc, sb ^ 1, pk0, Cfg::kPostB + g);
      else if constexpr (g < Cfg::kRestB + Cfg::kIssuesA) load_a(src, prev_a, k0, g - Cfg::kRestB);
      else if constexpr (dma) load_b(src, sb, k0, g - kBarrierUnit);
      const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < FM; ++i)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            fb[g % kRing], fa[step][i], (decltype(first)::value && step == 0) ? zero : acc[i][j], 0, 0, 0);
      // issue order: a read behind each of the first MFMAs, the request behind the third
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if constexpr (reads == 3) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if constexpr (reads == 3) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if constexpr (dma) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    });
    __builtin_amdgcn_sched_barrier(0);
    sa = next_a;
    sb ^= 1;
  };
  using First = std::true_type;
  using NotFirst = std::false_type;

  TileCtx cur;
  TileId nxt;
  if (!setup_tile(0, nxt)) return;
  materialize(nxt, cur);
  // k tile 0 whole, the A rows and the first B requests of k tile 1
#pragma unroll
  for (int u = 0; u < Cfg::kIssuesA; ++u) load_a(cur, 0, 0, u);
#pragma unroll
  for (int u = 0; u < Cfg::kIssuesB; ++u) load_b(cur, 0, 0, u);
#pragma unroll
  for (int u = 0; u < Cfg::kIssuesA; ++u) load_a(cur, 1, BK, u);
#pragma unroll
  for (int u = 0; u < Cfg::kPostB; ++u) load_b(cur, 1, BK, u);
  wait_vmcnt<0>();
  raw_barrier();
#pragma unroll
  for (int i = 0; i < FM; ++i) read_a(0, 0, 0, i);
  static_for<kLook>([&](auto c) __attribute__((always_inline)) { constexpr int u = decltype(c)::value; read_b(u % kRing, 0, u / FN, u % FN); });
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  for (int ti = 0;; ++ti) {
    const bool has_next = setup_tile(ti + 1, nxt);
    if (!has_next) nxt = static_cast<const TileId&>(cur);   // the last tile requests its own first k tiles again: in bounds, never read
    iteration(cur, 2 * BK, cur, 1 * BK, First{});
    for (int kt = 1; kt < nk - 2; ++kt) iteration(cur, (kt + 2) * BK, cur, (kt + 1) * BK, NotFirst{});
    iteration(nxt, 0, cur, (nk - 1) * BK, NotFirst{});
    iteration(nxt, BK, nxt, 0, NotFirst{});
    // acc[i][j][v] = C[row i * 16 + lane % 16][column j * 16 + (lane / 16) * 4 + v].
    const bf16_t* bias_src = bias + (size_t)cur.b * N;
    auto load_bias = [&](int j) {
      const int col = cur.col0 + wn * Cfg::TN + j * 16 + g4 * 4;
      return *reinterpret_cast<const uint2*>(bias_src + min(col, N - 4));
    };
    uint2 bias_next[2] = {};
    if constexpr (HAS_BIAS) {
      bias_next[0] = load_bias(0);
      bias_next[1] = load_bias(1);
    }
    mfma_result_fence();
    // Rows and columns past the edge leave through the range check of a buffer store.  Column
    // blocks leave in pairs: the lanes of an even group of 16 keep their own four columns of
    // block j and take the next four from the group above, the odd groups do the same for
    // block j + 1 (v_permlane16_swap), so a lane holds eight consecutive columns and a store
    // covers 16 rows x 64 contiguous bytes.
    bf16_t* Cb = C + (size_t)cur.b * R * N;
    const uint64_t cb_bits = reinterpret_cast<uint64_t>(Cb);
    bf16_t* cb_uniform = reinterpret_cast<bf16_t*>(
        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(cb_bits >> 32)) << 32) |
        (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)cb_bits));
    const __amdgpu_buffer_rsrc_t c_rsrc = __builtin_amdgcn_make_buffer_rsrc(cb_uniform, 0, R * N * 2, 0x00020000);
    const int wrow0 = cur.row0 + wm * Cfg::TM, wcol0 = cur.col0 + wn * Cfg::TN;
    const int lane_col = (g4 & 1) * 16 + (g4 >> 1) * 8;       // inside a pair of column blocks
    const uint32_t lane_off = (uint32_t)(n16 * N + lane_col) * 2u;
#pragma unroll
    for (int jp = 0; jp < FN / 2; ++jp) {
      const uint2 bias_pk[2] = {bias_next[0], bias_next[1]};
      if constexpr (HAS_BIAS) {
        if (jp + 1 < FN / 2) {
          bias_next[0] = load_bias(2 * jp + 2);
          bias_next[1] = load_bias(2 * jp + 3);
        }
      }
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const bool row_ok = n16 < cur.live - (wrow0 + i * 16);
        uint32_t p[2][2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int j = 2 * jp + t;
          const uint2 bp = bias_pk[t];
          const float bv[4] = {bf_lo(bp.x), bf_hi(bp.x), bf_lo(bp.y), bf_hi(bp.y)};
          p[t][0] = epilogue_pair<EPI, HAS_BIAS>(acc[i][j][0], acc[i][j][1], bv[0], bv[1]);
          p[t][1] = epilogue_pair<EPI, HAS_BIAS>(acc[i][j][2], acc[i][j][3], bv[2], bv[3]);
        }
        const auto x = __builtin_amdgcn_permlane16_swap(p[0][0], p[1][0], false, false);
        const auto y = __builtin_amdgcn_permlane16_swap(p[0][1], p[1][1], false, false);
        const u32x4_t v = {x[0], y[0], x[1], y[1]};
        const int col_s = wcol0 + jp * 32;
        const bool ok = row_ok && lane_col + 8 <= N - col_s;
        __builtin_amdgcn_raw_buffer_store_b128(v, c_rsrc, ok ? lane_off : 0xfffffff0u,
                                               ((wrow0 + i * 16) * N + col_s) * 2, EPI != kEpiBias ? 2 : 0);
        store_data_guard();
      }
    }
    if (!has_next) break;
    materialize(nxt, cur);
  }
  wait_vmcnt<0>();
#endif
}

// Whether this kernel covers the product: k a multiple of 64 and at least 256, operands
// addressable with 32-bit byte offsets from their start, N a multiple of 8, output of one
// batch below 2 GiB, and a ragged launch only with its plan.
template <int FN>
inline bool w8_gemm_ok(int batch, int R, int N, int Kd, const int32_t* rows, const int4* plan) {
  const GemmGeom g = gemm_geometry<W8Cfg<FN>>(batch, R, N, Kd);
  const uint64_t lim = 1ull << 32;
  return g.fast && Kd / 64 >= 4 && (N & 7) == 0 && (uint64_t)batch * R * Kd * 2 < lim &&
         (uint64_t)batch * N * Kd * 2 < lim && (uint64_t)R * N * 2 < (1ull << 31) &&
         g.tiles <= 0x7ffffff0LL && (rows == nullptr || plan != nullptr);
}

template <int EPI, int FN>
int launch_gemm_bf16_w8(const bf16_t* A, const bf16_t* Bt, const bf16_t* bias, bf16_t* C, int batch,
                         int R, int N, int Kd, hipStream_t stream, const int4* plan = nullptr,
                         int32_t* clear = nullptr, int clear_count = 0, int32_t* status = nullptr) {
  using Cfg = W8Cfg<FN>;
  const GemmGeom g = gemm_geometry<Cfg>(batch, R, N, Kd);
  auto kern = bias != nullptr ? gemm_bf16_w8_kernel<EPI, true, FN> : gemm_bf16_w8_kernel<EPI, false, FN>;
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::kLdsBytes);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3(kCusPerXcd * kNumXcd), dim3(Cfg::kThreads), Cfg::kLdsBytes,
                     stream, A, Bt, bias, C, R, N, Kd, g.tiles_m, g.tiles_n, (int)g.tiles,
                     g.tiles_per_xcd, g.panel_rows, plan_ref<Cfg>(g, plan, batch, R), clear,
                     clear_count, status, active_units().xcds, active_units().slots);
  return launch_status();
}

}  // namespace vmoe
#endif  // VMOE_GEMM_BF16_W8_H_
