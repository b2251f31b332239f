// Batched bf16 GEMM on the gfx950 matrix cores, float32 accumulate:
//   C[b] (R x N) = epilogue(A[b] (R x Kd) . Bt[b] (N x Kd)^T + bias[b])
// Both operands are K-contiguous, so a lane's MFMA fragment (8 consecutive k
// of one row) is a single 16-byte LDS read for A and for B alike.
//
// Tiling: a workgroup of WM x WN waves computes a BM x BN tile; each wave owns
// (BM/WM) x (BN/WN) of it as a grid of 32x32 v_mfma_f32_32x32x16_bf16 tiles held
// in accumulator registers.
//
// Operand path: global memory -> LDS directly (global_load_lds_dwordx4), no
// staging registers and no LDS write instructions.  A wave-wide load fills 1 KiB
// of consecutive LDS, lane L landing at base + 16*L, so each lane fetches the
// global 16-byte chunk that an XOR swizzle assigns to its LDS slot; the swizzle
// makes the 128-bit fragment reads conflict-free on the 64 LDS banks.
//
// Pipeline: K advances in BK-wide tiles through a ring of NSTAGE LDS stages; the
// DMA loads run NSTAGE-1 tiles ahead and are never drained (s_waitcnt vmcnt(n)
// covers only the tile needed next).  Inside a tile the fragment reads of the
// next 16-wide k slice are issued under the MFMAs of the current one (double
// buffered fragment registers), and the tile's one barrier sits before its last
// slice so that the next tile's first fragments are fetched under MFMAs too.
//
// The MFMA is issued with the weight fragment as its first operand, so the
// accumulator tile is C^T: a lane ends up with 4 consecutive output columns of
// one output row, which the epilogue packs into 8-byte LDS writes; the tile is
// then streamed out with 16-byte, row-contiguous global stores.
//
// Workgroup -> tile mapping: hardware hands consecutive workgroups to the 8 XCDs
// round-robin, each XCD has a private L2.  Workgroup w is therefore given
// logical tile (w % 8) * ceil(tiles/8) + w / 8, so that an XCD walks a contiguous
// run of tiles (whole experts), and within an expert tiles are ordered in panels
// of 8 row tiles so that the tiles in flight on an XCD share A and B panels.
//
// Two kernels share this scheme: gemm_bf16_kernel computes one tile per workgroup;
// gemm_bf16_persistent_kernel (long k, one workgroup per CU) walks a list of tiles
// and keeps the operand ring full across tile boundaries.
#ifndef VMOE_GEMM_BF16_H_
#define VMOE_GEMM_BF16_H_

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <type_traits>
#include <utility>
#include "vmoe_common.h"

namespace vmoe {

enum { kEpiBias = 0, kEpiBiasGeluTanh = 1, kEpiBiasGeluErf = 2 };

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order: a loop whose
// index is a constant in the body (register arrays, if constexpr).
template <int I>
using IntC = std::integral_constant<int, I>;
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(IntC<Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}


// 0.5 x (1 + tanh(c (x + 0.044715 x^3))) = x * sigmoid(2 c (x + 0.044715 x^3)),
// with the hardware exp2 and reciprocal (relative error ~1e-7, far inside bf16).
__device__ __forceinline__ float gelu_tanh_fast(float x) {
  const float k0 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
  const float k1 = k0 * 0.044715f;
  float z = x * fmaf(k1, x * x, k0);
  float e = __builtin_amdgcn_exp2f(z);
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

template <int EPI>
__device__ __forceinline__ float apply_epilogue(float acc, float bias, bool has_bias) {
  float o = bf16r(acc);
  if (has_bias) o = bf16r(o + bias);
  if (EPI == kEpiBiasGeluTanh) o = gelu_tanh_fast(o);
  if (EPI == kEpiBiasGeluErf) o = gelu_erf(o);
  return o;
}

// The same epilogue for two neighbouring outputs at once, as one bfloat16 pair:
// every rounding step is a single packed conversion (v_cvt_pk_bf16_f32) followed
// by a shift and a mask, instead of a conversion and a shift per element.
template <int EPI, bool HAS_BIAS>
__device__ __forceinline__ uint32_t epilogue_pair(float a0, float a1, float b0, float b1) {
  uint32_t p = pack_bf16x2(a0, a1);
  if (HAS_BIAS) p = pack_bf16x2(bf_lo(p) + b0, bf_hi(p) + b1);
  if (EPI == kEpiBiasGeluTanh) p = pack_bf16x2(gelu_tanh_fast(bf_lo(p)), gelu_tanh_fast(bf_hi(p)));
  if (EPI == kEpiBiasGeluErf) p = pack_bf16x2(gelu_erf(bf_lo(p)), gelu_erf(bf_hi(p)));
  return p;
}

template <int BM_, int BN_, int WM_, int WN_, int BK_ = 32, int NSTAGE_ = 4, int BLOCKS_PER_CU_ = 1>
struct GemmCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, NSTAGE = NSTAGE_;
  static constexpr int kBlocksPerCu = BLOCKS_PER_CU_;
  static constexpr int kWaves = WM * WN;
  static constexpr int kThreads = 64 * kWaves;
  static constexpr int TM = BM / WM, TN = BN / WN;   // wave tile
  static constexpr int FM = TM / 32, FN = TN / 32;   // 32x32 MFMA tiles per wave
  static constexpr int kRowBytes = BK * 2;           // LDS row of one k tile, XOR-swizzled 16-byte chunks
  static constexpr int kChunksPerRow = BK / 8;       // 4 (BK=32) or 8 (BK=64)
  static constexpr int kRowsPerLoad = 64 / kChunksPerRow;   // rows filled by one wave-wide DMA load
  // The gfx950 LDS serves 16 lanes of a 128-bit read per clock from 64 banks (256
  // bytes): the swizzle must spread 16 consecutive rows over all of them.
  static constexpr int kSwzShift = BK == 32 ? 2 : 1;  // log2(rows per 256-byte bank line)
  static constexpr int kStageBytes = (BM + BN) * kRowBytes;
  static constexpr int kOutLd = TN + 8;              // padded row of the staged output tile
  static constexpr size_t kMainBytes = (size_t)NSTAGE * kStageBytes;
  static constexpr size_t kOutBytes = (size_t)kWaves * TM * kOutLd * sizeof(bf16_t);
  static constexpr size_t kLdsBytes = kMainBytes > kOutBytes ? kMainBytes : kOutBytes;
  static constexpr int kAIssues = BM / kRowsPerLoad / kWaves;
  static constexpr int kBIssues = BN / kRowsPerLoad / kWaves;
  static constexpr int kLoads = kAIssues + kBIssues;  // DMA instructions per wave per k tile
  static_assert(BK == 32 || BK == 64, "BK");
  static_assert(NSTAGE >= 2 && NSTAGE * kLoads < 64, "vmcnt is a 6-bit counter");
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be 32-aligned");
  static_assert(BM % (kRowsPerLoad * kWaves) == 0 && BN % (kRowsPerLoad * kWaves) == 0,
                "tile loads must divide evenly");
  static_assert(kLdsBytes * kBlocksPerCu <= 160 * 1024, "LDS budget");
};

typedef const __attribute__((address_space(1))) void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// Epilogue of one wave: acc[i][j][v] = C[wrow0 + i*32 + m][wcol0 + j*32 + (v/4)*8 + h*4 + v%4]
// (the MFMA was issued with the weight fragment first, so a lane holds 4
// consecutive columns of one row).  Bias, rounding, GELU and the bf16 pack happen
// in registers; the wave tile is staged in a wave-private LDS region and leaves
// as 16-byte, row-contiguous global stores.
// Bias of the wave tile's columns for one lane: four consecutive bfloat16 per
// (column tile j, quad q), fetched before the main loop so that the epilogue does
// not start with a round trip to memory.
template <int TN>
__device__ __forceinline__ void load_bias(uint2 (&bias_pk)[TN / 8], const bf16_t* __restrict__ bias,
                                          int b, int N, int wcol0, int lane) {
  const int h = lane >> 5;
#pragma unroll
  for (int jq = 0; jq < TN / 8; ++jq) {
    bias_pk[jq] = make_uint2(0, 0);
    if (bias != nullptr) {
      const int col = wcol0 + jq * 8 + h * 4;
      const bf16_t* src = bias + (size_t)b * N;
      if ((N & 3) == 0) {
        bias_pk[jq] = *reinterpret_cast<const uint2*>(src + min(col, N - 4));
      } else {
        uint32_t v[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) v[t] = src[min(col + t, N - 1)];
        bias_pk[jq] = make_uint2(v[0] | (v[1] << 16), v[2] | (v[3] << 16));
      }
    }
  }
}

// The staged wave tile (TM rows of TN + 8 bfloat16 at `so`) to memory as 16-byte
// row-contiguous pieces.
template <int EPI, int TM, int TN>
__device__ __forceinline__ void store_staged_tile(const bf16_t* so, int lane, bf16_t* __restrict__ C,
                                                  int b, int R, int live, int N, int wrow0, int wcol0) {
  constexpr int OLD = TN + 8;
  bf16_t* Cb = C + (size_t)b * R * N;
  // Each wave reads back only what it wrote (LDS operations of a wave complete in order).
  constexpr int kChunksOut = TN / 8;                  // 16-byte chunks per staged row
  constexpr int kRowsPerPass = 64 / kChunksOut;
  static_assert(64 % kChunksOut == 0, "wave tile width must divide a wave");
  const int oc = (lane % kChunksOut) * 8;
  const int orow = lane / kChunksOut;
#if defined(__HIP_DEVICE_COMPILE__)
  // Rows and columns past the edge leave through the range check of a buffer store (the
  // lane's part of the address in the vector offset, which the check sees, the pass's part in
  // the scalar offset) instead of a branch around every store.
  if ((uint64_t)R * N * 2 < (1ull << 31)) {
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    const uint64_t cb_bits = reinterpret_cast<uint64_t>(Cb);      // the same in every lane
    bf16_t* cb_uniform = reinterpret_cast<bf16_t*>(
        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(cb_bits >> 32)) << 32) |
        (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)cb_bits));
    const __amdgpu_buffer_rsrc_t c_rsrc = __builtin_amdgcn_make_buffer_rsrc(cb_uniform, 0, R * N * 2, 0x00020000);
    const uint32_t lane_off = (uint32_t)(orow * N + oc) * 2u;
    const int row_u = __builtin_amdgcn_readfirstlane(wrow0), col_u = __builtin_amdgcn_readfirstlane(wcol0);
    const bool col_ok = oc + 8 <= N - col_u;
    // (four staged pieces are read before the first of them is stored: the guard behind a
    // store keeps every later instruction behind it, the reads of later pieces included)
    constexpr int kBatch = 4;
    static_assert(TM / kRowsPerPass % kBatch == 0, "passes come in batches of four");
#pragma unroll
    for (int r0 = 0; r0 < TM; r0 += kBatch * kRowsPerPass) {
      uint4 v[kBatch];
#pragma unroll
      for (int t = 0; t < kBatch; ++t)
        v[t] = *reinterpret_cast<const uint4*>(so + (r0 + t * kRowsPerPass + orow) * OLD + oc);
#pragma unroll
      for (int t = 0; t < kBatch; ++t) {
        const int rs = r0 + t * kRowsPerPass;
        const bool ok = col_ok && orow < live - (row_u + rs);
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v[t]), c_rsrc,
                                               ok ? lane_off : 0xfffffff0u,
                                               ((row_u + rs) * N + col_u) * 2, EPI != kEpiBias ? 2 : 0);
        store_data_guard();
      }
    }
    return;
  }
#endif
#pragma unroll
  for (int r0 = 0; r0 < TM; r0 += kRowsPerPass) {
    const int rl = r0 + orow;
    const int row = wrow0 + rl;
    const int col = wcol0 + oc;
    uint4 v = *reinterpret_cast<const uint4*>(so + rl * OLD + oc);
    if (row < live && col + 8 <= N) {
      // The activated hidden layer (hundreds of MB, read back once by the second product)
      // is larger than any cache: it leaves with streaming stores so that it does not
      // evict the operands.  The second product's output is read next by combine and
      // stays cacheable.
      if constexpr (EPI != kEpiBias) {
        typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(__builtin_bit_cast(u32x4_t, v),
                                    reinterpret_cast<u32x4_t*>(Cb + (size_t)row * N + col));
      } else {
        *reinterpret_cast<uint4*>(Cb + (size_t)row * N + col) = v;
      }
    }
  }
}

template <int EPI, int TM, int TN>
__device__ __forceinline__ void store_tile(floatx16 (&acc)[TM / 32][TN / 32], unsigned char* smem,
                                           int wave, int lane, const uint2 (&bias_pk)[TN / 8],
                                           bool has_bias, bf16_t* __restrict__ C, int b, int R,
                                           int live, int N, int wrow0, int wcol0) {
  constexpr int FM = TM / 32, FN = TN / 32, OLD = TN + 8;
  const int m = lane & 31, h = lane >> 5;
  bf16_t* so = reinterpret_cast<bf16_t*>(smem) + (size_t)wave * TM * OLD;
  auto stage = [&](auto has_bias_c) {
    constexpr bool kHasBias = decltype(has_bias_c)::value;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int cl = j * 32 + q * 8 + h * 4;          // column inside the wave tile
        const uint2 bp = bias_pk[j * 4 + q];
        const float bv[4] = {bf_lo(bp.x), bf_hi(bp.x), bf_lo(bp.y), bf_hi(bp.y)};
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          const uint32_t p0 = epilogue_pair<EPI, kHasBias>(acc[i][j][q * 4], acc[i][j][q * 4 + 1], bv[0], bv[1]);
          const uint32_t p1 = epilogue_pair<EPI, kHasBias>(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3], bv[2], bv[3]);
          *reinterpret_cast<uint2*>(so + (i * 32 + m) * OLD + cl) = make_uint2(p0, p1);
        }
      }
    }
  };
  if (has_bias) stage(std::true_type{});
  else stage(std::false_type{});
  store_staged_tile<EPI, TM, TN>(so, lane, C, b, R, live, N, wrow0, wcol0);
}

// XCD-aware workgroup -> (batch, tile_m, tile_n); returns false for padding workgroups.
__device__ __forceinline__ bool map_tile(int tiles_m, int tiles_n, int num_tiles, int tiles_per_xcd,
                                         int panel_rows, int& b, int& tile_m, int& tile_n) {
  const int logical = (blockIdx.x % kNumXcd) * tiles_per_xcd + blockIdx.x / kNumXcd;
  if (blockIdx.x / kNumXcd >= tiles_per_xcd || logical >= num_tiles) return false;
  const int per_batch = tiles_m * tiles_n;
  b = logical / per_batch;
  const int rem = logical - b * per_batch;
  const int panel = rem / (panel_rows * tiles_n);
  const int in_panel = rem - panel * panel_rows * tiles_n;
  const int rows_here = min(panel_rows, tiles_m - panel * panel_rows);
  tile_n = in_panel / rows_here;
  tile_m = panel * panel_rows + in_panel - tile_n * rows_here;
  return true;
}

// Ragged batches (only rows[b] leading rows of batch b are live).  A small kernel plans
// the launch first: the live row tiles of all batches, batch-major, form one list that
// is cut into kNumXcd equal runs, one per die, so that every die gets the same amount
// of work whatever the batches' sizes while a batch's weights are still read by one die
// (two, where a cut falls inside it).  Inside a die's run the tiles are ordered in
// panels as in map_tile.  plan[blockIdx] = (batch, tile_m, tile_n, live rows of the
// batch), batch -1 for a workgroup without work.  One launch plans up to two products
// (the two of an MLP differ in tile height and width).
// (RaggedGeom, PlanEntry and plan_entry, the scalar arithmetic of one plan entry, live in
// route_index.h; the kernels read an entry as one int4.)
static_assert(sizeof(PlanEntry) == sizeof(int4), "a plan entry is read as one int4");

__device__ __forceinline__ void plan_one(const RaggedGeom& g, const int32_t* tile_prefix,
                                         const int32_t* __restrict__ rows, int batch, int R,
                                         int i) {
  if (g.plan == nullptr || i >= g.num_blocks) return;
  g.plan[i] = plan_entry(g, tile_prefix, rows, batch, R, i);
}

// Entry num_blocks of a plan (one past its last workgroup) is its header: the number of live
// row tiles, from which a tile-walking kernel derives the length of its die's run, and the
// tag of the geometry the plan was written for (plan_tag).
// One workgroup of the planning launch (block = its index among the planning workgroups).
// With `fill` (G x batch fill counts of the slot assignment) the row counts are its column
// sums, added up here, and `rows` is not read: the plan then does not wait for the launch
// that writes the row counts and can share a launch with it.
__device__ __forceinline__ void plan_ragged_tiles_block(
    const int32_t* __restrict__ rows, const int32_t* __restrict__ fill, int G, int batch, int R,
    const RaggedGeom& ga, const RaggedGeom& gb, unsigned block, int32_t* tile_prefix) {
  // tile_prefix: 2 x (batch + 1) live row tiles before batch b, then `batch` row counts
  __shared__ int32_t wsum[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int32_t* pa = tile_prefix;
  int32_t* pb = tile_prefix + batch + 1;
  int32_t* rows_here = tile_prefix + 2 * (batch + 1);
  int carry_a = 0, carry_b = 0;
  for (int b0 = 0; b0 < batch; b0 += 256) {     // every workgroup scans all batches (few)
    const int bb = b0 + tid;
    int n = 0;
    if (bb < batch) {
      if (fill != nullptr) {
        for (int g = 0; g < G; ++g) n += fill[(size_t)g * batch + bb];
      } else {
        n = rows[bb];
      }
      n = min(max(n, 0), R);
      rows_here[bb] = n;
    }
    const int ta = (n + ga.bm - 1) / ga.bm, tb = (n + gb.bm - 1) / gb.bm;
    int xa = ta, xb = tb;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int ya = __shfl_up(xa, o, kWave), yb = __shfl_up(xb, o, kWave);
      if (lane >= o) { xa += ya; xb += yb; }
    }
    if (lane == 63) { wsum[0][wave] = xa; wsum[1][wave] = xb; }
    __syncthreads();
    int woff_a = 0, woff_b = 0, total_a = 0, total_b = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (w < wave) { woff_a += wsum[0][w]; woff_b += wsum[1][w]; }
      total_a += wsum[0][w];
      total_b += wsum[1][w];
    }
    if (bb < batch) {
      pa[bb] = carry_a + woff_a + xa - ta;
      pb[bb] = carry_b + woff_b + xb - tb;
    }
    carry_a += total_a;
    carry_b += total_b;
    __syncthreads();
  }
  if (tid == 0) { pa[batch] = carry_a; pb[batch] = carry_b; }
  __syncthreads();
  const int i = block * 256 + tid;
  plan_one(ga, pa, rows_here, batch, R, i);
  plan_one(gb, pb, rows_here, batch, R, i);
  if (block == 0) {
    if (tid == 0 && ga.plan != nullptr)
      ga.plan[ga.num_blocks] = PlanEntry{pa[batch], plan_tag(ga.bm, ga.tiles_n, ga.panel_rows, ga.num_blocks, batch, R), 0, 0};
    if (tid == 0 && gb.plan != nullptr)
      gb.plan[gb.num_blocks] = PlanEntry{pb[batch], plan_tag(gb.bm, gb.tiles_n, gb.panel_rows, gb.num_blocks, batch, R), 0, 0};
  }
}

// LDS of a planning workgroup.
inline size_t plan_ragged_tiles_lds(int batch) { return ((size_t)2 * (batch + 1) + batch) * sizeof(int32_t); }

__global__ __launch_bounds__(256) void plan_ragged_tiles_kernel(
    const int32_t* __restrict__ rows, int batch, int R, RaggedGeom ga, RaggedGeom gb) {
  extern __shared__ int32_t tile_prefix[];
  plan_ragged_tiles_block(rows, nullptr, 0, batch, R, ga, gb, blockIdx.x, tile_prefix);
}

// A launch plan as a product kernel is given it: the entries, the index of the header entry
// and the tag that the header must carry (plan_tag of the launch's own geometry).
struct PlanRef {
  const int4* entries;
  int blocks;
  int32_t tag;
};

// What the first launch of an expert MLP call does for the launches behind it on the stream
// (one workgroup's worth of stores, which would otherwise be a launch of their own): the
// counters of the second product's stream-K exchange start at zero in every call, and the
// call's status words are set to zero where the tag word does not say that they have been.
__device__ __forceinline__ void begin_call(int32_t* __restrict__ flags, int num_flags,
                                           int32_t* __restrict__ status, int tid, int threads) {
  if (flags != nullptr)
    for (int c = tid; c < num_flags; c += threads) flags[c] = 0;
  if (status != nullptr && tid == 0 && status[kStatusTagWord] != kStatusTag) {
    status[kStatusAbandonedWaits] = 0;
    status[kStatusPlanMismatches] = 0;
    status[kStatusTagWord] = kStatusTag;
  }
}

__global__ __launch_bounds__(256) void begin_call_kernel(int32_t* __restrict__ flags, int num_flags,
                                                         int32_t* __restrict__ status) {
  begin_call(flags, num_flags, status, threadIdx.x, 256);
}

// Reads a workgroup's plan entry.  False (and nothing may run) where the plan's header does
// not carry the launch's tag; workgroup 0 then counts the launch among the call's mismatches.
__device__ __forceinline__ bool read_plan(const PlanRef& ref, int32_t* __restrict__ status, int tid,
                                          int4& mine) {
  const int4 hdr = ref.entries[ref.blocks];
  mine = ref.entries[blockIdx.x];
  if (hdr.y == ref.tag) return true;
  if (blockIdx.x == 0 && tid == 0 && status != nullptr) status[kStatusPlanMismatches] += 1;
  return false;
}

// Fast path: Kd % BK == 0.  Global tiles go straight into LDS
// (global_load_lds_dwordx4: lane L of a wave lands at base + 16*L), so lane L
// fetches the global chunk that the XOR swizzle assigns to LDS slot L:
// row = L/8, slot = L%8, chunk = slot ^ (row & 7).
template <typename Cfg, int EPI>
__global__ __launch_bounds__(Cfg::kThreads, Cfg::kBlocksPerCu) void gemm_bf16_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bt, const bf16_t* __restrict__ bias,
    bf16_t* __restrict__ C, int R, int N, int Kd, int tiles_m, int tiles_n, int num_tiles,
    int tiles_per_xcd, int panel_rows, const int32_t* __restrict__ rows,
    PlanRef plan_ref, const int32_t* __restrict__ a_rows, int a_items,
    int32_t* __restrict__ clear, int clear_count, int32_t* __restrict__ status) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-resource builtins exist in the device pass only
  extern __shared__ __align__(1024) unsigned char smem[];
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
  constexpr int FM = Cfg::FM, FN = Cfg::FN;
  constexpr int RB = Cfg::kRowBytes;
  const int tid = threadIdx.x;
  const int4* plan = plan_ref.entries;
  if (blockIdx.x == 0) begin_call(clear, clear_count, status, tid, Cfg::kThreads);
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int m = lane & 31, h = lane >> 5;

  int b, tile_m, tile_n;
  // Ragged batches: only the first `live` rows of batch b hold data; tiles past them
  // have nothing to do, and the last tile stores only its live rows.
  int live = R;
  if (plan != nullptr) {
    int4 mine;
    if (!read_plan(plan_ref, status, tid, mine)) return;
    if (mine.x < 0) return;
    b = mine.x;
    tile_m = mine.y;
    tile_n = mine.z;
    live = mine.w;
  } else {
    if (!map_tile(tiles_m, tiles_n, num_tiles, tiles_per_xcd, panel_rows, b, tile_m, tile_n)) return;
    if (rows != nullptr) {
      live = min(rows[b], R);
      if (tile_m * BM >= live) return;
    }
  }
  const int row0 = tile_m * BM, col0 = tile_n * BN;
  // With a_rows, A is a matrix of items shared by all batches and a_rows[b * R + r] names
  // the item that row r of batch b holds: the gather of the dispatch step happens here,
  // in the operand load, and the dispatched buffer never exists.
  const unsigned char* Ab = reinterpret_cast<const unsigned char*>(
      a_rows != nullptr ? A : A + (size_t)b * R * Kd);
  const unsigned char* Bb = reinterpret_cast<const unsigned char*>(Bt + (size_t)b * N * Kd);

  // Byte offsets of this lane's chunk in each of its load instructions.  Lane L
  // of a DMA load lands in LDS slot L: row L / CPR, chunk slot L % CPR; it
  // therefore fetches global chunk  slot ^ swz(row).
  constexpr int CPR = Cfg::kChunksPerRow;
  constexpr int RPL = Cfg::kRowsPerLoad;
  const int lrow = lane / CPR;
  // (RPL * kWaves is a multiple of the swizzle period, so the row inside a wave's
  // load group determines the swizzle up to the wave's own offset.)
  const int chunk = (lane % CPR) ^ (((wave * RPL + lrow) >> Cfg::kSwzShift) & (CPR - 1));
  uint32_t a_goff[Cfg::kAIssues], b_goff[Cfg::kBIssues];
#pragma unroll
  for (int i = 0; i < Cfg::kAIssues; ++i) {
    int r = (i * Cfg::kWaves + wave) * RPL + lrow;
    int arow = min(row0 + r, (a_rows != nullptr ? live : R) - 1);
    // an entry outside the item matrix reads item 0 instead of leaving the buffer
    if (a_rows != nullptr) {
      arow = a_rows[(size_t)b * R + arow];
      arow = (unsigned)arow < (unsigned)a_items ? arow : 0;
    }
    a_goff[i] = (uint32_t)arow * (uint32_t)Kd * 2u + chunk * 16;
  }
#pragma unroll
  for (int i = 0; i < Cfg::kBIssues; ++i) {
    int r = (i * Cfg::kWaves + wave) * RPL + lrow;
    b_goff[i] = (uint32_t)min(col0 + r, N - 1) * (uint32_t)Kd * 2u + chunk * 16;
  }
  // A wave sustains about one 1 KB DMA load per 80 clocks, and a load that cannot be issued
  // (address FIFO full) holds up the MFMAs behind it: the loads of a k tile are spread out,
  // A rows under the second slice of one iteration, B rows under the first slice of the next.
  // Buffer addressing: the descriptor carries the operand's base, the lane's byte
  // offset is loop-invariant and the advance along k is a scalar, so a DMA load
  // needs no per-iteration address arithmetic and moves one address dword per
  // lane instead of two.
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<unsigned char*>(Ab), 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<unsigned char*>(Bb), 0, -1, 0x00020000);
  auto load_a = [&](int stage, int k0) {
    unsigned char* s = smem + stage * Cfg::kStageBytes;
#pragma unroll
    for (int i = 0; i < Cfg::kAIssues; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(s + (i * Cfg::kWaves + wave) * RPL * RB),
                                               16, a_goff[i], k0 * 2, 0, 0);
  };
  auto load_b = [&](int stage, int k0) {
    unsigned char* s = smem + stage * Cfg::kStageBytes;
#pragma unroll
    for (int i = 0; i < Cfg::kBIssues; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          b_rsrc, (lds_ptr_t)(s + BM * RB + (i * Cfg::kWaves + wave) * RPL * RB), 16, b_goff[i],
          k0 * 2, 0, 0);
  };

  floatx16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  bf16x8 fa[2][FM], fb[2][FN];
  const int a_row_off = (wm * Cfg::TM + m) * RB;
  const int b_row_off = BM * RB + (wn * Cfg::TN + m) * RB;
  const int swz = (m >> Cfg::kSwzShift) & (CPR - 1);
  auto load_frags = [&](int buf, int stage, int ks) {
    const unsigned char* s = smem + stage * Cfg::kStageBytes + (((2 * ks + h) ^ swz) * 16);
#pragma unroll
    for (int i = 0; i < FM; ++i)
      fa[buf][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(s + a_row_off + i * 32 * RB));
#pragma unroll
    for (int j = 0; j < FN; ++j)
      fb[buf][j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(s + b_row_off + j * 32 * RB));
  };

  // Main loop: a ring of NSTAGE LDS stages, the DMA loads run PD = NSTAGE-1 k
  // tiles ahead of the MFMAs and are never drained: the wait in front of the
  // tile barrier only covers the tile needed next (vmcnt leaves the younger
  // loads in flight).  The fragment reads of k slice s+1 are interleaved with
  // the MFMAs of slice s; the barrier of a tile sits before its last slice, so
  // the first fragments of the next tile are fetched under that slice's MFMAs.
  auto mfma_slice = [&](int buf) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
  };
  constexpr int KS = BK / 16;
  constexpr int NS = Cfg::NSTAGE, PD = NS - 1, L = Cfg::kLoads;
  constexpr int kReads = FM + FN;
  constexpr int kMfmas = FM * FN;
  static_assert(KS >= 2, "slice schedule");
  // Scheduling hints for one k slice (its own scheduling region): the LDS reads
  // of the next slice go out behind the first MFMAs (an MFMA leads, so the wait
  // for the previous slice's reads never covers a new read); the DMA loads
  // (first slice only) are spread over the remaining MFMAs.
  auto slice_schedule = [&](auto vmem_c) {
    constexpr int vmem = decltype(vmem_c)::value;
    constexpr int kLead = kReads < kMfmas ? kReads : kMfmas;
    constexpr int kReadsPer = (kReads + kLead - 1) / kLead;
    constexpr int kRest = kMfmas - kLead;
#pragma unroll
    for (int g = 0; g < kLead; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, kReadsPer, 0);
    }
    if constexpr (vmem > 0) {
      if constexpr (kRest > 0) {
        // one load in front of every (kRest / vmem)-th remaining MFMA
#pragma unroll
        for (int g = 0; g < kRest; ++g) {
          if (g * vmem / kRest != (g + 1) * vmem / kRest)
            __builtin_amdgcn_sched_group_barrier(0x020, (vmem + kRest - 1) / kRest, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
      } else {
        __builtin_amdgcn_sched_group_barrier(0x020, vmem, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // Waits until a k tile has landed, given how many tiles were issued after it.
  auto wait_tile = [&](int younger) {
    if (younger >= PD - 1) wait_vmcnt<(PD - 1) * L>();
    else if (PD >= 3 && younger == PD - 2) wait_vmcnt<(PD >= 3 ? PD - 2 : 0) * L>();
    else if (PD >= 4 && younger == PD - 3) wait_vmcnt<(PD >= 4 ? PD - 3 : 0) * L>();
    else wait_vmcnt<0>();
  };
  static_assert(PD <= 4, "wait_tile covers up to 4 tiles of prefetch");
  static_assert(KS == 2, "slice schedule");
  uint2 bias_pk[Cfg::TN / 8];
  load_bias<Cfg::TN>(bias_pk, bias, b, N, col0 + wn * Cfg::TN, lane);

  // All NS stages are in use: the barrier inside iteration kt (every wave has read
  // the last fragments of tile kt) frees stage kt % NS, and the loads of tile
  // kt + NS go out right behind it, under the MFMAs of the second k slice.
  const int nk = Kd / BK;
  const int pro = min(NS, nk);
  // Long k (more k tiles than stages): the B loads of a k tile go out one slice after its
  // A loads, under the first slice of the following iteration, so that a wave's DMA
  // requests come in two short bursts per iteration instead of one long one.
  const bool split = nk > NS;
#pragma unroll
  for (int t = 0; t < NS; ++t)
    if (t < pro) {
      load_a(t, t * BK);
      if (!split || t + 1 < NS) load_b(t, t * BK);
    }
  wait_tile(pro - 1);
  raw_barrier();
  load_frags(0, 0, 0);
  int stage = 0;
  if (split) {
    const int steady = nk - NS;
    int prev_stage = NS - 1;
    for (int kt = 0; kt < steady; ++kt) {
      const int next_stage = stage + 1 == NS ? 0 : stage + 1;
      load_frags(1, stage, 1);
      load_b(prev_stage, (kt + NS - 1) * BK);
      mfma_slice(0);
      slice_schedule(std::integral_constant<int, Cfg::kBIssues>{});
      wait_vmcnt<(PD - 1) * L>();
      wait_lgkmcnt0();
      raw_barrier();
      load_frags(0, next_stage, 0);
      load_a(stage, (kt + NS) * BK);
      mfma_slice(1);
      slice_schedule(std::integral_constant<int, Cfg::kAIssues>{});
      prev_stage = stage;
      stage = next_stage;
    }
    for (int kt = steady; kt < nk; ++kt) {
      const int next_stage = stage + 1 == NS ? 0 : stage + 1;
      load_frags(1, stage, 1);
      if (kt == steady) load_b(prev_stage, (nk - 1) * BK);
      mfma_slice(0);
      slice_schedule(std::integral_constant<int, 0>{});
      if (kt + 1 < nk) {
        wait_tile(nk - 2 - kt);
        wait_lgkmcnt0();
        raw_barrier();
        load_frags(0, next_stage, 0);
      }
      mfma_slice(1);
      slice_schedule(std::integral_constant<int, 0>{});
      stage = next_stage;
    }
  } else {
  // Steady state: the body is one basic block (no branches), so that the
  // scheduling hints hold and the fragment reads / DMA loads really are issued
  // under the MFMAs.  Tile kt + 1 has landed when only the PD - 1 tiles issued
  // after it are still in flight.
  const int steady = nk - NS;
  for (int kt = 0; kt < steady; ++kt) {
    const int next_stage = stage + 1 == NS ? 0 : stage + 1;
    const int load_k0 = (kt + NS) * BK;
    load_frags(1, stage, 1);
    mfma_slice(0);
    slice_schedule(std::integral_constant<int, 0>{});
    wait_vmcnt<(PD - 1) * L>();
    wait_lgkmcnt0();
    raw_barrier();
    load_frags(0, next_stage, 0);
    load_a(stage, load_k0);
    load_b(stage, load_k0);
    mfma_slice(1);
    slice_schedule(std::integral_constant<int, L>{});
    stage = next_stage;
  }
  // Drain: the last min(NS, nk) tiles, nothing left to load.
  for (int kt = steady > 0 ? steady : 0; kt < nk; ++kt) {
    const int next_stage = stage + 1 == NS ? 0 : stage + 1;
    load_frags(1, stage, 1);
    mfma_slice(0);
    slice_schedule(std::integral_constant<int, 0>{});
    if (kt + 1 < nk) {
      wait_tile(nk - 2 - kt);
      wait_lgkmcnt0();
      raw_barrier();
      load_frags(0, next_stage, 0);
    }
    mfma_slice(1);
    slice_schedule(std::integral_constant<int, 0>{});
    stage = next_stage;
  }
  }
  wait_lgkmcnt0();
  __syncthreads();   // all waves are done with the operand tiles: LDS is reused below
  mfma_result_fence();

  store_tile<EPI, Cfg::TM, Cfg::TN>(acc, smem, wave, lane, bias_pk, bias != nullptr, C, b, R, live,
                                    N, row0 + wm * Cfg::TM, col0 + wn * Cfg::TN);
#endif
}

// First-product form of gemm_bf16_kernel for k a multiple of 64 (128 x 256 tile, four waves,
// two workgroups per CU, same launch geometry and plan as GemmCfg<128, 256, 2, 2, 32, 3, 2>).
// The launch is bound by the rate at which the load path takes its DMA requests, and that
// rate depends on their shape: 64-byte row segments (32-wide k tiles) move at 9.5 TB/s,
// 128-byte segments at 13 and more.  The LDS that two workgroups per CU leave (80 KB each)
// does not hold two 64-wide stages of both operands, but it holds them for the B rows (the
// weights: two thirds of the requests): B sits in two slots of 64-wide k tiles (128-byte
// segments, 2 x 32 KB), A in two slots of 32-wide ones (64-byte segments, 2 x 8 KB).
// Iterations are 32 wide, one v_mfma_f32_16x16x32_bf16 deep: eight units of four MFMAs (the
// wave's four row blocks times one of its eight column blocks); a barrier stands in front of
// the first unit that reads fragments of the next k tile (unit 5).  The pair 2 J, 2 J + 1
// multiplies B slot J mod 2.
//   iteration 2 J      units 0-4: second half of the B rows of pair J + 1
//                      wait (that half may stay in flight), barrier
//                      units 5-7: A rows of k tile 2 J + 2
//   iteration 2 J + 1  units 0-4: nothing
//                      wait for everything, barrier (B slot J mod 2 is free from here on)
//                      units 5-7: A rows of k tile 2 J + 3, first half of the B rows of pair J + 2
// A load-only model of the launch: 350 us with 64-byte segments for both operands, 271 - 287
// with this mix.  The MFMA shape: the chip runs this product at its power limit, where the
// 16x16x32 instruction sustains about 14 % more flops than the 32x32x16 one; the same kernel
// written with 32x32x16 MFMAs (two slices of eight per iteration, barrier between them) took
// 0.970 - 0.977 ms per step of the B/16 layer against 0.949 - 0.957 (three alternating pairs).
// store_tile for sums in the layout of v_mfma_f32_16x16x32_bf16 with the B fragment first:
// acc[i][j][v] = C[row i * 16 + lane % 16][column j * 16 + (lane / 16) * 4 + v].
template <int EPI, int TM, int TN>
__device__ __forceinline__ void store_tile16(floatx4 (&acc)[TM / 16][TN / 16], unsigned char* smem,
                                             int wave, int lane, const uint2 (&bias_pk)[TN / 16],
                                             bool has_bias, bf16_t* __restrict__ C, int b, int R,
                                             int live, int N, int wrow0, int wcol0) {
  constexpr int FM = TM / 16, FN = TN / 16, OLD = TN + 8;
  const int n16 = lane & 15, g4 = lane >> 4;
  bf16_t* so = reinterpret_cast<bf16_t*>(smem) + (size_t)wave * TM * OLD;
  auto stage = [&](auto has_bias_c) {
    constexpr bool kHasBias = decltype(has_bias_c)::value;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int cl = j * 16 + g4 * 4;          // column inside the wave tile
      const uint2 bp = bias_pk[j];
      const float bv[4] = {bf_lo(bp.x), bf_hi(bp.x), bf_lo(bp.y), bf_hi(bp.y)};
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const uint32_t p0 = epilogue_pair<EPI, kHasBias>(acc[i][j][0], acc[i][j][1], bv[0], bv[1]);
        const uint32_t p1 = epilogue_pair<EPI, kHasBias>(acc[i][j][2], acc[i][j][3], bv[2], bv[3]);
        *reinterpret_cast<uint2*>(so + (i * 16 + n16) * OLD + cl) = make_uint2(p0, p1);
      }
    }
  };
  if (has_bias) stage(std::true_type{});
  else stage(std::false_type{});
  store_staged_tile<EPI, TM, TN>(so, lane, C, b, R, live, N, wrow0, wcol0);
}

template <int EPI>
__global__ __launch_bounds__(256, 2) void gemm_bf16_mixed_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bt, const bf16_t* __restrict__ bias,
    bf16_t* __restrict__ C, int R, int N, int Kd, int tiles_m, int tiles_n, int num_tiles,
    int tiles_per_xcd, int panel_rows, const int32_t* __restrict__ rows,
    PlanRef plan_ref, const int32_t* __restrict__ a_rows, int a_items,
    int32_t* __restrict__ clear, int clear_count, int32_t* __restrict__ status, int active_xcds) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-resource builtins exist in the device pass only
  extern __shared__ __align__(1024) unsigned char smem[];
  constexpr int BM = 128, BN = 256, TM = 64, TN = 128, FM = 4, FN = 8, kWaves = 4;   // FM x FN MFMA tiles of 16 x 16 per wave
  constexpr int kASlot = BM * 64, kBSlot = BN * 128, kBBase = 2 * kASlot;
  const int tid = threadIdx.x;
  const int4* plan = plan_ref.entries;
  if (blockIdx.x == 0) begin_call(clear, clear_count, status, tid, 256);
  if ((int)(blockIdx.x % kNumXcd) >= active_xcds) return;   // (measurement only, see active_units)
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int n16 = lane & 15, g4 = lane >> 4;

  int b, tile_m, tile_n;
  int live = R;
  if (plan != nullptr) {
    int4 mine;
    if (!read_plan(plan_ref, status, tid, mine)) return;
    if (mine.x < 0) return;
    b = mine.x;
    tile_m = mine.y;
    tile_n = mine.z;
    live = mine.w;
  } else {
    if (!map_tile(tiles_m, tiles_n, num_tiles, tiles_per_xcd, panel_rows, b, tile_m, tile_n)) return;
    if (rows != nullptr) {
      live = min(rows[b], R);
      if (tile_m * BM >= live) return;
    }
  }
  const int row0 = tile_m * BM, col0 = tile_n * BN;
  const unsigned char* Ab = reinterpret_cast<const unsigned char*>(
      a_rows != nullptr ? A : A + (size_t)b * R * Kd);
  const unsigned char* Bb = reinterpret_cast<const unsigned char*>(Bt + (size_t)b * N * Kd);

  // A request of A rows fills 16 rows x 64 bytes, one of B rows 8 rows x 128 bytes; lane L
  // lands in LDS position L of the request and fetches the piece that the XOR swizzle of its
  // row puts there.  Both swizzles go by row >> 1: for the fragment reads of this kernel (16
  // rows x one 16-byte piece per quarter wave) that is the one without bank conflicts on
  // 64-byte rows as well (a read-only probe: 1.89 ms against 2.70 with row >> 2, 2.52 without
  // a swizzle, 2.0 for the 128-byte rows).
  uint32_t a_goff[2], b_goff[8];
  {
    const int lrow = lane >> 2;
    const int piece = (lane & 3) ^ (((wave * 16 + lrow) >> 1) & 3);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int r = (i * kWaves + wave) * 16 + lrow;
      int arow = min(row0 + r, (a_rows != nullptr ? live : R) - 1);
      if (a_rows != nullptr) {
        arow = a_rows[(size_t)b * R + arow];
        arow = (unsigned)arow < (unsigned)a_items ? arow : 0;
      }
      a_goff[i] = (uint32_t)arow * (uint32_t)Kd * 2u + piece * 16;
    }
  }
  {
    const int lrow = lane >> 3;
    const int piece = (lane & 7) ^ (((wave * 8 + lrow) >> 1) & 7);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = (i * kWaves + wave) * 8 + lrow;
      b_goff[i] = (uint32_t)min(col0 + r, N - 1) * (uint32_t)Kd * 2u + piece * 16;
    }
  }
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<unsigned char*>(Ab), 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<unsigned char*>(Bb), 0, -1, 0x00020000);
  auto load_a = [&](int slot, int kt) {           // k tile kt (32 wide) -> A slot
    unsigned char* s = smem + slot * kASlot;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(s + (i * kWaves + wave) * 1024), 16,
                                               a_goff[i], kt * 64, 0, 0);
  };
  // B requests of a pair that go out with the first part (2, 3 and 4 measure the same, 5 and
  // 6 cost 3 and 11 us)
  constexpr int kBFirst = 4;
  auto load_b_half = [&](int slot, int pair, auto half) {   // pair of k tiles (64 wide) -> B slot
    unsigned char* s = smem + kBBase + slot * kBSlot;
    constexpr int i0 = decltype(half)::value ? kBFirst : 0;
    constexpr int i1 = decltype(half)::value ? 8 : kBFirst;
#pragma unroll
    for (int i = i0; i < i1; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (lds_ptr_t)(s + (i * kWaves + wave) * 1024), 16,
                                               b_goff[i], pair * 128, 0, 0);
  };
  using Half0 = std::integral_constant<int, 0>;
  using Half1 = std::integral_constant<int, 1>;

  floatx4 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;
  // v_mfma_f32_16x16x32_bf16: a lane supplies 8 consecutive k of one row (row = lane % 16,
  // k = 8 * (lane / 16) of the 32-wide iteration).  An iteration is FN units, one per column
  // block: four MFMAs (the wave's four row blocks times that column block).  The wave holds
  // the A fragments of the iteration, reads those of the next one during its last two units,
  // and keeps the B fragments of the next kLook units in flight.
  constexpr int kLook = 3, kRing = kLook + 1;
  static_assert(FN % kRing == 0, "fragment ring");
  constexpr int kBarrierUnit = FN - kLook;      // first unit that reads from the next k tile
  bf16x8 fa[2][FM], fb[kRing];
  const int a_row_off = (wm * TM + n16) * 64;
  const int b_row_off = kBBase + (wn * TN + n16) * 128;
  const int swz_a = (n16 >> 1) & 3, swz_b = (n16 >> 1) & 7;
  auto read_a = [&](int buf, int kt, int i) {
    fa[buf][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
        smem + (kt & 1) * kASlot + a_row_off + i * 16 * 64 + ((g4 ^ swz_a) * 16)));
  };
  auto read_b = [&](int buf, int kt, int j) {
    fb[buf] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
        smem + ((kt >> 1) & 1) * kBSlot + b_row_off + j * 16 * 128 + ((((kt & 1) * 4 + g4) ^ swz_b) * 16)));
  };
  uint2 bias_pk[FN];
#pragma unroll
  for (int j = 0; j < FN; ++j) {
    bias_pk[j] = make_uint2(0, 0);
    if (bias != nullptr) {
      const int col = col0 + wn * TN + j * 16 + g4 * 4;
      const bf16_t* src = bias + (size_t)b * N;
      if ((N & 3) == 0) {
        bias_pk[j] = *reinterpret_cast<const uint2*>(src + min(col, N - 4));
      } else {
        uint32_t v[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) v[t] = src[min(col + t, N - 1)];
        bias_pk[j] = make_uint2(v[0] | (v[1] << 16), v[2] | (v[3] << 16));
      }
    }
  }

  // Units lo .. hi - 1 of iteration kt (fragment set par = kt & 1 as a constant); `next`: the
  // k tile kt + 1 exists, so the units from kBarrierUnit on read its first fragments; `dma`
  // requests go out under these units, spread evenly.
  auto units = [&](auto lo_c, auto hi_c, auto par_c, int kt, auto next_c, auto dma_c) __attribute__((always_inline)) {
    constexpr int lo = decltype(lo_c)::value, hi = decltype(hi_c)::value, par = decltype(par_c)::value;
    constexpr bool next = decltype(next_c)::value;
    constexpr int dma = decltype(dma_c)::value;
    static_for<hi - lo>([&](auto c) __attribute__((always_inline)) {
      constexpr int j = lo + decltype(c)::value;
      constexpr int jl = j + kLook;
      constexpr bool rb = jl < FN || next;
      constexpr bool ra = next && j >= FN - 2;
      if constexpr (jl < FN) read_b(jl % kRing, kt, jl);
      else if constexpr (next) read_b(jl % kRing, kt + 1, jl - FN);
      if constexpr (ra) {
        read_a(par ^ 1, kt + 1, 2 * (j - (FN - 2)));
        read_a(par ^ 1, kt + 1, 2 * (j - (FN - 2)) + 1);
      }
#pragma unroll
      for (int i = 0; i < FM; ++i)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[j % kRing], fa[par][i], acc[i][j], 0, 0, 0);
      constexpr int u = j - lo, n = hi - lo;
      constexpr int dma_here = (u + 1) * dma / n - u * dma / n;
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if constexpr (rb) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if constexpr (ra) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if constexpr (ra) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if constexpr (dma_here > 0) __builtin_amdgcn_sched_group_barrier(0x020, dma_here, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    });
    __builtin_amdgcn_sched_barrier(0);
  };
  using U0 = std::integral_constant<int, 0>;
  using UB = std::integral_constant<int, kBarrierUnit>;
  using UN = std::integral_constant<int, FN>;
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;

  const int nk = Kd / 32;          // even, at least 4: the launcher checks
  load_a(0, 0);
  load_b_half(0, 0, Half0{});
  load_b_half(0, 0, Half1{});
  load_a(1, 1);
  load_b_half(1, 1, Half0{});
  wait_vmcnt<2 + kBFirst>();       // k tile 0 has landed: A rows of k tile 1 and the first part of a B slot may be in flight
  raw_barrier();
#pragma unroll
  for (int i = 0; i < FM; ++i) read_a(0, 0, i);
#pragma unroll
  for (int u = 0; u < kLook; ++u) read_b(u, 0, u);
  // Pair J = iterations 2 J and 2 J + 1 (B slot J mod 2).  B1: pair J + 1 exists; A2 / A3: k
  // tiles 2 J + 2 / 2 J + 3 exist; B2: pair J + 2 exists.  Requests and barriers as described
  // above the kernel; a barrier stands in front of the first unit that reads from the next k tile.
  auto pair = [&](int J, auto b1_c, auto a2_c, auto a3_c, auto b2_c) __attribute__((always_inline)) {
    constexpr bool B1 = decltype(b1_c)::value, A2 = decltype(a2_c)::value;
    constexpr bool A3 = decltype(a3_c)::value, B2 = decltype(b2_c)::value;
    const int kt = 2 * J;
    if constexpr (B1) load_b_half((J + 1) & 1, J + 1, Half1{});
    units(U0{}, UB{}, P0{}, kt, std::true_type{}, std::integral_constant<int, B1 ? 8 - kBFirst : 0>{});
    wait_vmcnt<B1 ? 8 - kBFirst : 0>();
    wait_lgkmcnt0();
    raw_barrier();
    if constexpr (A2) load_a(0, kt + 2);
    units(UB{}, UN{}, P0{}, kt, std::true_type{}, std::integral_constant<int, A2 ? 2 : 0>{});
    units(U0{}, UB{}, P1{}, kt + 1, std::bool_constant<A2>{}, U0{});
    if constexpr (A2) {
      wait_vmcnt<0>();
      wait_lgkmcnt0();
      raw_barrier();
    }
    if constexpr (A3) load_a(1, kt + 3);
    if constexpr (B2) load_b_half(J & 1, J + 2, Half0{});
    units(UB{}, UN{}, P1{}, kt + 1, std::bool_constant<A2>{},
          std::integral_constant<int, (A3 ? 2 : 0) + (B2 ? kBFirst : 0)>{});
  };
  using T = std::true_type;
  using F = std::false_type;
  const int npairs = nk / 2;
  for (int J = 0; J < npairs - 2; ++J) pair(J, T{}, T{}, T{}, T{});
  pair(npairs - 2, T{}, T{}, T{}, F{});
  pair(npairs - 1, F{}, F{}, F{}, F{});
  wait_lgkmcnt0();
  __syncthreads();   // all waves are done with the operand tiles: LDS is reused below
  mfma_result_fence();
  store_tile16<EPI, TM, TN>(acc, smem, wave, lane, bias_pk, bias != nullptr, C, b, R, live, N,
                            row0 + wm * TM, col0 + wn * TN);
#endif
}

// Generic path (any Kd % 8 == 0): 128x128 tile, operands staged through
// registers into padded LDS rows, out-of-range k chunks zero-filled.
// Persistent variant for long k (the second product of an MLP): one workgroup per CU
// walks its die's tiles.  The operand ring is never drained between tiles (the last
// NSTAGE iterations of a tile request the first k tiles of the next one, so a tile's
// first loads and the store traffic of the one before are off the critical path), and
// the output leaves through a staging region of its own, 32 rows per wave at a time.
// Operand offsets are relative to the whole arrays (the next tile may belong to another
// batch): batch * R * Kd * 2 and batch * N * Kd * 2 must fit 32 bits.
constexpr int kCusPerXcd = 32;

template <typename Cfg>
struct PersistentLds {
  // Two stages of 64-wide k tiles: the A rows get a ring of three slots and the B rows one
  // of two (all of the 160 KB of LDS), so that a k tile's A rows can be requested two
  // iterations ahead and stay in flight across the barrier of the iteration in between.
  static constexpr bool kDeepA = Cfg::NSTAGE == 2 && Cfg::BK == 64 &&
                                 (size_t)(3 * Cfg::BM + 2 * Cfg::BN) * Cfg::kRowBytes <= 160 * 1024;
  static constexpr size_t kABytes = (size_t)Cfg::BM * Cfg::kRowBytes;
  static constexpr size_t kBBytes = (size_t)Cfg::BN * Cfg::kRowBytes;
  static constexpr size_t kRing = kDeepA ? 3 * kABytes + 2 * kBBytes : (size_t)Cfg::NSTAGE * Cfg::kStageBytes;
  // The output is staged 32 rows per wave at a time, over the whole width of the wave tile
  // where the ring leaves room for that, else in two halves.  With the deep A ring the
  // staging region is the A slot that the finished tile's last k tile has just left.
  static constexpr size_t kFullStaging = (size_t)Cfg::kWaves * 32 * (Cfg::TN + 8) * sizeof(bf16_t);
  static constexpr size_t kRoom = kDeepA ? kABytes : 160 * 1024 - kRing;
  static constexpr int kStageCols = kFullStaging <= kRoom ? Cfg::TN : Cfg::TN / 2;
  static constexpr int kOutLd = kStageCols + 8;
  static constexpr size_t kStaging = (size_t)Cfg::kWaves * 32 * kOutLd * sizeof(bf16_t);
  static constexpr size_t kBytes = kDeepA ? kRing : kRing + kStaging;
  static_assert(kStageCols % 32 == 0, "staging covers whole MFMA tiles");
  static_assert(kStaging <= kRoom, "staging region");
  static_assert(kBytes <= 160 * 1024, "LDS budget");
};

// HAS_BIAS is a template parameter: a run-time choice between two epilogues keeps the
// accumulators alive across a branch and costs 556 bytes of scratch per lane.
template <typename Cfg, int EPI, bool HAS_BIAS>
__global__ __launch_bounds__(Cfg::kThreads, 1) void gemm_bf16_persistent_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bt, const bf16_t* __restrict__ bias,
    bf16_t* __restrict__ C, int R, int N, int Kd, int tiles_m, int tiles_n, int num_tiles,
    int tiles_per_xcd, int panel_rows, PlanRef plan_ref,
    float* __restrict__ sk_partials, int32_t* __restrict__ sk_flags, int32_t* __restrict__ status,
    int spin_limit, int wait_bias, int active_xcds, int active_slots) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-resource builtins exist in the device pass only
  extern __shared__ __align__(1024) unsigned char smem[];
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
  constexpr int FM = Cfg::FM, FN = Cfg::FN;
  constexpr int RB = Cfg::kRowBytes;
  constexpr int NS = Cfg::NSTAGE, PD = NS - 1, L = Cfg::kLoads;
  constexpr int KS = BK / 16;    // k slices (one MFMA deep) per k tile: 2 or 4
  const int tid = threadIdx.x;
  const int4* plan = plan_ref.entries;
  const int plan_blocks = plan_ref.blocks;
  // A plan whose header does not carry this launch's tag was written for other shapes, or
  // never: nothing runs, and the call's status words say so.
  if (plan != nullptr && plan[plan_blocks].y != plan_ref.tag) {
    if (blockIdx.x == 0 && tid == 0 && status != nullptr) atomicAdd(status + kStatusPlanMismatches, 1);
    return;
  }
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int m = lane & 31, h = lane >> 5;
  const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
  if (xcd >= active_xcds || slot >= active_slots) return;   // (measurement only, see active_units)
  constexpr int CPR = Cfg::kChunksPerRow;
  constexpr int RPL = Cfg::kRowsPerLoad;
  const int lrow = lane / CPR;
  const int chunk = (lane % CPR) ^ (((wave * RPL + lrow) >> Cfg::kSwzShift) & (CPR - 1));

  // Work of this workgroup: every kCusPerXcd-th entry of its die's run (the plan of a ragged
  // launch, else the static order of map_tile), so that the tiles in flight on a die at
  // any time are neighbours in that order, plus its share of the die's last, partial
  // round (stream-K pieces, see streamk_share).
  const int nk = Kd / BK;      // at least 2 * NS
  int die_tiles;
  if (plan != nullptr) {
    const int total = plan[plan_blocks].x;               // live row tiles of all batches
    const int share = (total + kNumXcd - 1) / kNumXcd;
    die_tiles = max(0, min(xcd * share + share, total) - xcd * share) * tiles_n;
  } else {
    die_tiles = max(0, min(tiles_per_xcd, num_tiles - xcd * tiles_per_xcd));
  }
  die_tiles = __builtin_amdgcn_readfirstlane(die_tiles);
  constexpr bool kCanShare = kStreamKGranule >= 2 * NS - 1;   // a piece covers the ring's fill and drain
  const StreamKShare share_ =
      streamk_share(die_tiles, kCusPerXcd, slot, nk, kCanShare && sk_partials != nullptr);
  const int num_items = share_.rounds + share_.pieces;
  struct TileCtx {
    int b, row0, col0, live;
    int kbeg, kcnt;       // k tiles of this item
    int shared;           // index of the tile among the die's shared ones (its sums and counter)
    int waits;            // deposits of the tile's other pieces that this item waits for and adds
    int leaves_sums;      // 1: the item deposits its sums; 0: it runs the epilogue
    uint32_t a[Cfg::kAIssues], bo[Cfg::kBIssues];
  };
  auto setup_tile = [&](int i, TileCtx& t) -> bool {
    if (i >= num_items) return false;
    int s_ = slot + i * kCusPerXcd;
    t.kbeg = 0;
    t.kcnt = nk;
    t.shared = 0;
    t.waits = 0;
    t.leaves_sums = 0;
    if (i >= share_.rounds) {
      s_ = share_.tile + (i - share_.rounds);
      t.kbeg = share_.kbeg;
      t.kcnt = share_.kcnt;
      t.shared = s_ - share_.rounds * kCusPerXcd;
      t.waits = share_.waits;
      t.leaves_sums = share_.last ? 0 : 1;
    }
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
    // (wave-uniform values, kept in scalar registers)
    t.b = __builtin_amdgcn_readfirstlane(t.b);
    t.live = __builtin_amdgcn_readfirstlane(t.live);
    t.row0 = __builtin_amdgcn_readfirstlane(tile_m * BM);
    t.col0 = __builtin_amdgcn_readfirstlane(tile_n * BN);
    t.kbeg = __builtin_amdgcn_readfirstlane(t.kbeg);
    t.kcnt = __builtin_amdgcn_readfirstlane(t.kcnt);
    t.shared = __builtin_amdgcn_readfirstlane(t.shared);
    t.waits = __builtin_amdgcn_readfirstlane(t.waits);
    t.leaves_sums = __builtin_amdgcn_readfirstlane(t.leaves_sums);
#pragma unroll
    for (int u = 0; u < Cfg::kAIssues; ++u) {
      const int r = (u * Cfg::kWaves + wave) * RPL + lrow;
      t.a[u] = (uint32_t)(t.b * R + min(t.row0 + r, R - 1)) * (uint32_t)Kd * 2u + chunk * 16;
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
  auto load_ktile = [&](const TileCtx& t, int stage, int k0) {
    unsigned char* s = smem + stage * Cfg::kStageBytes;
#pragma unroll
    for (int u = 0; u < Cfg::kAIssues; ++u)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(s + (u * Cfg::kWaves + wave) * RPL * RB),
                                               16, t.a[u], k0 * 2, 0, 0);
#pragma unroll
    for (int u = 0; u < Cfg::kBIssues; ++u)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          b_rsrc, (lds_ptr_t)(s + BM * RB + (u * Cfg::kWaves + wave) * RPL * RB), 16, t.bo[u], k0 * 2,
          0, 0);
  };

  floatx16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  bf16x8 fa[2][FM], fb[2][FN];
  const int a_row_off = (wm * Cfg::TM + m) * RB;
  const int b_row_off = BM * RB + (wn * Cfg::TN + m) * RB;
  const int swz = (m >> Cfg::kSwzShift) & (CPR - 1);
  auto load_frags = [&](int buf, int stage, int ks) {
    const unsigned char* s = smem + stage * Cfg::kStageBytes + (((2 * ks + h) ^ swz) * 16);
#pragma unroll
    for (int i = 0; i < FM; ++i)
      fa[buf][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(s + a_row_off + i * 32 * RB));
#pragma unroll
    for (int j = 0; j < FN; ++j)
      fb[buf][j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(s + b_row_off + j * 32 * RB));
  };
  auto mfma_slice = [&](int buf) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
  };
  // First slice of a tile: the sums start from zero in the MFMA itself, so the epilogue need
  // not clear 256 accumulator registers.
  auto mfma_slice_first = [&](int buf) {
    const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i], zero, 0, 0, 0);
  };
  // Same issue order inside a k slice as gemm_bf16_kernel: fragment reads behind the first
  // MFMAs, the DMA loads (second slice only) spread over the rest.
  constexpr int kReads = FM + FN, kMfmas = FM * FN;
  auto slice_schedule = [&](auto vmem_c) {
    constexpr int vmem = decltype(vmem_c)::value;
    constexpr int kLead = kReads < kMfmas ? kReads : kMfmas;
    constexpr int kReadsPer = (kReads + kLead - 1) / kLead;
    constexpr int kRest = kMfmas - kLead;
#pragma unroll
    for (int g = 0; g < kLead; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, kReadsPer, 0);
    }
    if constexpr (vmem > 0 && kRest > 0) {
#pragma unroll
      for (int g = 0; g < kRest; ++g) {
        if (g * vmem / kRest != (g + 1) * vmem / kRest)
          __builtin_amdgcn_sched_group_barrier(0x020, (vmem + kRest - 1) / kRest, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // Deep A ring (PersistentLds::kDeepA).  Iteration j multiplies k tile j out of A slot
  // j mod 3 and B slot j mod 2, four DMA requests per wave under each of its four slices:
  //   slice 0   second half of the B rows of k tile j + 1 (into the other B slot)
  //   slice 1   first half of the A rows of k tile j + 2 (into the A slot that k tile j - 1
  //   slice 2   second half of them                       left at the last barrier)
  //   wait until only those A requests are in flight; barrier (every wave has read the
  //   last fragments of k tile j)
  //   slice 3   first half of the B rows of k tile j + 2 (into k tile j's B slot)
  // A k tile's A rows (the operand that comes from HBM) have about 1.5 iterations to
  // arrive and stay in flight across a barrier, where two whole stages drained at every
  // barrier allowed 1 and 0.6; and no slice carries more than four requests (a request
  // that cannot be issued holds up the MFMAs behind it).  A model of the loop (these
  // requests, the fragment reads and the MFMAs on the second product's shape) takes 386 us
  // with two drained stages, 338 with the ring and two bursts of eight, 296 with this one.
  constexpr bool kDeepA = PersistentLds<Cfg>::kDeepA;
  constexpr int kABytes = (int)PersistentLds<Cfg>::kABytes, kBBytes = (int)PersistentLds<Cfg>::kBBytes;
  constexpr int kHalfA = Cfg::kAIssues / 2, kHalfB = Cfg::kBIssues / 2;
  auto ring_load_a = [&](const TileCtx& t, int slot_a, int k0, auto half) {
    unsigned char* s = smem + slot_a * kABytes;
    constexpr int u0 = decltype(half)::value * kHalfA;
#pragma unroll
    for (int u = u0; u < u0 + kHalfA; ++u)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(s + (u * Cfg::kWaves + wave) * RPL * RB),
                                               16, t.a[u], k0 * 2, 0, 0);
  };
  auto ring_load_b = [&](const TileCtx& t, int slot_b, int k0, auto half) {
    unsigned char* s = smem + 3 * kABytes + slot_b * kBBytes;
    constexpr int u0 = decltype(half)::value * kHalfB;
#pragma unroll
    for (int u = u0; u < u0 + kHalfB; ++u)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (lds_ptr_t)(s + (u * Cfg::kWaves + wave) * RPL * RB),
                                               16, t.bo[u], k0 * 2, 0, 0);
  };
  using Half0 = std::integral_constant<int, 0>;
  using Half1 = std::integral_constant<int, 1>;
  const int ring_b_row_off = 3 * kABytes + (wn * Cfg::TN + m) * RB;
  auto ring_frags = [&](int buf, int slot_a, int slot_b, int ks) {
    const int col = ((2 * ks + h) ^ swz) * 16;
    const unsigned char* pa = smem + slot_a * kABytes + a_row_off + col;
    const unsigned char* pb = smem + slot_b * kBBytes + ring_b_row_off + col;
#pragma unroll
    for (int i = 0; i < FM; ++i)
      fa[buf][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(pa + i * 32 * RB));
#pragma unroll
    for (int j = 0; j < FN; ++j)
      fb[buf][j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(pb + j * 32 * RB));
  };
  // SRC, K0: k tile j + 2; PSRC, PK0: k tile j + 1.
#define VMOE_PERSISTENT_K_ITERATION_RING(SRC, K0, PSRC, PK0, FIRST) do { \
    const int prev_a = sa == 0 ? 2 : sa - 1, next_a = sa == 2 ? 0 : sa + 1; \
    ring_frags(1, sa, sb, 1); \
    ring_load_b(PSRC, sb ^ 1, (PK0), Half1{}); \
    if constexpr (FIRST) mfma_slice_first(0); else mfma_slice(0); \
    slice_schedule(std::integral_constant<int, kHalfB>{}); \
    ring_frags(0, sa, sb, 2); \
    ring_load_a(SRC, prev_a, (K0), Half0{}); \
    mfma_slice(1); \
    slice_schedule(std::integral_constant<int, kHalfA>{}); \
    ring_frags(1, sa, sb, 3); \
    ring_load_a(SRC, prev_a, (K0), Half1{}); \
    mfma_slice(0); \
    slice_schedule(std::integral_constant<int, kHalfA>{}); \
    wait_vmcnt<Cfg::kAIssues>(); \
    wait_lgkmcnt0(); \
    raw_barrier(); \
    ring_frags(0, next_a, sb ^ 1, 0); \
    ring_load_b(SRC, sb, (K0), Half0{}); \
    mfma_slice(1); \
    slice_schedule(std::integral_constant<int, kHalfB>{}); \
    sa = next_a; \
    sb ^= 1; \
  } while (0)
  // One k tile of the plain ring of NS stages.  WAITED = the k tile needed next is known to
  // be complete (every wave drained its loads before the last output was staged, or in the
  // prologue).  Macros: as lambdas taking the tile by reference the offsets end up in
  // scratch memory.
#define VMOE_PERSISTENT_K_ITERATION(SRC, K0, WAITED) do { \
    const int next_stage = stage + 1 == NS ? 0 : stage + 1; \
    _Pragma("unroll") \
    for (int ks = 0; ks + 1 < KS; ++ks) { \
      load_frags((ks + 1) & 1, stage, ks + 1); \
      mfma_slice(ks & 1); \
      slice_schedule(std::integral_constant<int, 0>{}); \
    } \
    if constexpr (!(WAITED)) wait_vmcnt<(PD - 1) * L>(); \
    wait_lgkmcnt0(); \
    raw_barrier(); \
    load_frags(0, next_stage, 0); \
    load_ktile(SRC, stage, (K0)); \
    mfma_slice((KS - 1) & 1); \
    slice_schedule(std::integral_constant<int, L>{}); \
    stage = next_stage; \
  } while (0)

  TileCtx cur, nxt;
  if (!setup_tile(0, cur)) return;
  int stage = 0;
  int sa = 0, sb = 0;      // slots of the k tile that the next iteration multiplies (deep A ring)
  if constexpr (kDeepA) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      ring_load_a(cur, t, (cur.kbeg + t) * BK, Half0{});
      ring_load_a(cur, t, (cur.kbeg + t) * BK, Half1{});
      ring_load_b(cur, t, (cur.kbeg + t) * BK, Half0{});
      if (t == 0) ring_load_b(cur, t, (cur.kbeg + t) * BK, Half1{});   // (k tile 1's: first iteration)
    }
    wait_vmcnt<0>();
    raw_barrier();
    ring_frags(0, 0, 0, 0);
  } else {
#pragma unroll
    for (int t = 0; t < NS; ++t) load_ktile(cur, t, (cur.kbeg + t) * BK);
    wait_vmcnt<0>();
    raw_barrier();
    load_frags(0, 0, 0);
  }
  constexpr int OLD = PersistentLds<Cfg>::kOutLd;
  // Sums in memory: one tile per workgroup, in the order of the accumulator registers (a
  // wave's store or load covers 1 KB of consecutive memory).
  constexpr size_t kTileVecs = (size_t)BM * BN / 4;
  const __amdgpu_buffer_rsrc_t sums_rsrc = __builtin_amdgcn_make_buffer_rsrc(sk_partials, 0, -1, 0x00020000);
  const int vec0 = wave * FM * FN * 4 * 64 + lane;
  for (int ti = 0;; ++ti) {
    const bool has_next = setup_tile(ti + 1, nxt);
    if (!has_next) nxt = cur;   // the last tile requests its own first k tiles again: in bounds, never read
    uint2 bias_pk[Cfg::TN / 8];
    load_bias<Cfg::TN>(bias_pk, bias, cur.b, N, cur.col0 + wn * Cfg::TN, lane);
    const int kc = __builtin_amdgcn_readfirstlane(cur.kcnt);
    // (without the bounds the compiler plans for trip counts that cannot occur and spills)
    __builtin_assume(kc >= 2 * NS && kc <= nk);
    const int kb = __builtin_amdgcn_readfirstlane(cur.kbeg), nkb = __builtin_amdgcn_readfirstlane(nxt.kbeg);
    if constexpr (kDeepA) {
      VMOE_PERSISTENT_K_ITERATION_RING(cur, (kb + 2) * BK, cur, (kb + 1) * BK, true);
      for (int kt = 1; kt < kc - 2; ++kt)
        VMOE_PERSISTENT_K_ITERATION_RING(cur, (kb + kt + 2) * BK, cur, (kb + kt + 1) * BK, false);
      VMOE_PERSISTENT_K_ITERATION_RING(nxt, nkb * BK, cur, (kb + kc - 1) * BK, false);
      VMOE_PERSISTENT_K_ITERATION_RING(nxt, (nkb + 1) * BK, nxt, nkb * BK, false);
    } else {
#pragma unroll
      for (int kt = 0; kt < NS - 1; ++kt) VMOE_PERSISTENT_K_ITERATION(cur, (kb + kt + NS) * BK, true);
      for (int kt = NS - 1; kt < kc - NS; ++kt) VMOE_PERSISTENT_K_ITERATION(cur, (kb + kt + NS) * BK, false);
      for (int kt = kc - NS; kt < kc; ++kt) VMOE_PERSISTENT_K_ITERATION(nxt, (nkb + kt + NS - kc) * BK, false);
    }
    // The first NS k tiles of the next tile are complete before the staging region is
    // touched (no load that writes LDS is pending while the output is staged), and the
    // first NS - 1 iterations of the next tile need no wait of their own.
    wait_vmcnt<0>();
    mfma_result_fence();
    // Staging region: behind the ring, or (deep A ring) the A slot of the k tile multiplied
    // last, which no wave reads after that iteration's barrier and which the next request
    // for A rows (first slice of the next tile's first iteration) will fill: the barrier
    // at the end of the epilogue keeps that request behind every wave's staged rows.
    bf16_t* so = reinterpret_cast<bf16_t*>(
        smem + (kDeepA ? (size_t)(sa == 0 ? 2 : sa - 1) * kABytes : PersistentLds<Cfg>::kRing)) + (size_t)wave * 32 * OLD;
    // A piece of a shared tile that is not the first to finish adds the sums deposited so
    // far, chunk by chunk in the epilogue below, the loads kAhead chunks ahead of their
    // use.  The other pieces were computed at the same time as this one, in workgroups
    // with lower indices (placed before this one), so the wait is short.  That rests on all
    // workgroups of the launch being resident at once, which holds on a GPU this launch has
    // to itself; a kernel of another stream that holds compute units can keep a producer
    // from starting while its consumer waits.  The wait is therefore bounded, and a piece
    // that gives up does not pass off what it finds in memory as sums: it counts itself in
    // the call's status words and turns every sum it would have taken into NaN, which the
    // pieces behind it and the output rows then carry.
    const int waits = __builtin_amdgcn_readfirstlane(cur.waits);
    const bool adds_sums = waits > 0;
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    constexpr int kAhead = 8, kChunks = FM * FN * 4;
    // The sums are written through to memory and read past the caches (sc0 sc1 on both
    // sides): producer and consumer need no cache-wide write-back or invalidate (a
    // device-scope fence here writes back the whole L2, once per wave), and the exchange
    // does not depend on both workgroups sharing a die's L2.
    constexpr int kSumsAux = 1 | 16;
    const int shared_index = xcd * kCusPerXcd + __builtin_amdgcn_readfirstlane(cur.shared);
    const int sums_base = shared_index * (int)(kTileVecs * 16);
    u32x4_t ahead[kAhead];
    bool poisoned = false;
    if (adds_sums) {
      const int32_t* f = sk_flags + shared_index;
      const int awaited = waits + wait_bias;    // (wait_bias: 0 outside the test of this path)
      if (tid == 0) {
        int spins = 0;
        while (__hip_atomic_load(f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < awaited) {
          __builtin_amdgcn_s_sleep(16);
          if (++spins > spin_limit) {
            if (status != nullptr) atomicAdd(status + kStatusAbandonedWaits, 1);
            break;
          }
        }
      }
      __syncthreads();
      // (every wave looks for itself: the deposits are there, or its sums are poisoned)
      poisoned = __builtin_amdgcn_readfirstlane(
          (int)(__hip_atomic_load(f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < awaited)) != 0;
#pragma unroll
      for (int c = 0; c < kAhead; ++c)
        ahead[c] = __builtin_amdgcn_raw_buffer_load_b128(sums_rsrc, vec0 * 16, sums_base + c * 1024, kSumsAux);
    }
    const bool leaves_sums = __builtin_amdgcn_readfirstlane(cur.leaves_sums) != 0;
    // An item that ends inside its tile leaves its sums for the piece that continues it: the
    // epilogue below stores each group of four as float32 on its way (one code path for the
    // accumulators) and no row of the output.
    const int live_rows = leaves_sums ? 0 : cur.live;
    bf16_t* Cb = C + (size_t)cur.b * R * N;
    const int wrow0 = cur.row0 + wm * Cfg::TM, wcol0 = cur.col0 + wn * Cfg::TN;
    constexpr int SC = PersistentLds<Cfg>::kStageCols;   // columns staged at a time
    constexpr int kChunksOut = SC / 8;
    constexpr int kRowsPerPass = 64 / kChunksOut;
    static_assert(64 % kChunksOut == 0 && 32 % kRowsPerPass == 0, "staged width must divide a wave");
    const int oc = (lane % kChunksOut) * 8;
    const int orow = lane / kChunksOut;
    // A whole tile (the common case) takes a copy of the epilogue without the branches of
    // the shared ones: with two uniform branches per group of four sums and a divergent
    // one around every store the epilogue was some 250 basic blocks, 18 k clocks per tile
    // (14 % of the launch).  Rows and columns past the edge leave through the range check
    // of a buffer store instead of a branch.
    const bool c_small = (uint64_t)R * N * 2 < (1ull << 31);
    if (!adds_sums && !leaves_sums && c_small) {
      // (the tile's batch is the same in every lane; said explicitly, or every store
      // sits in a loop over the distinct descriptors of the wave)
      const uint64_t cb_bits = reinterpret_cast<uint64_t>(Cb);
      bf16_t* cb_uniform = reinterpret_cast<bf16_t*>(
          ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(cb_bits >> 32)) << 32) |
          (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)cb_bits));
      const __amdgpu_buffer_rsrc_t c_rsrc = __builtin_amdgcn_make_buffer_rsrc(cb_uniform, 0, R * N * 2, 0x00020000);
      const uint32_t lane_off = (uint32_t)(orow * N + oc) * 2u;
#pragma unroll
      for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int c0 = 0; c0 < Cfg::TN; c0 += SC) {
#pragma unroll
          for (int j = c0 / 32; j < (c0 + SC) / 32; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int cl = j * 32 - c0 + q * 8 + h * 4;
              const uint2 bp = bias_pk[j * 4 + q];
              const float bv[4] = {bf_lo(bp.x), bf_hi(bp.x), bf_lo(bp.y), bf_hi(bp.y)};
              float v[4];
              // (inline asm: the compiler's hazard recogniser does not see these reads of MFMA
              // results, which is why the mfma_result_fence() ahead of this epilogue is mandatory)
#pragma unroll
              for (int e = 0; e < 4; ++e)
                asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[e]) : "a"(acc[i][j][q * 4 + e]));
              const uint32_t p0 = epilogue_pair<EPI, HAS_BIAS>(v[0], v[1], bv[0], bv[1]);
              const uint32_t p1 = epilogue_pair<EPI, HAS_BIAS>(v[2], v[3], bv[2], bv[3]);
              *reinterpret_cast<uint2*>(so + m * OLD + cl) = make_uint2(p0, p1);
            }
          }
          // (all staged pieces are read before the first is stored: the guard behind a store
          // keeps every later instruction behind it)
          constexpr int kPasses = 32 / kRowsPerPass;
          uint4 staged[kPasses];
#pragma unroll
          for (int t = 0; t < kPasses; ++t)
            staged[t] = *reinterpret_cast<const uint4*>(so + (t * kRowsPerPass + orow) * OLD + oc);
#pragma unroll
          for (int t = 0; t < kPasses; ++t) {
            // (lane part of the address in the vector offset, which the range check sees;
            // the pass's part, uniform, in the scalar offset)
            const int row_s = wrow0 + i * 32 + t * kRowsPerPass, col_s = wcol0 + c0;
            const bool ok = orow < cur.live - row_s && oc + 8 <= N - col_s;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, staged[t]), c_rsrc,
                                                   ok ? lane_off : 0xfffffff0u,
                                                   (row_s * N + col_s) * 2, EPI != kEpiBias ? 2 : 0);
            store_data_guard();
          }
        }
      }
    } else {
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
      for (int c0 = 0; c0 < Cfg::TN; c0 += SC) {
#pragma unroll
        for (int j = c0 / 32; j < (c0 + SC) / 32; ++j) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int cl = j * 32 - c0 + q * 8 + h * 4;
            const uint2 bp = bias_pk[j * 4 + q];
            const float bv[4] = {bf_lo(bp.x), bf_hi(bp.x), bf_lo(bp.y), bf_hi(bp.y)};
            // (read here and nowhere earlier: hoisted above the branches below, the reads
            // of all 64 groups would need 256 registers at once; being inline asm they are
            // invisible to the compiler's hazard recogniser, so the mfma_result_fence() ahead
            // of this epilogue is what keeps them behind the last MFMA's write)
            floatx4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float x;
              asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x) : "a"(acc[i][j][q * 4 + e]));
              v[e] = x;
            }
            const int cidx = (i * FN + j) * 4 + q;
            if (adds_sums) {      // uniform over the workgroup
              v += __builtin_bit_cast(floatx4, ahead[cidx % kAhead]);
              if (poisoned) {
                const float nan = __builtin_nanf("");
                v = floatx4{nan, nan, nan, nan};
              }
              if (cidx + kAhead < kChunks)
                ahead[cidx % kAhead] = __builtin_amdgcn_raw_buffer_load_b128(
                    sums_rsrc, vec0 * 16, sums_base + (cidx + kAhead) * 1024, kSumsAux);
            }
            if (leaves_sums) {    // uniform over the workgroup
              __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v), sums_rsrc,
                                                     vec0 * 16, sums_base + cidx * 1024, kSumsAux);
              store_data_guard();
            } else {
              const uint32_t p0 = epilogue_pair<EPI, HAS_BIAS>(v[0], v[1], bv[0], bv[1]);
              const uint32_t p1 = epilogue_pair<EPI, HAS_BIAS>(v[2], v[3], bv[2], bv[3]);
              *reinterpret_cast<uint2*>(so + m * OLD + cl) = make_uint2(p0, p1);
            }
            if constexpr (!kDeepA) {
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[i][j][q * 4 + e] = 0.f;
            }
          }
        }
        if (leaves_sums) continue;
        // A wave reads back only what it wrote (its LDS operations complete in order).
#pragma unroll
        for (int r0 = 0; r0 < 32; r0 += kRowsPerPass) {
          const int rl = r0 + orow;
          const int row = wrow0 + i * 32 + rl;
          const int col = wcol0 + c0 + oc;
          const uint4 v = *reinterpret_cast<const uint4*>(so + rl * OLD + oc);
          if (row < live_rows && col + 8 <= N) {
            if constexpr (EPI != kEpiBias) {   // hidden layer: streaming store, as in store_tile
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
    }
    if (leaves_sums) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // every wave's sums have been written through
      __syncthreads();
      if (tid == 0)
        __hip_atomic_store(sk_flags + shared_index, waits + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (!has_next) break;
    if constexpr (kDeepA) raw_barrier();
    cur = nxt;
  }
  wait_vmcnt<0>();
#undef VMOE_PERSISTENT_K_ITERATION
#undef VMOE_PERSISTENT_K_ITERATION_RING
#endif
}

template <int EPI>
__global__ __launch_bounds__(256) void gemm_bf16_generic_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Bt, const bf16_t* __restrict__ bias,
    bf16_t* __restrict__ C, int R, int N, int Kd, int tiles_m, int tiles_n,
    const int32_t* __restrict__ rows) {
  constexpr int BM = 128, BN = 128, BK = 64, LD = BK + 8, NCH = 4;
  __shared__ __align__(16) bf16_t lds[(BM + BN) * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m = lane & 31, h = lane >> 5;
  const int per_batch = tiles_m * tiles_n;
  const int b = blockIdx.x / per_batch;
  const int rem = blockIdx.x - b * per_batch;
  const int tile_n = rem / tiles_m, tile_m = rem - tile_n * tiles_m;
  const int row0 = tile_m * BM, col0 = tile_n * BN;
  int live = R;
  if (rows != nullptr) {
    live = min(rows[b], R);
    if (row0 >= live) return;     // uniform over the workgroup: no barrier is skipped by a part of it
  }
  const bf16_t* Ab = A + (size_t)b * R * Kd;
  const bf16_t* Bb = Bt + (size_t)b * N * Kd;
  const int kc8 = (tid & 7) * 8;
  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  for (int k0 = 0; k0 < Kd; k0 += BK) {
    const bool ok = k0 + kc8 + 8 <= Kd;
    const int kk = ok ? k0 + kc8 : Kd - 8;
    uint4 ra[NCH], rb[NCH];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int r = (tid >> 3) + i * 32;
      ra[i] = *reinterpret_cast<const uint4*>(Ab + (size_t)min(row0 + r, R - 1) * Kd + kk);
      rb[i] = *reinterpret_cast<const uint4*>(Bb + (size_t)min(col0 + r, N - 1) * Kd + kk);
      if (!ok) { ra[i] = make_uint4(0, 0, 0, 0); rb[i] = make_uint4(0, 0, 0, 0); }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int r = (tid >> 3) + i * 32;
      *reinterpret_cast<uint4*>(lds + r * LD + kc8) = ra[i];
      *reinterpret_cast<uint4*>(lds + (BM + r) * LD + kc8) = rb[i];
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
            lds + (wm * 64 + i * 32 + m) * LD + ks * 16 + h * 8));
        fb[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
            lds + (BM + wn * 64 + i * 32 + m) * LD + ks * 16 + h * 8));
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
  }
  mfma_result_fence();
  const bf16_t* biasb = bias != nullptr ? bias + (size_t)b * N : nullptr;
  bf16_t* Cb = C + (size_t)b * R * N;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = row0 + wm * 64 + i * 32 + m;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int col = col0 + wn * 64 + j * 32 + (v >> 2) * 8 + h * 4 + (v & 3);
        if (row < live && col < N) {
          float bv = biasb != nullptr ? bf2f(biasb[col]) : 0.f;
          Cb[(size_t)row * N + col] = f2bf(apply_epilogue<EPI>(acc[i][j][v], bv, biasb != nullptr));
        }
      }
  }
}

struct GemmGeom {
  bool fast;             // the LDS-DMA kernel applies (else the generic one)
  int tiles_m, tiles_n, panel_rows, tiles_per_xcd;
  long long tiles;
  long long ragged_slots;   // workgroups per die of a planned (ragged) launch
};

template <typename Cfg>
GemmGeom gemm_geometry(int batch, int R, int N, int Kd) {
  GemmGeom g{};
  g.fast = !(Kd % Cfg::BK != 0 || (uint64_t)(R > N ? R : N) * Kd * 2 >= (1ull << 32));
  if (!g.fast) return g;
  g.tiles_m = (R + Cfg::BM - 1) / Cfg::BM;
  g.tiles_n = (N + Cfg::BN - 1) / Cfg::BN;
  g.tiles = (long long)batch * g.tiles_m * g.tiles_n;
  g.tiles_per_xcd = (int)((g.tiles + kNumXcd - 1) / kNumXcd);
  // Tile order inside a batch: panels of `panel_rows` row tiles, swept column tile
  // by column tile.  The tiles that run together on one die (32 compute units)
  // then form a block of about panel_rows x (concurrent / panel_rows) tiles, whose
  // operand footprint per tile is smallest when the block's A and B bytes match.
  const double concurrent = 32.0 * Cfg::kBlocksPerCu;
  int panel_rows = (int)(std::sqrt(concurrent * Cfg::BN / Cfg::BM) + 0.5);
  if (panel_rows < 1) panel_rows = 1;
  if (panel_rows > g.tiles_m) panel_rows = g.tiles_m;
  const int panels = (g.tiles_m + panel_rows / 2) / panel_rows > 0 ? (g.tiles_m + panel_rows / 2) / panel_rows : 1;
  g.panel_rows = (g.tiles_m + panels - 1) / panels;
  // Slots per die for the largest possible run (every row tile live).
  const long long share_max = ((long long)batch * g.tiles_m + kNumXcd - 1) / kNumXcd;
  g.ragged_slots = share_max * g.tiles_n;
  return g;
}

// The plan of a launch with geometry g as its kernel takes it (tag: what the planner wrote
// for the same geometry, batch count and rows per batch).
template <typename Cfg>
PlanRef plan_ref(const GemmGeom& g, const int4* plan, int batch, int R) {
  if (plan == nullptr) return PlanRef{nullptr, 0, 0};
  const int blocks = (int)(g.ragged_slots * kNumXcd);
  return PlanRef{plan, blocks, plan_tag(Cfg::BM, g.tiles_n, g.panel_rows, blocks, batch, R)};
}

// `plan`, if given, was filled by plan_ragged_tiles_kernel for this product's geometry.
// `clear` / `status`: see begin_call.
template <typename Cfg, int EPI>
int launch_gemm_bf16(const bf16_t* A, const bf16_t* Bt, const bf16_t* bias, bf16_t* C, int batch,
                     int R, int N, int Kd, hipStream_t stream, const int32_t* rows = nullptr,
                     const int4* plan = nullptr, const int32_t* a_rows = nullptr,
                     long long a_items = 0, int32_t* clear = nullptr, int clear_count = 0,
                     int32_t* status = nullptr) {
  const GemmGeom g = gemm_geometry<Cfg>(batch, R, N, Kd);
  if ((clear != nullptr || status != nullptr) && !g.fast) {
    hipLaunchKernelGGL(begin_call_kernel, dim3(1), dim3(256), 0, stream, clear, clear_count, status);
    clear = nullptr;
    status = nullptr;
  }
  if (a_rows != nullptr && (!g.fast || rows == nullptr ||
                            (unsigned long long)a_items * Kd * 2 >= (1ull << 32)))
    return VMOE_E_UNSUPPORTED;     // the gathering load exists in the LDS-DMA kernel only
  if (!g.fast) {
    const int tiles_m = (R + 127) / 128, tiles_n = (N + 127) / 128;
    const long long blocks = (long long)batch * tiles_m * tiles_n;
    if (blocks > 0x7fffffffLL) return VMOE_E_OVERFLOW;
    hipLaunchKernelGGL(gemm_bf16_generic_kernel<EPI>, dim3((unsigned)blocks), dim3(256), 0, stream,
                       A, Bt, bias, C, R, N, Kd, tiles_m, tiles_n, rows);
    return launch_status();
  }
  if (g.tiles > 0x7ffffff0LL) return VMOE_E_OVERFLOW;
  const unsigned blocks = (unsigned)(plan != nullptr ? g.ragged_slots : g.tiles_per_xcd) * kNumXcd;
  auto kern = gemm_bf16_kernel<Cfg, EPI>;
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::kLdsBytes);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, A, Bt, bias,
                     C, R, N, Kd, g.tiles_m, g.tiles_n, (int)g.tiles, g.tiles_per_xcd, g.panel_rows,
                     rows, plan_ref<Cfg>(g, plan, batch, R), a_rows, (int)a_items, clear, clear_count,
                     status);
  return launch_status();
}

// Measurement only: VMOE_GEMM_ACTIVE=<dies>x<compute units per die> in the environment makes
// the workgroups of the other dies (first and second product) and of the other compute units
// of a die (second product, one workgroup per compute unit) leave at once.  The work of those
// that left is not done, so the outputs are incomplete; what the launch then shows is the rate
// of a die or compute unit when its neighbours are idle, i.e. whether the products are held
// back by something the whole chip shares.  Unset: all 8 x 32.
struct ActiveUnits { int xcds, slots; };
inline ActiveUnits active_units() {
  ActiveUnits a{kNumXcd, 32};
  if (const char* t = getenv("VMOE_GEMM_ACTIVE")) {
    int x = 0, c = 0;
    if (sscanf(t, "%dx%d", &x, &c) == 2 && x >= 1 && x <= kNumXcd && c >= 1 && c <= 32) a = ActiveUnits{x, c};
  }
  return a;
}

// The first product of an MLP: gemm_bf16_mixed_kernel where it applies (k a multiple of 64
// and at least 128), else gemm_bf16_kernel with the same tiling; launch geometry and plan are
// those of GemmCfg<128, 256, 2, 2, 32, 3, 2> either way.  VMOE_FIRST_PRODUCT_K32=1 in the
// environment keeps the 32-wide k tiles for both operands (the switch behind the before /
// after figures).
template <int EPI>
int launch_gemm_bf16_first(const bf16_t* A, const bf16_t* Bt, const bf16_t* bias, bf16_t* C,
                           int batch, int R, int N, int Kd, hipStream_t stream,
                           const int32_t* rows, const int4* plan, const int32_t* a_rows,
                           long long a_items, int32_t* clear, int clear_count, int32_t* status) {
  using Cfg = GemmCfg<128, 256, 2, 2, 32, 3, 2>;
  const GemmGeom g = gemm_geometry<Cfg>(batch, R, N, Kd);
  const bool gather_ok = a_rows == nullptr ||
                         (rows != nullptr && (unsigned long long)a_items * Kd * 2 < (1ull << 32));
  if (!g.fast || Kd % 64 != 0 || Kd < 128 || !gather_ok || g.tiles > 0x7ffffff0LL ||
      getenv("VMOE_FIRST_PRODUCT_K32") != nullptr)
    return launch_gemm_bf16<Cfg, EPI>(A, Bt, bias, C, batch, R, N, Kd, stream, rows, plan, a_rows,
                                      a_items, clear, clear_count, status);
  constexpr size_t kLds = 2 * 128 * 64 + 2 * 256 * 128;
  static_assert(kLds * 2 <= 160 * 1024, "two workgroups per CU");
  const unsigned blocks = (unsigned)(plan != nullptr ? g.ragged_slots : g.tiles_per_xcd) * kNumXcd;
  auto kern = gemm_bf16_mixed_kernel<EPI>;
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), kLds);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), kLds, stream, A, Bt, bias, C, R, N, Kd,
                     g.tiles_m, g.tiles_n, (int)g.tiles, g.tiles_per_xcd, g.panel_rows, rows,
                     plan_ref<Cfg>(g, plan, batch, R), a_rows, (int)a_items, clear, clear_count, status,
                     active_units().xcds);
  return launch_status();
}

// Whether gemm_bf16_persistent_kernel covers the product: fast geometry, at least
// 2 * NSTAGE k tiles, operands addressable with 32-bit byte offsets from their start,
// and a ragged launch only with its plan.
template <typename Cfg>
bool persistent_gemm_ok(int batch, int R, int N, int Kd, const int32_t* rows, const int4* plan) {
  const GemmGeom g = gemm_geometry<Cfg>(batch, R, N, Kd);
  const uint64_t lim = 1ull << 32;
  return g.fast && Kd / Cfg::BK >= 2 * Cfg::NSTAGE && (N & 7) == 0 &&
         (uint64_t)batch * R * Kd * 2 < lim && (uint64_t)batch * N * Kd * 2 < lim &&
         g.tiles <= 0x7ffffff0LL && (rows == nullptr || plan != nullptr);
}

// Memory of the stream-K exchange of a tile-walking launch: one tile of float32 partial
// sums per workgroup, then one flag per workgroup.
template <typename Cfg>
struct StreamKWorkspace {
  static constexpr int kBlocks = kCusPerXcd * kNumXcd;
  static constexpr size_t kPartialBytes = (size_t)kBlocks * Cfg::BM * Cfg::BN * sizeof(float);
  static constexpr int kFlags = kBlocks;
  static constexpr size_t kBytes = kPartialBytes + (size_t)(kFlags + 63) / 64 * 256;
  static float* partials(void* ws) { return static_cast<float*>(ws); }
  static int32_t* flags(void* ws) {
    return reinterpret_cast<int32_t*>(static_cast<unsigned char*>(ws) + kPartialBytes);
  }
};

// Launches the persistent kernel; the caller checked persistent_gemm_ok.  `plan`, if
// given, was filled by plan_ragged_tiles_kernel for gemm_geometry<Cfg> (BM, BN and
// workgroups per CU decide it, not the number of stages).  `streamk`, if given, is
// StreamKWorkspace<Cfg>::kBytes of memory: the die's last, partial round is then shared
// along k; an earlier launch of the call has set its flags to zero (begin_call).  `status`:
// the call's status words.
// VMOE_STREAMK_TEST_GIVE_UP=<spins> in the environment (the test of the bounded wait): pieces
// wait for deposits that never come, for at most that many polls, and give up.
template <typename Cfg, int EPI>
int launch_gemm_bf16_persistent(const bf16_t* A, const bf16_t* Bt, const bf16_t* bias, bf16_t* C,
                                int batch, int R, int N, int Kd, hipStream_t stream,
                                const int4* plan, void* streamk, int32_t* status) {
  const GemmGeom g = gemm_geometry<Cfg>(batch, R, N, Kd);
  auto kern = bias != nullptr ? gemm_bf16_persistent_kernel<Cfg, EPI, true>
                              : gemm_bf16_persistent_kernel<Cfg, EPI, false>;
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), PersistentLds<Cfg>::kBytes);
  if (e != hipSuccess) return (int)e;
  using SK = StreamKWorkspace<Cfg>;
  float* partials = nullptr;
  int32_t* flags = nullptr;
  // (VMOE_WHOLE_TILES=1 in the environment keeps every tile whole: the switch behind the
  // before / after figures of the shared round)
  const ActiveUnits active = active_units();
  const bool all_active = active.xcds == kNumXcd && active.slots == kCusPerXcd;
  if (streamk != nullptr && getenv("VMOE_WHOLE_TILES") == nullptr && all_active) {
    partials = SK::partials(streamk);
    flags = SK::flags(streamk);
  }
  int spin_limit = 1 << 22, wait_bias = 0;     // polls ~0.5 us apart: about two seconds
  if (const char* t = getenv("VMOE_STREAMK_TEST_GIVE_UP")) {
    spin_limit = atoi(t) > 0 ? atoi(t) : 1;
    wait_bias = 1 << 20;
  }
  hipLaunchKernelGGL(kern, dim3(kCusPerXcd * kNumXcd), dim3(Cfg::kThreads),
                     PersistentLds<Cfg>::kBytes, stream, A, Bt, bias, C, R, N, Kd, g.tiles_m,
                     g.tiles_n, (int)g.tiles, g.tiles_per_xcd, g.panel_rows,
                     plan_ref<Cfg>(g, plan, batch, R), partials, flags, status, spin_limit, wait_bias,
                     active.xcds, active.slots);
  return launch_status();
}

}  // namespace vmoe
#endif  // VMOE_GEMM_BF16_H_
