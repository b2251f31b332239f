// bfloat16 einsum dispatch / combine of EinsumDispatcher (vmoe/moe.py:148-161)
// on v_mfma_f32_32x32x16_bf16, for weights, data and output that are all
// bfloat16 (products of two bfloat16 values are exact in float32, so this is the
// float32-accumulated einsum of the reference up to summation order).
//
// Both contractions are short (K = group size for dispatch, K = slots per group
// for combine), so the kernels are HBM-bound: every data row is read once, every
// output row written once.  The data operand is "k-major" in memory (the
// contraction index selects the row), while the matrix cores want eight
// consecutive k per lane.  Each thread therefore loads an 8 (k) x 8 (column)
// block with eight coalesced 16-byte loads, transposes it in registers with byte
// permutes and writes eight 16-byte runs of k into a rotated LDS tile; fragment
// reads are then single conflict-free 16-byte LDS reads.  The weight operand
// stays in registers for all tiles of a workgroup.  The operands are passed to
// the MFMA swapped (data as A, weights as B) so that a lane's four consecutive
// accumulator registers are four consecutive output columns: the tile leaves
// through a wave-private staging region as 16-byte row-contiguous stores.
#ifndef VMOE_EINSUM_BF16_H_
#define VMOE_EINSUM_BF16_H_
#include "vmoe_common.h"

namespace vmoe {
namespace ein {

constexpr int kTileD = 64;                  // data / output columns per tile
constexpr int kStageLd = kTileD + 8;        // row pitch of the staged output (elements)
constexpr int kStageElems = 32 * kStageLd;  // one wave's staging region
constexpr int kThreads = 256;

// Rotation of the 16-byte k chunks of tile row c.  Rows are a multiple of 256
// bytes long, so the rotation alone decides the bank group: 16 consecutive rows
// (one fragment read) get 16 distinct rotations, and the eight rows c, c+8, ...
// that neighbouring lanes write get even rotations 2 apart, which interleave
// with the next k chunk of the other half of the 16 lanes.
__device__ __forceinline__ int rot(int c) { return 2 * (c >> 3) + (c & 1) + 4 * ((c & 7) >> 1); }

__device__ __forceinline__ size_t bt_bytes(int KCP) { return (size_t)kTileD * KCP * 16; }

// Eight rows (k) x eight columns of data; rowidx < 0 or col >= D reads as zero.
__device__ __forceinline__ void load_block(uint4 (&r)[8], const bf16_t* __restrict__ data,
                                           const int (&rowidx)[8], int col, int D) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    r[i] = make_uint4(0, 0, 0, 0);
    if (rowidx[i] >= 0 && col < D)
      r[i] = *reinterpret_cast<const uint4*>(data + (size_t)rowidx[i] * D + col);
  }
}

// Transposes the block held in r (row i = k index kb*8+i, 8 columns cc*8..+8)
// and writes, for each column, its 8 consecutive k values as one 16-byte chunk.
__device__ __forceinline__ void write_block_transposed(const uint4 (&r)[8], bf16_t* bt, int kb,
                                                       int cc, int KCP) {
  uint32_t w[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    w[i][0] = r[i].x; w[i][1] = r[i].y; w[i][2] = r[i].z; w[i][3] = r[i].w;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
    uint32_t o[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] = __builtin_amdgcn_perm(w[2 * q + 1][j >> 1], w[2 * q][j >> 1], sel);
    const int c = cc * 8 + j;
    const int chunk = (kb + 2 * cc + (j & 1) + 4 * (j >> 1)) & (KCP - 1);
    *reinterpret_cast<uint4*>(bt + ((size_t)c * KCP + chunk) * 8) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

__device__ __forceinline__ bf16x8 read_frag(const bf16_t* bt, int c, int rc, int kb, int KCP) {
  const int chunk = (kb + rc) & (KCP - 1);
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(bt + ((size_t)c * KCP + chunk) * 8));
}

// Accumulators of a (64 columns) x (32 rows) wave tile -> staging region so[row][column].
__device__ __forceinline__ void stage_tile(const floatx16 (&acc)[2], bf16_t* so, int m, int h) {
#pragma unroll
  for (int jj = 0; jj < 2; ++jj)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int cl = jj * 32 + q * 8 + h * 4;
      const uint32_t p0 = (uint32_t)f2bf(acc[jj][q * 4 + 0]) | ((uint32_t)f2bf(acc[jj][q * 4 + 1]) << 16);
      const uint32_t p1 = (uint32_t)f2bf(acc[jj][q * 4 + 2]) | ((uint32_t)f2bf(acc[jj][q * 4 + 3]) << 16);
      *reinterpret_cast<uint2*>(so + m * kStageLd + cl) = make_uint2(p0, p1);
    }
}

// Staged rows -> global rows orow[p] (row p*8 + lane/8 of the wave tile), 16 bytes per lane.
__device__ __forceinline__ void store_staged(const bf16_t* so, bf16_t* __restrict__ out,
                                             const int (&orow)[4], int lane, int d0, int D) {
  const int oc = (lane & 7) * 8;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int rl = p * 8 + (lane >> 3);
    const uint4 v = *reinterpret_cast<const uint4*>(so + rl * kStageLd + oc);
    if (orow[p] >= 0 && d0 + oc < D)
      *reinterpret_cast<uint4*>(out + (size_t)orow[p] * D + d0 + oc) = v;
  }
}

// Workgroup -> (group, part of the group's work), such that all workgroups of a
// group run on the same die and share its L2 copy of the group's weights.
__device__ __forceinline__ bool map_group(int G, int per_group, int& g, int& rem) {
  const int xcd = blockIdx.x % kNumXcd, idx = blockIdx.x / kNumXcd;
  g = (idx / per_group) * kNumXcd + xcd;
  rem = idx % per_group;
  return g < G;
}

// out[slot(g, n), :] = sum_s w[g, s, n] * data[g, s, :]   (n = e*C + c)
// A workgroup owns 128 buffer rows n of one group (wave = 32 of them) and a run
// of column tiles; S <= 16 * KSMAX.  W_BLOCKS: the weights (k-major as well) go
// through the same transposing LDS tile, 64 buffer rows at a time; otherwise
// (E*C not a multiple of 8, or unaligned) each lane gathers its values one by one.
template <int KSMAX, bool W_BLOCKS>
__global__ __launch_bounds__(kThreads, 2) void einsum_dispatch_bf16_kernel(
    const bf16_t* __restrict__ w, const bf16_t* __restrict__ data, bf16_t* __restrict__ out, int G,
    int S, int E, int C, int D, int KS, int KCP, int d_splits, int n_blocks, int tiles_per_split) {
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* bt = reinterpret_cast<bf16_t*>(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, h = lane >> 5;
  bf16_t* so = reinterpret_cast<bf16_t*>(smem + bt_bytes(KCP)) + wave * kStageElems;
  int g, rem;
  if (!map_group(G, d_splits * n_blocks, g, rem)) return;
  const int nb = rem / d_splits, ds = rem - nb * d_splits;
  const int N = E * C;
  const int cc = tid & 7, kb = tid >> 3;
  const int rc0 = rot(m), rc1 = rot(32 + m);

  int rowidx[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) rowidx[i] = kb * 8 + i < S ? g * S + kb * 8 + i : -1;
  const int total_tiles = (D + kTileD - 1) / kTileD;
  const int t0 = ds * tiles_per_split, t1 = min(t0 + tiles_per_split, total_tiles);
  uint4 pre0[8], pre1[8];

  // Weights of this wave's 32 buffer rows, all k, kept in registers.
  bf16x8 wf[KSMAX];
  if constexpr (W_BLOCKS) {
    uint4 wa[8], wb[8];
    load_block(wa, w, rowidx, nb * 128 + cc * 8, N);
    load_block(wb, w, rowidx, nb * 128 + 64 + cc * 8, N);
    load_block(pre0, data, rowidx, t0 * kTileD + cc * 8, D);
    if (t0 + 1 < t1) load_block(pre1, data, rowidx, (t0 + 1) * kTileD + cc * 8, D);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      if (kb < 2 * KS) write_block_transposed(half == 0 ? wa : wb, bt, kb, cc, KCP);
      wait_lgkmcnt0();
      raw_barrier();
      if ((wave >> 1) == half) {
        const int c = (wave & 1) * 32 + m;
#pragma unroll
        for (int ks = 0; ks < KSMAX; ++ks)
          if (ks < KS) wf[ks] = read_frag(bt, c, (wave & 1) ? rc1 : rc0, 2 * ks + h, KCP);
      }
      wait_lgkmcnt0();
      raw_barrier();
    }
  } else {
    const int n = nb * 128 + wave * 32 + m;
    const bf16_t* wg = w + (size_t)g * S * N;
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) {
      uint32_t pk[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int k = ks * 16 + h * 8 + 2 * q;
        uint32_t lo = 0, hi = 0;
        if (n < N && k < S) lo = wg[(size_t)k * N + n];
        if (n < N && k + 1 < S) hi = wg[(size_t)(k + 1) * N + n];
        pk[q] = lo | (hi << 16);
      }
      wf[ks] = __builtin_bit_cast(bf16x8, make_uint4(pk[0], pk[1], pk[2], pk[3]));
    }
    load_block(pre0, data, rowidx, t0 * kTileD + cc * 8, D);
    if (t0 + 1 < t1) load_block(pre1, data, rowidx, (t0 + 1) * kTileD + cc * 8, D);
  }

  int orow[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int nn = nb * 128 + wave * 32 + p * 8 + (lane >> 3);
    orow[p] = nn < N ? slot_row(nn / C, g, nn % C, G, E, C) : -1;
  }

  // One column tile: the block loaded two tiles ago goes into the LDS tile, its
  // registers take the tile after next.
  auto tile = [&](uint4 (&pre)[8], int t) {
    if (kb < 2 * KS) write_block_transposed(pre, bt, kb, cc, KCP);
    wait_lgkmcnt0();
    raw_barrier();
    if (t + 2 < t1) load_block(pre, data, rowidx, (t + 2) * kTileD + cc * 8, D);
    floatx16 acc[2];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[jj][v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) {
      if (ks < KS) {
        const bf16x8 f0 = read_frag(bt, m, rc0, 2 * ks + h, KCP);
        const bf16x8 f1 = read_frag(bt, 32 + m, rc1, 2 * ks + h, KCP);
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f0, wf[ks], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f1, wf[ks], acc[1], 0, 0, 0);
      }
    }
    mfma_result_fence();
    stage_tile(acc, so, m, h);
    store_staged(so, out, orow, lane, t * kTileD, D);
    wait_lgkmcnt0();
    raw_barrier();
  };
  for (int t = t0; t < t1; t += 2) {
    tile(pre0, t);
    if (t + 1 < t1) tile(pre1, t + 1);
  }
}

// out[g, s, :] = sum_n w[g, s, n] * data[slot(g, n), :]   (n = e*C + c, N = E*C <= 128)
// A workgroup owns 256 item rows of one group (wave = 64 of them, as two 32-row
// tiles computed one after the other) and a run of column tiles.
__global__ __launch_bounds__(kThreads, 2) void einsum_combine_bf16_kernel(
    const bf16_t* __restrict__ w, const bf16_t* __restrict__ data, bf16_t* __restrict__ out, int G,
    int S, int E, int C, int D, int KS, int d_splits, int row_blocks, int tiles_per_split) {
  constexpr int KSMAX = 8, KCP = 16;
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* bt = reinterpret_cast<bf16_t*>(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, h = lane >> 5;
  bf16_t* so = reinterpret_cast<bf16_t*>(smem + bt_bytes(KCP)) + wave * kStageElems;
  int g, rem;
  if (!map_group(G, d_splits * row_blocks, g, rem)) return;
  const int rb = rem / d_splits, ds = rem - rb * d_splits;
  const int N = E * C;

  const int cc = tid & 7, kb = tid >> 3;
  int rowidx[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int nn = kb * 8 + i;
    rowidx[i] = nn < N ? slot_row(nn / C, g, nn % C, G, E, C) : -1;
  }
  const int total_tiles = (D + kTileD - 1) / kTileD;
  const int t0 = ds * tiles_per_split, t1 = min(t0 + tiles_per_split, total_tiles);
  uint4 pre0[8], pre1[8];
  load_block(pre0, data, rowidx, t0 * kTileD + cc * 8, D);
  if (t0 + 1 < t1) load_block(pre1, data, rowidx, (t0 + 1) * kTileD + cc * 8, D);

  // Combine weights of this wave's two 32-row tiles, all k, straight from memory
  // (k is the fast index of w here).
  const int row_base = rb * 256 + wave * 64;
  bf16x8 wf[2][KSMAX];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int s = row_base + i * 32 + m;
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) {
      const int k = ks * 16 + h * 8;
      uint4 raw = make_uint4(0, 0, 0, 0);
      if (s < S && k < N) raw = *reinterpret_cast<const uint4*>(w + ((size_t)g * S + s) * N + k);
      wf[i][ks] = __builtin_bit_cast(bf16x8, raw);
    }
  }
  const bool tile_on[2] = {row_base < S, row_base + 32 < S};
  int orow[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int s = row_base + i * 32 + p * 8 + (lane >> 3);
      orow[i][p] = s < S ? g * S + s : -1;
    }
  const int rc0 = rot(m), rc1 = rot(32 + m);

  auto tile = [&](uint4 (&pre)[8], int t) {
    if (kb < 2 * KS) write_block_transposed(pre, bt, kb, cc, KCP);
    wait_lgkmcnt0();
    raw_barrier();
    if (t + 2 < t1) load_block(pre, data, rowidx, (t + 2) * kTileD + cc * 8, D);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (tile_on[i]) {
        floatx16 acc[2];
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[jj][v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KSMAX; ++ks) {
          if (ks < KS) {
            const bf16x8 f0 = read_frag(bt, m, rc0, 2 * ks + h, KCP);
            const bf16x8 f1 = read_frag(bt, 32 + m, rc1, 2 * ks + h, KCP);
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f0, wf[i][ks], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f1, wf[i][ks], acc[1], 0, 0, 0);
          }
        }
        mfma_result_fence();
        stage_tile(acc, so, m, h);
        store_staged(so, out, orow[i], lane, t * kTileD, D);
      }
    }
    wait_lgkmcnt0();
    raw_barrier();
  };
  for (int t = t0; t < t1; t += 2) {
    tile(pre0, t);
    if (t + 1 < t1) tile(pre1, t + 1);
  }
}

// Column tiles per workgroup such that the launch has about two workgroups per
// compute unit (all resident at once) when the shape allows it.
inline void split_columns(int D, int64_t groups_x_blocks, int& d_splits, int& tiles_per_split) {
  const int tiles = (D + kTileD - 1) / kTileD;
  int64_t want = (512 + groups_x_blocks - 1) / groups_x_blocks;
  if (want < 1) want = 1;
  if (want > tiles) want = tiles;
  tiles_per_split = (int)((tiles + want - 1) / want);
  d_splits = (tiles + tiles_per_split - 1) / tiles_per_split;
}

inline bool dispatch_fast_ok(const VmoeEinsumParams* p) {
  return p->w_dtype == VMOE_W_BF16 && p->data_dtype == VMOE_BF16 && p->out_dtype == VMOE_BF16 &&
         p->D % 8 == 0 && aligned16(p->data) && aligned16(p->out) && p->S <= 256;
}

inline bool combine_fast_ok(const VmoeEinsumParams* p) {
  const int64_t N = (int64_t)p->E * p->C;
  return p->w_dtype == VMOE_W_BF16 && p->data_dtype == VMOE_BF16 && p->out_dtype == VMOE_BF16 &&
         p->D % 8 == 0 && aligned16(p->data) && aligned16(p->out) && aligned16(p->w) &&
         N % 8 == 0 && N <= 128;
}

inline int launch_dispatch_fast(const VmoeEinsumParams* p, hipStream_t stream) {
  const int N = p->E * p->C;
  const int KS = (p->S + 15) / 16, KCP = KS <= 8 ? 16 : 32;
  const int n_blocks = (N + 127) / 128;
  int d_splits, tiles_per_split;
  split_columns(p->D, (int64_t)p->G * n_blocks, d_splits, tiles_per_split);
  const int64_t blocks = (int64_t)((p->G + kNumXcd - 1) / kNumXcd) * kNumXcd * d_splits * n_blocks;
  if (blocks >= INT32_MAX) return VMOE_E_OVERFLOW;
  const size_t lds = (size_t)kTileD * KCP * 16 + 4 * kStageElems * sizeof(bf16_t);
  const bool w_blocks = N % 8 == 0 && aligned16(p->w);
  auto kern = KS <= 13 ? (w_blocks ? einsum_dispatch_bf16_kernel<13, true>
                                   : einsum_dispatch_bf16_kernel<13, false>)
                       : (w_blocks ? einsum_dispatch_bf16_kernel<16, true>
                                   : einsum_dispatch_bf16_kernel<16, false>);
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kThreads), lds, stream,
                     (const bf16_t*)p->w, (const bf16_t*)p->data, (bf16_t*)p->out, p->G, p->S, p->E,
                     p->C, p->D, KS, KCP, d_splits, n_blocks, tiles_per_split);
  return launch_status();
}

inline int launch_combine_fast(const VmoeEinsumParams* p, hipStream_t stream) {
  const int N = p->E * p->C;
  const int KS = (N + 15) / 16;
  const int row_blocks = (p->S + 255) / 256;
  int d_splits, tiles_per_split;
  split_columns(p->D, (int64_t)p->G * row_blocks, d_splits, tiles_per_split);
  const int64_t blocks = (int64_t)((p->G + kNumXcd - 1) / kNumXcd) * kNumXcd * d_splits * row_blocks;
  if (blocks >= INT32_MAX) return VMOE_E_OVERFLOW;
  const size_t lds = (size_t)kTileD * 16 * 16 + 4 * kStageElems * sizeof(bf16_t);
  hipLaunchKernelGGL(einsum_combine_bf16_kernel, dim3((unsigned)blocks), dim3(kThreads), lds, stream,
                     (const bf16_t*)p->w, (const bf16_t*)p->data, (bf16_t*)p->out, p->G, p->S, p->E,
                     p->C, p->D, KS, d_splits, row_blocks, tiles_per_split);
  return launch_status();
}

}  // namespace ein
}  // namespace vmoe
#endif  // VMOE_EINSUM_BF16_H_
