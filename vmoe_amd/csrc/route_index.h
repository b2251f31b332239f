// Index arithmetic of the routing kernels: sort keys, bitmap positions, slot rows, packed
// rows and launch-plan entries, as plain scalar functions.  The device kernels call them
// per thread; a host build (-DVMOE_CPU_ONLY, plain C++) runs the same functions under
// address and undefined-behaviour sanitizers.
#ifndef VMOE_ROUTE_INDEX_H_
#define VMOE_ROUTE_INDEX_H_

#include <stdint.h>

#if defined(VMOE_CPU_ONLY)
#define VMOE_HD inline
#else
#define VMOE_HD __host__ __device__ __forceinline__
#endif

namespace vmoe {

// Accelerator complex dies of the device; workgroup i is placed on die i % kNumXcd,
// and each die has its own L2.
constexpr int kNumXcd = 8;

// Monotone map float32 bits -> uint32 (larger float -> larger uint); -0.0 == +0.0.
VMOE_HD uint32_t orderable_bits(uint32_t u) {
  if (u == 0x80000000u) u = 0u;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Slot row of (expert e, group g, position c) in the (E, G*C) expert buffer: the row
// order of vmoe/moe.py:488-500.
VMOE_HD int slot_row(int e, int g, int c, int G, int E, int C) {
  int r;
  if (G % E == 0) {
    const int q = G / E;
    r = ((g % q) * E + g / q) * C + c;
  } else {
    r = g * C + c;
  }
  return e * (G * C) + r;
}

// Batch priority routing: items are visited by descending first-choice gate, equal gates
// by ascending item index (stable argsort of the negated gate, vmoe/moe.py:571).  The
// sort is ascending on these keys; padding keys (all ones) sort last.
VMOE_HD uint64_t bpr_key64(uint32_t gate_bits, int s) {
  return ((uint64_t)(~orderable_bits(gate_bits)) << 32) | (uint32_t)s;
}
// Gates that came out of a bfloat16 router are non-negative floats whose low 16 bits are
// zero: gate and item index then share one 32-bit key (S <= 65536).
VMOE_HD bool bpr_gate_is_narrow(uint32_t gate_bits) { return (gate_bits & 0x8000ffffu) == 0u; }
VMOE_HD uint32_t bpr_key32(uint32_t gate_bits, int s) {
  return ((~orderable_bits(gate_bits)) & 0xffff0000u) | (uint32_t)s;
}

// Choice k of the item with priority rank `rank` owns bit k*S + rank of its expert's
// bitmap: K-major, so that every first choice precedes every second choice
// (vmoe/moe.py:573-575).  The position of the choice in the expert's buffer -- the cumsum
// of the one-hot column, vmoe/moe.py:577-580 -- is the number of set bits before its own.
VMOE_HD int choice_bit(int k, int S, int rank) { return k * S + rank; }
VMOE_HD int position_from_bitmap(uint32_t bits_before_word, uint32_t word, int bit) {
  return (int)bits_before_word + __builtin_popcount(word & ((1u << (bit & 31)) - 1u));
}

// Hand-made (expert, position) pair -> slot row, as vmoe/moe.py:190-197 and :202-206 read
// it: pairs with expert >= E or position >= C are dropped (-1); *invalid is set for
// negative entries (also dropped).
VMOE_HD int slot_of_index_pair(int e, int c, int g, int G, int E, int C, bool* invalid) {
  *invalid = e < 0 || c < 0;
  if (*invalid || e >= E || c >= C) return -1;
  return slot_row(e, g, c, G, E, C);
}

// Packed rows: the slot row of a kept assignment of group g -> its row in the packed layout,
// expert e's items in rows 0 .. n_e-1 of its block, groups in order; rows_before is the
// number of rows of expert e taken by the groups before g.
VMOE_HD int slot_expert(int slot, int G, int C) { return slot / (G * C); }
VMOE_HD int packed_row(int slot, int rows_before, int G, int C) {
  const int per_expert = G * C;
  const int e = slot / per_expert;
  const int c = (slot - e * per_expert) % C;
  return e * per_expert + rows_before + c;
}

// ---- launch plan of a ragged batched product (see gemm_bf16.h) ----
struct alignas(16) PlanEntry {
  int32_t batch, tile_m, tile_n, live;     // batch -1: a workgroup without work
};
struct RaggedGeom {
  int bm, tiles_n, panel_rows, num_blocks;
  PlanEntry* plan;
};
// Entry num_blocks of a plan, one past its last workgroup's, is its header: (live row tiles
// of all batches, tag, 0, 0).  The tag names what the plan was written for -- tile height,
// column tiles, panel height, workgroups, batches and rows per batch -- and a product kernel
// that does not find the tag of its own launch there runs nothing: a workspace that was never
// planned, or was planned for other shapes, cannot drive its addressing.
VMOE_HD int32_t plan_tag(int bm, int tiles_n, int panel_rows, int num_blocks, int batch, int R) {
  const int v[6] = {bm, tiles_n, panel_rows, num_blocks, batch, R};
  uint32_t h = 0x564d4f45u;
  for (int i = 0; i < 6; ++i) {
    h = (h ^ (uint32_t)v[i]) * 0x9E3779B1u;
    h ^= h >> 15;
  }
  return (int32_t)(h | 1u);
}
// Status words of an expert MLP call (int32, in its workspace).  They only ever grow: the
// first launch of a call sets them to zero when the tag word does not yet say that it did.
enum { kStatusAbandonedWaits = 0, kStatusPlanMismatches = 1, kStatusTagWord = 2, kStatusWords = 3 };
constexpr int32_t kStatusTag = 0x56537461;

VMOE_HD int plan_min(int a, int b) { return a < b ? a : b; }
VMOE_HD int plan_max(int a, int b) { return a > b ? a : b; }

// Entry i of the plan.  tile_prefix[b] = live row tiles of the batches before b
// (tile_prefix[batch] = all of them).  The list of live row tiles, batch-major, is cut into
// kNumXcd equal runs, one per die (workgroup i belongs to die i % kNumXcd and is the die's
// slot i / kNumXcd); inside a die's run the tiles of one batch form panels of about
// panel_rows row tiles, each swept column tile by column tile.
VMOE_HD PlanEntry plan_entry(const RaggedGeom& g, const int32_t* tile_prefix, const int32_t* rows,
                             int batch, int R, int i) {
  const int total = tile_prefix[batch];
  const int share = (total + kNumXcd - 1) / kNumXcd;
  const int xcd = i % kNumXcd;
  int slot = i / kNumXcd;
  const int first = xcd * share;
  const int last = plan_min(first + share, total);      // this die's run of the tile list
  PlanEntry out{-1, 0, 0, 0};
  if (first < last && slot < (last - first) * g.tiles_n) {
    int lo = 0, hi = batch;                             // tile_prefix[lo] <= first < tile_prefix[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (tile_prefix[mid] <= first) lo = mid;
      else hi = mid;
    }
    // Walk the run batch by batch; the tiles of one batch are cut into panels of about
    // panel_rows row tiles (never across batches: a panel shares one batch's B operand),
    // each swept column tile by column tile.
    int pos = first;
    for (int b = lo; b < batch && pos < last; ++b) {
      const int seg_end = plan_min(tile_prefix[b + 1], last);
      const int seg = seg_end - pos;
      if (seg <= 0) continue;
      const int panels = plan_max(1, (seg + g.panel_rows / 2) / g.panel_rows);
      const int per_panel = (seg + panels - 1) / panels;
      if (slot < seg * g.tiles_n) {
        int q = slot / (per_panel * g.tiles_n);         // panels before the last are full
        if (q > panels - 1) q = panels - 1;
        const int rows_here = plan_min(per_panel, seg - q * per_panel);
        const int in_panel = slot - q * per_panel * g.tiles_n;
        const int tile_n = in_panel / rows_here;
        const int entry = pos + q * per_panel + (in_panel - tile_n * rows_here);
        out = PlanEntry{b, entry - tile_prefix[b], tile_n, plan_min(plan_max(rows[b], 0), R)};
        break;
      }
      slot -= seg * g.tiles_n;
      pos = seg_end;
    }
  }
  return out;
}

// ---- stream-K share of a die's last, partial round (see gemm_bf16_persistent_kernel) ----
// A die's run of n tiles is walked by `slots` workgroups, one tile per workgroup and round:
// q = n / slots whole rounds, and r = n % slots tiles that would leave slots - r workgroups
// idle for a whole tile's time.  Those r tiles are cut along k instead (at multiples of
// kStreamKGranule k tiles), after the whole rounds, and always so that the workgroups
// that run side by side compute the same k range of neighbouring tiles: the operands of
// neighbours then meet in the die's L2, as they do in a whole round (pieces at staggered
// k positions run at the rate of memory, which costs more than the idle workgroups did).
//  * r <= slots / 2: every tile in p = min(slots / r, 4) equal pieces; piece c of tile t
//    goes to slot c * r + t, so slots c * r .. c * r + r - 1 form a group in step.
//  * r <= 3/4 slots: each of the first slots - r workgroups computes the tails of
//    g = ceil(r / (slots - r)) <= 3 consecutive tiles, one after the other, and slot
//    slots - r + t the head of tile t; the cut is placed so that both kinds finish
//    together (a tail costs its k tiles and the store of its sums, a head its k tiles
//    and an epilogue: about 0.04 and 0.1 of a tile).
//  * more: the tiles run whole (a cut would save less than it costs).
// The pieces of a tile exchange float32 sums through one tile of memory and a counter per
// shared tile: a piece waits until the counter says that `waits` pieces have deposited,
// adds the sums found there to its own, and either deposits the result (counter + 1) or,
// as the tile's last piece, turns it into the output.  A piece only ever waits for
// workgroups with lower indices (placed before its own), and those never wait for it.
constexpr int kStreamKGranule = 4;
struct StreamKShare {
  int rounds;       // whole rounds: tiles slot + i * slots of the die's run, i < rounds
  // After the rounds: `pieces` pieces of consecutive run entries tile, tile + 1, ..., all
  // over k tiles kbeg .. kbeg + kcnt - 1, computed one after the other.
  int pieces;
  int tile, kbeg, kcnt;
  int waits;        // deposits a piece waits for and adds (0: none)
  int last;         // 1: the pieces run the epilogue; 0: they deposit their sums
};
VMOE_HD int streamk_cut(int U, int c, int parts) {     // k tile where part c of `parts` begins
  return (int)(((long long)U * c + parts / 2) / parts) * kStreamKGranule;
}
VMOE_HD StreamKShare streamk_share(int n, int slots, int j, int nk, bool sharing) {
  StreamKShare s{};
  s.rounds = n / slots;
  const int r = n - s.rounds * slots;
  const int U = nk / kStreamKGranule;
  const int base = s.rounds * slots;
  if (r == 0) return s;
  const bool cut = sharing && nk % kStreamKGranule == 0;
  if (cut && 2 * r <= slots) {
    int parts = slots / r;
    if (parts > 4) parts = 4;
    if (parts > U) parts = U;
    if (parts >= 2) {
      const int c = j / r, t = j - c * r;
      if (c < parts) {
        const int k0 = streamk_cut(U, c, parts), k1 = streamk_cut(U, c + 1, parts);
        s.pieces = 1;
        s.tile = base + t;
        s.kbeg = k0;
        s.kcnt = k1 - k0;
        s.waits = c;
        s.last = c + 1 == parts ? 1 : 0;
      }
      return s;
    }
  } else if (cut && 4 * r <= 3 * slots && U >= 4) {
    const int others = slots - r;
    const int g = (r + others - 1) / others;           // 2 or 3 tails per tail workgroup
    // head + 0.1 = g * (tail + 0.04), head + tail = 1 (in tiles)
    int head = (int)((U * (104LL * g - 10) + 50 * (g + 1)) / (100 * (g + 1)));
    if (head > U - 1) head = U - 1;
    if (head < 1) head = 1;
    const int k1 = head * kStreamKGranule;
    if (j >= others) {
      s.pieces = 1;
      s.tile = base + (j - others);
      s.kbeg = 0;
      s.kcnt = k1;
      s.waits = 1;
      s.last = 1;
    } else {
      const int t = g * j;
      s.pieces = t < r ? plan_min(g, r - t) : 0;
      s.tile = base + t;
      s.kbeg = k1;
      s.kcnt = nk - k1;
      s.waits = 0;
      s.last = 0;
    }
    return s;
  }
  if (j < r) {     // the tiles of the partial round run whole
    s.pieces = 1;
    s.tile = base + j;
    s.kbeg = 0;
    s.kcnt = nk;
    s.waits = 0;
    s.last = 1;
  }
  return s;
}

}  // namespace vmoe
#endif  // VMOE_ROUTE_INDEX_H_
