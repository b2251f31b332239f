// Host build of the routing kernels' index arithmetic (vmoe_amd/csrc/route_index.h compiled
// as plain C++ with -DVMOE_CPU_ONLY), meant to be run under -fsanitize=address,undefined:
// every array has exactly the size the C ABI documents, so an index that leaves a buffer
// is reported.  The cooperative parts of the device kernels (the bitonic sort, the LDS
// atomics, the wave scans) are replaced by sequential loops that call the same scalar
// functions the device threads call; results are compared with the sequential greedy
// statement of the assignment in oracle/route_greedy.c.
//
//   route_host_check [seed]     exit status 0 = every case agrees
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "route_index.h"

extern "C" {
void oracle_top_k(const float* gates, int32_t S, int32_t E, int32_t K, float* val, int32_t* idx);
void oracle_route_greedy(const int32_t* expert_idx, const float* top1, int32_t S, int32_t K,
                         int32_t E, int32_t batch_priority, int32_t* pos, int32_t* count);
}

using namespace vmoe;

static int failures = 0;
#define CHECK(cond, ...) do { if (!(cond)) { if (++failures < 20) { printf("FAIL %s:%d: ", __FILE__, __LINE__); printf(__VA_ARGS__); printf("\n"); } } } while (0)

static uint32_t float_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float bf16_round(float f) {
  uint32_t u = float_bits(f);
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  float r; memcpy(&r, &u, 4); return r;
}

struct Routed {
  std::vector<int32_t> indices, token_slot, slot_token, fill;
};

// What route_assign_group does for all groups, phase by phase.
static Routed route_assign_host(const std::vector<float>& val, const std::vector<int32_t>& idx, int G,
                                int S, int E, int K, int C, bool bpr, bool narrow_keys) {
  Routed out;
  out.indices.assign((size_t)G * S * K * 2, -7);
  out.token_slot.assign((size_t)G * S * K, -7);
  out.slot_token.assign((size_t)E * G * C, -7);
  out.fill.assign((size_t)G * E, -7);
  const int W = (S * K + 31) / 32;
  for (int g = 0; g < G; ++g) {
    const float* v = val.data() + (size_t)g * S * K;
    const int32_t* ix = idx.data() + (size_t)g * S * K;
    std::vector<int32_t> rank(S);
    if (bpr) {
      bool narrow = narrow_keys && S <= 65536;
      for (int s = 0; s < S && narrow; ++s) narrow = bpr_gate_is_narrow(float_bits(v[(size_t)s * K]));
      if (narrow) {
        std::vector<uint32_t> keys(S);
        for (int s = 0; s < S; ++s) keys[s] = bpr_key32(float_bits(v[(size_t)s * K]), s);
        std::sort(keys.begin(), keys.end());
        for (int r = 0; r < S; ++r) rank[keys[r] & 0xffffu] = r;
      } else {
        std::vector<uint64_t> keys(S);
        for (int s = 0; s < S; ++s) keys[s] = bpr_key64(float_bits(v[(size_t)s * K]), s);
        std::sort(keys.begin(), keys.end());
        for (int r = 0; r < S; ++r) rank[(uint32_t)keys[r]] = r;
      }
    } else {
      for (int s = 0; s < S; ++s) rank[s] = s;
    }
    std::vector<uint32_t> bitmap((size_t)E * W, 0u), prefix((size_t)E * W, 0u);
    std::vector<int32_t> total(E, 0);
    for (int i = 0; i < S * K; ++i) {
      const int s = i / K, k = i - s * K, e = ix[i];
      if (e >= 0 && e < E) {
        const int bit = choice_bit(k, S, rank[s]);
        bitmap[(size_t)e * W + (bit >> 5)] |= 1u << (bit & 31);
      }
    }
    for (int e = 0; e < E; ++e) {
      int carry = 0;
      for (int w = 0; w < W; ++w) {
        prefix[(size_t)e * W + w] = (uint32_t)carry;
        carry += __builtin_popcount(bitmap[(size_t)e * W + w]);
      }
      total[e] = carry;
    }
    for (int i = 0; i < S * K; ++i) {
      const int s = i / K, k = i - s * K, e = ix[i];
      int pos = -1, slot = -1;
      if (e >= 0 && e < E) {
        const int bit = choice_bit(k, S, rank[s]);
        const int w = bit >> 5;
        pos = position_from_bitmap(prefix[(size_t)e * W + w], bitmap[(size_t)e * W + w], bit);
        if (pos < C) {
          slot = slot_row(e, g, pos, G, E, C);
          out.slot_token.at(slot) = g * S + s;
        }
      }
      const size_t o = (size_t)g * S * K + i;
      out.indices.at(2 * o) = e;
      out.indices.at(2 * o + 1) = pos;
      out.token_slot.at(o) = slot;
    }
    for (int i = 0; i < E * C; ++i) {
      const int e = i / C, c = i - e * C;
      if (c >= total[e]) out.slot_token.at(slot_row(e, g, c, G, E, C)) = -1;
    }
    for (int e = 0; e < E; ++e) out.fill.at((size_t)g * E + e) = total[e] < C ? total[e] : C;
  }
  return out;
}

static void check_routing(std::mt19937& rng, int G, int S, int E, int K, int C, int flavour) {
  std::normal_distribution<float> normal(0.f, 2.f);
  std::vector<float> gates((size_t)G * S * E);
  for (int g = 0; g < G; ++g)
    for (int s = 0; s < S; ++s) {
      float* row = gates.data() + ((size_t)g * S + s) * E;
      float mx = -1e30f, sum = 0.f;
      for (int e = 0; e < E; ++e) { row[e] = normal(rng); if (flavour == 2) row[e] = (float)(int)row[e]; mx = std::max(mx, row[e]); }
      if (flavour == 3) { for (int e = 0; e < E; ++e) row[e] = (float)(int)(row[e] * 2) / 4; continue; }   // negative, zero, tied
      for (int e = 0; e < E; ++e) { row[e] = expf(row[e] - mx); sum += row[e]; }
      for (int e = 0; e < E; ++e) { row[e] /= sum; if (flavour >= 1) row[e] = bf16_round(row[e]); }
    }
  std::vector<float> val((size_t)G * S * K);
  std::vector<int32_t> idx((size_t)G * S * K);
  for (int g = 0; g < G; ++g)
    oracle_top_k(gates.data() + (size_t)g * S * E, S, E, K, val.data() + (size_t)g * S * K, idx.data() + (size_t)g * S * K);
  for (int bpr = 0; bpr < 2; ++bpr) {
    const Routed r = route_assign_host(val, idx, G, S, E, K, C, bpr, true);
    const Routed wide = route_assign_host(val, idx, G, S, E, K, C, bpr, false);
    CHECK(r.indices == wide.indices, "32- and 64-bit keys disagree: G=%d S=%d E=%d K=%d", G, S, E, K);
    std::vector<int32_t> pos((size_t)S * K), count(E);
    std::vector<float> top1(S);
    std::vector<char> claimed((size_t)E * G * C, 0);
    for (int g = 0; g < G; ++g) {
      for (int s = 0; s < S; ++s) top1[s] = val[((size_t)g * S + s) * K];
      oracle_route_greedy(idx.data() + (size_t)g * S * K, top1.data(), S, K, E, bpr, pos.data(), count.data());
      for (int i = 0; i < S * K; ++i) {
        const size_t o = (size_t)g * S * K + i;
        CHECK(r.indices[2 * o] == idx[o] && r.indices[2 * o + 1] == pos[i],
              "G=%d S=%d E=%d K=%d C=%d bpr=%d flavour=%d group %d choice %d: (%d,%d) want (%d,%d)", G, S, E, K, C,
              bpr, flavour, g, i, r.indices[2 * o], r.indices[2 * o + 1], idx[o], pos[i]);
        const int slot = r.token_slot[o];
        CHECK((slot >= 0) == (pos[i] < C), "kept flag: group %d choice %d", g, i);
        if (slot >= 0) {
          CHECK(slot < E * G * C && r.slot_token[slot] == g * S + i / K && !claimed[slot], "slot maps: slot %d", slot);
          claimed[slot] = 1;
        }
      }
      for (int e = 0; e < E; ++e) CHECK(r.fill[(size_t)g * E + e] == std::min(count[e], C), "fill");
    }
    for (size_t s = 0; s < claimed.size(); ++s)
      CHECK(claimed[s] ? r.slot_token[s] >= 0 : r.slot_token[s] == -1, "unclaimed slot %zu holds %d", s, r.slot_token[s]);

    // packed rows (compact_rows_kernel / compact_rows_fused_kernel per assignment)
    std::vector<int32_t> prefix((size_t)G * E), rows(E, 0);
    for (int e = 0; e < E; ++e) {
      int carry = 0;
      for (int g = 0; g < G; ++g) { prefix[(size_t)g * E + e] = carry; carry += r.fill[(size_t)g * E + e]; }
      rows[e] = carry;
    }
    std::vector<int32_t> token_row((size_t)G * S * K, -7), row_token((size_t)E * G * C, -1);
    for (size_t i = 0; i < token_row.size(); ++i) {
      const int slot = r.token_slot[i];
      int row = -1;
      if (slot >= 0) {
        const int g = (int)(i / ((size_t)S * K));
        row = packed_row(slot, prefix.at((size_t)g * E + slot_expert(slot, G, C)), G, C);
        CHECK(row_token.at(row) == -1, "packed row %d written twice", row);
        row_token.at(row) = (int)(i / K);
      }
      token_row[i] = row;
    }
    for (int e = 0; e < E; ++e)
      for (int q = 0; q < G * C; ++q)
        CHECK((row_token[(size_t)e * G * C + q] >= 0) == (q < rows[e]), "expert %d packed row %d of %d", e, q, rows[e]);

    // launch plans over these row counts, for the tile shapes the products use
    for (int bm : {128, 256, 384})
      for (int tiles_n : {1, 3, 12})
        for (int panel_rows : {1, 5, 13}) {
          const int R = G * C;
          const int share_max = (E * ((R + bm - 1) / bm) + kNumXcd - 1) / kNumXcd;
          const int num_blocks = share_max * tiles_n * kNumXcd;
          std::vector<PlanEntry> plan(num_blocks);
          RaggedGeom geom{bm, tiles_n, panel_rows, num_blocks, plan.data()};
          std::vector<int32_t> tile_prefix(E + 1, 0);
          for (int e = 0; e < E; ++e) tile_prefix[e + 1] = tile_prefix[e] + (std::min(std::max(rows[e], 0), R) + bm - 1) / bm;
          for (int i = 0; i < num_blocks; ++i) plan[i] = plan_entry(geom, tile_prefix.data(), rows.data(), E, R, i);
          std::vector<int> seen((size_t)tile_prefix[E] * tiles_n, 0);
          for (int x = 0; x < kNumXcd; ++x) {
            bool ended = false;
            for (int slot = 0; slot * kNumXcd + x < num_blocks; ++slot) {
              const PlanEntry p = plan[slot * kNumXcd + x];
              if (p.batch < 0) { ended = true; continue; }
              CHECK(!ended, "die %d: work after an empty slot", x);
              CHECK(p.batch < E && p.tile_n >= 0 && p.tile_n < tiles_n && p.live == rows[p.batch] && p.tile_m >= 0 &&
                    p.tile_m * bm < p.live, "plan entry out of range: batch %d tile (%d,%d) live %d", p.batch, p.tile_m, p.tile_n, p.live);
              if (p.batch < E && p.tile_m >= 0 && p.tile_m * bm < rows[p.batch] && p.tile_n < tiles_n)
                ++seen.at(((size_t)tile_prefix[p.batch] + p.tile_m) * tiles_n + p.tile_n);
            }
          }
          for (size_t t = 0; t < seen.size(); ++t) CHECK(seen[t] == 1, "bm=%d tiles_n=%d panel_rows=%d: tile %zu planned %d times", bm, tiles_n, panel_rows, t, seen[t]);
        }
  }
}

// indices_to_slots_kernel on hand-made pairs, out-of-range and negative entries included.
static void check_index_pairs(std::mt19937& rng, int G, int S, int E, int K, int C) {
  std::uniform_int_distribution<int> de(-1, E + 1), dc(-1, C + 1);
  const size_t n = (size_t)G * S * K;
  std::vector<int32_t> token_slot(n, -7), slot_token((size_t)E * G * C, -1);
  int invalid = 0, dup = 0, want_invalid = 0;
  for (size_t i = 0; i < n; ++i) {
    const int e = de(rng), c = dc(rng);
    const size_t item = i / K;
    bool inv;
    const int slot = slot_of_index_pair(e, c, (int)(item / S), G, E, C, &inv);
    invalid += inv;
    want_invalid += (e < 0 || c < 0);
    CHECK((slot >= 0) == (e >= 0 && c >= 0 && e < E && c < C), "pair (%d,%d) -> slot %d", e, c, slot);
    if (slot >= 0) {
      CHECK(slot / (G * C) == e, "slot %d is not in expert %d's block", slot, e);
      if (slot_token.at(slot) >= 0) ++dup;
      slot_token.at(slot) = (int)item;
    }
    token_slot[i] = slot;
  }
  CHECK(invalid == want_invalid, "invalid count");
  (void)dup;
}


// Stream-K share of a die's partial round (streamk_share): over die runs of 0 .. 200 tiles
// and several k lengths, every k tile of every tile is computed exactly once by pieces of
// at least three k tiles; the pieces of a tile wait for 0, 1, 2, ... deposits, in ascending
// slot order, and exactly the one that waits for all the others runs the epilogue; shared,
// the partial round costs a workgroup at most 0.85 of a tile's k tiles (plus rounding).
static int check_streamk() {
  int cases = 0;
  const int slots = 32;
  for (int sharing = 0; sharing < 2; ++sharing)
    for (int nk : {4, 8, 12, 16, 48, 64, 80, 50})
      for (int n = 0; n <= 200; ++n) {
        ++cases;
        struct Pc { int slot, kbeg, kcnt, last, waits; };
        std::vector<std::vector<Pc>> tiles(n);
        int maxpiece = 0;
        for (int j = 0; j < slots; ++j) {
          const StreamKShare s = streamk_share(n, slots, j, nk, sharing != 0);
          CHECK(s.rounds == n / slots && s.pieces >= 0 && s.pieces <= 3, "share n=%d j=%d", n, j);
          for (int i = 0; i < s.rounds; ++i) tiles[j + i * slots].push_back({j, 0, nk, 1, 0});
          int work = 0;
          for (int i = 0; i < s.pieces; ++i) {
            const int tile = s.tile + i;
            CHECK(tile >= s.rounds * slots && tile < n && tile - s.rounds * slots < slots && s.kbeg >= 0 &&
                  s.kcnt >= 3 && s.kbeg + s.kcnt <= nk, "piece n=%d nk=%d j=%d", n, nk, j);
            if (tile < 0 || tile >= n) continue;
            tiles[tile].push_back({j, s.kbeg, s.kcnt, s.last, s.waits});
            work += s.kcnt;
          }
          maxpiece = std::max(maxpiece, work);
        }
        for (int t = 0; t < n; ++t) {
          auto& v = tiles[t];
          std::sort(v.begin(), v.end(), [](const Pc& a, const Pc& b) { return a.kbeg < b.kbeg; });
          int k = 0;
          for (size_t a = 0; a < v.size(); ++a) {
            CHECK(v[a].kbeg == k, "pieces consecutive n=%d nk=%d t=%d", n, nk, t);
            k += v[a].kcnt;
          }
          CHECK(k == nk, "tile covered n=%d nk=%d t=%d", n, nk, t);
          std::sort(v.begin(), v.end(), [](const Pc& a, const Pc& b) { return a.waits < b.waits; });
          for (size_t a = 0; a < v.size(); ++a) {
            CHECK(v[a].waits == (int)a, "deposit order n=%d nk=%d t=%d", n, nk, t);
            if (a > 0) CHECK(v[a].slot > v[a - 1].slot, "a piece waits for lower slots only n=%d nk=%d t=%d", n, nk, t);
            CHECK((v[a].last != 0) == (a + 1 == v.size()), "last piece n=%d nk=%d t=%d", n, nk, t);
          }
        }
        const int r = n % slots;
        if (sharing && nk % kStreamKGranule == 0 && nk >= 4 * kStreamKGranule && r > 0 && 4 * r <= 3 * slots)
          CHECK(100 * maxpiece <= 85 * nk + 100 * kStreamKGranule, "partial round n=%d nk=%d: %d k tiles", n, nk, maxpiece);
      }
  return cases;
}

int main(int argc, char** argv) {
  std::mt19937 rng(argc > 1 ? (unsigned)atoi(argv[1]) : 2024u);
  const int sizes[] = {1, 2, 3, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1000,
                       1023, 1024, 1025, 1500, 2047, 2048, 2049, 3000, 4095, 4096, 4097};
  int cases = 0;
  for (int rep = 0; rep < 2; ++rep)
    for (int S : sizes) {
      const int E = 1 + (int)(rng() % 40);
      const int K = 1 + (int)(rng() % std::min(E, 4));
      const int G = 1 + (int)(rng() % 3);
      const int C = 1 + (int)(rng() % std::max(1, (S * K) / E + 2));
      check_routing(rng, G, S, E, K, C, cases % 4);
      check_index_pairs(rng, G, S, E, K, C);
      ++cases;
    }
  // groups divisible by experts (interleaved row order) and the benchmark shapes' group counts
  check_routing(rng, 8, 96, 4, 2, 40, 1);
  check_routing(rng, 32, 200, 32, 2, 13, 1);
  check_routing(rng, 16, 300, 32, 2, 10, 0);
  check_routing(rng, 6, 50, 3, 1, 100, 3);
  cases += 4;
  cases += check_streamk();
  printf("%d cases, %d failures\n", cases, failures);
  return failures == 0 ? 0 : 1;
}
