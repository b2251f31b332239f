/* Sequential greedy slot assignment (TEST INFRASTRUCTURE ONLY).
 *
 * An independent C statement of what vmoe/moe.py:547-590 + :626-652 evaluate
 * to for one group: every choice level k is walked in order (all first choices
 * before any second choice, moe.py:573-575), inside a level items are walked
 * by priority -- index order, or, with batch priority routing, descending
 * first-choice gate with the item index as tie break (stable argsort of the
 * negated gate, moe.py:571) -- and each visit takes the next free position of
 * the chosen expert.  Positions are NOT clipped to the capacity
 * (moe.py:646 keeps the raw cumsum value).
 *
 * Also holds top-k selection with the tie rule of jax.lax.top_k (descending,
 * lower index first) so the C side can route from gates alone.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct { float key; int32_t idx; } keyed_t;

static int cmp_desc_stable(const void* a, const void* b) {
  const keyed_t* x = (const keyed_t*)a;
  const keyed_t* y = (const keyed_t*)b;
  if (x->key > y->key) return -1;
  if (x->key < y->key) return 1;
  return (x->idx > y->idx) - (x->idx < y->idx);
}

/* gates (S,E) -> val (S,K), idx (S,K). */
void oracle_top_k(const float* gates, int32_t S, int32_t E, int32_t K,
                  float* val, int32_t* idx) {
  keyed_t* row = (keyed_t*)malloc(sizeof(keyed_t) * (size_t)E);
  for (int32_t s = 0; s < S; ++s) {
    for (int32_t e = 0; e < E; ++e) { row[e].key = gates[(size_t)s * E + e]; row[e].idx = e; }
    qsort(row, (size_t)E, sizeof(keyed_t), cmp_desc_stable);
    for (int32_t k = 0; k < K; ++k) { val[(size_t)s * K + k] = row[k].key; idx[(size_t)s * K + k] = row[k].idx; }
  }
  free(row);
}

/* expert_idx (S,K), top1 (S) or NULL -> pos (S,K), count (E). */
void oracle_route_greedy(const int32_t* expert_idx, const float* top1,
                         int32_t S, int32_t K, int32_t E, int32_t batch_priority,
                         int32_t* pos, int32_t* count) {
  keyed_t* order = (keyed_t*)malloc(sizeof(keyed_t) * (size_t)S);
  for (int32_t s = 0; s < S; ++s) { order[s].key = batch_priority ? top1[s] : 0.0f; order[s].idx = s; }
  if (batch_priority) qsort(order, (size_t)S, sizeof(keyed_t), cmp_desc_stable);
  memset(count, 0, sizeof(int32_t) * (size_t)E);
  for (int32_t k = 0; k < K; ++k)
    for (int32_t r = 0; r < S; ++r) {
      int32_t s = order[r].idx;
      int32_t e = expert_idx[(size_t)s * K + k];
      pos[(size_t)s * K + k] = count[e]++;
    }
  free(order);
}

/* Whole batch: gates (G,S,E) -> indices (G,S,K,2), weights (G,S,K). */
void oracle_route_batch(const float* gates, int32_t G, int32_t S, int32_t E, int32_t K,
                        int32_t batch_priority, int32_t* indices, float* weights) {
  int32_t* idx = (int32_t*)malloc(sizeof(int32_t) * (size_t)S * K);
  int32_t* pos = (int32_t*)malloc(sizeof(int32_t) * (size_t)S * K);
  int32_t* cnt = (int32_t*)malloc(sizeof(int32_t) * (size_t)E);
  float* top1 = (float*)malloc(sizeof(float) * (size_t)S);
  for (int32_t g = 0; g < G; ++g) {
    float* w = weights + (size_t)g * S * K;
    oracle_top_k(gates + (size_t)g * S * E, S, E, K, w, idx);
    for (int32_t s = 0; s < S; ++s) top1[s] = w[(size_t)s * K];
    oracle_route_greedy(idx, top1, S, K, E, batch_priority, pos, cnt);
    for (int32_t i = 0; i < S * K; ++i) {
      indices[((size_t)g * S * K + i) * 2 + 0] = idx[i];
      indices[((size_t)g * S * K + i) * 2 + 1] = pos[i];
    }
  }
  free(idx); free(pos); free(cnt); free(top1);
}
