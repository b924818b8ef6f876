// Host side of a compression: which block goes where.  No device work, no allocation on the device.
//
// One side (K or V) of a layer's cache is a set of precision classes, each a list of 32-token blocks in stored order;
// a compression ranks all blocks -- the kept history plus the new tokens -- and cuts the ranking into targets
// (fp16, 8, 4, 2, 1 bit, evicted) by the caller's token counts.  The reference realises the move class by class with
// mask gathers and torch.cat (quant/hqe_2.py:552-659, 672-836); what that sequence amounts to is fixed by three rules:
//   * a block only ever moves to a lower precision: one ranked into a higher class stays where it is;
//   * inside a class the members that stay come first, in their order; then the new tokens ranked into it; then what
//     comes down from the fp16, 8-, 4- and 2-bit classes, each in its source's order;
//   * after an eviction a block's position is its rank among the survivors (quant/hqe_2.py:661-670).
// hqekv_plan_side turns them into the block-level plan hqekv_cache_migrate executes.
#include <stdint.h>

#include <algorithm>
#include <vector>

#include "common.h"

using namespace hq;

extern "C" int hqekv_plan_side(const int32_t *const *old_blocks, const int32_t *old_counts, int32_t hist_blocks,
                               int32_t n_new_blocks, const int64_t *order, const int64_t *target_tokens, int32_t n_targets,
                               int32_t *counts_out, int32_t *plan_out, int32_t *alive_out, int32_t *n_alive_out) {
  constexpr int NCLS = 5, NEW = 5, EVICT = 5;
  if (hist_blocks < 0 || n_new_blocks < 0 || !order || !target_tokens || !counts_out || !plan_out || !alive_out || !n_alive_out ||
      (n_targets != 5 && n_targets != 6) || !old_counts || !old_blocks)
    return fail(HQEKV_E_ARG, "plan_side: null pointer or bad sizes");
  const int64_t total = (int64_t)hist_blocks + n_new_blocks;
  if (total >= (1 << 24)) return fail(HQEKV_E_UNSUPPORTED, "plan_side: %lld blocks (limit 2^24)", (long long)total);
  // ---- the target every block is ranked into
  int64_t sum = 0;
  for (int t = 0; t < n_targets; ++t) {
    if (target_tokens[t] < 0 || target_tokens[t] % HQEKV_GROUP) return fail(HQEKV_E_ARG, "plan_side: target %d holds %lld tokens (whole blocks of 32 only)", t, (long long)target_tokens[t]);
    sum += target_tokens[t] / HQEKV_GROUP;
  }
  if (sum != total) return fail(HQEKV_E_ARG, "plan_side: the targets hold %lld blocks, the side %lld", (long long)sum, (long long)total);
  std::vector<int8_t> label((size_t)total, (int8_t)-1);
  {
    int64_t r = 0;
    for (int t = 0; t < n_targets; ++t)
      for (int64_t k = 0; k < target_tokens[t] / HQEKV_GROUP; ++k, ++r) {
        const int64_t b = order[r];
        if (b < 0 || b >= total || label[(size_t)b] >= 0) return fail(HQEKV_E_ARG, "plan_side: the ranking is not a permutation of the blocks");
        label[(size_t)b] = (int8_t)t;
      }
  }
  // ---- the class every block is in now
  int64_t kept = 0;
  std::vector<int8_t> seen((size_t)total, 0);
  for (int c = 0; c < NCLS; ++c) {
    if (old_counts[c] < 0 || (old_counts[c] > 0 && !old_blocks[c])) return fail(HQEKV_E_ARG, "plan_side: class %d lacks its block list", c);
    for (int32_t j = 0; j < old_counts[c]; ++j) {
      const int32_t b = old_blocks[c][j];
      if (b < 0 || b >= hist_blocks || seen[(size_t)b]) return fail(HQEKV_E_ARG, "plan_side: the classes do not partition the history");
      seen[(size_t)b] = 1;
    }
    kept += old_counts[c];
  }
  if (kept != hist_blocks) return fail(HQEKV_E_ARG, "plan_side: the classes hold %lld blocks of a history of %d", (long long)kept, hist_blocks);
  // ---- lay the new classes out: destination class, then origin (stays / new / down from fp16, 8, 4, 2), then source order
  int32_t *plan_src = plan_out;
  std::vector<int32_t> plan_pos((size_t)total);
  int64_t u = 0;
  for (int d = 0; d < NCLS; ++d) {
    const int64_t begin = u;
    auto take = [&](int src, int32_t n_src, auto &&block_of) {   // blocks of source `src` whose destination is d
      for (int32_t j = 0; j < n_src; ++j) {
        const int32_t b = block_of(j);
        const int own = src == NEW ? -1 : src;
        const int dest = std::max(own, (int)label[(size_t)b]);
        if (dest != d) continue;
        plan_src[u] = (int32_t)(((uint32_t)src << 24) | (uint32_t)j);
        plan_pos[(size_t)u] = b;   // old position for now
        ++u;
      }
    };
    take(d, old_counts[d], [&](int32_t j) { return old_blocks[d][j]; });                    // stays
    take(NEW, n_new_blocks, [&](int32_t j) { return hist_blocks + j; });                     // new tokens
    for (int c = 0; c < d; ++c) take(c, old_counts[c], [&](int32_t j) { return old_blocks[c][j]; });   // comes down
    counts_out[d] = (int32_t)(u - begin);
  }
  // ---- survivors in position order (a block ranked "evicted" is dropped whatever class it is in); a block's new
  // number is its rank among them
  int32_t n_alive = 0;
  for (int64_t b = 0; b < total; ++b)
    if (label[(size_t)b] != EVICT) alive_out[n_alive++] = (int32_t)b;
  if (n_alive != u) return fail(HQEKV_E_ARG, "plan_side: internal count mismatch (%d survivors, %lld planned)", n_alive, (long long)u);
  if (n_alive != total) {
    std::vector<int32_t> rank_of((size_t)total, -1);
    for (int32_t r = 0; r < n_alive; ++r) rank_of[(size_t)alive_out[r]] = r;
    for (int64_t k = 0; k < u; ++k) plan_pos[(size_t)k] = rank_of[(size_t)plan_pos[(size_t)k]];
  }
  std::copy(plan_pos.begin(), plan_pos.begin() + u, plan_out + u);   // the new block numbers follow the u source entries
  *n_alive_out = n_alive;
  return HQEKV_OK;
}
