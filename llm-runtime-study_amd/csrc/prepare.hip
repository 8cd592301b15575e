// The host side of a step's metadata: fills the pinned staging buffer that one copy takes to the device.
//
// Nothing here touches the GPU.  The step function (engine/step.py) hands over what it knows of the step's
// entries as flat arrays, and this routine writes every array of the device metadata: token ids, positions,
// request row and state slot of each token, rows whose logits are wanted, per request cumulative query starts,
// context lengths and state slots, the query groups for mixers that ask for them, and per cache group the
// physical slot of each token (looked up in the host's block tables).  It is the inner loop of every step on the
// host; in Python it was half of a step's host time.  The Python routine that does the same stays as the
// reference (ModelRunner.prepare with native=False); a test runs both on random steps and compares every word.
#include "common.h"

#include <algorithm>
#include <vector>

extern "C" int lrs_attention_prefill_group_for(int tokens, int longest);

namespace {

// Order of the arrays in `offsets` (element offsets into the staging buffer); the per-group slot arrays follow.
enum {
  AT_TOKEN_IDS, AT_POSITIONS, AT_TOKEN_REQUEST, AT_TOKEN_SLOT, AT_LOGIT_ROWS, AT_CU_SEQLENS_Q, AT_SEQ_LENS_K, AT_SLOT_IDS,
  AT_QBLOCK_TOKEN0, AT_QBLOCK_COUNT, AT_COUNTS, AT_GROUP_SLOTS
};
// Order of the numbers handed back in `summary`.
enum { OUT_T, OUT_R, OUT_LOGIT_ROWS, OUT_QBLOCKS, OUT_MAX_QBLOCK, OUT_MAX_Q, OUT_MAX_K, OUT_SINGLE_ROWS, OUT_COUNT };

struct Group {
  int key, token0, count;
};

}  // namespace

// entries: n_entries requests; entry i brings entry_tokens[i] tokens (tokens_flat, in order), holds entry_length[i]
// positions after them (for a step prepared ahead of later steps of its launch: minus those), sits in state slot
// entry_slot[i], and wants the logits at the entry_wants[i] places listed in want_flat (places among its own tokens).
// pad_to > 0 (decode-only steps): rows up to pad_to belong to no request (token 0 at position 0 of the trash slot)
// and logits are wanted for every row.  tables[g] is the host block table of cache group g, [*, max_blocks], row =
// state slot (the trash slot's row names the trash page).  query_group: the most tokens in a query group, 0: no
// mixer asks for groups.  Returns 0, or 1 with a message for lrs_last_error().
LRS_API int lrs_step_prepare(int32_t* meta, const int64_t* offsets, int n_entries, const int32_t* entry_slot,
                             const int32_t* entry_length, const int32_t* entry_tokens, const int32_t* tokens_flat,
                             const int32_t* entry_wants, const int32_t* want_flat, int pad_to, int trash_slot,
                             int n_groups, const int32_t* const* tables, int max_blocks, int page_size, int query_group,
                             int32_t* summary) {
  LRS_REQUIRE(meta && offsets && n_entries > 0 && entry_slot && entry_length && entry_tokens && tokens_flat && entry_wants && summary,
              "step_prepare: missing arrays or no entries");
  LRS_REQUIRE(page_size > 0 && max_blocks > 0 && n_groups >= 0 && pad_to >= 0, "step_prepare: bad sizes");
  int32_t* ids = meta + offsets[AT_TOKEN_IDS];
  int32_t* pos = meta + offsets[AT_POSITIONS];
  int32_t* req = meta + offsets[AT_TOKEN_REQUEST];
  int32_t* of_token = meta + offsets[AT_TOKEN_SLOT];
  int32_t* rows = meta + offsets[AT_LOGIT_ROWS];
  int32_t* cu = meta + offsets[AT_CU_SEQLENS_Q];
  int32_t* lens = meta + offsets[AT_SEQ_LENS_K];
  int32_t* slots = meta + offsets[AT_SLOT_IDS];
  int32_t* counts = meta + offsets[AT_COUNTS];
  int cursor = 0, n_rows = 0, at_token = 0, at_want = 0, max_q = 0, max_k = 0, singles = -1;
  cu[0] = 0;
  for (int r = 0; r < n_entries; ++r) {
    const int n = entry_tokens[r], length = entry_length[r], start = length - n;
    LRS_REQUIRE(n > 0 && start >= 0, "step_prepare: entry %d brings %d tokens into a cache of %d", r, n, length);
    for (int i = 0; i < n; ++i) {
      ids[cursor + i] = tokens_flat[at_token + i];
      pos[cursor + i] = start + i;
      req[cursor + i] = r;
      of_token[cursor + i] = entry_slot[r];
    }
    for (int w = 0; w < entry_wants[r]; ++w) rows[n_rows++] = cursor + want_flat[at_want + w];
    at_token += n;
    at_want += entry_wants[r];
    cursor += n;
    cu[r + 1] = cursor;
    lens[r] = length;
    slots[r] = entry_slot[r];
    max_q = std::max(max_q, n);
    max_k = std::max(max_k, length);
    if (singles < 0 && n != 1) singles = r;
  }
  const int real = n_entries;
  const bool all_decode = max_q == 1;
  if (pad_to > real) {
    LRS_REQUIRE(all_decode, "step_prepare: only a decode-only step can be padded");
    for (int r = real; r < pad_to; ++r) {
      ids[cursor] = 0;
      pos[cursor] = 0;
      req[cursor] = r;
      of_token[cursor] = trash_slot;
      ++cursor;
      cu[r + 1] = cursor;
      lens[r] = 1;
      slots[r] = trash_slot;
    }
  }
  if (pad_to > 0) {
    for (int t = 0; t < cursor; ++t) rows[t] = t;
    n_rows = cursor;
  }
  counts[0] = real;
  int n_groups_q = 0, max_group = 0, single_rows = 0;
  if (query_group > 0) {
    int32_t* token0 = meta + offsets[AT_QBLOCK_TOKEN0];
    int32_t* count = meta + offsets[AT_QBLOCK_COUNT];
    std::vector<Group> groups;
    if (all_decode) {
      groups.reserve(cursor);
      for (int t = 0; t < cursor; ++t) groups.push_back(Group{pos[t], t, 1});
    } else {
      // the requests at the head of the step that bring one token each are left to the mixer as single rows;
      // the groups cover the rows after them and count their tokens from there
      single_rows = singles;
      int size = lrs_attention_prefill_group_for(cursor - singles, max_k);
      if (size > query_group) size = query_group;
      LRS_REQUIRE(size > 0, "step_prepare: no query group size for %d tokens", cursor - singles);
      for (int r = singles; r < real; ++r)
        for (int t0 = cu[r]; t0 < cu[r + 1]; t0 += size) {
          const int n = std::min(size, cu[r + 1] - t0);
          groups.push_back(Group{pos[t0 + n - 1], t0 - singles, n});
        }
    }
    std::stable_sort(groups.begin(), groups.end(), [](const Group& a, const Group& b) { return a.key > b.key; });   // longest context first
    for (size_t i = 0; i < groups.size(); ++i) {
      token0[i] = groups[i].token0;
      count[i] = groups[i].count;
      max_group = std::max(max_group, groups[i].count);
    }
    n_groups_q = (int)groups.size();
  }
  for (int g = 0; g < n_groups; ++g) {
    int32_t* gslots = meta + offsets[AT_GROUP_SLOTS + g];
    const int32_t* table = tables[g];
    for (int t = 0; t < cursor; ++t) {
      const int block = pos[t] / page_size;
      LRS_REQUIRE(block < max_blocks, "step_prepare: position %d lies beyond the block table's %d blocks", pos[t], max_blocks);
      const int32_t page = table[(int64_t)of_token[t] * max_blocks + block];
      gslots[t] = page >= 0 ? page * page_size + pos[t] % page_size : -1;
    }
  }
  summary[OUT_T] = cursor;
  summary[OUT_R] = std::max(real, pad_to);
  summary[OUT_LOGIT_ROWS] = n_rows;
  summary[OUT_QBLOCKS] = n_groups_q;
  summary[OUT_MAX_QBLOCK] = max_group;
  summary[OUT_MAX_Q] = max_q;
  summary[OUT_MAX_K] = max_k;
  summary[OUT_SINGLE_ROWS] = single_rows;
  return 0;
}

LRS_API int lrs_step_prepare_summary_size() { return OUT_COUNT; }
