// Host-side core of the cache manager and of the step description: page pools, block tables,
// request lengths, all-or-nothing reservation, window release, and the packing of one step's
// index arrays into the buffer that is uploaded.  Plain C++ (no GPU code); called through a C
// interface once or twice per step, so that a step of 64 lanes costs the host microseconds.
//
// What the bookkeeping mirrors in the reference: typed, side-effect-free exhaustion
// (crates/macllm-kv/src/cache.rs:649-658), reservation of all lanes' growth before a step
// (:2216-2323, :2331-2445), release at the end of a request (:1840-1852), the scan-based
// cross-check of the accounting (:3810-3841), and the per-step lane records built once and
// shared by all layers (:2707-2786).
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <vector>

namespace {

// Ids 0..total-1 with a free list; the id freed last is handed out first, so a small pool
// reuses its ids at once.
struct Pool {
  int total = 0;
  std::vector<int> free_ids;
  std::vector<uint8_t> held;

  explicit Pool(int n) : total(n), held(n, 0) {
    free_ids.reserve(n);
    for (int id = n - 1; id >= 0; --id) free_ids.push_back(id);
  }
  int free_count() const { return (int)free_ids.size(); }
  bool take(int count, int* out) {
    if (count < 0 || count > free_count()) return false;
    for (int i = 0; i < count; ++i) {
      const int id = free_ids.back();
      free_ids.pop_back();
      held[id] = 1;
      out[i] = id;
    }
    return true;
  }
  // nothing is changed unless every id is held (and named once)
  bool give(const int* ids, int count) {
    for (int i = 0; i < count; ++i) {
      if (ids[i] < 0 || ids[i] >= total || !held[ids[i]]) {
        for (int j = 0; j < i; ++j) held[ids[j]] = 1;
        return false;
      }
      held[ids[i]] = 0;               // a second mention of the same id fails the test above
    }
    free_ids.insert(free_ids.end(), ids, ids + count);
    return true;
  }
  // every id is either free or in `elsewhere`, exactly once: 0; lost or held twice: 1;
  // held elsewhere but marked free: 2
  int check(const int* elsewhere, int count) const {
    std::vector<int> seen(total, 0);
    for (int id : free_ids) {
      if (id < 0 || id >= total) return 1;
      ++seen[id];
    }
    for (int i = 0; i < count; ++i) {
      if (elsewhere[i] < 0 || elsewhere[i] >= total) return 1;
      ++seen[elsewhere[i]];
    }
    for (int id = 0; id < total; ++id)
      if (seen[id] != 1) return 1;
    for (int i = 0; i < count; ++i)
      if (!held[elsewhere[i]]) return 2;
    return 0;
  }
};

struct Table {
  std::vector<int> pages;   // logical page -> page id, or -1 once a window has passed it
  int first_live = 0;
};

struct Group {
  int page_size;
  int window;               // <= 0: every key is kept
  Pool pool;
  std::vector<Table> tables;   // by slot
  Group(int page_size_, int pages, int window_, int slots)
      : page_size(page_size_), window(window_), pool(pages), tables(slots) {}
  int missing(int slot, long new_length) const {
    const long wanted = (new_length + page_size - 1) / page_size;
    const long have = (long)tables[slot].pages.size();
    return wanted > have ? (int)(wanted - have) : 0;
  }
};

struct Core {
  std::vector<Group> groups;
  Pool slots;
  std::vector<int> length;       // tokens of each slot's request that are in the cache
  std::vector<int> scratch;
  Core(int max_slots) : slots(max_slots), length(max_slots, 0) {}
  bool live(int slot) const { return slot >= 0 && slot < slots.total && slots.held[slot]; }
};

}  // namespace

extern "C" {

// ---------------------------------------------------------------- a pool on its own
void* hc_pool_create(int total) { return total > 0 ? new Pool(total) : nullptr; }
void hc_pool_destroy(void* pool) { delete (Pool*)pool; }
int hc_pool_total(void* pool) { return ((Pool*)pool)->total; }
int hc_pool_free_count(void* pool) { return ((Pool*)pool)->free_count(); }
int hc_pool_take(void* pool, int count, int* out) { return ((Pool*)pool)->take(count, out) ? 0 : 1; }
int hc_pool_give(void* pool, const int* ids, int count) { return ((Pool*)pool)->give(ids, count) ? 0 : 1; }
int hc_pool_check(void* pool, const int* elsewhere, int count) { return ((Pool*)pool)->check(elsewhere, count); }

// ---------------------------------------------------------------- the core
void* hc_create(int num_groups, const int* page_size, const int* num_pages, const int* window, int max_slots) {
  if (num_groups < 0 || max_slots <= 0) return nullptr;
  for (int g = 0; g < num_groups; ++g)
    if (page_size[g] <= 0 || num_pages[g] <= 0) return nullptr;
  Core* core = new Core(max_slots);
  core->groups.reserve(num_groups);
  for (int g = 0; g < num_groups; ++g) core->groups.emplace_back(page_size[g], num_pages[g], window[g], max_slots);
  return core;
}
void hc_destroy(void* core) { delete (Core*)core; }
void* hc_group_pool(void* core, int group) { return &((Core*)core)->groups[group].pool; }
void* hc_slot_pool(void* core) { return &((Core*)core)->slots; }

// A state slot for a new request (its tables empty, its length 0), or -1 when none is free.
int hc_add_request(void* handle) {
  Core* core = (Core*)handle;
  int slot;
  if (!core->slots.take(1, &slot)) return -1;
  core->length[slot] = 0;
  for (Group& group : core->groups) {
    group.tables[slot].pages.clear();
    group.tables[slot].first_live = 0;
  }
  return slot;
}

// Everything the slot's request holds goes back.  0, or -1 when the slot is not live.
int hc_finish(void* handle, int slot) {
  Core* core = (Core*)handle;
  if (!core->live(slot)) return -1;
  for (Group& group : core->groups) {
    Table& table = group.tables[slot];
    std::vector<int>& live = core->scratch;
    live.clear();
    for (int page : table.pages)
      if (page >= 0) live.push_back(page);
    if (!group.pool.give(live.data(), (int)live.size())) return -2;
    table.pages.clear();
    table.first_live = 0;
  }
  core->slots.give(&slot, 1);
  return 0;
}

int hc_length(void* handle, int slot) {
  Core* core = (Core*)handle;
  return core->live(slot) ? core->length[slot] : -1;
}

void hc_lengths(void* handle, int n, const int* slots, int* out) {
  Core* core = (Core*)handle;
  for (int i = 0; i < n; ++i) out[i] = core->live(slots[i]) ? core->length[slots[i]] : -1;
}

// Pages for `tokens[i]` more tokens of every listed slot, all or nothing.
// 0: done.  1: not enough pages, nothing changed; info = {group, requested, free, total}.
// -1: a slot is not live or named twice, or a count is not positive; info[0] = the lane.
int hc_reserve(void* handle, int n, const int* slots, const int* tokens, int* info) {
  Core* core = (Core*)handle;
  for (int i = 0; i < n; ++i) {
    if (!core->live(slots[i]) || tokens[i] <= 0) {
      info[0] = i;
      return -1;
    }
    for (int j = 0; j < i; ++j)
      if (slots[j] == slots[i]) {
        info[0] = i;
        return -1;
      }
  }
  for (size_t g = 0; g < core->groups.size(); ++g) {
    const Group& group = core->groups[g];
    long missing = 0;
    for (int i = 0; i < n; ++i) missing += group.missing(slots[i], (long)core->length[slots[i]] + tokens[i]);
    if (missing > group.pool.free_count()) {
      info[0] = (int)g;
      info[1] = (int)std::min<long>(missing, 0x7fffffffL);
      info[2] = group.pool.free_count();
      info[3] = group.pool.total;
      return 1;
    }
  }
  for (Group& group : core->groups)
    for (int i = 0; i < n; ++i) {
      const int missing = group.missing(slots[i], (long)core->length[slots[i]] + tokens[i]);
      if (missing == 0) continue;
      std::vector<int>& pages = group.tables[slots[i]].pages;
      const size_t before = pages.size();
      pages.resize(before + missing);
      group.pool.take(missing, pages.data() + before);
    }
  return 0;
}

// The step ran: lengths advance, and a group with a window gives back every page all later
// queries are past (the next query, at position `length`, sees keys >= length - window + 1).
int hc_commit(void* handle, int n, const int* slots, const int* tokens) {
  Core* core = (Core*)handle;
  for (int i = 0; i < n; ++i)
    if (!core->live(slots[i]) || tokens[i] < 0) return -1;
  for (int i = 0; i < n; ++i) {
    const int slot = slots[i];
    core->length[slot] += tokens[i];
    for (Group& group : core->groups) {
      if (group.window <= 0) continue;
      Table& table = group.tables[slot];
      const long first_needed_key = (long)core->length[slot] - group.window + 1;
      if (first_needed_key <= 0) continue;
      const int first_needed_page = (int)std::min<long>(first_needed_key / group.page_size, (long)table.pages.size());
      if (first_needed_page <= table.first_live) continue;
      if (!group.pool.give(table.pages.data() + table.first_live, first_needed_page - table.first_live)) return -2;
      for (int page = table.first_live; page < first_needed_page; ++page) table.pages[page] = -1;
      table.first_live = first_needed_page;
    }
  }
  return 0;
}

// The slot's block table in a group: returns the number of logical pages and copies up to
// `capacity` page ids (-1 = given back) to `out`.
int hc_table(void* handle, int group, int slot, int* out, int capacity) {
  Core* core = (Core*)handle;
  const std::vector<int>& pages = core->groups[group].tables[slot].pages;
  const int count = (int)pages.size();
  if (out && capacity > 0) std::memcpy(out, pages.data(), sizeof(int) * std::min(count, capacity));
  return count;
}
int hc_first_live(void* handle, int group, int slot) { return ((Core*)handle)->groups[group].tables[slot].first_live; }

// Every page of every group is free or in exactly one live table: 0; else 1 + the group.
int hc_check(void* handle) {
  Core* core = (Core*)handle;
  for (size_t g = 0; g < core->groups.size(); ++g) {
    std::vector<int> held;
    for (int slot = 0; slot < core->slots.total; ++slot) {
      const Table& table = core->groups[g].tables[slot];
      if (!core->slots.held[slot]) {
        if (!table.pages.empty()) return 1 + (int)g;
        continue;
      }
      for (int page : table.pages)
        if (page >= 0) held.push_back(page);
    }
    if (core->groups[g].pool.check(held.data(), (int)held.size()) != 0) return 1 + (int)g;
  }
  return 0;
}

// The index arrays of one step, as 32-bit words in the order
//   token ids [T] | positions [T] | lane of token [T] | first token of each lane [L+1] |
//   start positions [L] | lengths after the step [L] | slot ids [L] | wanted rows [W] |
//   query tiles [tiles, 2] = (lane, first row) of runs of up to `query_tile` rows of one lane |
//   per group: cache cell of each token [T] | block table [L, width] |
//   per chunk size Q: chunks [n, 4] = (lane, first row, rows, index within the lane) of every lane cut from its
//                     first token into runs of Q rows | lane chunks [L, 2] = (first chunk, chunks) of every lane
// for `n` lanes of live slots (their pages already reserved) followed by `pad_lanes` padding lanes
// of `pad_lengths[i]` tokens (token id 0, position from 0) on the scratch slot and the scratch page
// of every group (ids one past the pools').  `max_pages` > 0 fixes every table's width; otherwise
// it is the longest table of the step.  `want_rows_fixed`, if given, replaces the wanted rows
// (`fixed_count` of them).
//
// A step of fixed capacity (one whose arrays a captured graph reads at fixed addresses, whatever lanes it
// holds) fixes the sizes of the sections that depend on how the tokens fall into lanes: `tiles_cap` > 0 makes
// the tile table that long (entries past the step's own hold lane -1: nothing to do), `wants_cap` > 0 the
// wanted rows (entries past the step's own name row 0: computed and dropped), `chunks_cap[c]` > 0 the chunk
// table of chunk size c (entries past the step's own hold lane -1 and no rows).
//
// meta receives: the 9 + 2*groups + 2*chunk_sizes section sizes, then each group's width, then the longest
// context after the step, then the step's own number of chunks for each chunk size.  Returns the words
// written, -1 when a slot is not live, a wanted place is outside its lane or the step's pages were not
// reserved, -2 when the step does not fit a fixed capacity, or -(words needed) - 2 when `capacity` is too small.
long hc_pack(void* handle, int n, const int* slots, const int* lengths, const int* tokens, const int* want_counts,
             const int* wants, int pad_lanes, const int* pad_lengths, int max_pages, int query_tile,
             const int* want_rows_fixed, int fixed_count, int tiles_cap, int wants_cap, int n_chunk_sizes,
             const int* chunk_sizes, const int* chunks_cap, int* out, long capacity, int* meta) {
  Core* core = (Core*)handle;
  const int L = n + pad_lanes;
  const int G = (int)core->groups.size();
  const int C = n_chunk_sizes;
  long T = 0, W = 0, tiles = 0;
  int longest = 0;
  std::vector<long> chunk_count(C, 0);
  for (int i = 0; i < L; ++i) {
    const int length = i < n ? lengths[i] : pad_lengths[i - n];
    if (length <= 0 || query_tile <= 0) return -1;
    if (i < n) {
      if (!core->live(slots[i])) return -1;
      W += want_counts[i];
      longest = std::max(longest, core->length[slots[i]] + length);
    } else {
      longest = std::max(longest, length);
    }
    T += length;
    tiles += (length + query_tile - 1) / query_tile;
    for (int c = 0; c < C; ++c) {
      if (chunk_sizes[c] <= 0) return -1;
      chunk_count[c] += (length + chunk_sizes[c] - 1) / chunk_sizes[c];
    }
  }
  if (want_rows_fixed) W = fixed_count;
  const long own_tiles = tiles, own_wants = W;
  if (tiles_cap > 0) {
    if (tiles > tiles_cap) return -2;
    tiles = tiles_cap;
  }
  if (wants_cap > 0) {
    if (W > wants_cap) return -2;
    W = wants_cap;
  }
  std::vector<long> chunk_rows(C);
  for (int c = 0; c < C; ++c) {
    chunk_rows[c] = chunk_count[c];
    if (chunks_cap && chunks_cap[c] > 0) {
      if (chunk_count[c] > chunks_cap[c]) return -2;
      chunk_rows[c] = chunks_cap[c];
    }
  }
  std::vector<int> width(G, 1);
  for (int g = 0; g < G; ++g) {
    const Group& group = core->groups[g];
    if (max_pages > 0) {
      width[g] = max_pages;
      continue;
    }
    for (int i = 0; i < n; ++i) width[g] = std::max(width[g], (int)group.tables[slots[i]].pages.size());
    for (int i = 0; i < pad_lanes; ++i)
      width[g] = std::max(width[g], (pad_lengths[i] + group.page_size - 1) / group.page_size);
  }
  long total = 3 * T + (L + 1) + 3L * L + W + 2 * tiles;
  for (int g = 0; g < G; ++g) total += T + (long)L * width[g];
  for (int c = 0; c < C; ++c) total += 4 * chunk_rows[c] + 2L * L;
  int* m = meta;
  *m++ = (int)T; *m++ = (int)T; *m++ = (int)T; *m++ = L + 1; *m++ = L; *m++ = L; *m++ = L; *m++ = (int)W;
  *m++ = (int)(2 * tiles);
  for (int g = 0; g < G; ++g) { *m++ = (int)T; *m++ = L * width[g]; }
  for (int c = 0; c < C; ++c) { *m++ = (int)(4 * chunk_rows[c]); *m++ = 2 * L; }
  for (int g = 0; g < G; ++g) *m++ = width[g];
  *m++ = longest;
  for (int c = 0; c < C; ++c) *m++ = (int)chunk_count[c];
  if (total > capacity) return -total - 2;

  int* token_ids = out;
  int* positions = token_ids + T;
  int* lane_of_token = positions + T;
  int* first_token = lane_of_token + T;
  int* start_pos = first_token + L + 1;
  int* seq_lens = start_pos + L;
  int* slot_ids = seq_lens + L;
  int* want_rows = slot_ids + L;
  int* tile_words = want_rows + W;
  int* cursor = tile_words + 2 * tiles;

  long row = 0, want_at = 0, want_out = 0;
  int* tile_at = tile_words;
  for (int i = 0; i < L; ++i) {
    const bool real = i < n;
    const int length = real ? lengths[i] : pad_lengths[i - n];
    const int start = real ? core->length[slots[i]] : 0;
    first_token[i] = (int)row;
    start_pos[i] = start;
    seq_lens[i] = start + length;
    slot_ids[i] = real ? slots[i] : core->slots.total;
    if (real) {
      std::memcpy(token_ids + row, tokens + row, sizeof(int) * length);
      if (!want_rows_fixed)
        for (int w = 0; w < want_counts[i]; ++w) {
          const int place = wants[want_at + w];
          if (place < 0 || place >= length) return -1;
          want_rows[want_out++] = (int)row + place;
        }
      want_at += want_counts[i];
    } else {
      std::memset(token_ids + row, 0, sizeof(int) * length);
    }
    for (int t = 0; t < length; ++t) {
      positions[row + t] = start + t;
      lane_of_token[row + t] = i;
    }
    for (int first = 0; first < length; first += query_tile) {
      *tile_at++ = i;
      *tile_at++ = (int)row + first;
    }
    row += length;
  }
  first_token[L] = (int)row;
  if (want_rows_fixed) std::memcpy(want_rows, want_rows_fixed, sizeof(int) * fixed_count);
  for (long w = own_wants; w < W; ++w) want_rows[w] = 0;
  for (long t = own_tiles; t < tiles; ++t) {
    *tile_at++ = -1;
    *tile_at++ = 0;
  }

  for (int g = 0; g < G; ++g) {
    const Group& group = core->groups[g];
    int* mapping = cursor;
    int* table_out = mapping + T;
    cursor = table_out + (long)L * width[g];
    const int page_size = group.page_size;
    const int scratch_page = group.pool.total;
    row = 0;
    for (int i = 0; i < L; ++i) {
      const bool real = i < n;
      const int length = real ? lengths[i] : pad_lengths[i - n];
      int* table_row = table_out + (long)i * width[g];
      int count;
      if (real) {
        const std::vector<int>& pages = group.tables[slots[i]].pages;
        count = std::min((int)pages.size(), width[g]);
        for (int p = 0; p < count; ++p) table_row[p] = std::max(pages[p], 0);
        const int start = core->length[slots[i]];
        for (int t = 0; t < length; ++t) {
          const int position = start + t;
          const int logical = position / page_size;
          const int page = logical < (int)pages.size() ? pages[logical] : -1;
          if (page < 0) return -1;                       // the step's pages were not reserved
          mapping[row + t] = page * page_size + position % page_size;
        }
      } else {
        count = std::min((length + page_size - 1) / page_size, width[g]);
        for (int p = 0; p < count; ++p) table_row[p] = scratch_page;
        for (int t = 0; t < length; ++t) mapping[row + t] = scratch_page * page_size + t % page_size;
      }
      for (int p = count; p < width[g]; ++p) table_row[p] = 0;
      row += length;
    }
  }

  for (int c = 0; c < C; ++c) {
    const int Q = chunk_sizes[c];
    int* chunk_out = cursor;
    int* lane_out = chunk_out + 4 * chunk_rows[c];
    cursor = lane_out + 2L * L;
    long at = 0;
    row = 0;
    for (int i = 0; i < L; ++i) {
      const int length = i < n ? lengths[i] : pad_lengths[i - n];
      const int count = (length + Q - 1) / Q;
      lane_out[2 * i] = (int)at;
      lane_out[2 * i + 1] = count;
      for (int index = 0; index < count; ++index) {
        chunk_out[4 * at] = i;
        chunk_out[4 * at + 1] = (int)row + index * Q;
        chunk_out[4 * at + 2] = std::min(Q, length - index * Q);
        chunk_out[4 * at + 3] = index;
        ++at;
      }
      row += length;
    }
    for (; at < chunk_rows[c]; ++at) {
      chunk_out[4 * at] = -1;
      chunk_out[4 * at + 1] = 0;
      chunk_out[4 * at + 2] = 0;
      chunk_out[4 * at + 3] = 1;                         // not the first chunk of anything
    }
  }
  return total;
}

}  // extern "C"
