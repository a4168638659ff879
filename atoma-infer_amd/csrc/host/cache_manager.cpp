// Page tables and free lists of the paged cache, and the slots of per-request fixed-size state.
//
// Layers with equal cache needs form a group; each group has its own pool of pages (its own page numbers) and each
// request has one block table per group.  A group may keep all tokens or only a window of the last W: pages
// that a window has passed are given back while the request is still running.  Pages come from a LIFO free
// list, so the page freed last is used next (the reference's allocator pops from a Vec the same way:
// backends/vllm/src/block_allocator.rs:59-111).  Unlike the reference (backends/vllm/src/block_manager.rs:195-237,
// 294-377) pages are reserved for whatever length the next step reaches, any number at a time, and all groups
// together or not at all.
//
// Plain C interface; no GPU code.  Not thread-safe: one engine thread owns a manager.
#include <cstdint>
#include <cstring>
#include <unordered_map>
#include <vector>

namespace {

struct Group {
  int page_size = 0;
  int num_pages = 0;
  int window = 0;  // 0: keep everything
  std::vector<int32_t> free_list;
  std::vector<uint8_t> in_use;
};

struct Request {
  int state_slot = -1;
  int64_t reserved_len = 0;                   // pages cover positions [0, reserved_len) except released ones
  std::vector<std::vector<int32_t>> tables;   // per group; -1 marks a released entry
  std::vector<int64_t> first_live;            // per group: index of the first entry not released
};

struct Manager {
  std::vector<Group> groups;
  std::unordered_map<int64_t, Request> requests;
  std::vector<int32_t> free_slots;
  std::vector<uint8_t> slot_in_use;
};

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// entries of the block table needed so that positions [0, len) are covered
inline int64_t blocks_for(const Group& g, int64_t len) { return ceil_div(len, g.page_size); }

// number of new pages group gi must hand out so that request r reaches new_len
int64_t pages_needed(const Manager& m, const Request* r, size_t gi, int64_t new_len) {
  const Group& g = m.groups[gi];
  const int64_t have = r ? (int64_t)r->tables[gi].size() : 0;
  const int64_t want = blocks_for(g, new_len);
  return want > have ? want - have : 0;
}

// pages of request r in group gi that are still held (table entries that a window has not released)
int64_t live_pages(const Request& r, size_t gi) { return (int64_t)r.tables[gi].size() - r.first_live[gi]; }

}  // namespace

extern "C" {

enum { CM_OK = 0, CM_NO_PAGES = -1, CM_EXISTS = -2, CM_UNKNOWN = -3, CM_NO_SLOT = -4, CM_BAD_ARG = -5,
       CM_CORRUPT = -6 };

void* cm_create(int n_groups, const int32_t* page_sizes, const int32_t* num_pages, const int32_t* windows,
                int n_state_slots) {
  if (n_groups < 0 || n_state_slots < 0) return nullptr;
  for (int i = 0; i < n_groups; ++i)
    if (page_sizes[i] <= 0 || num_pages[i] < 0 || windows[i] < 0) return nullptr;
  Manager* m = new Manager();
  m->groups.resize(n_groups);
  for (int i = 0; i < n_groups; ++i) {
    Group& g = m->groups[i];
    g.page_size = page_sizes[i];
    g.num_pages = num_pages[i];
    g.window = windows[i];
    g.in_use.assign(g.num_pages, 0);
    g.free_list.reserve(g.num_pages);
    // page 0 is handed out first
    for (int p = g.num_pages - 1; p >= 0; --p) g.free_list.push_back(p);
  }
  m->slot_in_use.assign(n_state_slots, 0);
  for (int s = n_state_slots - 1; s >= 0; --s) m->free_slots.push_back(s);
  return m;
}

void cm_destroy(void* h) { delete static_cast<Manager*>(h); }

// Registers a request and gives it a state slot.  Returns the slot, or a negative code.
int cm_add_request(void* h, int64_t id) {
  Manager* m = static_cast<Manager*>(h);
  if (m->requests.count(id)) return CM_EXISTS;
  if (m->free_slots.empty()) return CM_NO_SLOT;
  Request r;
  r.state_slot = m->free_slots.back();
  m->free_slots.pop_back();
  m->slot_in_use[r.state_slot] = 1;
  r.tables.resize(m->groups.size());
  r.first_live.assign(m->groups.size(), 0);
  m->requests.emplace(id, std::move(r));
  return m->requests[id].state_slot;
}

// 1 if cm_reserve(id, new_len) would succeed.  An unknown id is treated as a request that holds nothing yet.
int cm_can_reserve(void* h, int64_t id, int64_t new_len) {
  Manager* m = static_cast<Manager*>(h);
  auto it = m->requests.find(id);
  const Request* r = it == m->requests.end() ? nullptr : &it->second;
  if (!r && m->free_slots.empty()) return 0;
  for (size_t gi = 0; gi < m->groups.size(); ++gi)
    if (pages_needed(*m, r, gi, new_len) > (int64_t)m->groups[gi].free_list.size()) return 0;
  return 1;
}

// 1 if a request of new_len tokens could ever be held, with every page free.  A group with a window gives pages
// back as the request moves on: it must hold the window and the page that the next token opens.
int cm_fits_at_all(void* h, int64_t new_len) {
  Manager* m = static_cast<Manager*>(h);
  for (const Group& g : m->groups) {
    int64_t need = blocks_for(g, new_len);
    if (g.window > 0 && blocks_for(g, g.window) + 1 < need) need = blocks_for(g, g.window) + 1;
    if (need > g.num_pages) return 0;
  }
  return 1;
}

// 1 if a new request of total_len tokens may start with a first portion of first_len tokens.  Beside the pages of
// that portion, a group with a window must have room for what the newcomer and every request already held will
// need once they have moved on: the window and the page that the next token opens, each.  Without that, a request
// admitted into pages that the others are about to ask for is preempted again at once, step after step.
int cm_can_admit(void* h, int64_t total_len, int64_t first_len) {
  Manager* m = static_cast<Manager*>(h);
  if (m->free_slots.empty() || first_len > total_len) return 0;
  for (size_t gi = 0; gi < m->groups.size(); ++gi) {
    const Group& g = m->groups[gi];
    int64_t need = blocks_for(g, first_len);
    if (g.window > 0) {
      const int64_t steady = blocks_for(g, g.window) + 1;
      const int64_t own = blocks_for(g, total_len) < steady ? blocks_for(g, total_len) : steady;
      if (own > need) need = own;
      for (const auto& kv : m->requests) {
        const int64_t lack = steady - live_pages(kv.second, gi);
        if (lack > 0) need += lack;
      }
    }
    if (need > (int64_t)g.free_list.size()) return 0;
  }
  return 1;
}

// 1 if some group keeps a window only.
int cm_has_window(void* h) {
  for (const Group& g : static_cast<Manager*>(h)->groups)
    if (g.window > 0) return 1;
  return 0;
}

// Makes every group cover positions [0, new_len).  All groups or none.
int cm_reserve(void* h, int64_t id, int64_t new_len) {
  Manager* m = static_cast<Manager*>(h);
  auto it = m->requests.find(id);
  if (it == m->requests.end()) return CM_UNKNOWN;
  if (new_len < 0) return CM_BAD_ARG;
  Request& r = it->second;
  for (size_t gi = 0; gi < m->groups.size(); ++gi)
    if (pages_needed(*m, &r, gi, new_len) > (int64_t)m->groups[gi].free_list.size()) return CM_NO_PAGES;
  for (size_t gi = 0; gi < m->groups.size(); ++gi) {
    Group& g = m->groups[gi];
    for (int64_t n = pages_needed(*m, &r, gi, new_len); n > 0; --n) {
      const int32_t p = g.free_list.back();
      g.free_list.pop_back();
      g.in_use[p] = 1;
      r.tables[gi].push_back(p);
    }
  }
  if (new_len > r.reserved_len) r.reserved_len = new_len;
  return CM_OK;
}

// Gives back, in windowed groups, the pages that no token at position >= computed_len can see any more:
// a query at position p sees keys p - W + 1 .. p, so every key below computed_len - W + 1 is dead.
// Returns the number of pages released.
int cm_release_behind(void* h, int64_t id, int64_t computed_len) {
  Manager* m = static_cast<Manager*>(h);
  auto it = m->requests.find(id);
  if (it == m->requests.end()) return CM_UNKNOWN;
  Request& r = it->second;
  int released = 0;
  for (size_t gi = 0; gi < m->groups.size(); ++gi) {
    Group& g = m->groups[gi];
    if (g.window <= 0) continue;
    const int64_t first_needed = computed_len - g.window + 1;
    if (first_needed <= 0) continue;
    int64_t dead_blocks = first_needed / g.page_size;  // blocks wholly below first_needed
    if (dead_blocks > (int64_t)r.tables[gi].size()) dead_blocks = (int64_t)r.tables[gi].size();
    for (int64_t b = r.first_live[gi]; b < dead_blocks; ++b) {
      const int32_t p = r.tables[gi][b];
      if (p >= 0) {
        g.in_use[p] = 0;
        g.free_list.push_back(p);
        r.tables[gi][b] = -1;
        ++released;
      }
    }
    if (dead_blocks > r.first_live[gi]) r.first_live[gi] = dead_blocks;
  }
  return released;
}

// Returns everything the request holds.  Freeing an unknown id is an error, so a double free is seen.
int cm_free(void* h, int64_t id) {
  Manager* m = static_cast<Manager*>(h);
  auto it = m->requests.find(id);
  if (it == m->requests.end()) return CM_UNKNOWN;
  Request& r = it->second;
  for (size_t gi = 0; gi < m->groups.size(); ++gi) {
    Group& g = m->groups[gi];
    // last page first, so that a following request receives them in ascending order of position
    for (auto p = r.tables[gi].rbegin(); p != r.tables[gi].rend(); ++p) {
      if (*p < 0) continue;
      g.in_use[*p] = 0;
      g.free_list.push_back(*p);
    }
  }
  m->slot_in_use[r.state_slot] = 0;
  m->free_slots.push_back(r.state_slot);
  m->requests.erase(it);
  return CM_OK;
}

int cm_num_groups(void* h) { return (int)static_cast<Manager*>(h)->groups.size(); }
int cm_num_free_pages(void* h, int group) { return (int)static_cast<Manager*>(h)->groups[group].free_list.size(); }
int cm_num_pages(void* h, int group) { return static_cast<Manager*>(h)->groups[group].num_pages; }
int cm_num_free_slots(void* h) { return (int)static_cast<Manager*>(h)->free_slots.size(); }
int cm_num_requests(void* h) { return (int)static_cast<Manager*>(h)->requests.size(); }

int cm_state_slot(void* h, int64_t id) {
  Manager* m = static_cast<Manager*>(h);
  auto it = m->requests.find(id);
  return it == m->requests.end() ? CM_UNKNOWN : it->second.state_slot;
}

int64_t cm_reserved_len(void* h, int64_t id) {
  Manager* m = static_cast<Manager*>(h);
  auto it = m->requests.find(id);
  return it == m->requests.end() ? CM_UNKNOWN : it->second.reserved_len;
}

// Copies the block table of (id, group) into out (at most cap entries); returns its length.
int cm_table(void* h, int64_t id, int group, int32_t* out, int cap) {
  Manager* m = static_cast<Manager*>(h);
  auto it = m->requests.find(id);
  if (it == m->requests.end()) return CM_UNKNOWN;
  if (group < 0 || group >= (int)m->groups.size()) return CM_BAD_ARG;
  const auto& t = it->second.tables[group];
  const int n = (int)t.size();
  if (out && cap > 0) std::memcpy(out, t.data(), sizeof(int32_t) * (size_t)(n < cap ? n : cap));
  return n;
}

// Step metadata of one group for n entries: entry e brings counts[e] tokens of request ids[e] at positions
// starts[e] ...  Writes, per token, the cache slot page * page_size + offset into slot_mapping (tokens of all
// entries in order) and, per entry, the block table padded with zeros into block_tables[e * max_blocks ...].
// Fails if a token has no live page.
int cm_fill_step(void* h, int group, int n, const int64_t* ids, const int32_t* starts, const int32_t* counts,
                 int32_t* slot_mapping, int32_t* block_tables, int max_blocks) {
  Manager* m = static_cast<Manager*>(h);
  if (group < 0 || group >= (int)m->groups.size()) return CM_BAD_ARG;
  const Group& g = m->groups[group];
  int64_t tok = 0;
  for (int e = 0; e < n; ++e) {
    auto it = m->requests.find(ids[e]);
    if (it == m->requests.end()) return CM_UNKNOWN;
    const auto& t = it->second.tables[group];
    if ((int64_t)t.size() > max_blocks) return CM_BAD_ARG;
    int32_t* row = block_tables + (size_t)e * max_blocks;
    for (int b = 0; b < max_blocks; ++b) row[b] = b < (int)t.size() && t[b] >= 0 ? t[b] : 0;
    for (int i = 0; i < counts[e]; ++i) {
      const int64_t pos = (int64_t)starts[e] + i;
      const int64_t b = pos / g.page_size;
      if (b >= (int64_t)t.size() || t[b] < 0) return CM_NO_PAGES;
      slot_mapping[tok++] = (int32_t)((int64_t)t[b] * g.page_size + pos % g.page_size);
    }
  }
  return CM_OK;
}

// One step's reservations in one call: every entry's request is made to cover its tokens.  Returns CM_OK, or the
// code of the first reservation that failed, with that entry's index in *failed (earlier entries keep what they
// got, as after a loop of cm_reserve calls).
int cm_reserve_all(void* h, int n, const int64_t* ids, const int32_t* starts, const int32_t* counts, int* failed) {
  for (int e = 0; e < n; ++e) {
    const int rc = cm_reserve(h, ids[e], (int64_t)starts[e] + counts[e]);
    if (rc != CM_OK) {
      if (failed) *failed = e;
      return rc;
    }
  }
  return CM_OK;
}

// After a step: pages that a window has passed go back, for every entry; done[e] is what request ids[e] now holds.
int cm_release_behind_all(void* h, int n, const int64_t* ids, const int32_t* done) {
  for (int e = 0; e < n; ++e) {
    const int rc = cm_release_behind(h, ids[e], done[e]);
    if (rc < 0) return rc;
  }
  return CM_OK;
}

// The metadata of a step, written into one staging buffer of int32 (the layout is the caller's: off[] gives where
// each array starts).  Entry e brings counts[e] tokens of request ids[e] at positions starts[e] ...; tokens holds
// them one entry after the other; feeds[e] >= 0 names the row of a device array that supplies the entry's one token
// instead; wants holds, per entry, want_counts[e] places among its tokens.  Written: token ids, positions and
// entry index per token; first row per entry (n + 1 values); length after the step and state slot per entry; the
// batch rows of the wanted places; per group, cache slot per token and padded block table per entry; and
// (row, feed) pairs.  Returns the number of such pairs, or a negative code.
//   off: tokens, positions, token->entry, first rows, lengths, state slots, wanted rows, slot mappings (groups one
//   after the other, a step's tokens each), block tables (groups one after the other, n * max_blocks each), pairs
int cm_pack_step(void* h, int n, const int64_t* ids, const int32_t* starts, const int32_t* counts,
                 const int32_t* tokens, const int32_t* feeds, const int32_t* want_counts, const int32_t* wants,
                 int32_t* buf, const int64_t* off, int max_blocks) {
  Manager* m = static_cast<Manager*>(h);
  if (n <= 0 || max_blocks <= 0) return CM_BAD_ARG;
  int32_t* o_tok = buf + off[0];
  int32_t* o_pos = buf + off[1];
  int32_t* o_seq = buf + off[2];
  int32_t* o_qs = buf + off[3];
  int32_t* o_len = buf + off[4];
  int32_t* o_slot = buf + off[5];
  int32_t* o_want = buf + off[6];
  int32_t* o_feed = buf + off[9];
  int64_t row = 0, wi = 0;
  int n_feed = 0;
  for (int e = 0; e < n; ++e) {
    auto it = m->requests.find(ids[e]);
    if (it == m->requests.end()) return CM_UNKNOWN;
    const int32_t c = counts[e];
    if (c <= 0) return CM_BAD_ARG;
    if (feeds[e] >= 0) {
      if (c != 1) return CM_BAD_ARG;
      o_feed[2 * n_feed] = (int32_t)row;
      o_feed[2 * n_feed + 1] = feeds[e];
      ++n_feed;
    }
    for (int32_t i = 0; i < c; ++i) {
      o_tok[row + i] = tokens[row + i];
      o_pos[row + i] = starts[e] + i;
      o_seq[row + i] = e;
    }
    for (int32_t w = 0; w < want_counts[e]; ++w) {
      const int32_t place = wants[wi + w];
      if (place < 0 || place >= c) return CM_BAD_ARG;
      o_want[wi + w] = (int32_t)row + place;
    }
    wi += want_counts[e];
    o_qs[e] = (int32_t)row;
    o_len[e] = starts[e] + c;
    o_slot[e] = it->second.state_slot;
    row += c;
  }
  o_qs[n] = (int32_t)row;
  const int64_t t = row;
  for (int g = 0; g < (int)m->groups.size(); ++g) {
    const int rc = cm_fill_step(h, g, n, ids, starts, counts, buf + off[7] + (int64_t)g * t,
                                buf + off[8] + (int64_t)g * n * max_blocks, max_blocks);
    if (rc != CM_OK) return rc;
  }
  return n_feed;
}

// Consistency: every page is either free or held by exactly one table entry, and likewise every state slot.
int cm_check(void* h) {
  Manager* m = static_cast<Manager*>(h);
  for (size_t gi = 0; gi < m->groups.size(); ++gi) {
    const Group& g = m->groups[gi];
    std::vector<int> seen(g.num_pages, 0);
    for (int32_t p : g.free_list) {
      if (p < 0 || p >= g.num_pages || g.in_use[p]) return CM_CORRUPT;
      if (++seen[p] > 1) return CM_CORRUPT;
    }
    for (const auto& kv : m->requests)
      for (int32_t p : kv.second.tables[gi]) {
        if (p < 0) continue;
        if (p >= g.num_pages || !g.in_use[p]) return CM_CORRUPT;
        if (++seen[p] > 1) return CM_CORRUPT;
      }
    for (int p = 0; p < g.num_pages; ++p)
      if (seen[p] != 1) return CM_CORRUPT;
  }
  std::vector<int> seen(m->slot_in_use.size(), 0);
  for (int32_t s : m->free_slots) {
    if (s < 0 || s >= (int)seen.size() || m->slot_in_use[s] || ++seen[s] > 1) return CM_CORRUPT;
  }
  for (const auto& kv : m->requests) {
    const int s = kv.second.state_slot;
    if (s < 0 || s >= (int)seen.size() || !m->slot_in_use[s] || ++seen[s] > 1) return CM_CORRUPT;
  }
  for (int v : seen)
    if (v != 1) return CM_CORRUPT;
  return CM_OK;
}

}  // extern "C"
