// The decisions of continuous batching with chunked prefill: which requests run how many tokens in the next step.
//
// One plan is made under a token budget and a request budget, as the reference's chunked policy does
// (backends/vllm/src/scheduler.rs:1257-1379, budget :40-149):
//   1. running requests that decode, in order of arrival (policy.rs:56-61);
//   2. running requests still in their prompt: the next portion, as large as the budget left allows
//      (scheduler.rs:1588-1623);
//   3. waiting requests, first come first served, while budget, pages and state slots last; the head of the queue
//      blocks those behind it (scheduler.rs:897-1016).
// Pages are reserved for what a step adds.  When they run out for a running request, the running request that
// arrived last is preempted by recomputation (scheduler.rs:650-690, 1778-1896): what it holds goes back and it
// returns to the front of the waiting queue.  A request that runs alone tries shorter portions, and is finished
// ("capped") when not even one token finds a page.  A waiting request longer than the model length, or than the whole
// pool, is dropped ("ignored").  With a window of keys (pages come back as a request moves on) portions are
// shortened before anything is preempted, the first portion of a request that finds the pool idle is shortened until
// it fits, and a request is admitted only if the window of every request already there still finds its pages.
//
// The scheduler keeps four counters per request (tokens held, tokens computed, tokens sampled, frozen); whoever
// runs the steps reports them before each plan.  It calls the cache manager of the same library directly and lists
// what it registered and released there, so that the caller's own books can follow.
//
// Plain C interface; not thread-safe: one engine thread owns a scheduler.
#include <algorithm>
#include <cstdint>
#include <deque>
#include <unordered_map>
#include <vector>

#include "cache_manager.h"

namespace {

struct Req {
  int64_t uid = 0;
  double arrival = 0.0;
  int32_t length = 0;     // prompt + generated tokens, those still on their way included
  int32_t computed = 0;   // tokens whose keys and values are in the cache
  int32_t sampled = 0;    // tokens generated so far
  bool frozen = false;    // its last token is on its way: nothing more is planned for it
  bool running = false;
  int32_t uncomputed() const { return length - computed; }
  bool in_prefill() const { return uncomputed() > 1 || sampled == 0; }
};

struct Entry {
  int64_t uid;
  int32_t n, start;
  uint8_t sample;
};

struct Sched {
  void* cm = nullptr;
  int max_tokens = 0, max_seqs = 0, max_model_len = 0, chunked = 1, max_chunk = 0;
  bool windowed = false;  // some cache group keeps a window of keys only
  int chunk_align = 1;    // where a prompt may be cut
  double delay_factor = 0.0;
  std::deque<int64_t> waiting;
  std::vector<int64_t> running;
  std::unordered_map<int64_t, Req> reqs;
  double last_prompt_latency = 0.0, prev_time = 0.0;
  bool prev_prompt = false;
  int64_t num_preemptions = 0;
  // the last plan
  std::vector<Entry> entries;
  std::vector<int64_t> preempted, ignored, capped, admitted;

  int used_tokens() const {
    int s = 0;
    for (const Entry& e : entries) s += e.n;
    return s;
  }

  // A portion that does not end what the request holds ends at a multiple of chunk_align (a mixer that scans its
  // tokens in blocks asks for that); 0 if no such portion of at most n tokens exists.
  int aligned(const Req& r, int n) const {
    if (chunk_align <= 1 || n >= r.uncomputed()) return n;
    const int end = (r.computed + n) / chunk_align * chunk_align;
    return end > r.computed ? end - r.computed : 0;
  }

  int chunk(const Req& r, int budget) const {
    int n = std::min(r.uncomputed(), budget);
    if (max_chunk > 0 && r.uncomputed() > 1) n = std::min(n, max_chunk);
    if (!chunked && n < r.uncomputed()) return 0;  // prompts are not cut: wait for a step with room for all of it
    return aligned(r, n);
  }

  void release(int64_t uid) {
    if (cm_state_slot(cm, uid) >= 0) cm_free(cm, uid);
  }

  void drop_running(int64_t uid) { running.erase(std::remove(running.begin(), running.end(), uid), running.end()); }

  void preempt(Req& v) {
    drop_running(v.uid);
    release(v.uid);
    v.computed = 0;
    v.running = false;
    waiting.push_front(v.uid);
    ++num_preemptions;
    preempted.push_back(v.uid);
    // a victim already planned into this step gives its place back
    entries.erase(std::remove_if(entries.begin(), entries.end(), [&](const Entry& e) { return e.uid == v.uid; }),
                  entries.end());
  }

  // the reference's optional batching delay (scheduler.rs:2077-2097)
  bool passed_delay(double now) {
    if (prev_prompt) last_prompt_latency = now - prev_time;
    prev_time = now;
    prev_prompt = false;
    if (delay_factor > 0 && !waiting.empty()) {
      double earliest = reqs[waiting.front()].arrival;
      for (int64_t u : waiting) earliest = std::min(earliest, reqs[u].arrival);
      return (now - earliest) > delay_factor * last_prompt_latency || running.empty();
    }
    return true;
  }

  int plan(double now) {
    entries.clear();
    preempted.clear();
    ignored.clear();
    capped.clear();
    admitted.clear();
    std::stable_sort(running.begin(), running.end(),
                     [&](int64_t a, int64_t b) { return reqs[a].arrival < reqs[b].arrival; });

    // 1 and 2: running requests, decodes before portions of prompts
    std::vector<int64_t> order;
    for (int pass = 0; pass < 2; ++pass)
      for (int64_t u : running) {
        const Req& r = reqs[u];
        if (!r.frozen && r.in_prefill() == (pass == 1)) order.push_back(u);
      }
    size_t first = 0;
    bool all_single = (int)order.size() <= max_seqs && (int)order.size() <= max_tokens;
    for (size_t i = 0; all_single && i < order.size(); ++i) all_single = reqs[order[i]].uncomputed() == 1;
    if (all_single) {
      // the common step: everything running adds one token and fits both budgets; pages are taken request by
      // request, and the general path below takes over at the first that finds none
      for (; first < order.size(); ++first) {
        Req& r = reqs[order[first]];
        if (!cm_can_reserve(cm, r.uid, r.computed + 1)) break;
        if (cm_reserve(cm, r.uid, r.computed + 1) != 0) return -1;
        entries.push_back({r.uid, 1, r.computed, 1});
      }
    }
    for (size_t i = first; i < order.size(); ++i) {
      Req& r = reqs[order[i]];
      if (!r.running) continue;  // preempted while serving an earlier request
      if ((int)entries.size() >= max_seqs) break;
      const int n_whole = chunk(r, max_tokens - used_tokens());
      int n = n_whole;
      if (n <= 0) continue;
      while (!cm_can_reserve(cm, r.uid, r.computed + n)) {
        // the latest arrival that is not just waiting for its last token (that one frees its pages soon)
        Req* victim = &r;
        for (auto it = running.rbegin(); it != running.rend(); ++it)
          if (!reqs[*it].frozen) {
            victim = &reqs[*it];
            break;
          }
        const bool alone = victim == &r && running.size() == 1;
        // A shorter portion may still find its pages: when nothing else could give any back, and, with a window
        // of keys, always (pages come back as the request moves on, so a portion too long for what is free now
        // is no reason to throw away what another request has computed).
        const int shorter = n > 1 ? aligned(r, n / 2) : 0;
        if (shorter > 0 && chunked && (alone || windowed)) {
          n = shorter;
          continue;
        }
        if (alone) {
          // not even one token finds a page: the pool cannot hold this request
          drop_running(r.uid);
          release(r.uid);
          r.running = false;
          capped.push_back(r.uid);
          break;
        }
        preempt(*victim);
        if (victim == &r) break;
        n = n_whole;      // what came back may hold the whole portion
      }
      if (!r.running) continue;
      if (cm_reserve(cm, r.uid, r.computed + n) != 0) return -1;
      entries.push_back({r.uid, n, r.computed, (uint8_t)(r.computed + n == r.length)});
    }

    // 3: admissions, unless something was preempted in this step (its pages are meant for the running ones)
    if (preempted.empty() && passed_delay(now)) {
      while (!waiting.empty()) {
        Req& r = reqs[waiting.front()];
        if (r.length > max_model_len || !cm_fits_at_all(cm, r.length)) {
          waiting.pop_front();
          ignored.push_back(r.uid);
          continue;
        }
        if ((int)entries.size() >= max_seqs || (int)running.size() >= max_seqs) break;
        int n = chunk(r, max_tokens - used_tokens());
        if (n <= 0 || cm_num_free_slots(cm) == 0) break;
        // If nothing holds pages, waiting frees none: only a shorter first portion helps (a prompt longer than
        // the pool gets in through a window of keys); when one token finds no page the request can never run.
        const bool pool_is_idle = cm_num_requests(cm) == 0;
        while (n > 1 && chunked && pool_is_idle && !cm_can_admit(cm, r.length, n)) n = aligned(r, n / 2);
        if (n <= 0 || !cm_can_admit(cm, r.length, n)) {
          if (!pool_is_idle) break;  // later
          waiting.pop_front();
          ignored.push_back(r.uid);
          continue;
        }
        waiting.pop_front();
        if (cm_add_request(cm, r.uid) < 0) return -1;
        if (cm_reserve(cm, r.uid, n) != 0) return -1;
        r.running = true;
        running.push_back(r.uid);
        admitted.push_back(r.uid);
        entries.push_back({r.uid, n, 0, (uint8_t)(n == r.length)});
        prev_prompt = true;
      }
    }
    for (int64_t u : ignored) reqs.erase(u);
    for (int64_t u : capped) reqs.erase(u);
    return (int)entries.size();
  }
};

int copy_out(const std::vector<int64_t>& v, int64_t* out, int cap) {
  const int n = (int)v.size();
  for (int i = 0; i < n && i < cap; ++i) out[i] = v[i];
  return n;
}

}  // namespace

extern "C" {

void* sc_create(void* cache_manager, int max_tokens, int max_seqs, int max_model_len, int chunked, int max_chunk,
                double delay_factor, int chunk_align) {
  if (!cache_manager || max_tokens <= 0 || max_seqs <= 0 || max_model_len <= 0 || max_chunk < 0 || chunk_align <= 0)
    return nullptr;
  // a cut prompt needs room for one aligned portion, also in a step in which every other request decodes a token
  // (decoding requests are planned first: with less room a prompt would stand still for as long as they run)
  if (chunked && chunk_align > 1 &&
      (max_tokens < chunk_align + max_seqs - 1 || (max_chunk > 0 && max_chunk < chunk_align)))
    return nullptr;
  Sched* s = new Sched();
  s->cm = cache_manager;
  s->max_tokens = max_tokens;
  s->max_seqs = max_seqs;
  s->max_model_len = max_model_len;
  s->chunked = chunked;
  s->max_chunk = max_chunk;
  s->delay_factor = delay_factor;
  s->windowed = cm_has_window(cache_manager) != 0;
  s->chunk_align = chunk_align;
  return s;
}

void sc_destroy(void* h) { delete static_cast<Sched*>(h); }

// A new request joins the back of the waiting queue.  0, or -1 if the number is in use.
int sc_add(void* h, int64_t uid, double arrival, int32_t length) {
  Sched* s = static_cast<Sched*>(h);
  if (s->reqs.count(uid)) return -1;
  Req r;
  r.uid = uid;
  r.arrival = arrival;
  r.length = length;
  s->reqs.emplace(uid, r);
  s->waiting.push_back(uid);
  return 0;
}

// Takes a request out wherever it is (aborted, or it has its last token) and gives back what it holds.
// Returns 1 if pages and slot went back, 0 if it held none, -1 if the number is unknown.
int sc_remove(void* h, int64_t uid) {
  Sched* s = static_cast<Sched*>(h);
  auto it = s->reqs.find(uid);
  if (it == s->reqs.end()) return -1;
  if (it->second.running)
    s->drop_running(uid);
  else
    s->waiting.erase(std::remove(s->waiting.begin(), s->waiting.end(), uid), s->waiting.end());
  const int held = cm_state_slot(s->cm, uid) >= 0;
  if (held) cm_free(s->cm, uid);
  s->reqs.erase(it);
  return held;
}

// The counters of n requests as they stand now: rows of (number, length, computed, sampled, frozen).
// -1 if one of them is unknown.
int sc_sync(void* h, int n, const int64_t* rows) {
  Sched* s = static_cast<Sched*>(h);
  for (int i = 0; i < n; ++i, rows += 5) {
    auto it = s->reqs.find(rows[0]);
    if (it == s->reqs.end()) return -1;
    Req& r = it->second;
    r.length = (int32_t)rows[1];
    r.computed = (int32_t)rows[2];
    r.sampled = (int32_t)rows[3];
    r.frozen = rows[4] != 0;
  }
  return 0;
}

// Plans one step at time `now`; returns the number of entries, or -1 if the cache manager refused what it had
// just promised (its books and the scheduler's have come apart).
int sc_schedule(void* h, double now) { return static_cast<Sched*>(h)->plan(now); }

// The entries of the last plan as rows of (number, tokens, start, sample?); returns their number and copies at
// most cap rows.
int sc_entries(void* h, int64_t* rows, int cap) {
  Sched* s = static_cast<Sched*>(h);
  const int m = (int)s->entries.size();
  for (int i = 0; i < m && i < cap; ++i, rows += 4) {
    rows[0] = s->entries[i].uid;
    rows[1] = s->entries[i].n;
    rows[2] = s->entries[i].start;
    rows[3] = s->entries[i].sample;
  }
  return m;
}

// Lists of request numbers: 0 preempted, 1 ignored, 2 capped, 3 admitted (all of the last plan), 4 the waiting
// queue from its head, 5 the running requests.  Returns the list's length; copies at most cap of them.
int sc_list(void* h, int kind, int64_t* out, int cap) {
  Sched* s = static_cast<Sched*>(h);
  switch (kind) {
    case 0: return copy_out(s->preempted, out, cap);
    case 1: return copy_out(s->ignored, out, cap);
    case 2: return copy_out(s->capped, out, cap);
    case 3: return copy_out(s->admitted, out, cap);
    case 4: return copy_out(std::vector<int64_t>(s->waiting.begin(), s->waiting.end()), out, cap);
    case 5: return copy_out(s->running, out, cap);
  }
  return -1;
}

int sc_num_waiting(void* h) { return (int)static_cast<Sched*>(h)->waiting.size(); }
int sc_num_running(void* h) { return (int)static_cast<Sched*>(h)->running.size(); }
int64_t sc_num_preemptions(void* h) { return static_cast<Sched*>(h)->num_preemptions; }
double sc_last_prompt_latency(void* h) { return static_cast<Sched*>(h)->last_prompt_latency; }

}  // extern "C"
