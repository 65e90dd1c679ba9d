// Continuous batching: which requests run in the next step, and how many of their tokens.  Bookkeeping over the
// cache manager's books (cache.cpp); no GPU.  allpaca_amd/engine/scheduler.py is the Python face of this file, keeps
// the requests' tokens and says what the rules are; here a request is its counts.
//
// Every step, under a budget of tokens: (1) every running request that is decoding gets its one token, oldest
// admission first; if a page is missing, the most recently admitted running request that is not yet part of the step
// gives way (its pages go back, it returns to the front of the queue and is computed again from its prompt and the
// tokens it has generated); (2) running requests still in their prompt get a portion, oldest first, cut to what the
// budget and the free pages allow; (3) waiting requests are admitted in arrival order while fewer than
// `max_active` run and pages for a first portion are free; (4) a step whose rows overshoot a multiple of `row_tile`
// by up to a quarter tile has its last prompt portion cut back to the multiple.  If nobody can advance, the most
// recently admitted gives way until someone can.
// The reference advances one request per tick (crates/allpaca-core/src/scheduler.rs:607-664) by its chunk size
// (crates/allpaca-core/src/engine.rs:4717-4756) and takes a request's pages up front (engine.rs:3341-3349).
#include "cache.h"

#include <algorithm>
#include <deque>

using namespace apc_host;

#define APC_SCHED_TOO_LARGE (-40)     // a request cannot get a page although it runs alone
#define APC_SCHED_UNKNOWN (-41)
#define APC_SCHED_ROOM (-42)          // the caller's arrays are too short for the plan

namespace {

enum { WAITING = 0, RUNNING = 1, FINISHED = 2 };

struct Req {
  long long id;                       // its name in the cache manager's books
  int prompt = 0, out = 0, max_tokens = 0, computed = 0, status = WAITING, order = 0, preemptions = 0;
  int n_tokens() const { return prompt + out; }
  int left() const { return n_tokens() - computed; }
  bool decoding() const { return left() == 1 && out > 0; }
};

struct Item {
  long long id;
  int start, count, samples;
};

struct Sched {
  Cache* C;
  int max_active, budget, chunk, row_tile;
  std::unordered_map<long long, Req> reqs;
  std::deque<long long> waiting;
  std::vector<long long> running;
  int admissions = 0, preemption_count = 0;
  // the plan in work
  std::vector<Item> scheduled;
  std::vector<long long> preempted, admitted;

  Req& req(long long id) { return reqs.at(id); }

  bool fits(const Req& r, int n, const int* promised) {
    int need[APC_MAX_GROUPS];
    C->pages_needed(*C->find(r.id), n, need);
    for (size_t g = 0; g < C->pools.size(); ++g)
      if (need[g] + promised[g] > C->pools[g].free_count()) return false;
    return true;
  }
  void promise(const Req& r, int n, int* promised) {
    int need[APC_MAX_GROUPS];
    C->pages_needed(*C->find(r.id), n, need);
    for (size_t g = 0; g < C->pools.size(); ++g) promised[g] += need[g];
  }
  // the largest portion below n that the free pages allow (0 if none)
  int shrink(const Req& r, int n, const int* promised) {
    const Seq& s = *C->find(r.id);
    int room = 0, have = 0;
    if (!C->pools.empty()) {
      room = C->pools[0].free_count() - promised[0];
      have = (int)s.tables[0].size();
      for (size_t g = 1; g < C->pools.size(); ++g) {
        room = std::min(room, C->pools[g].free_count() - promised[g]);
        have = std::min(have, (int)s.tables[g].size());
      }
    }
    const int can = (have + std::max(room, 0)) * C->page_tokens - s.length;
    return std::max(0, std::min(n - 1, can));
  }
  void preempt(long long id) {
    Req& v = req(id);
    C->release(id);
    running.erase(std::find(running.begin(), running.end(), id));
    v.status = WAITING;
    v.computed = 0;
    ++v.preemptions;
    ++preemption_count;
    waiting.push_front(id);
    preempted.push_back(id);
  }
  bool is_scheduled(long long id) const {
    for (const Item& s : scheduled)
      if (s.id == id) return true;
    return false;
  }
  std::vector<long long> by_order(bool want_decoding) {
    std::vector<long long> out;
    for (long long id : running)
      if (req(id).decoding() == want_decoding) out.push_back(id);
    std::sort(out.begin(), out.end(), [&](long long a, long long b) { return req(a).order < req(b).order; });
    return out;
  }
  long long newest(const std::vector<long long>& among) {
    long long best = among[0];
    for (long long id : among)
      if (req(id).order > req(best).order) best = id;
    return best;
  }

  int plan_once() {
    scheduled.clear();
    int left_budget = budget;
    int promised[APC_MAX_GROUPS] = {0};
    // 1. decodes, oldest admission first
    for (long long id : by_order(true)) {
      Req& r = req(id);
      if (r.status != RUNNING || left_budget <= 0) continue;
      while (r.status == RUNNING && !fits(r, 1, promised)) {
        std::vector<long long> victims;
        for (long long v : running)
          if (!is_scheduled(v)) victims.push_back(v);
        if (victims.size() == 1 && victims[0] == id && running.size() == 1) return APC_SCHED_TOO_LARGE;
        preempt(newest(victims));
      }
      if (r.status != RUNNING) continue;
      promise(r, 1, promised);
      scheduled.push_back({id, r.computed, 1, 1});
      --left_budget;
    }
    // 2. portions of prompts that are under way
    for (long long id : by_order(false)) {
      if (left_budget <= 0) break;
      Req& r = req(id);
      if (r.status != RUNNING) continue;
      int n = std::min({r.left(), chunk, left_budget});
      while (n > 0 && !fits(r, n, promised)) n = shrink(r, n, promised);
      if (n <= 0) continue;
      promise(r, n, promised);
      scheduled.push_back({id, r.computed, n, n == r.left() ? 1 : 0});
      left_budget -= n;
    }
    // 3. admissions, in arrival order; the first that does not fit blocks the ones behind it
    while (!waiting.empty() && left_budget > 0 && (int)running.size() < max_active) {
      const long long id = waiting.front();
      if (std::find(preempted.begin(), preempted.end(), id) != preempted.end()) break;
      if (C->slots.free_count() <= 0) break;
      Req& r = req(id);
      if (C->admit(id) < 0) break;
      int n = std::min({r.left(), chunk, left_budget});
      while (n > 0 && !fits(r, n, promised)) n = shrink(r, n, promised);
      if (n <= 0) {
        C->release(id);
        break;
      }
      waiting.pop_front();
      r.status = RUNNING;
      r.order = ++admissions;
      running.push_back(id);
      admitted.push_back(id);
      promise(r, n, promised);
      scheduled.push_back({id, r.computed, n, n == r.left() ? 1 : 0});
      left_budget -= n;
    }
    trim_to_tiles();
    return 0;
  }

  void trim_to_tiles() {
    if (!row_tile) return;
    int total = 0;
    for (const Item& s : scheduled) total += s.count;
    const int over = total % row_tile;
    if (total < 2 * row_tile || !(over > 0 && over <= row_tile / 4)) return;
    for (auto it = scheduled.rbegin(); it != scheduled.rend(); ++it)
      if (!req(it->id).decoding() && 2 * (it->count - over) >= it->count) {
        it->count -= over;
        it->samples = 0;
        return;
      }
  }

  int plan() {
    preempted.clear();
    admitted.clear();
    int rc = plan_once();
    while (!rc && scheduled.empty() && running.size() > 1) {
      preempt(newest(running));
      rc = plan_once();
    }
    return rc;
  }
};

}  // namespace

// ==================================================================================================== interface
APC_HOST_EXPORT void* apc_sched_new(void* cache, int max_active, int budget, int chunk, int row_tile) {
  if (!cache || max_active <= 0 || budget <= 0 || chunk <= 0 || row_tile < 0) return nullptr;
  Sched* s = new Sched();
  s->C = (Cache*)cache;
  s->max_active = max_active;
  s->budget = budget;
  s->chunk = chunk;
  s->row_tile = row_tile;
  return s;
}
APC_HOST_EXPORT void apc_sched_free(void* s) { delete (Sched*)s; }

// Pages the request may come to hold at worst, per group, against the pools: 0 if it can fit, else the pages of the
// first group it is too large for (`group` says which).
APC_HOST_EXPORT int apc_sched_too_large(void* sp, int prompt, int max_tokens, int* group) {
  Sched& S = *(Sched*)sp;
  const Cache& C = *S.C;
  const int P = C.page_tokens;
  const int need = (prompt + max_tokens + P - 1) / P;
  for (size_t g = 0; g < C.pools.size(); ++g) {
    int worst = need;
    if (C.windows[g] >= 0) worst = std::min(need, (C.windows[g] + P - 1) / P + 1 + (S.chunk + P - 1) / P);
    if (worst > C.pools[g].n) {
      if (group) *group = (int)g;
      return worst;
    }
  }
  return 0;
}

APC_HOST_EXPORT int apc_sched_add(void* sp, long long id, int prompt, int out, int max_tokens) {
  Sched& S = *(Sched*)sp;
  if (prompt <= 0 || S.reqs.count(id)) return -1;
  Req r;
  r.id = id;
  r.prompt = prompt;
  r.out = out;
  r.max_tokens = max_tokens;
  S.reqs.emplace(id, r);
  S.waiting.push_back(id);
  return 0;
}

// One step's plan.  scheduled: (id, start, count, samples) per entry into `items` (4 long longs each); the requests
// that gave way and those admitted, in the order it happened, into `preempted` and `admitted` (with the order number
// of each admission in `orders`); the counts into n[0..2].
APC_HOST_EXPORT int apc_sched_plan(void* sp, long long* items, int cap_items, long long* preempted, long long* admitted,
                                   int* orders, int cap_ids, int* n) {
  Sched& S = *(Sched*)sp;
  const int rc = S.plan();
  if (rc) return rc;
  n[0] = (int)S.scheduled.size();
  n[1] = (int)S.preempted.size();
  n[2] = (int)S.admitted.size();
  if (n[0] > cap_items || n[1] > cap_ids || n[2] > cap_ids) return APC_SCHED_ROOM;
  for (int i = 0; i < n[0]; ++i) {
    items[4 * i] = S.scheduled[i].id;
    items[4 * i + 1] = S.scheduled[i].start;
    items[4 * i + 2] = S.scheduled[i].count;
    items[4 * i + 3] = S.scheduled[i].samples;
  }
  std::copy(S.preempted.begin(), S.preempted.end(), preempted);
  for (int i = 0; i < n[2]; ++i) {
    admitted[i] = S.admitted[i];
    orders[i] = S.req(S.admitted[i]).order;
  }
  return 0;
}

APC_HOST_EXPORT int apc_sched_advance(void* sp, long long id, int count) {
  Sched& S = *(Sched*)sp;
  auto it = S.reqs.find(id);
  if (it == S.reqs.end()) return APC_SCHED_UNKNOWN;
  it->second.computed += count;
  return 0;
}
APC_HOST_EXPORT int apc_sched_token(void* sp, long long id) {  // a sampled token was appended
  Sched& S = *(Sched*)sp;
  auto it = S.reqs.find(id);
  if (it == S.reqs.end()) return APC_SCHED_UNKNOWN;
  return ++it->second.out;
}
// The request ends: out of the queues, its pages and slot go back, its record is dropped.
APC_HOST_EXPORT int apc_sched_finish(void* sp, long long id) {
  Sched& S = *(Sched*)sp;
  auto it = S.reqs.find(id);
  if (it == S.reqs.end()) return APC_SCHED_UNKNOWN;
  auto w = std::find(S.waiting.begin(), S.waiting.end(), id);
  if (w != S.waiting.end()) S.waiting.erase(w);
  auto r = std::find(S.running.begin(), S.running.end(), id);
  if (r != S.running.end()) S.running.erase(r);
  if (S.C->find(id)) S.C->release(id);
  S.reqs.erase(it);
  return 0;
}
APC_HOST_EXPORT int apc_sched_counts(void* sp, int* out) {  // waiting, running, preemptions so far
  Sched& S = *(Sched*)sp;
  out[0] = (int)S.waiting.size();
  out[1] = (int)S.running.size();
  out[2] = S.preemption_count;
  return 0;
}
