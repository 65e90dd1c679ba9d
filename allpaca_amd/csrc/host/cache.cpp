// The cache manager's books: pools of page ids handed out from a stack (last freed, first reused), block tables per
// request and paged group, state slots.  No GPU is touched here; the device memory that the ids index lives with
// the caller (allpaca_amd/cache/storage.py).  allpaca_amd/cache/pages.py is the Python face of this file and says
// what each call means; requests are named by 64-bit ids that the face hands out.
// The reference takes a request's pages at admission and frees them when its handle drops
// (crates/allpaca-core/src/engine.rs:3341-3349, crates/allpaca-core/src/kv_tier.rs:341-532).
#include "cache.h"

#include <algorithm>
#include <string>

namespace apc_host {

int Pool::alloc() {
  if (free_.empty()) return APC_CACHE_OUT_OF_PAGES;
  const int p = free_.back();
  if (held[p]) return APC_CACHE_CORRUPT;
  free_.pop_back();
  held[p] = 1;
  ++allocations;
  return p;
}

int Pool::give_back(int page) {
  if (page < 0 || page >= n) return APC_CACHE_PAGE_OUTSIDE;
  if (!held[page]) return APC_CACHE_FREED_TWICE;
  held[page] = 0;
  free_.push_back(page);
  if (log_frees) freed.push_back(page);
  return 0;
}

Pool::Pool(int pages) : n(pages), held((size_t)pages, 0) {
  free_.reserve(pages);
  for (int p = pages - 1; p >= 0; --p) free_.push_back(p);  // page 0 goes out first
}

Cache::Cache(int page_tokens_, const std::vector<int>& windows_, const std::vector<int>& pages, int max_requests_)
    : page_tokens(page_tokens_), windows(windows_), slots(max_requests_), max_requests(max_requests_) {
  for (int n : pages) pools.emplace_back(n);
}

int Cache::first_needed(int group, int next_pos) const {
  const int w = windows[group];
  return w < 0 ? 0 : std::max(0, next_pos - w + 1);
}

Seq* Cache::find(long long id) {
  auto it = seqs.find(id);
  return it == seqs.end() ? nullptr : &it->second;
}

int Cache::admit(long long id) {
  if (seqs.count(id)) return APC_CACHE_ALREADY_LIVE;
  const int slot = slots.alloc();
  if (slot == APC_CACHE_OUT_OF_PAGES) return APC_CACHE_OUT_OF_SLOTS;
  if (slot < 0) return slot;
  Seq s;
  s.slot = slot;
  s.tables.resize(pools.size());
  s.version = ++versions;
  seqs.emplace(id, std::move(s));
  return slot;
}

void Cache::pages_needed(const Seq& s, int n_new, int* out) const {
  const int want = (s.length + n_new + page_tokens - 1) / page_tokens;
  for (size_t g = 0; g < pools.size(); ++g) out[g] = std::max(0, want - (int)s.tables[g].size());
}

int Cache::reserve(long long id, int n_new) {
  Seq* s = find(id);
  if (!s) return APC_CACHE_UNKNOWN;
  int need[APC_MAX_GROUPS];
  pages_needed(*s, n_new, need);
  for (size_t g = 0; g < pools.size(); ++g)
    if (need[g] > pools[g].free_count()) return APC_CACHE_OUT_OF_PAGES;
  for (size_t g = 0; g < pools.size(); ++g)
    for (int i = 0; i < need[g]; ++i) {
      const int p = pools[g].alloc();
      if (p < 0) return p;
      s->tables[g].push_back(p);
    }
  s->reserved = std::max(s->reserved, s->length + n_new);
  return 0;
}

int Cache::commit(long long id, int n_new) {
  Seq* s = find(id);
  if (!s) return APC_CACHE_UNKNOWN;
  if (s->length + n_new > s->reserved) return APC_CACHE_COMMIT_BEYOND;
  s->length += n_new;
  for (size_t g = 0; g < pools.size(); ++g) {
    auto& t = s->tables[g];
    const int passed = std::min(first_needed((int)g, s->length) / page_tokens, (int)t.size());
    for (int i = 0; i < passed; ++i)
      if (t[i] != APC_PAGE_FREED) {
        const int rc = pools[g].give_back(t[i]);
        if (rc) return rc;
        t[i] = APC_PAGE_FREED;
        s->version = ++versions;
      }
  }
  return 0;
}

int Cache::truncate(long long id, int length) {
  Seq* s = find(id);
  if (!s) return APC_CACHE_UNKNOWN;
  if (length > s->length) return APC_CACHE_TRUNCATE_BEYOND;
  const int keep = (length + page_tokens - 1) / page_tokens;
  for (size_t g = 0; g < pools.size(); ++g) {
    auto& t = s->tables[g];
    for (int i = first_needed((int)g, length) / page_tokens; i < std::min(keep, (int)t.size()); ++i)
      if (t[i] == APC_PAGE_FREED) return APC_CACHE_TRUNCATE_WINDOW;
  }
  for (size_t g = 0; g < pools.size(); ++g) {
    auto& t = s->tables[g];
    while ((int)t.size() > keep) {
      const int p = t.back();
      t.pop_back();
      s->version = ++versions;
      if (p != APC_PAGE_FREED) {
        const int rc = pools[g].give_back(p);
        if (rc) return rc;
      }
    }
  }
  s->length = length;
  s->reserved = std::min(s->reserved, keep * page_tokens);
  return 0;
}

int Cache::release(long long id) {
  auto it = seqs.find(id);
  if (it == seqs.end()) return APC_CACHE_UNKNOWN;
  Seq& s = it->second;
  int rc = 0;
  for (size_t g = 0; g < pools.size(); ++g)
    for (int p : s.tables[g])
      if (p != APC_PAGE_FREED) {
        const int e = pools[g].give_back(p);
        if (e && !rc) rc = e;
      }
  const int e = slots.give_back(s.slot);
  if (e && !rc) rc = e;
  seqs.erase(it);
  return rc;
}

// No page lost, none held twice, free + held = pool; slots and live requests agree.
int Cache::check(std::string& why) const {
  for (size_t g = 0; g < pools.size(); ++g) {
    std::vector<long long> owner((size_t)pools[g].n, -1);
    std::vector<char> seen((size_t)pools[g].n, 0);
    for (const auto& kv : seqs)
      for (int p : kv.second.tables[g]) {
        if (p == APC_PAGE_FREED) continue;
        if (p < 0 || p >= pools[g].n) {
          why = "group " + std::to_string(g) + ": a block table holds page " + std::to_string(p) + " outside the pool";
          return APC_CACHE_CHECK_FAILED;
        }
        if (seen[p]) {
          why = "group " + std::to_string(g) + ": page " + std::to_string(p) + " held by two requests";
          return APC_CACHE_CHECK_FAILED;
        }
        seen[p] = 1;
      }
    int held = 0;
    for (int p = 0; p < pools[g].n; ++p) {
      if ((pools[g].held[p] != 0) != (seen[p] != 0)) {
        why = "group " + std::to_string(g) + ": page " + std::to_string(p) +
              (pools[g].held[p] ? " is held by the pool but in no block table" : " is in a block table but not held");
        return APC_CACHE_CHECK_FAILED;
      }
      held += pools[g].held[p] ? 1 : 0;
    }
    if (held + pools[g].free_count() != pools[g].n) {
      why = "group " + std::to_string(g) + ": " + std::to_string(held) + " held + " +
            std::to_string(pools[g].free_count()) + " free != " + std::to_string(pools[g].n);
      return APC_CACHE_CHECK_FAILED;
    }
  }
  std::vector<char> slot_seen((size_t)slots.n, 0);
  for (const auto& kv : seqs) {
    const int sl = kv.second.slot;
    if (sl < 0 || sl >= slots.n || slot_seen[sl] || !slots.held[sl]) {
      why = "state slots and live requests disagree";
      return APC_CACHE_CHECK_FAILED;
    }
    slot_seen[sl] = 1;
  }
  for (int sl = 0; sl < slots.n; ++sl)
    if ((slots.held[sl] != 0) != (slot_seen[sl] != 0)) {
      why = "state slots and live requests disagree";
      return APC_CACHE_CHECK_FAILED;
    }
  return 0;
}

}  // namespace apc_host

using namespace apc_host;

// ==================================================================================================== interface
APC_HOST_EXPORT void* apc_pool_new(int pages) { return pages > 0 ? new Pool(pages) : nullptr; }
APC_HOST_EXPORT void apc_pool_free(void* pool) { delete (Pool*)pool; }
APC_HOST_EXPORT int apc_pool_alloc(void* pool) { return ((Pool*)pool)->alloc(); }
APC_HOST_EXPORT int apc_pool_give_back(void* pool, int page) { return ((Pool*)pool)->give_back(page); }
APC_HOST_EXPORT int apc_pool_free_count(void* pool) { return ((Pool*)pool)->free_count(); }
APC_HOST_EXPORT int apc_pool_pages(void* pool) { return ((Pool*)pool)->n; }
APC_HOST_EXPORT long long apc_pool_allocations(void* pool) { return ((Pool*)pool)->allocations; }
APC_HOST_EXPORT int apc_pool_held(void* pool, int* out, int cap) {  // the held page ids, ascending; returns their number
  Pool& p = *(Pool*)pool;
  int k = 0;
  for (int i = 0; i < p.n; ++i)
    if (p.held[i]) {
      if (k < cap) out[k] = i;
      ++k;
    }
  return k;
}
// With the log on, every page that comes back is noted; `apc_pool_drain` hands the notes out and forgets them.
APC_HOST_EXPORT void apc_pool_log_frees(void* pool, int on) {
  Pool& p = *(Pool*)pool;
  p.log_frees = on != 0;
  if (!on) p.freed.clear();
}
APC_HOST_EXPORT int apc_pool_drain(void* pool, int* out, int cap) {
  Pool& p = *(Pool*)pool;
  const int k = (int)std::min((size_t)cap, p.freed.size());
  std::copy(p.freed.begin(), p.freed.begin() + k, out);
  p.freed.erase(p.freed.begin(), p.freed.begin() + k);
  return k;
}

APC_HOST_EXPORT void* apc_cache_new(int page_tokens, int n_groups, const int* windows, const int* pages,
                                    int max_requests) {
  if (page_tokens <= 0 || n_groups < 0 || n_groups > APC_MAX_GROUPS || max_requests <= 0) return nullptr;
  for (int g = 0; g < n_groups; ++g)
    if (pages[g] <= 0) return nullptr;
  return new Cache(page_tokens, std::vector<int>(windows, windows + n_groups), std::vector<int>(pages, pages + n_groups),
                   max_requests);
}
APC_HOST_EXPORT void apc_cache_free(void* c) { delete (Cache*)c; }
APC_HOST_EXPORT void* apc_cache_pool(void* c, int group) {  // group -1: the state slots
  Cache& C = *(Cache*)c;
  if (group < 0) return &C.slots;
  return group < (int)C.pools.size() ? &C.pools[group] : nullptr;
}
APC_HOST_EXPORT int apc_cache_admit(void* c, long long id) { return ((Cache*)c)->admit(id); }
APC_HOST_EXPORT int apc_cache_release(void* c, long long id) { return ((Cache*)c)->release(id); }
APC_HOST_EXPORT int apc_cache_reserve(void* c, long long id, int n_new) { return ((Cache*)c)->reserve(id, n_new); }
APC_HOST_EXPORT int apc_cache_commit(void* c, long long id, int n_new) { return ((Cache*)c)->commit(id, n_new); }
APC_HOST_EXPORT int apc_cache_truncate(void* c, long long id, int length) { return ((Cache*)c)->truncate(id, length); }
APC_HOST_EXPORT int apc_cache_length(void* c, long long id) {
  const Seq* s = ((Cache*)c)->find(id);
  return s ? s->length : APC_CACHE_UNKNOWN;
}
APC_HOST_EXPORT int apc_cache_slot(void* c, long long id) {
  const Seq* s = ((Cache*)c)->find(id);
  return s ? s->slot : APC_CACHE_UNKNOWN;
}
APC_HOST_EXPORT long long apc_cache_version(void* c, long long id) {
  const Seq* s = ((Cache*)c)->find(id);
  return s ? s->version : APC_CACHE_UNKNOWN;
}
APC_HOST_EXPORT int apc_cache_pages_needed(void* c, long long id, int n_new, int* out) {
  Cache& C = *(Cache*)c;
  const Seq* s = C.find(id);
  if (!s) return APC_CACHE_UNKNOWN;
  C.pages_needed(*s, n_new, out);
  return 0;
}
// The request's block table in `group` (APC_PAGE_FREED where a window has passed); returns its length.
APC_HOST_EXPORT int apc_cache_table(void* c, long long id, int group, int* out, int cap) {
  Cache& C = *(Cache*)c;
  const Seq* s = C.find(id);
  if (!s || group < 0 || group >= (int)C.pools.size()) return APC_CACHE_UNKNOWN;
  const auto& t = s->tables[group];
  std::copy(t.begin(), t.begin() + std::min((size_t)cap, t.size()), out);
  return (int)t.size();
}
APC_HOST_EXPORT int apc_cache_check(void* c) {
  Cache& C = *(Cache*)c;
  return C.check(C.why);
}
APC_HOST_EXPORT const char* apc_cache_why(void* c) { return ((Cache*)c)->why.c_str(); }
