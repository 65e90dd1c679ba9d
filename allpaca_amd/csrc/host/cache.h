// The cache manager's books (cache.cpp), as the step packer and the scheduler see them.
#pragma once
#include "host.h"

#include <string>
#include <unordered_map>
#include <vector>

#define APC_MAX_GROUPS 8
#define APC_PAGE_FREED (-1)           // block-table entry of a page that a window has passed

#define APC_CACHE_ALREADY_LIVE (-20)
#define APC_CACHE_OUT_OF_SLOTS (-21)
#define APC_CACHE_OUT_OF_PAGES (-22)
#define APC_CACHE_COMMIT_BEYOND (-23)
#define APC_CACHE_TRUNCATE_BEYOND (-24)
#define APC_CACHE_TRUNCATE_WINDOW (-25)
#define APC_CACHE_UNKNOWN (-26)
#define APC_CACHE_PAGE_OUTSIDE (-27)
#define APC_CACHE_FREED_TWICE (-28)
#define APC_CACHE_CORRUPT (-29)       // a page was on the free list while held
#define APC_CACHE_CHECK_FAILED (-30)

namespace apc_host {

struct Pool {
  int n;
  std::vector<int> free_;
  std::vector<char> held;
  long long allocations = 0;  // how many times a page was handed out (reuse shows as allocations > n)
  bool log_frees = false;
  std::vector<int> freed;
  explicit Pool(int pages);
  int free_count() const { return (int)free_.size(); }
  int alloc();                // a page id, or an error code (< 0)
  int give_back(int page);
};

struct Seq {
  int slot = 0;
  int length = 0;             // positions committed
  int reserved = 0;           // positions that pages exist for
  std::vector<std::vector<int>> tables;  // per paged group
  long long version = 0;      // changes whenever an entry of a table was taken away or replaced
};

struct Cache {
  int page_tokens;
  std::vector<int> windows;   // per paged group: -1 none
  std::vector<Pool> pools;
  Pool slots;
  int max_requests;
  std::unordered_map<long long, Seq> seqs;
  long long versions = 0;
  std::string why;
  Cache(int page_tokens, const std::vector<int>& windows, const std::vector<int>& pages, int max_requests);
  int first_needed(int group, int next_pos) const;
  Seq* find(long long id);
  int admit(long long id);    // the slot, or an error code
  void pages_needed(const Seq& s, int n_new, int* out) const;
  int reserve(long long id, int n_new);
  int commit(long long id, int n_new);
  int truncate(long long id, int length);
  int release(long long id);
  int check(std::string& why) const;
};

}  // namespace apc_host
