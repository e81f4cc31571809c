// Paged cache bookkeeping: which physical pages hold which positions of which
// request, in every group of layers; fixed-size state slots; prefix-page reuse.
//
// It owns numbers only.  The tensors that the pages and slots index belong to
// the engine.
//
// Groups.  Layers with the same need share a group: a group keeps all keys of a
// request (window == 0) or only the last `window` of them.  Each group has its
// own pool of pages and its own block table per request; all groups use one
// page size.  Position i of a request lives in logical page i / page_size of
// each group, at slot  page * page_size + i % page_size.
//
// Life of a request:
//   add_request   takes a state slot; with a prompt and the prefix cache on, it
//                 attaches the longest chain of published pages that match
//   reserve       (optional) takes pages in all-keys groups up to a token count
//   extend        takes pages, in every group, for the next n tokens
//   commit        the n tokens were computed: pages that became full are
//                 published for reuse; pages a window has passed are given back
//   finish        gives everything back
//
// The behaviours follow the reference's cache scheduler
// (src/exec/cache_scheduler): page arithmetic admission.rs:1166-1174; the free
// queue hands out its head and takes released pages at its head
// (availability_queue.rs:746-780, reclamation.rs:1185); the prefix hash chain
// mod.rs:939-958; matching leaves at least one prompt token uncached
// (prefix_cache.rs:3187); published pages whose last holder left stay resident,
// children before parents, and are evicted from the head under pressure
// (reclamation.rs:534-992, eviction_policy.rs:34-65); the first writer of a
// hash wins (prefix_cache.rs:264-272).
#pragma once
#include <cstdint>
#include <deque>
#include <list>
#include <string>
#include <unordered_map>
#include <vector>

namespace vosti {

using RequestId = uint64_t;

enum Status : int {
  OK = 0,
  NO_PAGES = 1,
  NO_SLOT = 2,
  UNKNOWN_REQUEST = 3,
  DUPLICATE_REQUEST = 4,
  BAD_ARGUMENT = 5,
  STEP_PENDING = 6,
};

struct GroupSpec {
  int window;     // 0: the group keeps every key
  int num_pages;
};

class CacheManager {
 public:
  CacheManager(int page_size, std::vector<GroupSpec> groups, int num_slots, bool prefix_cache);

  Status add_request(RequestId id, const int32_t* prompt, int n_prompt, int* cached_tokens);
  Status reserve(RequestId id, int total_tokens);
  Status extend(RequestId id, const int32_t* tokens, int n);
  Status commit(RequestId id);
  Status abort_step(RequestId id);
  Status finish(RequestId id);

  bool has_request(RequestId id) const { return requests_.count(id) != 0; }
  int page_size() const { return page_size_; }
  int num_groups() const { return (int)groups_.size(); }
  int window(int group) const { return groups_[group].window; }
  int length(RequestId id) const;        // tokens committed
  int pending(RequestId id) const;       // tokens of the step in flight
  int state_slot(RequestId id) const;
  int num_logical_pages(RequestId id, int group) const;   // block-table width this request needs
  // Pages this request could take right now: free ones plus evictable cached ones.
  int available_pages(int group) const;
  int free_pages(int group) const { return (int)groups_[group].free.size(); }
  int pages_needed(RequestId id, int group, int n_more) const;   // fresh pages extend(n_more) would take
  int free_slots() const { return (int)free_slots_.size(); }
  int num_requests() const { return (int)requests_.size(); }

  // Block table row (released or absent pages read as page 0) and slots of
  // positions [start, start + n).
  Status fill_block_table(RequestId id, int group, int32_t* out, int width) const;
  Status fill_slots(RequestId id, int group, int start, int n, int32_t* out) const;

  // Counters for tests and logs.  An admission that is taken back before any
  // step was planned for the request (no pages for the rest of its prompt)
  // leaves them as they were.
  int64_t prefix_hits() const { return prefix_hit_pages_; }
  int64_t prefix_hit_requests() const { return prefix_hit_requests_; }   // admissions that found a cached prefix
  int64_t evictions() const { return evictions_; }
  int cached_blocks() const { return (int)lru_.size(); }
  // Gives every cached page (published, held by no request) back to the free queues; returns how many
  // there were.  A caller that wants the next requests to find nothing to reuse calls it between them
  // (the reference's reclaim_cached_leaves_until(capacity), examples/support/engine_calls.rs:72-82).
  int drop_cached();

  // Empty string if every invariant holds, else a description of the first
  // violation: every page is free, cached or held, and never twice.
  std::string check() const;

 private:
  struct Group {
    int window;
    int num_pages;
    std::deque<int> free;
    std::vector<int> holders;   // per page, its state: PAGE_FREE (in the free queue), PAGE_PRIVATE (one request's own) or PAGE_NODE (in a prefix node)
  };
  // A published full page per group ("block"): node of the prefix tree.
  struct Node {
    uint64_t hash = 0;
    int parent = -1;
    int depth = 0;               // 1 for the first page of a prompt
    int refcount = 0;            // live requests holding it
    int children = 0;
    bool alive = false;
    std::vector<int> pages;      // one per group
    std::vector<int32_t> tokens;
    std::list<int>::iterator lru_it;
    bool in_lru = false;
  };
  struct Request {
    int slot = -1;
    int length = 0;
    int pending = 0;
    std::vector<int32_t> tokens;              // committed + pending
    std::vector<std::vector<int>> pages;      // [group][logical page] physical page or -1
    std::vector<int> first_live;              // [group] first logical page a window has not passed yet
    std::vector<int> nodes;                   // [logical page] node index or -1 (prefix cache only)
    int published = 0;                        // leading pages that are nodes of this request's chain
    bool chain_broken = false;                // a page lost the race for its hash: nothing later is published
    int attached = 0;                         // cached pages found at admission
    bool ran = false;                         // a step was planned for it: its admission stands in the counters
  };

  int take_page(int g);
  void give_page(int g, int page);
  bool evict_one();
  int alloc_node();
  void publish(Request& r);
  void release_window(Request& r);
  Status grow(Request& r, int upto_tokens, bool all_keys_only);
  int fresh_needed(const Request& r, int g, int upto_tokens) const;
  static uint64_t chain_hash(uint64_t prev, const int32_t* tokens, int n);

  int page_size_;
  bool prefix_cache_;
  std::vector<Group> groups_;
  std::vector<int> free_slots_;
  std::unordered_map<RequestId, Request> requests_;
  std::vector<Node> nodes_;
  std::vector<int> free_nodes_;
  std::unordered_map<uint64_t, int> by_hash_;
  std::list<int> lru_;   // cached (refcount 0) nodes, eviction from the front
  int64_t prefix_hit_pages_ = 0;
  int64_t prefix_hit_requests_ = 0;
  int64_t evictions_ = 0;
};

}  // namespace vosti
