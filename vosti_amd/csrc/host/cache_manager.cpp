#include "cache_manager.h"

#include <algorithm>
#include <sstream>

namespace vosti {

static constexpr int8_t PAGE_FREE = 0, PAGE_PRIVATE = 1, PAGE_NODE = 2;

CacheManager::CacheManager(int page_size, std::vector<GroupSpec> groups, int num_slots, bool prefix_cache)
    : page_size_(page_size), prefix_cache_(prefix_cache) {
  for (const GroupSpec& s : groups) {
    Group g;
    g.window = s.window;
    g.num_pages = s.num_pages;
    for (int p = 0; p < s.num_pages; ++p) g.free.push_back(p);
    g.holders.assign(s.num_pages, PAGE_FREE);
    groups_.push_back(std::move(g));
    // A page of a windowed group is given back while its request lives, so it
    // cannot be shared: prefix reuse needs every group to keep all keys.
    if (s.window != 0) prefix_cache_ = false;
  }
  for (int s = num_slots - 1; s >= 0; --s) free_slots_.push_back(s);
}

uint64_t CacheManager::chain_hash(uint64_t prev, const int32_t* tokens, int n) {
  uint64_t h = prev ^ 0xcbf29ce484222325ull;
  for (int i = 0; i < n; ++i) h = (h ^ (uint64_t)(uint32_t)tokens[i]) * 0x100000001b3ull;
  return h;
}

int CacheManager::take_page(int g) {
  Group& grp = groups_[g];
  const int p = grp.free.front();
  grp.free.pop_front();
  grp.holders[p] = PAGE_PRIVATE;
  return p;
}

void CacheManager::give_page(int g, int page) {
  Group& grp = groups_[g];
  grp.holders[page] = PAGE_FREE;
  grp.free.push_front(page);
}

int CacheManager::alloc_node() {
  if (!free_nodes_.empty()) {
    const int i = free_nodes_.back();
    free_nodes_.pop_back();
    return i;
  }
  nodes_.emplace_back();
  return (int)nodes_.size() - 1;
}

bool CacheManager::evict_one() {
  for (auto it = lru_.begin(); it != lru_.end(); ++it) {
    Node& n = nodes_[*it];
    if (n.children != 0) continue;   // parents stay until their children have gone
    const int idx = *it;
    lru_.erase(it);
    n.in_lru = false;
    by_hash_.erase(n.hash);
    if (n.parent >= 0) nodes_[n.parent].children -= 1;
    for (int g = 0; g < (int)groups_.size(); ++g) give_page(g, n.pages[g]);
    n.alive = false;
    n.pages.clear();
    n.tokens.clear();
    free_nodes_.push_back(idx);
    evictions_ += 1;
    return true;
  }
  return false;
}

int CacheManager::drop_cached() {
  int n = 0;
  while (evict_one()) n += 1;
  return n;
}

int CacheManager::available_pages(int g) const {
  return (int)groups_[g].free.size() + (prefix_cache_ ? (int)lru_.size() : 0);
}

int CacheManager::fresh_needed(const Request& r, int g, int upto_tokens) const {
  const int need = (upto_tokens + page_size_ - 1) / page_size_;
  return std::max(0, need - (int)r.pages[g].size());
}

int CacheManager::pages_needed(RequestId id, int group, int n_more) const {
  auto it = requests_.find(id);
  if (it == requests_.end()) return (n_more + page_size_ - 1) / page_size_;
  const Request& r = it->second;
  return fresh_needed(r, group, r.length + r.pending + n_more);
}

Status CacheManager::grow(Request& r, int upto_tokens, bool all_keys_only) {
  const int G = (int)groups_.size();
  for (int g = 0; g < G; ++g) {
    if (all_keys_only && groups_[g].window != 0) continue;
    if (fresh_needed(r, g, upto_tokens) > available_pages(g)) return NO_PAGES;
  }
  for (int g = 0; g < G; ++g) {
    if (all_keys_only && groups_[g].window != 0) continue;
    int fresh = fresh_needed(r, g, upto_tokens);
    while (fresh > 0) {
      if (groups_[g].free.empty() && !evict_one()) return NO_PAGES;   // not reached: checked above
      r.pages[g].push_back(take_page(g));
      fresh -= 1;
    }
  }
  if (prefix_cache_) r.nodes.resize(r.pages.empty() ? 0 : r.pages[0].size(), -1);
  return OK;
}

Status CacheManager::add_request(RequestId id, const int32_t* prompt, int n_prompt, int* cached_tokens) {
  if (cached_tokens) *cached_tokens = 0;
  if (requests_.count(id)) return DUPLICATE_REQUEST;
  if (n_prompt < 0 || (n_prompt > 0 && prompt == nullptr)) return BAD_ARGUMENT;
  if (free_slots_.empty()) return NO_SLOT;
  Request r;
  r.slot = free_slots_.back();
  free_slots_.pop_back();
  r.pages.resize(groups_.size());
  r.first_live.assign(groups_.size(), 0);
  if (prefix_cache_ && n_prompt > 0) {
    const int c_max = (n_prompt - 1) / page_size_;   // at least one prompt token stays uncached
    uint64_t h = 0;
    int parent = -1;
    for (int j = 0; j < c_max; ++j) {
      const int32_t* blk = prompt + (int64_t)j * page_size_;
      h = chain_hash(h, blk, page_size_);
      auto it = by_hash_.find(h);
      if (h == 0 || it == by_hash_.end()) break;
      Node& n = nodes_[it->second];
      if (!n.alive || n.depth != j + 1 || n.parent != parent) break;
      if (!std::equal(n.tokens.begin(), n.tokens.end(), blk)) break;
      if (n.in_lru) {
        lru_.erase(n.lru_it);
        n.in_lru = false;
      }
      n.refcount += 1;
      for (int g = 0; g < (int)groups_.size(); ++g) r.pages[g].push_back(n.pages[g]);
      r.nodes.push_back(it->second);
      parent = it->second;
      r.published = j + 1;
    }
    r.length = r.published * page_size_;
    r.tokens.assign(prompt, prompt + r.length);
    r.attached = r.published;
    prefix_hit_pages_ += r.published;
    if (r.published > 0) ++prefix_hit_requests_;
    if (cached_tokens) *cached_tokens = r.length;
  }
  requests_.emplace(id, std::move(r));
  return OK;
}

Status CacheManager::reserve(RequestId id, int total_tokens) {
  auto it = requests_.find(id);
  if (it == requests_.end()) return UNKNOWN_REQUEST;
  if (total_tokens < 0) return BAD_ARGUMENT;
  return grow(it->second, total_tokens, /*all_keys_only=*/true);
}

Status CacheManager::extend(RequestId id, const int32_t* tokens, int n) {
  auto it = requests_.find(id);
  if (it == requests_.end()) return UNKNOWN_REQUEST;
  Request& r = it->second;
  if (n <= 0 || tokens == nullptr) return BAD_ARGUMENT;
  if (r.pending != 0) return STEP_PENDING;
  const Status st = grow(r, r.length + n, /*all_keys_only=*/false);
  if (st != OK) return st;
  r.tokens.insert(r.tokens.end(), tokens, tokens + n);
  r.ran = true;
  r.pending = n;
  return OK;
}

Status CacheManager::abort_step(RequestId id) {
  auto it = requests_.find(id);
  if (it == requests_.end()) return UNKNOWN_REQUEST;
  Request& r = it->second;
  r.tokens.resize(r.length);
  r.pending = 0;
  return OK;
}

void CacheManager::publish(Request& r) {
  while (!r.chain_broken && (r.published + 1) * page_size_ <= r.length) {
    const int j = r.published;
    const int parent = j > 0 ? r.nodes[j - 1] : -1;
    const uint64_t prev = parent >= 0 ? nodes_[parent].hash : 0;
    const int32_t* blk = r.tokens.data() + (int64_t)j * page_size_;
    const uint64_t h = chain_hash(prev, blk, page_size_);
    if (h == 0 || by_hash_.count(h)) {
      // The first writer of a hash keeps it; this request's copy stays private,
      // and so does everything after it, which could only hang below it.
      r.chain_broken = true;
      break;
    }
    const int idx = alloc_node();
    Node& n = nodes_[idx];
    n.hash = h;
    n.parent = parent;
    n.depth = j + 1;
    n.refcount = 1;
    n.children = 0;
    n.alive = true;
    n.in_lru = false;
    n.tokens.assign(blk, blk + page_size_);
    n.pages.clear();
    for (int g = 0; g < (int)groups_.size(); ++g) {
      n.pages.push_back(r.pages[g][j]);
      groups_[g].holders[r.pages[g][j]] = PAGE_NODE;
    }
    if (parent >= 0) nodes_[parent].children += 1;
    by_hash_[h] = idx;
    r.nodes[j] = idx;
    r.published = j + 1;
  }
}

void CacheManager::release_window(Request& r) {
  for (int g = 0; g < (int)groups_.size(); ++g) {
    const int w = groups_[g].window;
    if (w == 0) continue;
    // The next query stands at position >= length and sees keys >= length - w + 1.
    const int first_needed = std::max(0, r.length - w + 1);
    const int upto = std::min((int)r.pages[g].size(), first_needed / page_size_);
    for (int j = r.first_live[g]; j < upto; ++j) {
      if (r.pages[g][j] >= 0) {
        give_page(g, r.pages[g][j]);
        r.pages[g][j] = -1;
      }
    }
    r.first_live[g] = std::max(r.first_live[g], upto);
  }
}

Status CacheManager::commit(RequestId id) {
  auto it = requests_.find(id);
  if (it == requests_.end()) return UNKNOWN_REQUEST;
  Request& r = it->second;
  r.length += r.pending;
  r.pending = 0;
  if (prefix_cache_) publish(r);
  release_window(r);
  return OK;
}

Status CacheManager::finish(RequestId id) {
  auto it = requests_.find(id);
  if (it == requests_.end()) return UNKNOWN_REQUEST;
  Request& r = it->second;
  if (!r.ran && r.attached > 0) {
    prefix_hit_pages_ -= r.attached;
    prefix_hit_requests_ -= 1;
  }
  const int n_logical = r.pages.empty() ? 0 : (int)r.pages[0].size();
  // Tail to root, so that in the cached queue children stand before parents.
  for (int j = n_logical - 1; j >= 0; --j) {
    const int node = (prefix_cache_ && j < (int)r.nodes.size()) ? r.nodes[j] : -1;
    if (node >= 0) {
      Node& n = nodes_[node];
      n.refcount -= 1;
      if (n.refcount == 0) {
        lru_.push_back(node);
        n.lru_it = std::prev(lru_.end());
        n.in_lru = true;
      }
    }
  }
  for (int g = 0; g < (int)groups_.size(); ++g) {
    for (int j = (int)r.pages[g].size() - 1; j >= 0; --j) {
      const int p = r.pages[g][j];
      if (p < 0) continue;
      const bool shared = prefix_cache_ && j < (int)r.nodes.size() && r.nodes[j] >= 0;
      if (!shared) give_page(g, p);
    }
  }
  free_slots_.push_back(r.slot);
  requests_.erase(it);
  return OK;
}

int CacheManager::length(RequestId id) const {
  auto it = requests_.find(id);
  return it == requests_.end() ? -1 : it->second.length;
}

int CacheManager::pending(RequestId id) const {
  auto it = requests_.find(id);
  return it == requests_.end() ? -1 : it->second.pending;
}

int CacheManager::state_slot(RequestId id) const {
  auto it = requests_.find(id);
  return it == requests_.end() ? -1 : it->second.slot;
}

int CacheManager::num_logical_pages(RequestId id, int group) const {
  auto it = requests_.find(id);
  if (it == requests_.end() || group < 0 || group >= (int)groups_.size()) return -1;
  return (int)it->second.pages[group].size();
}

Status CacheManager::fill_block_table(RequestId id, int group, int32_t* out, int width) const {
  auto it = requests_.find(id);
  if (it == requests_.end()) return UNKNOWN_REQUEST;
  if (group < 0 || group >= (int)groups_.size()) return BAD_ARGUMENT;
  const std::vector<int>& pg = it->second.pages[group];
  if ((int)pg.size() > width) return BAD_ARGUMENT;
  for (int j = 0; j < width; ++j) out[j] = (j < (int)pg.size() && pg[j] >= 0) ? pg[j] : 0;
  return OK;
}

Status CacheManager::fill_slots(RequestId id, int group, int start, int n, int32_t* out) const {
  auto it = requests_.find(id);
  if (it == requests_.end()) return UNKNOWN_REQUEST;
  if (group < 0 || group >= (int)groups_.size() || start < 0 || n < 0) return BAD_ARGUMENT;
  const std::vector<int>& pg = it->second.pages[group];
  for (int i = 0; i < n; ++i) {
    const int pos = start + i, j = pos / page_size_;
    if (j >= (int)pg.size() || pg[j] < 0) return BAD_ARGUMENT;
    out[i] = pg[j] * page_size_ + pos % page_size_;
  }
  return OK;
}

std::string CacheManager::check() const {
  std::ostringstream err;
  const int G = (int)groups_.size();
  for (int g = 0; g < G; ++g) {
    const Group& grp = groups_[g];
    std::vector<int> seen(grp.num_pages, 0);
    for (int p : grp.free) {
      if (p < 0 || p >= grp.num_pages) { err << "group " << g << ": free list holds page " << p; return err.str(); }
      if (grp.holders[p] != PAGE_FREE) { err << "group " << g << ": page " << p << " is free and held"; return err.str(); }
      if (seen[p]++) { err << "group " << g << ": page " << p << " is free twice"; return err.str(); }
    }
    for (size_t i = 0; i < nodes_.size(); ++i) {
      const Node& n = nodes_[i];
      if (!n.alive) continue;
      const int p = n.pages[g];
      if (grp.holders[p] != PAGE_NODE) { err << "group " << g << ": published page " << p << " has the wrong state"; return err.str(); }
      if (seen[p]++) { err << "group " << g << ": page " << p << " is held twice"; return err.str(); }
      if (n.refcount < 0) { err << "node " << i << " has a negative count"; return err.str(); }
      if ((n.refcount == 0) != n.in_lru) { err << "node " << i << ": cached-queue membership disagrees with its count"; return err.str(); }
    }
    std::vector<int> node_refs(nodes_.size(), 0);
    for (const auto& kv : requests_) {
      const Request& r = kv.second;
      for (size_t j = 0; j < r.pages[g].size(); ++j) {
        const int p = r.pages[g][j];
        if (p < 0) continue;
        const int node = (prefix_cache_ && j < r.nodes.size()) ? r.nodes[j] : -1;
        if (node >= 0) {
          if (nodes_[node].pages[g] != p) { err << "request " << kv.first << ": page " << j << " disagrees with its node"; return err.str(); }
          node_refs[node] += 1;
        } else {
          if (grp.holders[p] != PAGE_PRIVATE) { err << "group " << g << ": private page " << p << " has the wrong state"; return err.str(); }
          if (seen[p]++) { err << "group " << g << ": page " << p << " is held twice"; return err.str(); }
        }
      }
    }
    for (size_t i = 0; i < nodes_.size(); ++i)
      if (nodes_[i].alive && node_refs[i] != nodes_[i].refcount) { err << "node " << i << ": count " << nodes_[i].refcount << " but " << node_refs[i] << " holders"; return err.str(); }
    for (int p = 0; p < grp.num_pages; ++p)
      if (!seen[p]) { err << "group " << g << ": page " << p << " is lost"; return err.str(); }
  }
  std::vector<int> slot_seen(free_slots_.size() + requests_.size(), 0);
  for (int s : free_slots_) {
    if (s < 0 || s >= (int)slot_seen.size() || slot_seen[s]++) { err << "state slot " << s << " is free twice or out of range"; return err.str(); }
  }
  for (const auto& kv : requests_) {
    const int s = kv.second.slot;
    if (s < 0 || s >= (int)slot_seen.size() || slot_seen[s]++) { err << "state slot " << s << " is held twice"; return err.str(); }
  }
  // Cached queue: a child never stands behind its parent.
  std::unordered_map<int, int> order;
  int k = 0;
  for (int idx : lru_) order[idx] = k++;
  for (int idx : lru_) {
    const int parent = nodes_[idx].parent;
    if (parent >= 0 && order.count(parent) && order[parent] < order[idx]) { err << "cached queue: node " << idx << " stands behind its parent"; return err.str(); }
  }
  return "";
}

}  // namespace vosti
