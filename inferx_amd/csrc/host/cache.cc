// Host-side bookkeeping of what requests keep between steps: page pools, block
// lists, state slots, and the flat layout of one step's batch.  No GPU code;
// built with the host compiler into libinferx_host.so and driven from Python
// through a C interface (inferx_amd/cache/manager.py documents the rules).
//
// Reference: KvBlockPool / BlockTable (src/core/kv_cache.cc:58-104,
// include/inferx/core/kv_cache.h:158-186), Reserve / ReleaseBlocks
// (src/scheduler/scheduler.cc:99-111, 170-190), batch emission (:524-668).
#include <cstdint>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace {

struct Pool {
  int32_t num = 0;
  std::vector<int32_t> free_list;  // LIFO; page 0 is handed out first
  std::vector<uint8_t> is_free;

  explicit Pool(int32_t n) : num(n), is_free(static_cast<size_t>(n), 1) {
    free_list.reserve(static_cast<size_t>(n));
    for (int32_t p = n - 1; p >= 0; --p) free_list.push_back(p);
  }
  int32_t allocate() {
    if (free_list.empty()) return -1;
    const int32_t p = free_list.back();
    free_list.pop_back();
    is_free[static_cast<size_t>(p)] = 0;
    return p;
  }
  // 0 ok, -1 outside the pool, -2 freed twice
  int release(int32_t p) {
    if (p < 0 || p >= num) return -1;
    if (is_free[static_cast<size_t>(p)]) return -2;
    is_free[static_cast<size_t>(p)] = 1;
    free_list.push_back(p);
    return 0;
  }
  int32_t free_pages() const { return static_cast<int32_t>(free_list.size()); }
};

struct Request {
  int64_t cached = 0;
  int64_t reserved = 0;  // tokens that pages have been reserved for (>= cached)
  int32_t slot = -1;
  std::vector<std::vector<int32_t>> blocks;  // per group, by logical page; -1 = given back
};

struct Cache {
  std::vector<int32_t> windows;
  std::vector<Pool> pools;
  int32_t page_size = 0, max_requests = 0, max_blocks = 0;
  int64_t max_seq_len = 0;
  int64_t step_cap = 0;  // > 0: no step brings more tokens of a request than this (see reserve)
  std::vector<int32_t> free_slots;
  std::unordered_map<int64_t, Request> requests;
  std::vector<int64_t> order;  // live requests in the order they were added
  std::string error;

  Request* get(int64_t rid) {
    auto it = requests.find(rid);
    if (it == requests.end()) {
      error = "unknown request";
      return nullptr;
    }
    return &it->second;
  }
  int64_t first_live_page(size_t g, int64_t cached) const {
    const int64_t w = windows[g];
    if (w <= 0) return 0;
    const int64_t start = cached + 1 - w;
    return (start > 0 ? start : 0) / page_size;
  }
  bool release_page(size_t g, int32_t page) {
    const int rc = pools[g].release(page);
    if (rc == -1) error = "page " + std::to_string(page) + " is outside the pool";
    if (rc == -2) error = "page " + std::to_string(page) + " freed twice";
    return rc == 0;
  }
  bool drop_pages(Request& r) {
    bool ok = true;
    for (size_t g = 0; g < r.blocks.size(); ++g) {
      for (int32_t p : r.blocks[g])
        if (p >= 0) ok = release_page(g, p) && ok;
      r.blocks[g].clear();
    }
    return ok;
  }
  // pages that no query at or after the request's next position can read go back
  bool release_passed(Request& r) {
    bool ok = true;
    for (size_t g = 0; g < r.blocks.size(); ++g) {
      auto& b = r.blocks[g];
      int64_t first = first_live_page(g, r.cached);
      if (first > static_cast<int64_t>(b.size())) first = static_cast<int64_t>(b.size());
      for (int64_t j = 0; j < first; ++j)
        if (b[static_cast<size_t>(j)] >= 0) {
          ok = release_page(g, b[static_cast<size_t>(j)]) && ok;
          b[static_cast<size_t>(j)] = -1;
        }
    }
    return ok;
  }
  // Pages of group g that a request which has `cached` tokens and a reservation up to `upto` holds now.  A group
  // that keeps every token holds all of them.  A windowed group, when the largest step is known (step_cap), holds
  // only what the next step can touch, cached + step_cap tokens at most: its pages beyond that are taken when the
  // steps get there (its pool is sized so that they are there, see pages_for_window in cache/manager.py), so
  // that a long prompt does not claim a context's worth of pages in a group that only ever reads a window.
  int64_t pages_held(size_t g, int64_t cached, int64_t upto) const {
    if (windows[g] > 0 && step_cap > 0 && upto > cached + step_cap) upto = cached + step_cap;
    return (upto + page_size - 1) / page_size;
  }
  // 0 ok, 1 pool empty, 2 context full, -1 error
  int reserve(int64_t rid, int64_t new_len) {
    Request* r = get(rid);
    if (!r) return -1;
    if (new_len > max_seq_len) return 2;
    if (!release_passed(*r)) return -1;
    const int64_t upto = new_len > r->reserved ? new_len : r->reserved;
    for (size_t g = 0; g < pools.size(); ++g) {
      const int64_t need = pages_held(g, r->cached, upto) - static_cast<int64_t>(r->blocks[g].size());
      if (need > pools[g].free_pages()) return 1;  // all groups or nothing
    }
    for (size_t g = 0; g < pools.size(); ++g) {
      const int64_t want_pages = pages_held(g, r->cached, upto);
      while (static_cast<int64_t>(r->blocks[g].size()) < want_pages) r->blocks[g].push_back(pools[g].allocate());
    }
    r->reserved = upto;
    return 0;
  }
};

Cache* C(void* h) { return static_cast<Cache*>(h); }

}  // namespace

extern "C" {

void* ixh_cache_create(int n_groups, const int32_t* windows, const int32_t* pages, int page_size, int max_requests,
                       int64_t max_seq_len, int64_t step_cap) {
  if (n_groups < 0 || page_size <= 0 || max_requests <= 0 || max_seq_len <= 0 || step_cap < 0) return nullptr;
  for (int g = 0; g < n_groups; ++g)
    if (pages[g] <= 0) return nullptr;
  Cache* c = new Cache();
  c->windows.assign(windows, windows + n_groups);
  for (int g = 0; g < n_groups; ++g) c->pools.emplace_back(pages[g]);
  c->page_size = page_size;
  c->max_requests = max_requests;
  c->max_seq_len = max_seq_len;
  c->step_cap = step_cap;
  c->max_blocks = static_cast<int32_t>((max_seq_len + page_size - 1) / page_size);
  for (int32_t s = max_requests - 1; s >= 0; --s) c->free_slots.push_back(s);
  return c;
}

void ixh_cache_destroy(void* h) { delete C(h); }
const char* ixh_cache_error(void* h) { return C(h)->error.c_str(); }
int ixh_cache_max_blocks(void* h) { return C(h)->max_blocks; }

int ixh_cache_add(void* h, int64_t rid) {
  Cache* c = C(h);
  if (c->requests.count(rid)) {
    c->error = "request is already live";
    return -1;
  }
  if (c->free_slots.empty()) {
    c->error = "all " + std::to_string(c->max_requests) + " request slots are taken";
    return -1;
  }
  Request r;
  r.slot = c->free_slots.back();
  c->free_slots.pop_back();
  r.blocks.resize(c->pools.size());
  c->requests.emplace(rid, std::move(r));
  c->order.push_back(rid);
  return c->requests[rid].slot;
}

int ixh_cache_free(void* h, int64_t rid) {
  Cache* c = C(h);
  Request* r = c->get(rid);
  if (!r) return -1;
  const bool ok = c->drop_pages(*r);
  c->free_slots.push_back(r->slot);
  c->requests.erase(rid);
  for (size_t i = 0; i < c->order.size(); ++i)
    if (c->order[i] == rid) {
      c->order.erase(c->order.begin() + static_cast<long>(i));
      break;
    }
  return ok ? 0 : -1;
}

int ixh_cache_reset(void* h, int64_t rid) {
  Cache* c = C(h);
  Request* r = c->get(rid);
  if (!r) return -1;
  const bool ok = c->drop_pages(*r);
  r->cached = r->reserved = 0;
  return ok ? 0 : -1;
}

int ixh_cache_reserve(void* h, int64_t rid, int64_t new_len) { return C(h)->reserve(rid, new_len); }

int ixh_cache_commit(void* h, int64_t rid, int64_t tokens) {
  Cache* c = C(h);
  Request* r = c->get(rid);
  if (!r) return -1;
  if (tokens < 0 || r->cached + tokens > r->reserved) {
    c->error = "commit of " + std::to_string(tokens) + " tokens beyond the " + std::to_string(r->reserved) + " reserved";
    return -1;
  }
  r->cached += tokens;
  return c->release_passed(*r) ? 0 : -1;
}

int64_t ixh_cache_cached(void* h, int64_t rid) {
  Request* r = C(h)->get(rid);
  return r ? r->cached : -1;
}
int ixh_cache_slot(void* h, int64_t rid) {
  Request* r = C(h)->get(rid);
  return r ? r->slot : -1;
}
int ixh_cache_contains(void* h, int64_t rid) { return C(h)->requests.count(rid) ? 1 : 0; }
int ixh_cache_can_add(void* h) { return C(h)->free_slots.empty() ? 0 : 1; }
int ixh_cache_num_live(void* h) { return static_cast<int>(C(h)->order.size()); }
int ixh_cache_live(void* h, int64_t* out, int cap) {
  Cache* c = C(h);
  int n = 0;
  for (int64_t rid : c->order)
    if (n < cap) out[n++] = rid;
  return n;
}

// the request's pages in this group by logical page number, -1 where none is held; returns the count or -1
int ixh_cache_block_row(void* h, int64_t rid, int group, int32_t* out, int cap) {
  Cache* c = C(h);
  Request* r = c->get(rid);
  if (!r) return -1;
  if (group < 0 || group >= static_cast<int>(c->pools.size())) {
    c->error = "no such page group";
    return -1;
  }
  const auto& b = r->blocks[static_cast<size_t>(group)];
  for (size_t j = 0; j < b.size() && static_cast<int>(j) < cap; ++j) out[j] = b[j];
  return static_cast<int>(b.size());
}

int64_t ixh_cache_slot_index(void* h, int64_t rid, int group, int64_t position) {
  Cache* c = C(h);
  Request* r = c->get(rid);
  if (!r) return -1;
  const auto& b = r->blocks[static_cast<size_t>(group)];
  const int64_t j = position / c->page_size;
  if (position < 0 || j >= static_cast<int64_t>(b.size()) || b[static_cast<size_t>(j)] < 0) {
    c->error = "no page holds position " + std::to_string(position) + " in group " + std::to_string(group);
    return -1;
  }
  return static_cast<int64_t>(b[static_cast<size_t>(j)]) * c->page_size + position % c->page_size;
}

void ixh_cache_pool_stats(void* h, int group, int32_t* num, int32_t* free_pages) {
  const Pool& p = C(h)->pools[static_cast<size_t>(group)];
  *num = p.num;
  *free_pages = p.free_pages();
}

// every page is free or held exactly once; every slot likewise.  0 or -1 with the error text set
int ixh_cache_check(void* h) {
  Cache* c = C(h);
  for (size_t g = 0; g < c->pools.size(); ++g) {
    const Pool& pool = c->pools[g];
    std::vector<uint8_t> held(static_cast<size_t>(pool.num), 0);
    int64_t n_held = 0;
    for (const auto& kv : c->requests)
      for (int32_t p : kv.second.blocks[g]) {
        if (p < 0) continue;
        if (p >= pool.num) { c->error = "group " + std::to_string(g) + ": a held page is outside the pool"; return -1; }
        if (held[static_cast<size_t>(p)]) { c->error = "group " + std::to_string(g) + ": a page is held twice"; return -1; }
        if (pool.is_free[static_cast<size_t>(p)]) {
          c->error = "group " + std::to_string(g) + ": a held page is on the free list";
          return -1;
        }
        held[static_cast<size_t>(p)] = 1;
        ++n_held;
      }
    std::unordered_set<int32_t> seen;
    for (int32_t p : pool.free_list)
      if (!seen.insert(p).second) { c->error = "group " + std::to_string(g) + ": a page is on the free list twice"; return -1; }
    if (n_held + pool.free_pages() != pool.num) {
      c->error = "group " + std::to_string(g) + ": " + std::to_string(pool.num - n_held - pool.free_pages()) + " pages lost";
      return -1;
    }
  }
  std::unordered_set<int32_t> slots(c->free_slots.begin(), c->free_slots.end());
  size_t n = c->free_slots.size();
  for (const auto& kv : c->requests) {
    slots.insert(kv.second.slot);
    ++n;
  }
  if (slots.size() != static_cast<size_t>(c->max_requests) || n != static_cast<size_t>(c->max_requests)) {
    c->error = "a state slot is lost or held twice";
    return -1;
  }
  return 0;
}

// Reserve pages for every entry and lay the step out flat (inferx_amd/engine/batch.py: StepBatch).
// Entries: rids[n], n_tokens[n], tokens_flat, n_want[n], want_flat (places among an entry's tokens).
// Out: token_ids, positions, seq_of_token [T]; q_start [n + 1]; seq_lens, state_slots [n]; logits_rows [sum
// n_want]; slots [G][T]; tables [G][n][max_blocks] (-1 where no page is held).
// Returns 0; 1 / 2 = pages / context ran out for entry *failed (earlier entries keep what they reserved);
// -1 = misuse (error text set; *failed names the entry).
int ixh_build_batch(void* h, int n, const int64_t* rids, const int32_t* n_tokens, const int32_t* tokens_flat,
                    const int32_t* n_want, const int32_t* want_flat, int32_t* token_ids, int32_t* positions,
                    int32_t* seq_of_token, int32_t* q_start, int32_t* seq_lens, int32_t* state_slots,
                    int32_t* logits_rows, int32_t* slots, int32_t* tables, int* failed) {
  Cache* c = C(h);
  const size_t G = c->pools.size();
  std::unordered_set<int64_t> seen;
  int64_t T = 0;
  {
    int64_t w_at = 0;
    for (int s = 0; s < n; ++s) {
      *failed = s;
      if (!seen.insert(rids[s]).second) { c->error = "appears twice in one step"; return -1; }
      if (!c->requests.count(rids[s])) { c->error = "is not live"; return -1; }
      if (n_tokens[s] < 0) { c->error = "negative token count"; return -1; }
      if (c->step_cap > 0 && n_tokens[s] > c->step_cap) {
        c->error = "brings " + std::to_string(n_tokens[s]) + " tokens in one step, the cache was made for " +
                   std::to_string(c->step_cap) + " at most";
        return -1;
      }
      for (int i = 0; i < n_want[s]; ++i)
        if (want_flat[w_at + i] < 0 || want_flat[w_at + i] >= n_tokens[s]) {
          c->error = "wanted place " + std::to_string(want_flat[w_at + i]) + " is outside its " +
                     std::to_string(n_tokens[s]) + " tokens";
          return -1;
        }
      w_at += n_want[s];
      T += n_tokens[s];
    }
  }
  for (int s = 0; s < n; ++s) {
    *failed = s;
    Request& r = c->requests[rids[s]];
    const int rc = c->reserve(rids[s], r.cached + n_tokens[s]);
    if (rc != 0) return rc;
  }
  const int32_t P = c->page_size, MB = c->max_blocks;
  for (int64_t i = 0; i < static_cast<int64_t>(G) * n * MB; ++i) tables[i] = -1;
  int64_t row = 0, t_at = 0, w_at = 0, r_at = 0;
  for (int s = 0; s < n; ++s) {
    const Request& r = c->requests[rids[s]];
    const int32_t cnt = n_tokens[s];
    q_start[s] = static_cast<int32_t>(row);
    seq_lens[s] = static_cast<int32_t>(r.cached + cnt);
    state_slots[s] = r.slot;
    for (size_t g = 0; g < G; ++g) {
      const auto& b = r.blocks[g];
      int32_t* trow = tables + (static_cast<int64_t>(g) * n + s) * MB;
      for (size_t j = 0; j < b.size() && static_cast<int32_t>(j) < MB; ++j) trow[j] = b[j];
    }
    for (int32_t i = 0; i < cnt; ++i) {
      const int64_t pos = r.cached + i;
      token_ids[row + i] = tokens_flat[t_at + i];
      positions[row + i] = static_cast<int32_t>(pos);
      seq_of_token[row + i] = s;
      for (size_t g = 0; g < G; ++g)
        slots[static_cast<int64_t>(g) * T + row + i] =
            r.blocks[g][static_cast<size_t>(pos / P)] * P + static_cast<int32_t>(pos % P);
    }
    for (int i = 0; i < n_want[s]; ++i) logits_rows[r_at++] = static_cast<int32_t>(row + want_flat[w_at + i]);
    w_at += n_want[s];
    t_at += cnt;
    row += cnt;
  }
  q_start[n] = static_cast<int32_t>(row);
  return 0;
}

// ---- a pool on its own (tests, tools) ----
void* ixh_pool_create(int n) { return n > 0 ? new Pool(n) : nullptr; }
void ixh_pool_destroy(void* p) { delete static_cast<Pool*>(p); }
int ixh_pool_allocate(void* p) { return static_cast<Pool*>(p)->allocate(); }
int ixh_pool_release(void* p, int page) { return static_cast<Pool*>(p)->release(page); }
int ixh_pool_free_pages(void* p) { return static_cast<Pool*>(p)->free_pages(); }
int ixh_host_abi_version() { return 1; }

}  // extern "C"
