// Host-side bookkeeping of the engine, with a C interface:
//   * pools of pages and state slots with one owner per item, block tables per
//     request and cache group, pages behind a group's window given back on commit;
//   * the scheduler's decisions: which requests run in the next step and with how
//     many tokens, admission, preemption by recomputation, finishing;
//   * the integer buffer of a step (token ids, positions, request of each token,
//     block tables, cache places of the new tokens, attention work items);
//   * the per-request streams of uniform numbers the sampler draws from.
// No device code and no device memory: the cache's tensors live on the Python side.
//
// The reference keeps the same state in its allocator, block tables and scheduler
// (/root/reference/src/paged_attention/allocator.zig:19-118, block_table.zig:20-93,
// scheduler.zig:6-245); the differences are stated at the functions below.
//
// Every function returns 0 or one of the ZA_HOST_* codes; za_host_last_error() gives
// the message of the calling thread's last failure.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <deque>
#include <string>
#include <unordered_map>
#include <vector>

#define ZA_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

enum {
  ZA_HOST_OK = 0,
  ZA_HOST_OUT_OF_PAGES = 1,
  ZA_HOST_OUT_OF_SLOTS = 2,
  ZA_HOST_POOL = 3,      // a bookkeeping invariant was violated (double free, foreign page, ...)
  ZA_HOST_ARG = 4,
  ZA_HOST_STEP = 5,      // the entries of a step are malformed
};

constexpr int FREED = -1;      // block-table entry of a page that was given back
constexpr int64_t NOBODY = INT64_MIN;

thread_local std::string g_error;

template <typename... A>
int fail(int code, const char* fmt, A... args) {
  char buf[512];
  std::snprintf(buf, sizeof buf, fmt, args...);
  g_error = buf;
  return code;
}
inline int fail(int code, const char* message) {   // no arguments: not a format string
  g_error = message;
  return code;
}

// ------------------------------------------------------------------ pools
// `size` numbered items; take() pops the most recently returned one.  A LIFO free
// list like the reference's (allocator.zig:72-86) with its reference count replaced
// by a single owner per item, which makes "held twice" and "freed twice" detectable.
struct Pool {
  int size = 0;
  bool pages = true;
  std::vector<int> free_;
  std::vector<int64_t> owner;
  int high_water = 0;
  long long total_taken = 0;

  // `scatter`: hand the items out in a fixed pseudo-random order instead of 0, 1, 2 ...
  // Requests that are filled one after the other and then decode in step would
  // otherwise read pages a constant distance apart, which can keep hitting the same
  // memory channels (measured: 64 requests of 2,048 tokens decode 5 % faster scattered).
  void init(int n, bool is_pages, bool scatter = false) {
    size = n;
    pages = is_pages;
    free_.resize(n);
    for (int i = 0; i < n; ++i) free_[i] = n - 1 - i;   // pop yields 0 first
    if (scatter) {
      uint64_t x = 0x9E3779B97F4A7C15ull ^ (uint64_t)n;
      for (int i = n - 1; i > 0; --i) {                 // Fisher-Yates with splitmix64
        x += 0x9E3779B97F4A7C15ull;
        uint64_t z = x;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        std::swap(free_[i], free_[(size_t)(z % (uint64_t)(i + 1))]);
      }
    }
    owner.assign(n, NOBODY);
  }
  const char* what() const { return pages ? "page" : "slot"; }
  int out_of() const { return pages ? ZA_HOST_OUT_OF_PAGES : ZA_HOST_OUT_OF_SLOTS; }
  int free_count() const { return (int)free_.size(); }
  int used_count() const { return size - (int)free_.size(); }

  int take(int64_t who, int* item) {
    if (who == NOBODY) return fail(ZA_HOST_POOL, "an owner is needed");
    if (free_.empty()) return fail(out_of(), "no free %s (all %d in use)", what(), size);
    const int it = free_.back();
    if (owner[it] != NOBODY)
      return fail(ZA_HOST_POOL, "%s %d was on the free list while owned", what(), it);
    free_.pop_back();
    owner[it] = who;
    ++total_taken;
    high_water = std::max(high_water, used_count());
    *item = it;
    return ZA_HOST_OK;
  }
  int give(int item, int64_t who) {
    if (item < 0 || item >= size) return fail(ZA_HOST_POOL, "%s %d does not exist", what(), item);
    if (owner[item] == NOBODY) return fail(ZA_HOST_POOL, "%s %d freed twice", what(), item);
    if (owner[item] != who)
      return fail(ZA_HOST_POOL, "%s %d belongs to another owner", what(), item);
    owner[item] = NOBODY;
    free_.push_back(item);
    return ZA_HOST_OK;
  }
  // every item is either free exactly once or owned, never both
  int check() const {
    std::vector<char> seen(size, 0);
    for (int it : free_) {
      if (it < 0 || it >= size) return fail(ZA_HOST_POOL, "%s %d on the free list does not exist", what(), it);
      if (seen[it]) return fail(ZA_HOST_POOL, "%s %d is on the free list twice", what(), it);
      seen[it] = 1;
      if (owner[it] != NOBODY) return fail(ZA_HOST_POOL, "%s %d is free and owned", what(), it);
    }
    int owned = 0;
    for (int i = 0; i < size; ++i) owned += owner[i] != NOBODY;
    if (owned + (int)free_.size() != size)
      return fail(ZA_HOST_POOL, "%d owned + %d free != %d %ss", owned, (int)free_.size(), size, what());
    return ZA_HOST_OK;
  }
};

// ------------------------------------------------------------------ cache
struct Group {
  int window = 0;
  Pool pool;
  std::vector<char> ever_used;
};

struct RequestCache {
  int slot = -1;
  int num_tokens = 0;
  int reserved = 0;            // tokens the tables cover
  long long serial = 0;        // number of this admission
  std::vector<std::vector<int>> tables;   // per group: page ids
};

struct Cache {
  int page_size = 0;
  std::vector<Group> groups;
  Pool slots;
  std::unordered_map<int64_t, RequestCache> requests;
  long long pages_reused = 0;
  long long admissions = 0;

  RequestCache* find(int64_t req) {
    auto it = requests.find(req);
    return it == requests.end() ? nullptr : &it->second;
  }
  int pages_wanted(const RequestCache& rc, int g, int n_new) const {
    const int want = (rc.num_tokens + n_new + page_size - 1) / page_size;
    return std::max(0, want - (int)rc.tables[g].size());
  }
  bool can_reserve(const RequestCache& rc, int n_new, const int* spare) const {
    for (size_t g = 0; g < groups.size(); ++g) {
      const int free_pages = groups[g].pool.free_count() - (spare ? spare[g] : 0);
      if (pages_wanted(rc, (int)g, n_new) > free_pages) return false;
    }
    return true;
  }
  int admit(int64_t req, int* slot_out) {
    if (requests.count(req)) return fail(ZA_HOST_POOL, "the request is already admitted");
    int slot = 0;
    if (int rc = slots.take(req, &slot)) return rc;
    RequestCache r;
    r.slot = slot;
    r.serial = ++admissions;
    r.tables.resize(groups.size());
    requests.emplace(req, std::move(r));
    if (slot_out) *slot_out = slot;
    return ZA_HOST_OK;
  }
  // make the request's tables cover n_new more tokens; all groups or none
  int reserve(int64_t req, int n_new) {
    RequestCache* rc = find(req);
    if (!rc) return fail(ZA_HOST_ARG, "the request is not admitted");
    if (n_new < 0) return fail(ZA_HOST_ARG, "a negative number of tokens");
    for (size_t g = 0; g < groups.size(); ++g) {
      const int n = pages_wanted(*rc, (int)g, n_new);
      if (n > groups[g].pool.free_count())
        return fail(ZA_HOST_OUT_OF_PAGES, "the request needs %d pages of group %d, %d of %d free", n,
                    (int)g, groups[g].pool.free_count(), groups[g].pool.size);
    }
    for (size_t g = 0; g < groups.size(); ++g) {
      const int n = pages_wanted(*rc, (int)g, n_new);
      for (int i = 0; i < n; ++i) {
        int page = 0;
        if (int e = groups[g].pool.take(req, &page)) return e;
        if (groups[g].ever_used[page]) ++pages_reused;
        groups[g].ever_used[page] = 1;
        rc->tables[g].push_back(page);
      }
    }
    rc->reserved = std::max(rc->reserved, rc->num_tokens + n_new);
    return ZA_HOST_OK;
  }
  // n_new tokens were written; give back pages no later query can read
  int commit(int64_t req, int n_new) {
    RequestCache* rc = find(req);
    if (!rc) return fail(ZA_HOST_ARG, "the request is not admitted");
    if (n_new < 0 || rc->num_tokens + n_new > rc->reserved)
      return fail(ZA_HOST_POOL, "the request commits %d tokens beyond its reservation", n_new);
    rc->num_tokens += n_new;
    for (size_t g = 0; g < groups.size(); ++g) {
      const int w = groups[g].window;
      if (w <= 0) continue;
      // the next query sits at position >= num_tokens and reads keys > position - w
      const int first_needed = rc->num_tokens - w + 1;
      if (first_needed <= 0) continue;
      auto& table = rc->tables[g];
      const int upto = std::min(first_needed / page_size, (int)table.size());
      for (int p = 0; p < upto; ++p)
        if (table[p] != FREED) {
          if (int e = groups[g].pool.give(table[p], req)) return e;
          table[p] = FREED;
        }
    }
    return ZA_HOST_OK;
  }
  int release(int64_t req) {
    auto it = requests.find(req);
    if (it == requests.end()) return fail(ZA_HOST_ARG, "the request is not admitted");
    RequestCache rc = std::move(it->second);
    requests.erase(it);
    for (size_t g = 0; g < groups.size(); ++g)
      for (int page : rc.tables[g])
        if (page != FREED)
          if (int e = groups[g].pool.give(page, req)) return e;
    return slots.give(rc.slot, req);
  }
  // no page lost, held twice or freed twice; tables agree with the pools
  int check() const {
    if (int e = slots.check()) return e;
    std::vector<char> seen_slot(slots.size, 0);
    for (const auto& kv : requests) {
      const RequestCache& rc = kv.second;
      if (rc.slot < 0 || rc.slot >= slots.size) return fail(ZA_HOST_POOL, "slot %d does not exist", rc.slot);
      if (seen_slot[rc.slot]) return fail(ZA_HOST_POOL, "slot %d held twice", rc.slot);
      seen_slot[rc.slot] = 1;
      if (slots.owner[rc.slot] != kv.first)
        return fail(ZA_HOST_POOL, "slot %d is owned by another request", rc.slot);
    }
    if ((int)requests.size() != slots.used_count())
      return fail(ZA_HOST_POOL, "slots in use do not match the admitted requests");
    for (size_t g = 0; g < groups.size(); ++g) {
      const Pool& pool = groups[g].pool;
      if (int e = pool.check()) return e;
      std::vector<char> held(pool.size, 0);
      int n_held = 0;
      for (const auto& kv : requests)
        for (int page : kv.second.tables[g]) {
          if (page == FREED) continue;
          if (page < 0 || page >= pool.size) return fail(ZA_HOST_POOL, "page %d does not exist", page);
          if (held[page]) return fail(ZA_HOST_POOL, "page %d of group %d held twice", page, (int)g);
          held[page] = 1;
          ++n_held;
          if (pool.owner[page] != kv.first)
            return fail(ZA_HOST_POOL, "page %d of group %d is owned by another request", page, (int)g);
        }
      if (n_held != pool.used_count())
        return fail(ZA_HOST_POOL, "group %d: %d pages in use but %d in tables (page lost)", (int)g,
                    pool.used_count(), n_held);
    }
    return ZA_HOST_OK;
  }
};

// ------------------------------------------------------------------ scheduler
// Kept from the reference's scheduler (scheduler.zig:97-245): requests wait in arrival
// order, are admitted head of the line first while the cache has room, decode until
// they reach max_new_tokens, and give their pages back when they finish; when pages
// run out the running request that arrived last is preempted (156-168).  Different by
// design: a token budget per step shared by decoding requests (one token each, served
// first) and portions of prompts of at most chunk_size tokens; pages are taken portion
// by portion; preemption is by recomputation (the victim gives back everything and
// returns to the FRONT of the line with prompt + generated tokens to run again); a
// request is never preempted to admit a waiting one; a request that cannot fit even
// alone is an error instead of waiting forever.
enum Phase { WAITING = 0, RUNNING = 1, FINISHED = 2 };
enum Reason { NONE = 0, EOS = 1, LENGTH = 2, MAX_MODEL_LEN = 3 };

struct SchedRequest {
  int64_t id = 0;
  int prompt_len = 0;
  int out_len = 0;
  int max_new = 0;
  bool has_eos = false;
  int eos = 0;
  long long number = 0;
  int num_computed = 0;
  int phase = WAITING;
  int reason = NONE;
  int preemptions = 0;
  int total() const { return prompt_len + out_len; }
  int remaining() const { return total() - num_computed; }
};

struct PlanEntry {
  int64_t id;
  int start, count, samples;
};

struct Scheduler {
  Cache* cache = nullptr;
  int max_num_seqs = 0, max_tokens = 0, chunk = 0, max_model_len = 0;
  std::unordered_map<int64_t, SchedRequest> reqs;
  std::deque<int64_t> waiting;
  std::vector<int64_t> running;
  long long arrivals = 0;
  long long preemption_count = 0;
  std::vector<int64_t> preempted_now;   // victims of the last schedule()

  void preempt(SchedRequest& v) {
    cache->release(v.id);
    v.num_computed = 0;
    v.phase = WAITING;
    ++v.preemptions;
    ++preemption_count;
    waiting.push_front(v.id);
    preempted_now.push_back(v.id);
  }
  void finish(SchedRequest& r, int reason) {
    if (cache->find(r.id)) cache->release(r.id);
    r.phase = FINISHED;
    r.reason = reason;
  }
  void drop_not_running() {
    running.erase(std::remove_if(running.begin(), running.end(),
                                 [&](int64_t id) { return reqs[id].phase != RUNNING; }),
                  running.end());
  }

  int schedule(std::vector<PlanEntry>& plan) {
    plan.clear();
    preempted_now.clear();
    int budget = max_tokens;
    const size_t G = cache->groups.size();
    std::vector<int> promised(G, 0);
    auto fits = [&](const SchedRequest& r, int n) {
      return cache->can_reserve(*cache->find(r.id), n, promised.data());
    };
    auto promise = [&](const SchedRequest& r, int n, int sign) {
      const RequestCache& rc = *cache->find(r.id);
      for (size_t g = 0; g < G; ++g) promised[g] += sign * cache->pages_wanted(rc, (int)g, n);
    };
    // decoding requests first (one token each), then running prompts, in arrival order
    std::vector<int64_t> order = running;
    std::stable_sort(order.begin(), order.end(), [&](int64_t a, int64_t b) {
      const SchedRequest &ra = reqs[a], &rb = reqs[b];
      const bool pa = ra.remaining() != 1, pb = rb.remaining() != 1;
      if (pa != pb) return pb;
      return ra.number < rb.number;
    });
    for (int64_t id : order) {
      SchedRequest& r = reqs[id];
      if (r.phase != RUNNING) continue;   // preempted while serving an earlier one
      if (budget == 0) break;
      const int n = std::min(std::min(r.remaining(), budget), chunk);
      while (!fits(r, n)) {
        SchedRequest* victim = nullptr;
        int n_running = 0;
        for (int64_t o : running) {
          SchedRequest& c = reqs[o];
          if (c.phase != RUNNING) continue;
          ++n_running;
          if (!victim || c.number > victim->number) victim = &c;
        }
        if (victim == &r && n_running == 1 && plan.empty())
          return fail(ZA_HOST_OUT_OF_PAGES,
                      "a request needs more pages for %d tokens than the whole pool holds",
                      r.num_computed + n);
        auto planned = std::find_if(plan.begin(), plan.end(),
                                    [&](const PlanEntry& e) { return e.id == victim->id; });
        if (planned != plan.end()) {
          // its pages for this step were only promised, not taken
          promise(*victim, planned->count, -1);
          budget += planned->count;
          plan.erase(planned);
        }
        preempt(*victim);
        if (victim == &r) break;
      }
      if (r.phase != RUNNING) continue;
      promise(r, n, +1);
      plan.push_back({r.id, r.num_computed, n, r.num_computed + n == r.total() ? 1 : 0});
      budget -= n;
    }
    drop_not_running();
    // admit waiting requests, head of the line first, while everything fits
    while (!waiting.empty() && budget > 0 && (int)running.size() < max_num_seqs &&
           cache->slots.free_count() > 0) {
      SchedRequest& r = reqs[waiting.front()];
      const int n = std::min(std::min(r.remaining(), budget), chunk);
      if (int e = cache->admit(r.id, nullptr)) return e;
      if (!fits(r, n)) {
        cache->release(r.id);
        if (running.empty())
          return fail(ZA_HOST_OUT_OF_PAGES,
                      "a request needs more pages for its first %d tokens than the whole pool holds", n);
        break;
      }
      waiting.pop_front();
      r.phase = RUNNING;
      running.push_back(r.id);
      promise(r, n, +1);
      plan.push_back({r.id, 0, n, n == r.total() ? 1 : 0});
      budget -= n;
    }
    return ZA_HOST_OK;
  }
};

// ------------------------------------------------------------------ uniform streams
// Philox-4x32 with 10 rounds (Salmon et al., "Parallel random numbers: as easy as 1, 2,
// 3", 2011): the number is a pure function of (seed, request number, index).
inline uint32_t mulhilo(uint32_t a, uint32_t b, uint32_t* hi) {
  const uint64_t p = (uint64_t)a * b;
  *hi = (uint32_t)(p >> 32);
  return (uint32_t)p;
}
float philox_uniform(uint64_t seed, uint64_t request, uint64_t index) {
  uint32_t c[4] = {(uint32_t)index, (uint32_t)(index >> 32), (uint32_t)request, (uint32_t)(request >> 32)};
  uint32_t k[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  for (int round = 0; round < 10; ++round) {
    uint32_t hi0, hi1;
    const uint32_t lo0 = mulhilo(0xD2511F53u, c[0], &hi0);
    const uint32_t lo1 = mulhilo(0xCD9E8D57u, c[2], &hi1);
    const uint32_t n0 = hi1 ^ c[1] ^ k[0], n1 = lo1, n2 = hi0 ^ c[3] ^ k[1], n3 = lo0;
    c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
    k[0] += 0x9E3779B9u;
    k[1] += 0xBB67AE85u;
  }
  return (float)(c[0] >> 8) * (1.0f / 16777216.0f);   // 24 bits: in [0, 1)
}

}  // namespace

// ====================================================================== C interface
ZA_EXPORT const char* za_host_last_error() { return g_error.c_str(); }

// ---- standalone pool (the cache below embeds the same type)
ZA_EXPORT void* za_pool_new(int size, int is_pages) {
  if (size < 0) return nullptr;
  Pool* p = new Pool();
  p->init(size, is_pages != 0);
  return p;
}
ZA_EXPORT void za_pool_free(void* p) { delete static_cast<Pool*>(p); }
ZA_EXPORT int za_pool_take(void* p, int64_t owner, int* item) { return static_cast<Pool*>(p)->take(owner, item); }
ZA_EXPORT int za_pool_take_many(void* p, int64_t owner, int n, int* items) {
  Pool* pool = static_cast<Pool*>(p);
  if (n > pool->free_count())   // all n or none
    return fail(pool->out_of(), "%d %ss wanted, %d of %d free", n, pool->what(), pool->free_count(), pool->size);
  for (int i = 0; i < n; ++i)
    if (int e = pool->take(owner, items + i)) return e;
  return ZA_HOST_OK;
}
ZA_EXPORT int za_pool_give(void* p, int item, int64_t owner) { return static_cast<Pool*>(p)->give(item, owner); }
ZA_EXPORT int za_pool_check(void* p) { return static_cast<Pool*>(p)->check(); }
// out: size, free, high water, total taken
ZA_EXPORT void za_pool_stats(void* p, long long* out) {
  Pool* pool = static_cast<Pool*>(p);
  out[0] = pool->size; out[1] = pool->free_count(); out[2] = pool->high_water; out[3] = pool->total_taken;
}
// 1 and *owner if the item is owned, 0 if free, -1 if it does not exist
ZA_EXPORT int za_pool_owner(void* p, int item, int64_t* owner) {
  Pool* pool = static_cast<Pool*>(p);
  if (item < 0 || item >= pool->size) return -1;
  if (pool->owner[item] == NOBODY) return 0;
  *owner = pool->owner[item];
  return 1;
}

// ---- cache
// `scatter_pages`: see Pool::init (slots are never scattered).
ZA_EXPORT void* za_cache_new(int n_groups, const int* windows, const int* num_pages, int page_size,
                             int num_slots, int scatter_pages) {
  if (n_groups < 0 || page_size <= 0 || num_slots < 0) return nullptr;
  Cache* c = new Cache();
  c->page_size = page_size;
  c->groups.resize(n_groups);
  for (int g = 0; g < n_groups; ++g) {
    if (num_pages[g] < 0) { delete c; return nullptr; }
    c->groups[g].window = windows[g];
    c->groups[g].pool.init(num_pages[g], true, scatter_pages != 0);
    c->groups[g].ever_used.assign(num_pages[g], 0);
  }
  c->slots.init(num_slots, false);
  return c;
}
ZA_EXPORT void za_cache_free(void* c) { delete static_cast<Cache*>(c); }
ZA_EXPORT void* za_cache_pool(void* c, int group) {   // group -1: the slots
  Cache* cache = static_cast<Cache*>(c);
  if (group < 0) return &cache->slots;
  if (group >= (int)cache->groups.size()) return nullptr;
  return &cache->groups[group].pool;
}
ZA_EXPORT int za_cache_admit(void* c, int64_t req, int* slot) { return static_cast<Cache*>(c)->admit(req, slot); }
ZA_EXPORT int za_cache_pages_needed(void* c, int64_t req, int n_new, int* out) {
  Cache* cache = static_cast<Cache*>(c);
  RequestCache* rc = cache->find(req);
  if (!rc) return fail(ZA_HOST_ARG, "the request is not admitted");
  for (size_t g = 0; g < cache->groups.size(); ++g) out[g] = cache->pages_wanted(*rc, (int)g, n_new);
  return ZA_HOST_OK;
}
// spare (may be null): pages promised to others, subtracted from the free counts first
ZA_EXPORT int za_cache_can_reserve(void* c, int64_t req, int n_new, const int* spare, int* ok) {
  Cache* cache = static_cast<Cache*>(c);
  RequestCache* rc = cache->find(req);
  if (!rc) return fail(ZA_HOST_ARG, "the request is not admitted");
  *ok = cache->can_reserve(*rc, n_new, spare) ? 1 : 0;
  return ZA_HOST_OK;
}
ZA_EXPORT int za_cache_reserve(void* c, int64_t req, int n_new) { return static_cast<Cache*>(c)->reserve(req, n_new); }
ZA_EXPORT int za_cache_commit(void* c, int64_t req, int n_new) { return static_cast<Cache*>(c)->commit(req, n_new); }
ZA_EXPORT int za_cache_release(void* c, int64_t req) { return static_cast<Cache*>(c)->release(req); }
// pages for every entry of a step: all of them or none
ZA_EXPORT int za_cache_reserve_many(void* c, int n, const int64_t* reqs, const int* counts) {
  Cache* cache = static_cast<Cache*>(c);
  std::vector<long long> wanted(cache->groups.size(), 0);
  for (int i = 0; i < n; ++i) {
    RequestCache* rc = cache->find(reqs[i]);
    if (!rc) return fail(ZA_HOST_STEP, "entry %d: the request is not admitted", i);
    if (counts[i] < 0) return fail(ZA_HOST_ARG, "a negative number of tokens");
    for (size_t g = 0; g < wanted.size(); ++g) wanted[g] += cache->pages_wanted(*rc, (int)g, counts[i]);
  }
  for (size_t g = 0; g < wanted.size(); ++g)
    if (wanted[g] > cache->groups[g].pool.free_count())
      return fail(ZA_HOST_OUT_OF_PAGES, "the step needs %lld pages of group %d, %d of %d are free",
                  wanted[g], (int)g, cache->groups[g].pool.free_count(), cache->groups[g].pool.size);
  for (int i = 0; i < n; ++i)
    if (int e = cache->reserve(reqs[i], counts[i])) return e;
  return ZA_HOST_OK;
}
ZA_EXPORT int za_cache_commit_many(void* c, int n, const int64_t* reqs, const int* counts) {
  for (int i = 0; i < n; ++i)
    if (int e = static_cast<Cache*>(c)->commit(reqs[i], counts[i])) return e;
  return ZA_HOST_OK;
}
// out: slot, tokens in the cache, tokens the tables cover, admission number; 1 if admitted else 0
ZA_EXPORT int za_cache_request(void* c, int64_t req, long long* out) {
  RequestCache* rc = static_cast<Cache*>(c)->find(req);
  if (!rc) return 0;
  out[0] = rc->slot; out[1] = rc->num_tokens; out[2] = rc->reserved; out[3] = rc->serial;
  return 1;
}
ZA_EXPORT int za_cache_num_requests(void* c) { return (int)static_cast<Cache*>(c)->requests.size(); }
ZA_EXPORT long long za_cache_pages_reused(void* c) { return static_cast<Cache*>(c)->pages_reused; }
// length of the table, or -1; copies at most cap entries
ZA_EXPORT int za_cache_table(void* c, int64_t req, int group, int* out, int cap) {
  Cache* cache = static_cast<Cache*>(c);
  RequestCache* rc = cache->find(req);
  if (!rc || group < 0 || group >= (int)cache->groups.size()) return -1;
  const auto& t = rc->tables[group];
  for (int i = 0; i < (int)t.size() && i < cap; ++i) out[i] = t[i];
  return (int)t.size();
}
// physical places page * page_size + offset of positions start .. start + n - 1
ZA_EXPORT int za_cache_token_slots(void* c, int64_t req, int group, int start, int n, int* out) {
  Cache* cache = static_cast<Cache*>(c);
  RequestCache* rc = cache->find(req);
  if (!rc || group < 0 || group >= (int)cache->groups.size()) return fail(ZA_HOST_ARG, "no such request or group");
  const auto& t = rc->tables[group];
  const int ps = cache->page_size;
  for (int i = 0; i < n; ++i) {
    const int pos = start + i;
    if (pos < 0 || pos / ps >= (int)t.size())
      return fail(ZA_HOST_POOL, "position %d lies beyond the request's pages", pos);
    const int page = t[pos / ps];
    if (page == FREED) return fail(ZA_HOST_POOL, "position %d lies in a page given back", pos);
    out[i] = page * ps + pos % ps;
  }
  return ZA_HOST_OK;
}
ZA_EXPORT int za_cache_check(void* c) { return static_cast<Cache*>(c)->check(); }

// ---- the step's integer buffer
// Sections, in this order, each starting at a multiple of 4 entries: token_ids[T],
// positions[T], token_seq[T], seq_start[S+1], ctx_len[S], slot_id[S], logit_rows[R];
// per group slots[T], table[S * width]; per granularity item_seq, item_row0,
// item_count.  The layout is a function of (tokens per entry, wanted rows per entry,
// table width) only.  `sections` receives (offset, length) pairs in that order,
// `meta` = {T, S, R, table width, longest context (cached + new), total entries}.
// With out == null only sections and meta are computed.  Every request must be
// admitted and its pages for this step reserved; nothing is committed here.
ZA_EXPORT int za_step_build(void* c, int S, const int64_t* reqs, const int* counts, const int* tokens,
                            const int* want_counts, const int* wants, int vocab, int n_gran,
                            const int* grans, int max_position, int min_pages, int* out,
                            long long out_cap, long long* sections, long long* meta,
                            int* ctx_lens, int* slot_ids) {
  Cache* cache = static_cast<Cache*>(c);
  if (S <= 0) return fail(ZA_HOST_STEP, "a step needs at least one entry");
  const int G = (int)cache->groups.size();
  std::vector<RequestCache*> rcs(S);
  long long T = 0, R = 0;
  int max_pages = 1, longest = 0;
  {
    std::vector<int64_t> sorted(reqs, reqs + S);
    std::sort(sorted.begin(), sorted.end());
    if (std::adjacent_find(sorted.begin(), sorted.end()) != sorted.end())
      return fail(ZA_HOST_STEP, "a request appears twice in one step");
  }
  for (int s = 0; s < S; ++s) {
    rcs[s] = cache->find(reqs[s]);
    if (!rcs[s]) return fail(ZA_HOST_STEP, "entry %d: the request is not admitted", s);
    const int n = counts[s];
    if (n <= 0) return fail(ZA_HOST_STEP, "entry %d brings no tokens", s);
    for (int i = 0; i < n; ++i) {
      const int t = tokens[T + i];
      if (t < 0 || t >= vocab)
        return fail(ZA_HOST_STEP, "entry %d: token id %d is outside the vocabulary of %d", s, t, vocab);
    }
    for (int i = 0; i < want_counts[s]; ++i) {
      const int w = wants[R + i];
      if (w < 0 || w >= n)
        return fail(ZA_HOST_STEP, "entry %d wants logits at place %d of %d tokens", s, w, n);
    }
    const int ctx = rcs[s]->num_tokens;
    if (max_position && ctx + n > max_position)
      return fail(ZA_HOST_STEP, "entry %d would reach position %d, beyond max_position_embeddings %d", s,
                  ctx + n - 1, max_position);
    if (ctx + n > rcs[s]->reserved)
      return fail(ZA_HOST_STEP, "entry %d: pages for %d tokens were not reserved", s, ctx + n);
    ctx_lens[s] = ctx;
    slot_ids[s] = rcs[s]->slot;
    longest = std::max(longest, ctx + n);
    for (int g = 0; g < G; ++g) max_pages = std::max(max_pages, (int)rcs[s]->tables[g].size());
    T += n;
    R += want_counts[s];
  }
  max_pages = std::max(max_pages, min_pages);
  // work items: at most `gran` consecutive query rows of one request
  std::vector<long long> item_counts(n_gran, 0);
  for (int k = 0; k < n_gran; ++k) {
    if (grans[k] <= 0) return fail(ZA_HOST_ARG, "a work-item size must be positive");
    for (int s = 0; s < S; ++s) item_counts[k] += (counts[s] + grans[k] - 1) / grans[k];
  }
  long long total = 0;
  int sec = 0;
  auto place = [&](long long n) {
    sections[2 * sec] = total;
    sections[2 * sec + 1] = n;
    ++sec;
    const long long at = total;
    total += (n + 3) / 4 * 4;   // keep every section 16-byte aligned
    return at;
  };
  const long long o_tok = place(T), o_pos = place(T), o_seq = place(T), o_start = place(S + 1),
                  o_ctx = place(S), o_slot = place(S), o_rows = place(R);
  std::vector<long long> o_slots(G), o_table(G);
  for (int g = 0; g < G; ++g) {
    o_slots[g] = place(T);
    o_table[g] = place((long long)S * max_pages);
  }
  std::vector<long long> o_iseq(n_gran), o_irow(n_gran), o_icnt(n_gran);
  for (int k = 0; k < n_gran; ++k) {
    o_iseq[k] = place(item_counts[k]);
    o_irow[k] = place(item_counts[k]);
    o_icnt[k] = place(item_counts[k]);
  }
  if (total < 4) total = 4;
  meta[0] = T; meta[1] = S; meta[2] = R; meta[3] = max_pages; meta[4] = longest; meta[5] = total;
  if (!out) return ZA_HOST_OK;
  if (out_cap < total)
    return fail(ZA_HOST_STEP, "the step needs %lld int32 entries, the buffer holds %lld", total, out_cap);
  std::fill(out, out + total, FREED);
  const int ps = cache->page_size;
  long long row = 0, r = 0;
  for (int s = 0; s < S; ++s) {
    const int n = counts[s], ctx = ctx_lens[s];
    out[o_start + s] = (int)row;
    out[o_ctx + s] = ctx;
    out[o_slot + s] = slot_ids[s];
    for (int i = 0; i < n; ++i) {
      out[o_tok + row + i] = tokens[row + i];
      out[o_pos + row + i] = ctx + i;
      out[o_seq + row + i] = s;
    }
    for (int i = 0; i < want_counts[s]; ++i) out[o_rows + r + i] = (int)row + wants[r + i];
    for (int g = 0; g < G; ++g) {
      const auto& table = rcs[s]->tables[g];
      for (int i = 0; i < n; ++i) {
        const int pos = ctx + i, page = table[pos / ps];
        if (page == FREED)
          return fail(ZA_HOST_POOL, "entry %d: position %d lies in a page given back", s, pos);
        out[o_slots[g] + row + i] = page * ps + pos % ps;
      }
      std::copy(table.begin(), table.end(), out + o_table[g] + (long long)s * max_pages);
    }
    row += n;
    r += want_counts[s];
  }
  out[o_start + S] = (int)row;
  for (int k = 0; k < n_gran; ++k) {
    long long at = 0, first = 0;
    for (int s = 0; s < S; ++s) {
      for (int done = 0; done < counts[s]; done += grans[k]) {
        out[o_iseq[k] + at] = s;
        out[o_irow[k] + at] = (int)(first + done);
        out[o_icnt[k] + at] = std::min(grans[k], counts[s] - done);
        ++at;
      }
      first += counts[s];
    }
  }
  return ZA_HOST_OK;
}

// A step of single tokens, first half: check the entries (admitted, no request twice,
// token ids inside the vocabulary, positions inside max_position), take the pages the
// new tokens need (all or none), and report the widest block table and the longest
// context (cached + 1) among them in extent[0..1].  The second half is za_step_build
// with counts and want_counts of 1.
ZA_EXPORT int za_decode_prepare(void* c, int S, const int64_t* reqs, const int* tokens, int vocab,
                                int max_position, long long* extent) {
  Cache* cache = static_cast<Cache*>(c);
  if (S <= 0) return fail(ZA_HOST_STEP, "a step needs at least one entry");
  const size_t G = cache->groups.size();
  std::vector<long long> wanted(G, 0);
  for (int s = 0; s < S; ++s) {
    for (int o = 0; o < s; ++o)
      if (reqs[o] == reqs[s]) return fail(ZA_HOST_STEP, "a request appears twice in one step");
    RequestCache* rc = cache->find(reqs[s]);
    if (!rc) return fail(ZA_HOST_STEP, "entry %d: the request is not admitted", s);
    if (tokens[s] < 0 || tokens[s] >= vocab)
      return fail(ZA_HOST_STEP, "entry %d: token id %d is outside the vocabulary of %d", s, tokens[s], vocab);
    if (max_position && rc->num_tokens + 1 > max_position)
      return fail(ZA_HOST_STEP, "entry %d would reach position %d, beyond max_position_embeddings %d", s,
                  rc->num_tokens, max_position);
    for (size_t g = 0; g < G; ++g) wanted[g] += cache->pages_wanted(*rc, (int)g, 1);
  }
  for (size_t g = 0; g < G; ++g)
    if (wanted[g] > cache->groups[g].pool.free_count())
      return fail(ZA_HOST_OUT_OF_PAGES, "the step needs %lld pages of group %d, %d of %d are free",
                  wanted[g], (int)g, cache->groups[g].pool.free_count(), cache->groups[g].pool.size);
  long long widest = 1, longest = 0;
  for (int s = 0; s < S; ++s) {
    if (int e = cache->reserve(reqs[s], 1)) return e;
    RequestCache* rc = cache->find(reqs[s]);
    longest = std::max<long long>(longest, rc->num_tokens + 1);
    for (size_t g = 0; g < G; ++g) widest = std::max<long long>(widest, (long long)rc->tables[g].size());
  }
  extent[0] = widest;
  extent[1] = longest;
  return ZA_HOST_OK;
}

// ---- scheduler
ZA_EXPORT void* za_sched_new(void* cache, int max_num_seqs, int max_tokens, int chunk, int max_model_len) {
  if (!cache || max_num_seqs < 1 || max_tokens < 1 || chunk < 1) return nullptr;
  Scheduler* s = new Scheduler();
  s->cache = static_cast<Cache*>(cache);
  s->max_num_seqs = max_num_seqs;
  s->max_tokens = max_tokens;
  s->chunk = chunk;
  s->max_model_len = max_model_len;
  return s;
}
ZA_EXPORT void za_sched_free(void* s) { delete static_cast<Scheduler*>(s); }
// a request with max_new == 0 is finished at once ("length"); *number is its arrival number
ZA_EXPORT int za_sched_add(void* sp, int64_t id, int prompt_len, int max_new, int has_eos, int eos,
                           long long* number) {
  Scheduler* s = static_cast<Scheduler*>(sp);
  if (prompt_len <= 0) return fail(ZA_HOST_ARG, "a request has an empty prompt");
  if (max_new < 0) return fail(ZA_HOST_ARG, "max_new_tokens must be >= 0");
  if (s->reqs.count(id)) return fail(ZA_HOST_ARG, "a request with this id is already known");
  SchedRequest r;
  r.id = id;
  r.prompt_len = prompt_len;
  r.max_new = max_new;
  r.has_eos = has_eos != 0;
  r.eos = eos;
  r.number = s->arrivals++;
  *number = r.number;
  if (max_new == 0) {
    r.phase = FINISHED;
    r.reason = LENGTH;
  } else {
    s->waiting.push_back(id);
  }
  s->reqs.emplace(id, r);
  return ZA_HOST_OK;
}
// forget a finished request
ZA_EXPORT int za_sched_forget(void* sp, int64_t id) {
  Scheduler* s = static_cast<Scheduler*>(sp);
  auto it = s->reqs.find(id);
  if (it == s->reqs.end() || it->second.phase != FINISHED) return fail(ZA_HOST_ARG, "not a finished request");
  s->reqs.erase(it);
  return ZA_HOST_OK;
}
// take a request out, whatever it is doing: what it holds is given back
ZA_EXPORT int za_sched_abort(void* sp, int64_t id) {
  Scheduler* s = static_cast<Scheduler*>(sp);
  auto it = s->reqs.find(id);
  if (it == s->reqs.end()) return fail(ZA_HOST_ARG, "not a request of this scheduler");
  if (s->cache->find(id)) s->cache->release(id);
  s->waiting.erase(std::remove(s->waiting.begin(), s->waiting.end(), id), s->waiting.end());
  s->running.erase(std::remove(s->running.begin(), s->running.end(), id), s->running.end());
  s->reqs.erase(it);
  return ZA_HOST_OK;
}
ZA_EXPORT int za_sched_has_work(void* sp) {
  Scheduler* s = static_cast<Scheduler*>(sp);
  return !s->waiting.empty() || !s->running.empty();
}
// The next step's entries (request, first token, count, whether a token is drawn) and
// the requests preempted while planning it.  *n_plan and *n_preempted receive the
// numbers; at most cap of each are written.
ZA_EXPORT int za_sched_schedule(void* sp, int cap, int64_t* ids, int* starts, int* counts, int* samples,
                                int* n_plan, int64_t* preempted, int* n_preempted) {
  Scheduler* s = static_cast<Scheduler*>(sp);
  std::vector<PlanEntry> plan;
  const int rc = s->schedule(plan);
  *n_preempted = (int)s->preempted_now.size();
  for (int i = 0; i < *n_preempted && i < cap; ++i) preempted[i] = s->preempted_now[i];
  if (rc) { *n_plan = 0; return rc; }
  *n_plan = (int)plan.size();
  for (int i = 0; i < *n_plan && i < cap; ++i) {
    ids[i] = plan[i].id; starts[i] = plan[i].start; counts[i] = plan[i].count; samples[i] = plan[i].samples;
  }
  return ZA_HOST_OK;
}
// Record a step: tokens computed, tokens drawn (tokens[i] is read where samples[i]);
// finish and free what is done.  finished/reasons receive the requests that ended
// (1 eos, 2 length, 3 max_model_len).
ZA_EXPORT int za_sched_update(void* sp, int n, const int64_t* ids, const int* counts, const int* samples,
                              const int* tokens, int64_t* finished, int* reasons, int* n_finished) {
  Scheduler* s = static_cast<Scheduler*>(sp);
  int nf = 0;
  for (int i = 0; i < n; ++i) {
    auto it = s->reqs.find(ids[i]);
    if (it == s->reqs.end()) return fail(ZA_HOST_ARG, "entry %d: unknown request", i);
    SchedRequest& r = it->second;
    r.num_computed += counts[i];
    if (!samples[i]) continue;
    ++r.out_len;
    if (r.has_eos && tokens[i] == r.eos) s->finish(r, EOS);
    else if (r.out_len >= r.max_new) s->finish(r, LENGTH);
    else if (s->max_model_len && r.total() >= s->max_model_len) s->finish(r, MAX_MODEL_LEN);
    if (r.phase == FINISHED) {
      finished[nf] = r.id;
      reasons[nf] = r.reason;
      ++nf;
    }
  }
  s->drop_not_running();
  *n_finished = nf;
  return ZA_HOST_OK;
}
// out: phase (0 waiting, 1 running, 2 finished), tokens computed, preemptions, reason,
// arrival number, generated tokens; 1 if known else 0
ZA_EXPORT int za_sched_request(void* sp, int64_t id, long long* out) {
  Scheduler* s = static_cast<Scheduler*>(sp);
  auto it = s->reqs.find(id);
  if (it == s->reqs.end()) return 0;
  const SchedRequest& r = it->second;
  out[0] = r.phase; out[1] = r.num_computed; out[2] = r.preemptions; out[3] = r.reason;
  out[4] = r.number; out[5] = r.out_len;
  return 1;
}
// which: 0 the waiting line, 1 the running requests; returns the length
ZA_EXPORT int za_sched_queue(void* sp, int which, int64_t* out, int cap) {
  Scheduler* s = static_cast<Scheduler*>(sp);
  int n = 0;
  if (which == 0) {
    for (int64_t id : s->waiting) { if (n < cap) out[n] = id; ++n; }
  } else {
    for (int64_t id : s->running) { if (n < cap) out[n] = id; ++n; }
  }
  return n;
}
ZA_EXPORT long long za_sched_preemptions(void* sp) { return static_cast<Scheduler*>(sp)->preemption_count; }

// ---- uniform numbers: out[i] = number `index[i]` of the stream of (seed[i], request[i])
ZA_EXPORT void za_uniforms(int n, const uint64_t* seeds, const uint64_t* requests, const uint64_t* index,
                           float* out) {
  for (int i = 0; i < n; ++i) out[i] = philox_uniform(seeds[i], requests[i], index[i]);
}
