// Host runtime in C++: the page pool, the cache manager's accounting with the
// layout of a step, and the scheduler. Integers only; no GPU call is made here.
// The Python classes of the same names are thin faces over these through a C API:
// a call returns a value >= 0, or minus an error code of the list below with the
// message kept for alofa_host_last_error().
//
// Pool: src/alofa/runtime/kv/pool.mojo:28-114 of the reference (first allocations
// 0, 1, 2, ..., a released page is the next one handed out). Scheduler: the policy
// and its order within a tick of src/alofa/engine/scheduler.mojo:639-767.
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <vector>

namespace {

enum Err : int { kInvalidArgument = 1, kOutOfRange = 2, kCapacity = 5, kDoubleFree = 11 };

thread_local char g_error[512];

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return -code;
}

int64_t blocks_for(int64_t tokens, int64_t block_size) { return tokens <= 0 ? 0 : (tokens + block_size - 1) / block_size; }

// ------------------------------------------------------------------------ pool

struct Pool {
  int n_blocks;
  std::vector<int> refcnt, free_stack;
  int high_water = 0;

  explicit Pool(int n) : n_blocks(n), refcnt(n, 0) {
    free_stack.reserve(n);
    for (int b = n - 1; b >= 0; --b) free_stack.push_back(b);  // pop yields 0 first
  }
  int n_free() const { return static_cast<int>(free_stack.size()); }
  int used() const { return n_blocks - n_free(); }
  int alloc_one() {
    if (free_stack.empty()) return fail(kCapacity, "kv block pool is exhausted [n_blocks=%d]", n_blocks);
    const int b = free_stack.back();
    free_stack.pop_back();
    refcnt[b] = 1;
    high_water = std::max(high_water, used());
    return b;
  }
  int held(int b) const {
    if (b < 0 || b >= n_blocks) return fail(kOutOfRange, "block id is outside the pool [block=%d n_blocks=%d]", b, n_blocks);
    if (refcnt[b] <= 0) return fail(kDoubleFree, "block is not held [block=%d]", b);
    return 0;
  }
  int retain(int b) {
    if (int e = held(b)) return e;
    ++refcnt[b];
    return 0;
  }
  int release(int b) {  // 1 when the block went back to the pool
    if (int e = held(b)) return e;
    if (--refcnt[b] == 0) {
      free_stack.push_back(b);
      return 1;
    }
    return 0;
  }
};

// ----------------------------------------------------------------------- cache

struct Group {
  int64_t window;  // -1: every key stays visible
  Pool pool;
};

struct Request {
  bool live = false;
  int64_t length = 0;
  std::vector<std::vector<int>> tables;  // per group: logical block -> physical or -1
  std::vector<int> first_held;
};

struct Cache {
  int block_size, max_requests;
  std::vector<Group> groups;
  std::vector<Request> reqs;  // by slot
  std::vector<int> free_slots;

  Request* get(int slot) {
    if (slot < 0 || slot >= max_requests || !reqs[slot].live) {
      fail(kInvalidArgument, "no such request [slot=%d]", slot);
      return nullptr;
    }
    return &reqs[slot];
  }
  int needed(const Request& r, int g, int64_t target) const {
    return static_cast<int>(std::max<int64_t>(0, blocks_for(target, block_size) - static_cast<int64_t>(r.tables[g].size())));
  }
  int reserve(int slot, int64_t target) {
    Request* r = get(slot);
    if (!r) return -kInvalidArgument;
    if (target < r->length) return fail(kInvalidArgument, "a request cannot shrink [slot=%d length=%lld target=%lld]", slot, (long long)r->length, (long long)target);
    for (size_t g = 0; g < groups.size(); ++g)
      if (needed(*r, g, target) > groups[g].pool.n_free())
        return fail(kCapacity, "kv block pool is exhausted [slot=%d group=%d need=%d free=%d]", slot, (int)g, needed(*r, g, target), groups[g].pool.n_free());
    for (size_t g = 0; g < groups.size(); ++g)
      for (int i = needed(*r, g, target); i > 0; --i) r->tables[g].push_back(groups[g].pool.alloc_one());
    return 0;
  }
  // freed pages are appended to freed[g] when given
  int commit(int slot, int64_t target, std::vector<std::vector<int>>* freed) {
    Request* r = get(slot);
    if (!r) return -kInvalidArgument;
    bool short_of = target < r->length;
    for (size_t g = 0; g < groups.size(); ++g) short_of |= blocks_for(target, block_size) > static_cast<int64_t>(r->tables[g].size());
    if (short_of) return fail(kInvalidArgument, "commit beyond what was reserved [slot=%d length=%lld target=%lld]", slot, (long long)r->length, (long long)target);
    r->length = target;
    for (size_t g = 0; g < groups.size(); ++g) {
      if (groups[g].window < 0) continue;
      // the next query stands at position `target` and sees keys >= target - window + 1
      const int64_t first_needed = std::max<int64_t>(0, target - groups[g].window + 1) / block_size;
      const int upto = static_cast<int>(std::min<int64_t>(first_needed, r->tables[g].size()));
      for (int b = r->first_held[g]; b < upto; ++b) {
        int& page = r->tables[g][b];
        if (page >= 0) {
          groups[g].pool.release(page);
          if (freed) (*freed)[g].push_back(page);
          page = -1;
        }
      }
      r->first_held[g] = std::max(r->first_held[g], upto);
    }
    return 0;
  }
};

// ------------------------------------------------------------------- scheduler

constexpr int ST_FREE = 0, ST_WAITING = 1, ST_RUNNING = 2;
constexpr int64_t DIGEST_MOD = 2147483647, DIGEST_MUL = 1000003;

// What the scheduler knows of one group of layers: its pool's pages, and the most tokens a request holds pages
// for in it at any time: below zero for no bound (a group that keeps every key, the reference's only case), a
// window's length plus what a step adds where the group gives back what its window has passed, 0 where it keeps
// no pages at all.
struct GroupRule {
  int64_t capacity, held_tokens;
};

struct SchedConfig {
  int64_t token_budget, max_chunk, block_size, watermark_permille, max_wait_ticks;
  int n_slots;
  std::vector<GroupRule> groups;  // at least one; the first is the one the reference's single count stands for
  int n_groups() const { return static_cast<int>(groups.size()); }
  int64_t threshold(int g) const { return groups[g].capacity * watermark_permille / 1000; }
  // pages a request of this many tokens holds in group g
  int64_t blocks(int g, int64_t tokens) const {
    const int64_t held = groups[g].held_tokens;
    return blocks_for(held < 0 ? tokens : std::min(tokens, held), block_size);
  }
};

// cfg: token_budget, max_chunk, block_size, capacity_blocks, watermark_permille, max_wait_ticks, n_slots, held_tokens,
// n_more, then (capacity_blocks, held_tokens) of every further group
SchedConfig config_from(const int64_t* cfg) {
  SchedConfig c{cfg[0], cfg[1], cfg[2], cfg[4], cfg[5], static_cast<int>(cfg[6]), {GroupRule{cfg[3], cfg[7]}}};
  for (int64_t g = 0; g < cfg[8]; ++g) c.groups.push_back(GroupRule{cfg[9 + 2 * g], cfg[10 + 2 * g]});
  return c;
}

struct Action {
  std::vector<int64_t> prefill;  // triples id, start, end
  std::vector<int64_t> decode, preempted, finished;
};

// Every count of pages is kept per group of layers, and every decision holds for all groups at once: a request
// is admitted, a chunk runs, a decode proceeds only where no group's bound is passed; the group that binds
// decides. With one group this is the reference's arithmetic number for number.
struct Sched {
  SchedConfig cfg;
  std::vector<int64_t> ids, prompt_len, done, generated, max_new, state, wait_ticks, preempt_count;
  std::vector<int64_t> blocks_used, cached_blocks;  // per group
  int64_t preempt_total = 0, tick_seq = 0;

  explicit Sched(const SchedConfig& c) : cfg(c), blocks_used(c.groups.size(), 0), cached_blocks(c.groups.size(), 0) {
    for (auto* v : {&ids, &prompt_len, &done, &generated, &max_new, &state, &wait_ticks, &preempt_count}) v->assign(c.n_slots, 0);
  }
  int G() const { return cfg.n_groups(); }
  int find(int64_t req) const {
    for (int i = 0; i < cfg.n_slots; ++i)
      if (state[i] != ST_FREE && ids[i] == req) return i;
    return -1;
  }
  int n_live() const { return static_cast<int>(std::count_if(state.begin(), state.end(), [](int64_t s) { return s != ST_FREE; })); }
  int64_t blocks_held(int g) const {
    int64_t t = 0;
    for (int i = 0; i < cfg.n_slots; ++i)
      if (state[i] != ST_FREE) t += cfg.blocks(g, done[i] + generated[i]);
    return t;
  }
  int64_t blocks_wanted(int g) const {
    int64_t t = 0;
    for (int i = 0; i < cfg.n_slots; ++i)
      if (state[i] == ST_WAITING) t += std::max<int64_t>(0, cfg.blocks(g, prompt_len[i]) - cfg.blocks(g, done[i]));
    return t;
  }
  int64_t digest() const {
    int64_t h = 0;
    for (int i = 0; i < cfg.n_slots; ++i)
      for (int64_t x : {state[i], ids[i], prompt_len[i], done[i], generated[i], max_new[i], wait_ticks[i], preempt_count[i]})
        h = (h * DIGEST_MUL + x) % DIGEST_MOD;
    for (int64_t x : {blocks_used[0], cached_blocks[0], preempt_total}) h = (h * DIGEST_MUL + x) % DIGEST_MOD;
    for (int g = 1; g < G(); ++g)  // (further groups follow; with one group the value is the reference's)
      for (int64_t x : {blocks_used[g], cached_blocks[g]}) h = (h * DIGEST_MUL + x) % DIGEST_MOD;
    return h;
  }
  int64_t committed(int g) const {
    int64_t t = 0;
    for (int i = 0; i < cfg.n_slots; ++i)
      if (state[i] != ST_FREE) t += cfg.blocks(g, prompt_len[i] + max_new[i]);
    return t;
  }
  // pages the growth from `from` to `to` tokens takes, per group, and whether they fit under every group's capacity
  // (a group that is asked for nothing is looked at only with `also_idle`: the reference's decode phase does not, its
  // prefill phase does)
  bool growth_fits(int64_t from, int64_t to, std::vector<int64_t>& need, bool also_idle) const {
    bool fits = true;
    need.resize(G());
    for (int g = 0; g < G(); ++g) {
      need[g] = cfg.blocks(g, to) - cfg.blocks(g, from);
      fits &= (need[g] <= 0 && !also_idle) || blocks_used[g] + need[g] <= cfg.groups[g].capacity;
    }
    return fits;
  }
  bool over_watermark() const {
    for (int g = 0; g < G(); ++g)
      if (blocks_used[g] > cfg.threshold(g)) return true;
    return false;
  }
  int admit(int64_t req, int64_t p_len, int64_t m_new) {
    if (p_len <= 0) return fail(kInvalidArgument, "prompt_len must be positive [request=%lld]", (long long)req);
    if (m_new <= 0) return fail(kInvalidArgument, "max_new must be positive [request=%lld]", (long long)req);
    if (find(req) >= 0) return fail(kInvalidArgument, "duplicate request id [request=%lld]", (long long)req);
    for (int g = 0; g < G(); ++g)
      if (cfg.blocks(g, p_len) > cfg.groups[g].capacity) return fail(kCapacity, "prompt does not fit in the kv pool [request=%lld]", (long long)req);
    for (int g = 0; g < G(); ++g)
      if (committed(g) + cfg.blocks(g, p_len + m_new) > cfg.threshold(g))
        return fail(kCapacity, "concurrent sequences exceed the kv watermark [request=%lld]", (long long)req);
    int slot = -1;
    for (int i = 0; i < cfg.n_slots && slot < 0; ++i)
      if (state[i] == ST_FREE) slot = i;
    if (slot < 0) return fail(kCapacity, "scheduler is full [request=%lld]", (long long)req);
    ids[slot] = req, prompt_len[slot] = p_len, max_new[slot] = m_new;
    done[slot] = generated[slot] = wait_ticks[slot] = preempt_count[slot] = 0;
    state[slot] = ST_WAITING;
    return 0;
  }
  void release(int slot, bool to_cache) {
    for (int g = 0; g < G(); ++g) {
      const int64_t held = cfg.blocks(g, done[slot] + generated[slot]);
      if (to_cache) {
        const int64_t whole = cfg.blocks(g, prompt_len[slot] + max_new[slot]);
        blocks_used[g] += whole - held;
        cached_blocks[g] += whole;
      } else {
        blocks_used[g] -= held;
      }
    }
    ids[slot] = prompt_len[slot] = done[slot] = generated[slot] = max_new[slot] = wait_ticks[slot] = preempt_count[slot] = 0;
    state[slot] = ST_FREE;
  }
  bool preempt_one(Action& act, int protect) {  // the newest running request: the highest slot, never `protect`
    for (int i = cfg.n_slots - 1; i >= 0; --i) {
      if (i != protect && state[i] == ST_RUNNING && done[i] + generated[i] > 0) {
        act.preempted.push_back(ids[i]);
        for (int g = 0; g < G(); ++g) blocks_used[g] -= cfg.blocks(g, done[i] + generated[i]);
        done[i] = generated[i] = wait_ticks[i] = 0;
        ++preempt_count[i];
        ++preempt_total;
        state[i] = ST_WAITING;
        return true;
      }
    }
    return false;
  }
  int64_t try_prefill(int slot, int64_t budget, Action& act, std::vector<char>& progressed) {
    if (budget <= 0 || state[slot] != ST_WAITING || progressed[slot]) return budget;
    const int64_t chunk = std::min({cfg.max_chunk, prompt_len[slot] - done[slot], budget});
    if (chunk <= 0) return budget;
    const int64_t new_done = done[slot] + chunk;
    std::vector<int64_t> need;
    if (!growth_fits(done[slot], new_done, need, true)) return budget;  // pages ran out: this request waits for a later tick
    act.prefill.insert(act.prefill.end(), {ids[slot], done[slot], new_done});
    for (int g = 0; g < G(); ++g) blocks_used[g] += need[g];
    done[slot] = new_done;
    progressed[slot] = 1;
    wait_ticks[slot] = 0;
    return budget - chunk;
  }
  // freed: per group, cache blocks the engine gave back
  int step(const int64_t* arrivals, int n_arr, const int64_t* cancelled, int n_c, const int64_t* finished, int n_f, const int64_t* freed, Action& act) {
    const int n = cfg.n_slots;
    ++tick_seq;
    std::vector<char> progressed(n, 0);
    for (int g = 0; g < G(); ++g)  // 0
      if (freed[g] > cached_blocks[g]) return fail(kInvalidArgument, "engine freed more blocks than the scheduler holds cached");
    for (int g = 0; g < G(); ++g)
      if (freed[g] > 0) cached_blocks[g] -= freed[g], blocks_used[g] -= freed[g];
    for (int i = 0; i < n_c; ++i) {  // 1
      const int slot = find(cancelled[i]);
      if (slot >= 0) release(slot, false);
    }
    for (int i = 0; i < n_f; ++i) {  // 2
      const int slot = find(finished[i]);
      if (slot >= 0) {
        act.finished.push_back(ids[slot]);
        release(slot, true);
      }
    }
    for (int i = 0; i < n; ++i)  // 3
      if (state[i] == ST_WAITING) ++wait_ticks[i];
    std::vector<int64_t> admitted;  // 4: atomic per tick
    for (int i = 0; i < n_arr; ++i) {
      const int64_t req = arrivals[3 * i];
      if (std::find(cancelled, cancelled + n_c, req) != cancelled + n_c) continue;
      if (int e = admit(req, arrivals[3 * i + 1], arrivals[3 * i + 2])) {
        for (int64_t a : admitted) {
          const int slot = find(a);
          if (slot >= 0) release(slot, false);
        }
        return e;
      }
      admitted.push_back(req);
    }
    for (int i = 0; i < n; ++i)  // 5
      if (state[i] == ST_WAITING && done[i] >= prompt_len[i] && prompt_len[i] > 0) state[i] = ST_RUNNING, wait_ticks[i] = 0;
    int64_t budget = cfg.token_budget;
    std::vector<int64_t> need;
    for (int i = 0; i < n && budget > 0; ++i) {  // 6
      if (state[i] != ST_RUNNING) continue;
      const int64_t seq = done[i] + generated[i];
      while (!growth_fits(seq, seq + 1, need, false))
        if (!preempt_one(act, i)) return fail(kCapacity, "kv pool too small for this batch");
      for (int g = 0; g < G(); ++g) blocks_used[g] += need[g];
      ++generated[i];
      act.decode.push_back(ids[i]);
      --budget;
      if (generated[i] >= max_new[i]) {
        act.finished.push_back(ids[i]);
        release(i, true);
      }
    }
    for (int i = 0; i < n; ++i)  // 7
      if (state[i] == ST_WAITING && wait_ticks[i] >= cfg.max_wait_ticks) budget = try_prefill(i, budget, act, progressed);
    for (int i = 0; i < n; ++i)  // 8
      if (state[i] == ST_WAITING) budget = try_prefill(i, budget, act, progressed);
    while (over_watermark())  // 9
      if (!preempt_one(act, -1)) break;
    return 0;
  }
};

int copy_out(const std::vector<int64_t>& v, int64_t* out, int cap) {
  if (static_cast<int>(v.size()) > cap) return fail(kCapacity, "output buffer too small [need=%d cap=%d]", (int)v.size(), cap);
  std::copy(v.begin(), v.end(), out);
  return static_cast<int>(v.size());
}

}  // namespace

extern "C" {

const char* alofa_host_last_error() { return g_error; }

// ---- pool
void* alofa_pool_new(int n) { return n > 0 ? new Pool(n) : nullptr; }
void alofa_pool_free(void* p) { delete static_cast<Pool*>(p); }
int alofa_pool_alloc_one(void* p) { return static_cast<Pool*>(p)->alloc_one(); }
int alofa_pool_retain(void* p, int b) { return static_cast<Pool*>(p)->retain(b); }
int alofa_pool_release(void* p, int b) { return static_cast<Pool*>(p)->release(b); }
int alofa_pool_refcnt_of(void* p, int b) {
  Pool* pool = static_cast<Pool*>(p);
  if (b < 0 || b >= pool->n_blocks) return fail(kOutOfRange, "block id is outside the pool [block=%d n_blocks=%d]", b, pool->n_blocks);
  return pool->refcnt[b];
}
int alofa_pool_n_free(void* p) { return static_cast<Pool*>(p)->n_free(); }
int alofa_pool_high_water(void* p) { return static_cast<Pool*>(p)->high_water; }
int alofa_pool_n_blocks(void* p) { return static_cast<Pool*>(p)->n_blocks; }

// ---- cache
// n_blocks: the pages of every group's own pool
void* alofa_cache_new(int n_groups, const int64_t* windows, const int64_t* n_blocks, int block_size, int max_requests) {
  if (n_groups < 0 || block_size <= 0 || max_requests <= 0) return nullptr;
  for (int g = 0; g < n_groups; ++g)
    if (n_blocks[g] <= 0 || n_blocks[g] > INT32_MAX) return nullptr;
  Cache* c = new Cache{block_size, max_requests, {}, {}, {}};
  for (int g = 0; g < n_groups; ++g) c->groups.push_back(Group{windows[g], Pool(static_cast<int>(n_blocks[g]))});
  c->reqs.resize(max_requests);
  for (int s = max_requests - 1; s >= 0; --s) c->free_slots.push_back(s);
  return c;
}
void alofa_cache_free(void* c) { delete static_cast<Cache*>(c); }
void* alofa_cache_pool(void* c, int g) { return &static_cast<Cache*>(c)->groups[g].pool; }
int alofa_cache_admit(void* cv) {  // takes the lowest free request slot
  Cache* c = static_cast<Cache*>(cv);
  if (c->free_slots.empty()) return fail(kCapacity, "no request slot is free [max_requests=%d]", c->max_requests);
  const int slot = c->free_slots.back();
  c->free_slots.pop_back();
  Request& r = c->reqs[slot];
  r.live = true;
  r.length = 0;
  r.tables.assign(c->groups.size(), {});
  r.first_held.assign(c->groups.size(), 0);
  return slot;
}
int alofa_cache_drop(void* cv, int slot) {  // the request ends: every page and its slot are given back
  Cache* c = static_cast<Cache*>(cv);
  Request* r = c->get(slot);
  if (!r) return -kInvalidArgument;
  for (size_t g = 0; g < c->groups.size(); ++g)
    for (int page : r->tables[g])
      if (page >= 0) c->groups[g].pool.release(page);
  r->live = false;
  r->tables.clear();
  c->free_slots.push_back(slot);
  return 0;
}
int64_t alofa_cache_length(void* cv, int slot) {
  Request* r = static_cast<Cache*>(cv)->get(slot);
  return r ? r->length : -kInvalidArgument;
}
int alofa_cache_blocks_needed(void* cv, int slot, int64_t target, int* out) {
  Cache* c = static_cast<Cache*>(cv);
  Request* r = c->get(slot);
  if (!r) return -kInvalidArgument;
  for (size_t g = 0; g < c->groups.size(); ++g) out[g] = c->needed(*r, g, target);
  return 0;
}
int alofa_cache_reserve(void* cv, int slot, int64_t target) { return static_cast<Cache*>(cv)->reserve(slot, target); }
// freed: [n_groups][cap] pages given back; counts[g] how many
int alofa_cache_commit(void* cv, int slot, int64_t target, int* freed, int cap, int* counts) {
  Cache* c = static_cast<Cache*>(cv);
  std::vector<std::vector<int>> got(c->groups.size());
  if (int e = c->commit(slot, target, &got)) return e;
  for (size_t g = 0; g < got.size(); ++g) {
    counts[g] = static_cast<int>(got[g].size());
    if (counts[g] > cap) return fail(kCapacity, "output buffer too small");
    std::copy(got[g].begin(), got[g].end(), freed + g * cap);
  }
  return 0;
}
int alofa_cache_share_prefix(void* cv, int src, int dst, int64_t n_tokens) {
  Cache* c = static_cast<Cache*>(cv);
  Request *s = c->get(src), *d = c->get(dst);
  if (!s || !d) return -kInvalidArgument;
  bool empty = d->length == 0;
  for (auto& t : d->tables) empty &= t.empty();
  if (!empty) return fail(kInvalidArgument, "only an empty request can take a shared prefix [slot=%d]", dst);
  for (auto& g : c->groups)
    if (g.window >= 0) return 0;  // only groups that keep every key can share
  const int n_blocks = static_cast<int>(std::min(n_tokens, s->length) / c->block_size);
  for (size_t g = 0; g < c->groups.size(); ++g)
    for (int b = 0; b < n_blocks; ++b) {
      c->groups[g].pool.retain(s->tables[g][b]);
      d->tables[g].push_back(s->tables[g][b]);
    }
  d->length = static_cast<int64_t>(n_blocks) * c->block_size;
  return static_cast<int>(d->length);
}
int alofa_cache_table(void* cv, int slot, int g, int* out, int cap) {
  Cache* c = static_cast<Cache*>(cv);
  Request* r = c->get(slot);
  if (!r) return -kInvalidArgument;
  const auto& t = r->tables[g];
  if (static_cast<int>(t.size()) > cap) return fail(kCapacity, "output buffer too small");
  std::copy(t.begin(), t.end(), out);
  return static_cast<int>(t.size());
}
int alofa_cache_table_len(void* cv, int slot, int g) {
  Request* r = static_cast<Cache*>(cv)->get(slot);
  return r ? static_cast<int>(r->tables[g].size()) : -kInvalidArgument;
}
int alofa_cache_slots(void* cv, int slot, int g, int64_t start, int n, int64_t* out) {
  Cache* c = static_cast<Cache*>(cv);
  Request* r = c->get(slot);
  if (!r) return -kInvalidArgument;
  const auto& t = r->tables[g];
  for (int i = 0; i < n; ++i) {
    const int64_t p = start + i, b = p / c->block_size;
    const int page = b < static_cast<int64_t>(t.size()) ? t[b] : -1;
    if (page < 0) return fail(kCapacity, "no page is held for this position [slot=%d group=%d position=%lld]", slot, g, (long long)p);
    out[i] = static_cast<int64_t>(page) * c->block_size + p % c->block_size;
  }
  return 0;
}
int alofa_cache_max_blocks(void* cv) {
  Cache* c = static_cast<Cache*>(cv);
  size_t m = 0;
  for (auto& r : c->reqs)
    if (r.live)
      for (auto& t : r.tables) m = std::max(m, t.size());
  return static_cast<int>(m);
}
int alofa_cache_n_free_slots(void* cv) { return static_cast<int>(static_cast<Cache*>(cv)->free_slots.size()); }
// no page lost, held twice without a count, or freed twice; slots neither lost nor held twice
int alofa_cache_check(void* cv) {
  Cache* c = static_cast<Cache*>(cv);
  for (size_t g = 0; g < c->groups.size(); ++g) {
    Pool& pool = c->groups[g].pool;
    std::vector<int> counts(pool.n_blocks, 0);
    for (auto& r : c->reqs)
      if (r.live)
        for (int page : r.tables[g])
          if (page >= 0) ++counts[page];
    if (counts != pool.refcnt) return fail(kInvalidArgument, "tables and pool disagree on who holds which page [group=%d]", (int)g);
    std::vector<char> on_stack(pool.n_blocks, 0);
    for (int b : pool.free_stack) {
      if (on_stack[b] || pool.refcnt[b] != 0) return fail(kDoubleFree, "a page is on the free stack twice or while held [group=%d]", (int)g);
      on_stack[b] = 1;
    }
    int held = 0;
    for (int x : counts) held += x > 0;
    if (pool.n_free() + held != pool.n_blocks) return fail(kInvalidArgument, "a page is neither free nor held [group=%d]", (int)g);
  }
  int live = 0;
  std::vector<char> seen(c->max_requests, 0);
  for (int s : c->free_slots) {
    if (seen[s] || c->reqs[s].live) return fail(kInvalidArgument, "request slots are lost or held twice");
    seen[s] = 1;
  }
  for (auto& r : c->reqs) live += r.live;
  if (live + static_cast<int>(c->free_slots.size()) != c->max_requests) return fail(kInvalidArgument, "request slots are lost or held twice");
  return 0;
}

// Longest table (in blocks) that a step with these entries will need.
int alofa_cache_step_width(void* cv, int n_entries, const int* slots, const int* n_tokens) {
  Cache* c = static_cast<Cache*>(cv);
  int64_t w = 1;
  for (int i = 0; i < n_entries; ++i) {
    Request* r = c->get(slots[i]);
    if (!r) return -kInvalidArgument;
    w = std::max(w, blocks_for(r->length + n_tokens[i], c->block_size));
    for (auto& t : r->tables) w = std::max<int64_t>(w, t.size());
  }
  return static_cast<int>(w);
}

// The layout of one step. Entry i brings n_tokens[i] tokens of the request in slots[i]. Either every
// entry gets its pages or nothing is changed (capacity error). Filled: pos0[i]; per row its position,
// entry index; per group the entries' tables ([entry][width], -1 padded; width >= the longest) and the
// rows' cache slots. Returns the number of rows.
int alofa_cache_plan_step(void* cv, int n_entries, const int* slots, const int* n_tokens, int64_t max_positions, int width,
                          int64_t* pos0, int* positions, int* req_of_token, int* tables, int64_t* row_slots, int64_t total_rows) {
  Cache* c = static_cast<Cache*>(cv);
  const int G = static_cast<int>(c->groups.size());
  std::vector<int> need(G, 0);
  int64_t rows = 0;
  for (int i = 0; i < n_entries; ++i) {
    Request* r = c->get(slots[i]);
    if (!r) return -kInvalidArgument;
    if (n_tokens[i] <= 0) return fail(kInvalidArgument, "an entry brings no tokens [entry=%d]", i);
    for (int j = 0; j < i; ++j)
      if (slots[j] == slots[i]) return fail(kInvalidArgument, "a request appears twice in one step [slot=%d]", slots[i]);
    if (r->length + n_tokens[i] > max_positions)
      return fail(kCapacity, "the request would pass the context bound [slot=%d length=%lld bound=%lld]", slots[i], (long long)(r->length + n_tokens[i]), (long long)max_positions);
    for (int g = 0; g < G; ++g) {
      need[g] += c->needed(*r, g, r->length + n_tokens[i]);
      const int64_t wide = std::max<int64_t>(blocks_for(r->length + n_tokens[i], c->block_size), r->tables[g].size());
      if (wide > width) return fail(kCapacity, "table is wider than the buffer [width=%d need=%d]", width, (int)wide);
      // pages held already for positions this step writes (reserved earlier, or the tail of the last one) must still be there
      const int64_t last = std::min<int64_t>(blocks_for(r->length + n_tokens[i], c->block_size), r->tables[g].size());
      for (int64_t b = r->length / c->block_size; b < last; ++b)
        if (r->tables[g][b] < 0)
          return fail(kCapacity, "no page is held for this position [slot=%d group=%d position=%lld]", slots[i], g, (long long)std::max<int64_t>(r->length, b * c->block_size));
    }
    rows += n_tokens[i];
  }
  if (rows != total_rows) return fail(kInvalidArgument, "row count does not fit the buffers [rows=%lld buffers=%lld]", (long long)rows, (long long)total_rows);
  for (int g = 0; g < G; ++g)
    if (need[g] > c->groups[g].pool.n_free()) return fail(kCapacity, "kv block pool is exhausted [group=%d need=%d free=%d]", g, need[g], c->groups[g].pool.n_free());
  int64_t row = 0;
  for (int i = 0; i < n_entries; ++i) {
    Request& r = c->reqs[slots[i]];
    c->reserve(slots[i], r.length + n_tokens[i]);
    pos0[i] = r.length;
    for (int g = 0; g < G; ++g) {
      const auto& t = r.tables[g];  // (no wider than the buffer: checked above, before anything was taken)
      int* dst = tables + (static_cast<int64_t>(g) * n_entries + i) * width;
      std::copy(t.begin(), t.end(), dst);
      std::fill(dst + t.size(), dst + width, -1);
    }
    for (int k = 0; k < n_tokens[i]; ++k, ++row) {
      const int64_t p = r.length + k;
      positions[row] = static_cast<int>(p);
      req_of_token[row] = i;
      for (int g = 0; g < G; ++g) {
        const int page = r.tables[g][p / c->block_size];  // (held: checked above, or taken just now)
        row_slots[static_cast<int64_t>(g) * total_rows + row] = static_cast<int64_t>(page) * c->block_size + p % c->block_size;
      }
    }
  }
  return static_cast<int>(rows);
}
// The step's tokens are written: lengths advance, pages a window has passed go back.
int alofa_cache_commit_step(void* cv, int n_entries, const int* slots, const int* n_tokens) {
  Cache* c = static_cast<Cache*>(cv);
  for (int i = 0; i < n_entries; ++i) {
    Request* r = c->get(slots[i]);
    if (!r) return -kInvalidArgument;
    if (int e = c->commit(slots[i], r->length + n_tokens[i], nullptr)) return e;
  }
  return 0;
}

// ---- scheduler
// cfg: see config_from
void* alofa_sched_new(const int64_t* cfg) {
  if (cfg[8] < 0) return nullptr;
  return new Sched(config_from(cfg));
}
void alofa_sched_free(void* s) { delete static_cast<Sched*>(s); }
// a new configuration for the next ticks (neither the slot count nor the number of groups can change)
int alofa_sched_set_config(void* sv, const int64_t* cfg) {
  Sched* s = static_cast<Sched*>(sv);
  if (cfg[6] != s->cfg.n_slots) return fail(kInvalidArgument, "the slot count of a scheduler cannot change");
  if (cfg[8] + 1 != s->G()) return fail(kInvalidArgument, "the number of groups of a scheduler cannot change");
  s->cfg = config_from(cfg);
  return 0;
}
// freed: per group, the cache blocks the engine gave back.
// out: prefill triples, then decode, preempted, finished ids, each at offset k * cap of `out` (4 * cap long);
// counts[4]; scalars: tick_seq, preempt_total, state_digest
int alofa_sched_step(void* sv, const int64_t* arrivals, int n_arr, const int64_t* cancelled, int n_c, const int64_t* finished, int n_f,
                     const int64_t* freed, int64_t* out, int cap, int* counts, int64_t* scalars) {
  Sched* s = static_cast<Sched*>(sv);
  Action act;
  if (int e = s->step(arrivals, n_arr, cancelled, n_c, finished, n_f, freed, act)) return e;
  const std::vector<int64_t>* lists[4] = {&act.prefill, &act.decode, &act.preempted, &act.finished};
  for (int k = 0; k < 4; ++k) {
    const int n = copy_out(*lists[k], out + static_cast<int64_t>(k) * cap, cap);
    if (n < 0) return n;
    counts[k] = n;
  }
  scalars[0] = s->tick_seq, scalars[1] = s->preempt_total, scalars[2] = s->digest();
  return 0;
}
int alofa_sched_find(void* s, int64_t req) { return static_cast<Sched*>(s)->find(req); }
int alofa_sched_would_admit(void* sv, int64_t p_len, int64_t m_new, const int64_t* pending, int n_pending) {
  Sched* s = static_cast<Sched*>(sv);
  const SchedConfig& c = s->cfg;
  if (p_len <= 0 || m_new <= 0) return 0;
  for (int g = 0; g < s->G(); ++g) {
    if (c.blocks(g, p_len) > c.groups[g].capacity) return 0;
    int64_t committed = s->committed(g);
    for (int i = 0; i < n_pending; ++i) committed += c.blocks(g, pending[2 * i] + pending[2 * i + 1]);
    if (committed + c.blocks(g, p_len + m_new) > c.threshold(g)) return 0;
  }
  return s->n_live() + n_pending < c.n_slots;
}
// which: 0 ids, 1 prompt_len, 2 done, 3 generated, 4 max_new, 5 state, 6 wait_ticks, 7 preempt_count
int alofa_sched_slots(void* sv, int which, int64_t* out) {
  Sched* s = static_cast<Sched*>(sv);
  const std::vector<int64_t>* v[8] = {&s->ids, &s->prompt_len, &s->done, &s->generated, &s->max_new, &s->state, &s->wait_ticks, &s->preempt_count};
  if (which < 0 || which > 7) return fail(kOutOfRange, "no such per-slot field [which=%d]", which);
  std::copy(v[which]->begin(), v[which]->end(), out);
  return 0;
}
// which: 0 blocks_used, 1 cached_blocks, 2 preempt_total, 3 tick_seq, 4 blocks_held, 5 blocks_wanted, 6 digest, 7 n_live;
// the counts of pages are those of group `g`
int64_t alofa_sched_scalar_of(void* sv, int which, int g) {
  Sched* s = static_cast<Sched*>(sv);
  if (g < 0 || g >= s->G()) return fail(kOutOfRange, "no such group [group=%d]", g);
  switch (which) {
    case 0: return s->blocks_used[g];
    case 1: return s->cached_blocks[g];
    case 2: return s->preempt_total;
    case 3: return s->tick_seq;
    case 4: return s->blocks_held(g);
    case 5: return s->blocks_wanted(g);
    case 6: return s->digest();
    case 7: return s->n_live();
  }
  return fail(kOutOfRange, "no such scalar [which=%d]", which);
}
int64_t alofa_sched_scalar(void* sv, int which) { return alofa_sched_scalar_of(sv, which, 0); }

}  // extern "C"
