// Host-side bookkeeping of the paged cache: page pools, block tables per request slot, groups
// of layers with different needs, window release.  No device code; the tables live in host
// memory that Python views directly (numpy) and copies to the device when a step needs them.
//
// Reference: src/runtime/block_manager.cpp:14-141 (LIFO free list, allocated bitmap, all-or-
// nothing allocation, double-free checks), src/runtime/kv_cache_manager.cpp and
// src/runtime/block_table.cpp (one block id list per sequence).  Ours: several groups, pages on
// demand, pages given back when a window has passed them, one slot per live request.
//
// Every call returns a status: 0 ok, 1 out of pages (nothing was changed), 2 misuse (nothing
// was changed); pi_cache_error() has the text of the last failure on that handle.
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

namespace {

enum { OK = 0, OUT_OF_PAGES = 1, MISUSE = 2 };

struct Pool {
  int num_pages = 0;
  std::vector<int> free_list;          // back() is handed out next; starts so that page 0 goes first
  std::vector<uint8_t> allocated;
  std::string error;

  void reset() {
    free_list.resize(num_pages);
    for (int i = 0; i < num_pages; ++i) free_list[i] = num_pages - 1 - i;
    allocated.assign(num_pages, 0);
  }
  int num_free() const { return (int)free_list.size(); }
  int take() {
    const int p = free_list.back();
    free_list.pop_back();
    allocated[p] = 1;
    return p;
  }
};

std::string format(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  return buf;
}

// Check all pages before changing anything: ids in range, allocated, none named twice.
int pool_free(Pool& pool, const int* pages, int n, std::string& error) {
  int bad = -1;
  bool outside = false;
  for (int i = 0; i < n && bad < 0; ++i) {
    const int p = pages[i];
    if (p < 0 || p >= pool.num_pages) { bad = i; outside = true; }
    else if (pool.allocated[p] != 1) bad = i;      // free already, or seen earlier in this call
    else pool.allocated[p] = 2;                    // seen in this call
  }
  if (bad >= 0) {
    for (int i = 0; i < bad; ++i) pool.allocated[pages[i]] = 1;
    error = outside ? format("page id %d is outside the pool of %d", pages[bad], pool.num_pages)
                    : format("page %d is freed twice", pages[bad]);
    return MISUSE;
  }
  for (int i = 0; i < n; ++i) {
    pool.allocated[pages[i]] = 0;
    pool.free_list.push_back(pages[i]);
  }
  return OK;
}

struct Group {
  int window = -1;                     // -1: keep every key
  Pool pool;
  std::vector<int32_t> table;          // [max_slots][max_blocks], -1 = no page
  std::vector<int32_t> next_block;     // [max_slots] blocks ever handed out (index of the next one)
  std::vector<int32_t> first_block;    // [max_slots] first block still held
};

struct Cache {
  int page_size = 0, max_slots = 0, max_model_len = 0, max_blocks = 0;
  std::vector<Group> groups;
  std::vector<int32_t> length;         // [max_slots] tokens whose keys are in the cache
  std::vector<int32_t> reserved;       // [max_slots] tokens that pages are held for
  std::vector<uint8_t> live;           // [max_slots]
  std::vector<int> free_slots;
  std::string error;

  int32_t* row(Group& g, int slot) { return g.table.data() + (size_t)slot * max_blocks; }
  bool is_live(int slot) const { return slot >= 0 && slot < max_slots && live[slot]; }
  int blocks_for(int tokens) const { return (tokens + page_size - 1) / page_size; }
  int needed(const Group& g, int slot, int new_tokens) const {
    const int target = (slot >= 0 ? length[slot] : 0) + new_tokens;
    const int have = slot >= 0 ? g.next_block[slot] : 0;
    const int more = blocks_for(target) - have;
    return more > 0 ? more : 0;
  }
};

}  // namespace

extern "C" {

// ---------------------------------------------------------------- a pool on its own
void* pi_pool_create(int num_pages) {
  if (num_pages <= 0) return nullptr;
  Pool* p = new Pool;
  p->num_pages = num_pages;
  p->reset();
  return p;
}
void pi_pool_destroy(void* h) { delete static_cast<Pool*>(h); }
const char* pi_pool_error(void* h) { return static_cast<Pool*>(h)->error.c_str(); }
int pi_pool_num_free(void* h) { return static_cast<Pool*>(h)->num_free(); }
int pi_pool_is_allocated(void* h, int page) {
  Pool* p = static_cast<Pool*>(h);
  return page >= 0 && page < p->num_pages && p->allocated[page];
}
int pi_pool_allocate(void* h, int n, int* out) {
  Pool* p = static_cast<Pool*>(h);
  if (n < 0) { p->error = format("cannot allocate %d pages", n); return MISUSE; }
  if (n > p->num_free()) {
    p->error = format("%d pages asked for, %d of %d free", n, p->num_free(), p->num_pages);
    return OUT_OF_PAGES;
  }
  for (int i = 0; i < n; ++i) out[i] = p->take();
  return OK;
}
int pi_pool_free(void* h, const int* pages, int n) {
  Pool* p = static_cast<Pool*>(h);
  return pool_free(*p, pages, n, p->error);
}
void pi_pool_reset(void* h) { static_cast<Pool*>(h)->reset(); }

// ---------------------------------------------------------------- the cache manager
void* pi_cache_create(int n_groups, const int* windows, int page_size, const int* num_pages, int max_slots, int max_model_len) {
  if (n_groups < 0 || page_size <= 0 || max_slots <= 0 || max_model_len <= 0) return nullptr;
  for (int g = 0; g < n_groups; ++g)
    if (num_pages[g] <= 0) return nullptr;
  Cache* c = new Cache;
  c->page_size = page_size;
  c->max_slots = max_slots;
  c->max_model_len = max_model_len;
  c->max_blocks = (max_model_len + page_size - 1) / page_size;
  c->groups.resize(n_groups);
  for (int g = 0; g < n_groups; ++g) {
    Group& grp = c->groups[g];
    grp.window = windows[g];
    grp.pool.num_pages = num_pages[g];
    grp.pool.reset();
    grp.table.assign((size_t)max_slots * c->max_blocks, -1);
    grp.next_block.assign(max_slots, 0);
    grp.first_block.assign(max_slots, 0);
  }
  c->length.assign(max_slots, 0);
  c->reserved.assign(max_slots, 0);
  c->live.assign(max_slots, 0);
  c->free_slots.resize(max_slots);
  for (int i = 0; i < max_slots; ++i) c->free_slots[i] = max_slots - 1 - i;   // slot 0 goes first
  return c;
}
void pi_cache_destroy(void* h) { delete static_cast<Cache*>(h); }
const char* pi_cache_error(void* h) { return static_cast<Cache*>(h)->error.c_str(); }
int pi_cache_max_blocks(void* h) { return static_cast<Cache*>(h)->max_blocks; }
int32_t* pi_cache_table(void* h, int g) { return static_cast<Cache*>(h)->groups[g].table.data(); }
int32_t* pi_cache_next_block(void* h, int g) { return static_cast<Cache*>(h)->groups[g].next_block.data(); }
int32_t* pi_cache_first_block(void* h, int g) { return static_cast<Cache*>(h)->groups[g].first_block.data(); }
int32_t* pi_cache_lengths(void* h) { return static_cast<Cache*>(h)->length.data(); }
int pi_cache_free_slots(void* h) { return (int)static_cast<Cache*>(h)->free_slots.size(); }
int pi_cache_free_pages(void* h, int g) { return static_cast<Cache*>(h)->groups[g].pool.num_free(); }
int pi_cache_page_allocated(void* h, int g, int page) {
  const Pool& p = static_cast<Cache*>(h)->groups[g].pool;
  return page >= 0 && page < p.num_pages && p.allocated[page];
}

int pi_cache_admit(void* h) {
  Cache* c = static_cast<Cache*>(h);
  if (c->free_slots.empty()) {
    c->error = format("no free slot: %d requests are live", c->max_slots);
    return -1;
  }
  const int slot = c->free_slots.back();
  c->free_slots.pop_back();
  c->live[slot] = 1;
  c->length[slot] = 0;
  c->reserved[slot] = 0;
  return slot;
}

// Pages each group must still hand out for the slot (-1: a request not admitted yet) to grow.
int pi_cache_pages_needed(void* h, int slot, int new_tokens, int* out) {
  Cache* c = static_cast<Cache*>(h);
  if (slot >= 0 && !c->is_live(slot)) { c->error = format("slot %d is not live in the cache", slot); return MISUSE; }
  for (size_t g = 0; g < c->groups.size(); ++g) out[g] = c->needed(c->groups[g], slot, new_tokens);
  return OK;
}

// Whether reserve would succeed; held_back[g] pages of group g count as taken (may be null).
int pi_cache_can_reserve(void* h, int slot, int new_tokens, const int* held_back) {
  Cache* c = static_cast<Cache*>(h);
  if (slot >= 0 && !c->is_live(slot)) return 0;
  for (size_t g = 0; g < c->groups.size(); ++g)
    if (c->needed(c->groups[g], slot, new_tokens) > c->groups[g].pool.num_free() - (held_back ? held_back[g] : 0)) return 0;
  return 1;
}

// Hold pages for positions length .. length + new_tokens - 1 in every group, all or nothing.
int pi_cache_reserve(void* h, int slot, int new_tokens) {
  Cache* c = static_cast<Cache*>(h);
  if (!c->is_live(slot)) { c->error = format("slot %d is not live in the cache", slot); return MISUSE; }
  if (new_tokens < 0) { c->error = format("cannot reserve %d tokens", new_tokens); return MISUSE; }
  const int target = c->length[slot] + new_tokens;
  if (target > c->max_model_len) {
    c->error = format("would hold %d tokens; the limit is %d", target, c->max_model_len);
    return MISUSE;
  }
  for (size_t g = 0; g < c->groups.size(); ++g) {
    const int n = c->needed(c->groups[g], slot, new_tokens);
    if (n > c->groups[g].pool.num_free()) {
      c->error = format("needs %d more pages in cache group %d, %d are free", n, (int)g, c->groups[g].pool.num_free());
      return OUT_OF_PAGES;
    }
  }
  for (Group& grp : c->groups) {
    const int n = c->needed(grp, slot, new_tokens);
    int32_t* row = c->row(grp, slot);
    for (int i = 0; i < n; ++i) row[grp.next_block[slot]++] = grp.pool.take();
  }
  if (target > c->reserved[slot]) c->reserved[slot] = target;
  return OK;
}

// The step wrote new_tokens more keys: advance the length, give back what every window has passed.
int pi_cache_commit(void* h, int slot, int new_tokens) {
  Cache* c = static_cast<Cache*>(h);
  if (!c->is_live(slot)) { c->error = format("slot %d is not live in the cache", slot); return MISUSE; }
  if (c->length[slot] + new_tokens > c->reserved[slot]) {
    c->error = format("committing to %d tokens but pages are held for %d", c->length[slot] + new_tokens, c->reserved[slot]);
    return MISUSE;
  }
  c->length[slot] += new_tokens;
  for (Group& grp : c->groups) {
    if (grp.window < 0) continue;
    // the next query sits at position >= length and reads keys >= length - window + 1
    int first_key = c->length[slot] - grp.window + 1;
    if (first_key < 0) first_key = 0;
    const int lo = grp.first_block[slot];
    int hi = first_key / c->page_size;
    if (hi > grp.next_block[slot]) hi = grp.next_block[slot];
    if (hi > lo) {
      int32_t* row = c->row(grp, slot);
      const int st = pool_free(grp.pool, row + lo, hi - lo, c->error);
      if (st != OK) return st;
      for (int b = lo; b < hi; ++b) row[b] = -1;
      grp.first_block[slot] = hi;
    }
  }
  return OK;
}

// The request ended (or was preempted): give back its pages and its slot.
int pi_cache_release(void* h, int slot) {
  Cache* c = static_cast<Cache*>(h);
  if (!c->is_live(slot)) { c->error = format("slot %d is not live in the cache", slot); return MISUSE; }
  for (Group& grp : c->groups) {
    int32_t* row = c->row(grp, slot);
    const int lo = grp.first_block[slot], hi = grp.next_block[slot];
    if (hi > lo) {
      const int st = pool_free(grp.pool, row + lo, hi - lo, c->error);
      if (st != OK) return st;
    }
    for (int b = 0; b < c->max_blocks; ++b) row[b] = -1;
    grp.next_block[slot] = 0;
    grp.first_block[slot] = 0;
  }
  c->live[slot] = 0;
  c->length[slot] = 0;
  c->reserved[slot] = 0;
  c->free_slots.push_back(slot);
  return OK;
}

// Pages each group must hand out for a whole step: every slot growing by its number of tokens.
int pi_cache_pages_needed_many(void* h, const int* slots, const int* new_tokens, int n, int* out) {
  Cache* c = static_cast<Cache*>(h);
  for (size_t g = 0; g < c->groups.size(); ++g) out[g] = 0;
  for (int i = 0; i < n; ++i) {
    if (!c->is_live(slots[i])) { c->error = format("slot %d is not live in the cache", slots[i]); return MISUSE; }
    for (size_t g = 0; g < c->groups.size(); ++g) out[g] += c->needed(c->groups[g], slots[i], new_tokens[i]);
  }
  return OK;
}

// A whole step at once: check that everything fits (nothing is taken otherwise), then reserve.
int pi_cache_reserve_many(void* h, const int* slots, const int* new_tokens, int n) {
  Cache* c = static_cast<Cache*>(h);
  std::vector<int> want(c->groups.size(), 0);
  for (int i = 0; i < n; ++i) {
    if (!c->is_live(slots[i])) { c->error = format("slot %d is not live in the cache", slots[i]); return MISUSE; }
    if (new_tokens[i] < 0 || c->length[slots[i]] + new_tokens[i] > c->max_model_len) {
      c->error = format("slot %d would hold %d tokens; the limit is %d", slots[i], c->length[slots[i]] + new_tokens[i], c->max_model_len);
      return MISUSE;
    }
    for (size_t g = 0; g < c->groups.size(); ++g) want[g] += c->needed(c->groups[g], slots[i], new_tokens[i]);
  }
  for (size_t g = 0; g < c->groups.size(); ++g)
    if (want[g] > c->groups[g].pool.num_free()) {
      c->error = format("the step needs %d more pages in cache group %d, %d are free", want[g], (int)g, c->groups[g].pool.num_free());
      return OUT_OF_PAGES;
    }
  for (int i = 0; i < n; ++i) {
    const int st = pi_cache_reserve(h, slots[i], new_tokens[i]);
    if (st != OK) return st;
  }
  return OK;
}

int pi_cache_commit_many(void* h, const int* slots, const int* new_tokens, int n) {
  for (int i = 0; i < n; ++i) {
    const int st = pi_cache_commit(h, slots[i], new_tokens[i]);
    if (st != OK) return st;
  }
  return OK;
}

// No page lost, none held twice: every allocated page appears exactly once in the tables of
// live slots, every page in a table is allocated, free slots hold nothing.
int pi_cache_check(void* h) {
  Cache* c = static_cast<Cache*>(h);
  int live = 0;
  for (int s = 0; s < c->max_slots; ++s) live += c->live[s] ? 1 : 0;
  if (live + (int)c->free_slots.size() != c->max_slots) { c->error = "a slot was lost"; return MISUSE; }
  for (int s : c->free_slots)
    if (s < 0 || s >= c->max_slots || c->live[s]) { c->error = "slot bookkeeping is inconsistent"; return MISUSE; }
  for (size_t gi = 0; gi < c->groups.size(); ++gi) {
    Group& grp = c->groups[gi];
    std::vector<uint8_t> seen(grp.pool.num_pages, 0);
    int held = 0;
    for (int s = 0; s < c->max_slots; ++s) {
      const int32_t* row = c->row(grp, s);
      int pages = 0;
      for (int b = 0; b < c->max_blocks; ++b) {
        const int p = row[b];
        if (p < 0) continue;
        ++pages;
        if (b < grp.first_block[s] || b >= grp.next_block[s]) {
          c->error = format("group %d: slot %d table does not match its block range", (int)gi, s);
          return MISUSE;
        }
        if (p >= grp.pool.num_pages || !grp.pool.allocated[p]) {
          c->error = format("group %d: %d pages allocated but a table names a free one", (int)gi, grp.pool.num_pages - grp.pool.num_free());
          return MISUSE;
        }
        if (seen[p]) { c->error = format("group %d: a page is held twice", (int)gi); return MISUSE; }
        seen[p] = 1;
      }
      if (!c->live[s] && pages) { c->error = format("group %d: free slot %d still holds pages", (int)gi, s); return MISUSE; }
      if (pages != grp.next_block[s] - grp.first_block[s]) {
        c->error = format("group %d: slot %d table does not match its block range", (int)gi, s);
        return MISUSE;
      }
      held += pages;
    }
    if (held != grp.pool.num_pages - grp.pool.num_free()) {
      c->error = format("group %d: %d pages allocated but %d in tables", (int)gi, grp.pool.num_pages - grp.pool.num_free(), held);
      return MISUSE;
    }
  }
  return OK;
}

}  // extern "C"
