// The cache manager's bookkeeping on the host: which pages of each group's pool are free, which
// request holds which, the block table of every request in every group, the slots of
// per-request state, and the block tables and slot mappings of a step, packed for the device.
// Pure host code: it never touches a device; the pools themselves are tensors of the caller's.
//
// The reference keeps one contiguous buffer per request and layer, sized at creation
// (src/model/runtime/optimized_kv_cache/cache.zig:21-107,350-404), and recycles it with reset()
// (:109-111); its error.CacheFull (:96) is kept as the error of a pool that has run out.
// Paging, groups, windows that give pages back and slots are this engine's own.
//
// Every function returns 0, or 1 (a pool or the slots have run out: CacheFull) or 2 (a call
// that does not fit the state: a request that is not live, a page freed twice) with a text for
// the caller's exception in zc_last_error(); nothing has changed then.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace {

constexpr int NO_PAGE = -1;
enum { OK = 0, FULL = 1, BAD = 2 };

thread_local std::string last_error;

int fail(int code, const std::string& text) {
  last_error = text;
  return code;
}

// Pages 0 .. num_pages - 1 with a last-in-first-out free list, so that a page given back is the
// next one handed out (reuse happens early, which is what tests with few pages need).  Handing
// out is all-or-nothing; a page is never held twice nor freed twice.
struct PagePool {
  int num_pages = 0;
  std::vector<int> free_list;
  std::vector<uint8_t> held;
  long long handed_out = 0;      // pages handed out over the pool's life
  int high_water = 0;

  explicit PagePool(int n) : num_pages(n), held((size_t)n, 0) {
    free_list.reserve((size_t)n);
    for (int p = n - 1; p >= 0; --p) free_list.push_back(p);
  }
  int num_free() const { return (int)free_list.size(); }
  int num_held() const { return num_pages - num_free(); }
  int take() {      // (the caller has checked that one is free)
    const int p = free_list.back();
    free_list.pop_back();
    held[(size_t)p] = 1;
    ++handed_out;
    high_water = std::max(high_water, num_held());
    return p;
  }
  bool give(int p) {
    if (p < 0 || p >= num_pages || !held[(size_t)p]) return false;
    held[(size_t)p] = 0;
    free_list.push_back(p);
    return true;
  }
  bool consistent(std::string* why) const {
    std::unordered_set<int> seen;
    for (int p : free_list) {
      if (!seen.insert(p).second) { *why = "a page is on the free list twice"; return false; }
      if (held[(size_t)p]) { *why = "page " + std::to_string(p) + " is free and held"; return false; }
    }
    long long h = 0;
    for (uint8_t x : held) h += x;
    if (h + (long long)free_list.size() != num_pages) { *why = "a page was lost"; return false; }
    return true;
  }
};

struct Request {
  int length = 0;
  int slot = 0;
  std::vector<std::vector<int>> tables;      // per group: logical page -> page of the pool
};

struct Group {
  int window;      // -1: every key is kept
  PagePool pages;
  std::vector<int> freed;      // what the last call gave back, in the order it was freed
  Group(int w, int n) : window(w), pages(n) {}
};

struct Core {
  int page_size;
  int max_requests;
  std::vector<Group> groups;
  PagePool slots;
  std::unordered_map<long long, Request> requests;

  Core(int ps, int max_req) : page_size(ps), max_requests(max_req), slots(max_req) {}

  int pages_for(int tokens) const { return (tokens + page_size - 1) / page_size; }
  // logical index of the first page a query at position >= length can still read
  int first_needed(const Group& g, int length) const {
    if (g.window < 0) return 0;
    return std::max(0, length - g.window + 1) / page_size;
  }
  int missing(const Group& g, const std::vector<int>& table, int length, int new_len) const {
    const int last = pages_for(new_len);
    if (g.window < 0) return std::max(0, last - (int)table.size());      // no holes
    int n = 0;
    for (int i = first_needed(g, length); i < last; ++i)
      if (i >= (int)table.size() || table[(size_t)i] == NO_PAGE) ++n;
    return n;
  }
  void missing_all(long long rid, int new_len, int* out) const {
    auto it = requests.find(rid);
    for (size_t g = 0; g < groups.size(); ++g) {
      if (it != requests.end())
        out[g] = missing(groups[g], it->second.tables[g], it->second.length, new_len);
      else
        out[g] = pages_for(new_len) - first_needed(groups[g], 0);
    }
  }
  // pages go back in the reverse of the order given (the first of them is handed out next)
  void give_back(Group& g, const std::vector<int>& pages) {
    for (auto it = pages.rbegin(); it != pages.rend(); ++it) {
      g.pages.give(*it);
      g.freed.push_back(*it);
    }
  }
  void forget_freed() {
    for (Group& g : groups) g.freed.clear();
  }
};

std::string rid_text(long long rid) { return "#" + std::to_string(rid); }

}  // namespace

extern "C" {

const char* zc_last_error() { return last_error.c_str(); }

// windows[g] < 0: the group keeps every key
void* zc_create(int n_groups, const int* windows, int page_size, int num_pages, int max_requests) {
  if (n_groups < 0 || page_size < 1 || num_pages < 0 || max_requests < 0) return nullptr;
  Core* c = new Core(page_size, max_requests);
  for (int g = 0; g < n_groups; ++g) c->groups.emplace_back(windows[g], num_pages);
  return c;
}
void zc_destroy(void* h) { delete (Core*)h; }

int zc_has_request(void* h, long long rid) { return ((Core*)h)->requests.count(rid) ? 1 : 0; }
int zc_length(void* h, long long rid, int* out) {
  Core* c = (Core*)h;
  auto it = c->requests.find(rid);
  if (it == c->requests.end()) return fail(BAD, "request " + rid_text(rid) + " is not live");
  *out = it->second.length;
  return OK;
}
int zc_state_slot(void* h, long long rid, int* out) {
  Core* c = (Core*)h;
  auto it = c->requests.find(rid);
  if (it == c->requests.end()) return fail(BAD, "request " + rid_text(rid) + " is not live");
  *out = it->second.slot;
  return OK;
}

int zc_add_request(void* h, long long rid, int* slot_out) {
  Core* c = (Core*)h;
  if (c->requests.count(rid)) return fail(BAD, "request " + rid_text(rid) + " is already live");
  if (c->slots.num_free() == 0)
    return fail(FULL, "CacheFull: all " + std::to_string(c->max_requests) + " request slots are in use");
  Request r;
  r.slot = c->slots.take();
  r.tables.resize(c->groups.size());
  *slot_out = r.slot;
  c->requests.emplace(rid, std::move(r));
  return OK;
}

// pages each group would have to hand out for rid (live or not yet) to hold new_len tokens
void zc_pages_missing(void* h, long long rid, int new_len, int* out) {
  ((Core*)h)->missing_all(rid, new_len, out);
}

// whether all (request, new_len) of a step fit together
int zc_can_reserve(void* h, int n, const long long* rids, const int* new_lens) {
  Core* c = (Core*)h;
  std::vector<long long> total(c->groups.size(), 0);
  std::vector<int> need(c->groups.size());
  int fresh = 0;
  for (int i = 0; i < n; ++i) {
    if (!c->requests.count(rids[i])) ++fresh;
    c->missing_all(rids[i], new_lens[i], need.data());
    for (size_t g = 0; g < need.size(); ++g) total[g] += need[g];
  }
  if (fresh > c->slots.num_free()) return 0;
  for (size_t g = 0; g < total.size(); ++g)
    if (total[g] > c->groups[g].pages.num_free()) return 0;
  return 1;
}

// pages for positions up to new_len (all groups or none)
int zc_reserve(void* h, long long rid, int new_len) {
  Core* c = (Core*)h;
  auto it = c->requests.find(rid);
  if (it == c->requests.end()) return fail(BAD, "request " + rid_text(rid) + " is not live");
  Request& r = it->second;
  if (new_len < r.length)
    return fail(BAD, "request " + rid_text(rid) + " holds " + std::to_string(r.length) +
                         " tokens, cannot shrink to " + std::to_string(new_len));
  for (size_t g = 0; g < c->groups.size(); ++g) {
    const int n = c->missing(c->groups[g], r.tables[g], r.length, new_len);
    if (n > c->groups[g].pages.num_free())
      return fail(FULL, "CacheFull: request " + rid_text(rid) + " needs " + std::to_string(n) +
                            " more pages of " + std::to_string(c->page_size) + " tokens, " +
                            std::to_string(c->groups[g].pages.num_free()) + " of " +
                            std::to_string(c->groups[g].pages.num_pages) + " free");
  }
  const int last = c->pages_for(new_len);
  for (size_t g = 0; g < c->groups.size(); ++g) {
    std::vector<int>& table = r.tables[g];
    if ((int)table.size() < last) table.resize((size_t)last, NO_PAGE);
    for (int i = c->first_needed(c->groups[g], r.length); i < last; ++i)
      if (table[(size_t)i] == NO_PAGE) table[(size_t)i] = c->groups[g].pages.take();
  }
  return OK;
}

// the request now holds new_len tokens; pages a window has passed go back
int zc_commit(void* h, long long rid, int new_len) {
  Core* c = (Core*)h;
  auto it = c->requests.find(rid);
  if (it == c->requests.end()) return fail(BAD, "request " + rid_text(rid) + " is not live");
  c->forget_freed();
  Request& r = it->second;
  r.length = new_len;
  for (size_t g = 0; g < c->groups.size(); ++g) {
    Group& grp = c->groups[g];
    if (grp.window < 0) continue;
    std::vector<int>& table = r.tables[g];
    const int first = std::min(c->first_needed(grp, new_len), (int)table.size());
    std::vector<int> gone;
    for (int i = 0; i < first; ++i)
      if (table[(size_t)i] != NO_PAGE) {
        gone.push_back(table[(size_t)i]);
        table[(size_t)i] = NO_PAGE;
      }
    c->give_back(grp, gone);
  }
  return OK;
}

// gives back the pages reserved beyond the tokens the request holds (a step that reserved them
// did not run)
int zc_trim(void* h, long long rid) {
  Core* c = (Core*)h;
  auto it = c->requests.find(rid);
  if (it == c->requests.end()) return fail(BAD, "request " + rid_text(rid) + " is not live");
  c->forget_freed();
  Request& r = it->second;
  const size_t keep = (size_t)c->pages_for(r.length);
  for (size_t g = 0; g < c->groups.size(); ++g) {
    std::vector<int>& table = r.tables[g];
    std::vector<int> gone;
    for (size_t i = keep; i < table.size(); ++i)
      if (table[i] != NO_PAGE) gone.push_back(table[i]);
    c->give_back(c->groups[g], gone);
    if (table.size() > keep) table.resize(keep);
  }
  return OK;
}

// everything the request holds goes back: pages of every group and the state slot
int zc_release(void* h, long long rid) {
  Core* c = (Core*)h;
  auto it = c->requests.find(rid);
  if (it == c->requests.end()) return fail(BAD, "request " + rid_text(rid) + " is not live");
  c->forget_freed();
  for (size_t g = 0; g < c->groups.size(); ++g) {
    std::vector<int> gone;
    for (int p : it->second.tables[g])
      if (p != NO_PAGE) gone.push_back(p);
    c->give_back(c->groups[g], gone);
  }
  c->slots.give(it->second.slot);
  c->requests.erase(it);
  return OK;
}

// what the last commit, trim or release gave back in a group (for a caller that poisons them)
int zc_last_freed(void* h, int group, int* out, int cap) {
  const std::vector<int>& f = ((Core*)h)->groups[(size_t)group].freed;
  const int n = std::min((int)f.size(), cap);
  std::copy(f.begin(), f.begin() + n, out);
  return (int)f.size();
}

// the block table of a request in a group: its length; the first min(length, cap) entries in out
int zc_table(void* h, int group, long long rid, int* out, int cap) {
  Core* c = (Core*)h;
  auto it = c->requests.find(rid);
  if (it == c->requests.end()) return -1;
  const std::vector<int>& t = it->second.tables[(size_t)group];
  const int n = std::min((int)t.size(), cap);
  std::copy(t.begin(), t.begin() + n, out);
  return (int)t.size();
}
// (a debugging aid: a test of the device-side table check plants a page that is not the pool's)
int zc_set_table_entry(void* h, int group, long long rid, int index, int page) {
  Core* c = (Core*)h;
  auto it = c->requests.find(rid);
  if (it == c->requests.end() || index < 0 || index >= (int)it->second.tables[(size_t)group].size())
    return fail(BAD, "no such table entry");
  it->second.tables[(size_t)group][(size_t)index] = page;
  return OK;
}

// A step's block tables and slot mapping of one group: request i brings q_lens[i] tokens
// behind the starts[i] it holds, its tokens are rows q_start[i] .. of the step.  table_out
// [n, max_pages] (NO_PAGE where the request has none), slots_out [sum q_lens]: page * page_size
// + row of every token's own key and value.
int zc_pack_group(void* h, int group, int n, const long long* rids, const int* starts,
                  const int* q_lens, int max_pages, int* table_out, int* slots_out) {
  Core* c = (Core*)h;
  const int ps = c->page_size;
  int row = 0;
  for (int i = 0; i < n; ++i) {
    auto it = c->requests.find(rids[i]);
    if (it == c->requests.end()) return fail(BAD, "request " + rid_text(rids[i]) + " is not live");
    const std::vector<int>& t = it->second.tables[(size_t)group];
    if ((int)t.size() > max_pages)
      return fail(BAD, "a block table of " + std::to_string(t.size()) + " pages does not fit " +
                           std::to_string(max_pages));
    int* dst = table_out + (size_t)i * max_pages;
    std::copy(t.begin(), t.end(), dst);
    std::fill(dst + t.size(), dst + max_pages, NO_PAGE);
    for (int p = starts[i]; p < starts[i] + q_lens[i]; ++p, ++row) {
      const int page = p / ps < (int)t.size() ? t[(size_t)(p / ps)] : NO_PAGE;
      if (page < 0) return fail(BAD, "a token would be written to a page that is not held");
      slots_out[row] = page * ps + p % ps;
    }
  }
  return OK;
}

// accounting: what[0] free, [1] held, [2] pages of the pool, [3] high water; handed_out apart
void zc_group_counts(void* h, int group, int* what, long long* handed_out) {
  const PagePool& p = ((Core*)h)->groups[(size_t)group].pages;
  what[0] = p.num_free();
  what[1] = p.num_held();
  what[2] = p.num_pages;
  what[3] = p.high_water;
  *handed_out = p.handed_out;
}
void zc_slot_counts(void* h, int* what) {
  const PagePool& p = ((Core*)h)->slots;
  what[0] = p.num_free();
  what[1] = p.num_held();
  what[2] = p.num_pages;
  what[3] = p.high_water;
}

// no page lost, none held twice: the pages in all tables are exactly the held ones
int zc_check(void* h) {
  Core* c = (Core*)h;
  std::string why;
  for (size_t g = 0; g < c->groups.size(); ++g) {
    if (!c->groups[g].pages.consistent(&why)) return fail(BAD, why);
    std::unordered_set<int> held;
    size_t n = 0;
    for (const auto& kv : c->requests)
      for (int p : kv.second.tables[g])
        if (p != NO_PAGE) {
          held.insert(p);
          ++n;
        }
    if (held.size() != n) return fail(BAD, "a page is in two tables");
    if ((int)n != c->groups[g].pages.num_held()) return fail(BAD, "held pages and tables disagree");
  }
  if (!c->slots.consistent(&why)) return fail(BAD, why);
  std::unordered_set<int> slots;
  for (const auto& kv : c->requests) slots.insert(kv.second.slot);
  if (slots.size() != c->requests.size() || (int)slots.size() != c->slots.num_held())
    return fail(BAD, "slots and requests disagree");
  return OK;
}

// ---- a pool on its own (the same bookkeeping, for callers that hand out something else)
void* zp_create(int n) { return n < 0 ? nullptr : new PagePool(n); }
void zp_destroy(void* h) { delete (PagePool*)h; }
int zp_alloc(void* h, int n, int* out) {
  PagePool* p = (PagePool*)h;
  if (n > p->num_free())
    return fail(FULL, "CacheFull: " + std::to_string(n) + " pages wanted, " +
                          std::to_string(p->num_free()) + " of " + std::to_string(p->num_pages) + " free");
  for (int i = 0; i < n; ++i) out[i] = p->take();
  return OK;
}
int zp_free(void* h, const int* pages, int n) {
  PagePool* p = (PagePool*)h;
  for (int i = 0; i < n; ++i)
    if (!p->give(pages[i])) return fail(BAD, "page " + std::to_string(pages[i]) + " freed but not held");
  return OK;
}
void zp_counts(void* h, int* what, long long* handed_out) {
  const PagePool* p = (const PagePool*)h;
  what[0] = p->num_free();
  what[1] = p->num_held();
  what[2] = p->num_pages;
  what[3] = p->high_water;
  *handed_out = p->handed_out;
}
int zp_check(void* h) {
  std::string why;
  return ((PagePool*)h)->consistent(&why) ? OK : fail(BAD, why);
}

}  // extern "C"
