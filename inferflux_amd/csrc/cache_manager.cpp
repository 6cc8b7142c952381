// Accounting of the paged cache on the host: pools of pages with reference counts, a block table per live
// request and cache group, state slots, and the arrays a step needs of them.  No device memory, no GPU.
//
// A request is known here by its state slot (0 .. max_requests - 1), which it holds from add to free.
// Groups: entry g of ``windows`` is the number of positions the group's layers look back (-1: all of them);
// a windowed group gives a page back as soon as every position in it lies before the window of the next
// query.  Pages are handed out most recently freed first; a page returns to its pool when its reference
// count reaches zero.  Every call either succeeds or changes nothing.
//
// The reference accounts pages on the host in the same units (16-token blocks with reference counts:
// runtime/kv_cache/paged_kv_cache.cpp:40-86, 211-246, 360-371; scheduler/scheduler.cpp:293, 2327-2335); it
// has no groups and no state slots.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <vector>

namespace {

thread_local char g_error[512];

struct Pool {
  int num_pages = 0;
  std::vector<int> free_list;   // back() is handed out next
  std::vector<int> refs;
  explicit Pool(int n) : num_pages(n), refs(n, 0) {
    free_list.reserve(n);
    for (int p = n - 1; p >= 0; --p) free_list.push_back(p);   // page 0 first
  }
  int num_free() const { return (int)free_list.size(); }
  int take() {
    const int p = free_list.back();
    free_list.pop_back();
    refs[p] = 1;
    return p;
  }
  bool release(int p) {
    if (p < 0 || p >= num_pages || refs[p] <= 0) return false;
    if (--refs[p] == 0) free_list.push_back(p);
    return true;
  }
};

struct Request {
  bool live = false;
  long long epoch = 0;   // a number no other request ever had: tells a request from a later one in the same slot
  int length = 0;        // committed positions
  int reserved = 0;      // positions with pages, >= length
  std::vector<std::vector<int>> tables;   // per group: page of block b, or -1 once given back
};

struct Manager {
  int page_size, max_requests;
  std::vector<Pool> pools;
  std::vector<int> windows;
  std::vector<int> free_slots;   // back() is handed out next
  std::vector<Request> requests;
  long long epochs = 0;
  int blocks_for(int positions) const { return (positions + page_size - 1) / page_size; }
};

#define FAIL(code, ...)                                   \
  do {                                                    \
    snprintf(g_error, sizeof(g_error), __VA_ARGS__);      \
    return code;                                          \
  } while (0)

Request* live_request(Manager* m, int slot) {
  if (slot < 0 || slot >= m->max_requests || !m->requests[slot].live) return nullptr;
  return &m->requests[slot];
}

}  // namespace

extern "C" {

const char* ifx_last_error() { return g_error; }

void* cm_create(int n_groups, const int* num_pages, const int* windows, int page_size, int max_requests) {
  if (n_groups < 0 || page_size <= 0 || max_requests < 0) {
    snprintf(g_error, sizeof(g_error), "cache manager: %d groups, page size %d, %d requests", n_groups, page_size, max_requests);
    return nullptr;
  }
  for (int g = 0; g < n_groups; ++g)
    if (num_pages[g] <= 0) {
      snprintf(g_error, sizeof(g_error), "a pool needs at least one page");
      return nullptr;
    }
  Manager* m = new Manager();
  m->page_size = page_size;
  m->max_requests = max_requests;
  for (int g = 0; g < n_groups; ++g) {
    m->pools.emplace_back(num_pages[g]);
    m->windows.push_back(windows[g]);
  }
  for (int s = max_requests - 1; s >= 0; --s) m->free_slots.push_back(s);   // slot 0 first
  m->requests.resize(max_requests);
  return m;
}

void cm_destroy(void* h) { delete (Manager*)h; }

// ---- pools ----------------------------------------------------------------------------------------------
int cm_pool_num_pages(void* h, int g) { return ((Manager*)h)->pools[g].num_pages; }
int cm_pool_num_free(void* h, int g) { return ((Manager*)h)->pools[g].num_free(); }
int cm_pool_take(void* h, int g) {
  Pool& p = ((Manager*)h)->pools[g];
  if (p.free_list.empty()) FAIL(-1, "no free page");
  return p.take();
}
int cm_pool_retain(void* h, int g, int page) {
  Pool& p = ((Manager*)h)->pools[g];
  if (page < 0 || page >= p.num_pages || p.refs[page] <= 0) FAIL(-1, "page %d is not in use", page);
  ++p.refs[page];
  return 0;
}
int cm_pool_release(void* h, int g, int page) {
  if (!((Manager*)h)->pools[g].release(page)) FAIL(-1, "page %d released but not in use (freed twice?)", page);
  return 0;
}
int cm_pool_refs(void* h, int g, int page) {
  Pool& p = ((Manager*)h)->pools[g];
  return page >= 0 && page < p.num_pages ? p.refs[page] : -1;
}
int cm_pool_free_list(void* h, int g, int* out) {   // in the order pages will be handed out, last first
  Pool& p = ((Manager*)h)->pools[g];
  std::copy(p.free_list.begin(), p.free_list.end(), out);
  return p.num_free();
}

// ---- requests -------------------------------------------------------------------------------------------
int cm_free_slots(void* h) { return (int)((Manager*)h)->free_slots.size(); }

int cm_add(void* h) {   // -> the request's slot
  Manager* m = (Manager*)h;
  if (m->free_slots.empty()) FAIL(-1, "all %d request slots are in use", m->max_requests);
  const int slot = m->free_slots.back();
  m->free_slots.pop_back();
  Request& r = m->requests[slot];
  r.live = true;
  r.epoch = ++m->epochs;
  r.length = r.reserved = 0;
  r.tables.assign(m->pools.size(), std::vector<int>());
  return slot;
}

int cm_free(void* h, int slot) {
  Manager* m = (Manager*)h;
  Request* r = live_request(m, slot);
  if (!r) FAIL(-1, "slot %d holds no live request (freed twice?)", slot);
  for (size_t g = 0; g < r->tables.size(); ++g)
    for (int p : r->tables[g])
      if (p >= 0) m->pools[g].release(p);
  r->live = false;
  r->tables.clear();
  m->free_slots.push_back(slot);
  return 0;
}

int cm_length(void* h, int slot) {
  Request* r = live_request((Manager*)h, slot);
  if (!r) FAIL(-1, "slot %d holds no live request", slot);
  return r->length;
}
int cm_reserved(void* h, int slot) {
  Request* r = live_request((Manager*)h, slot);
  if (!r) FAIL(-1, "slot %d holds no live request", slot);
  return r->reserved;
}
long long cm_epoch(void* h, int slot) {
  Request* r = live_request((Manager*)h, slot);
  return r ? r->epoch : -1;
}

// New pages per group for the request's next n_new positions.
int cm_pages_needed(void* h, int slot, int n_new, int* out) {
  Manager* m = (Manager*)h;
  Request* r = live_request(m, slot);
  if (!r) FAIL(-1, "slot %d holds no live request", slot);
  for (size_t g = 0; g < r->tables.size(); ++g) out[g] = std::max(0, m->blocks_for(r->length + n_new) - (int)r->tables[g].size());
  return 0;
}

// Whether every (slot, n_new) of the list fits at once: 1 / 0; totals per group go to ``totals`` if given.
int cm_can_reserve(void* h, const int* slots, const int* n_new, int count, int* totals) {
  Manager* m = (Manager*)h;
  std::vector<int> tot(m->pools.size(), 0);
  for (int i = 0; i < count; ++i) {
    Request* r = live_request(m, slots[i]);
    if (!r) FAIL(-1, "slot %d holds no live request", slots[i]);
    for (size_t g = 0; g < tot.size(); ++g) tot[g] += std::max(0, m->blocks_for(r->length + n_new[i]) - (int)r->tables[g].size());
  }
  int ok = 1;
  for (size_t g = 0; g < tot.size(); ++g) {
    if (totals) totals[g] = tot[g];
    if (tot[g] > m->pools[g].num_free()) ok = 0;
  }
  return ok;
}

// Pages for positions [length, length + n_new) in every group, or nothing: 0, or 1 with fail = {group, needed, free}.
int cm_reserve(void* h, int slot, int n_new, int* fail) {
  Manager* m = (Manager*)h;
  Request* r = live_request(m, slot);
  if (!r) FAIL(-1, "slot %d holds no live request", slot);
  if (n_new <= 0) FAIL(-2, "reserve needs a positive token count");
  const int blocks = m->blocks_for(r->length + n_new);
  for (size_t g = 0; g < r->tables.size(); ++g) {
    const int k = std::max(0, blocks - (int)r->tables[g].size());
    if (k > m->pools[g].num_free()) {
      fail[0] = (int)g; fail[1] = k; fail[2] = m->pools[g].num_free();
      return 1;
    }
  }
  for (size_t g = 0; g < r->tables.size(); ++g)
    while ((int)r->tables[g].size() < blocks) r->tables[g].push_back(m->pools[g].take());
  r->reserved = std::max(r->reserved, r->length + n_new);
  return 0;
}

// The step that wrote n_new positions has run: they count now; windowed groups give back what no later query sees.
int cm_commit(void* h, int slot, int n_new) {
  Manager* m = (Manager*)h;
  Request* r = live_request(m, slot);
  if (!r) FAIL(-1, "slot %d holds no live request", slot);
  if (n_new < 0 || r->length + n_new > r->reserved)
    FAIL(-2, "commit of %d beyond the %d reserved positions", n_new, r->reserved - r->length);
  r->length += n_new;
  for (size_t g = 0; g < r->tables.size(); ++g) {
    if (m->windows[g] < 0) continue;
    const int first_needed = r->length - m->windows[g] + 1;   // oldest position the next query reads
    if (first_needed <= 0) continue;
    std::vector<int>& t = r->tables[g];
    const int dead = std::min(first_needed / m->page_size, (int)t.size());
    for (int b = dead - 1; b >= 0; --b) {   // released blocks form a prefix: stop at the first -1
      if (t[b] < 0) break;
      m->pools[g].release(t[b]);
      t[b] = -1;
    }
  }
  return 0;
}

// commit(n_new) for each of the requests, after checking that all of them can: 0, or -2 and nothing changed.
int cm_commit_each(void* h, const int* slots, int count, int n_new) {
  Manager* m = (Manager*)h;
  for (int i = 0; i < count; ++i) {
    Request* r = live_request(m, slots[i]);
    if (!r) FAIL(-1, "slot %d holds no live request", slots[i]);
    if (n_new < 0 || r->length + n_new > r->reserved)
      FAIL(-2, "commit of %d beyond the %d reserved positions", n_new, r->reserved - r->length);
  }
  for (int i = 0; i < count; ++i) cm_commit(h, slots[i], n_new);
  return 0;
}

// Whether the slots still hold the requests with these epochs, at these lengths: 1 / 0.
int cm_unchanged(void* h, const int* slots, const long long* epochs, const int* lengths, int count) {
  Manager* m = (Manager*)h;
  for (int i = 0; i < count; ++i) {
    Request* r = live_request(m, slots[i]);
    if (!r || r->epoch != epochs[i] || r->length != lengths[i]) return 0;
  }
  return 1;
}

int cm_table_len(void* h, int slot, int g) {
  Request* r = live_request((Manager*)h, slot);
  if (!r) FAIL(-1, "slot %d holds no live request", slot);
  return (int)r->tables[g].size();
}
int cm_table(void* h, int slot, int g, int* out, int cap) {
  Request* r = live_request((Manager*)h, slot);
  if (!r) FAIL(-1, "slot %d holds no live request", slot);
  const int n = std::min(cap, (int)r->tables[g].size());
  std::copy(r->tables[g].begin(), r->tables[g].begin() + n, out);
  return (int)r->tables[g].size();
}

// ---- a step's arrays ----------------------------------------------------------------------------------
// Width of each group's block tables for the step of these requests: the longest table, rounded up to a
// multiple of ``width_multiple`` (at least one multiple).
int cm_step_widths(void* h, const int* slots, int R, int width_multiple, int* widths) {
  Manager* m = (Manager*)h;
  for (size_t g = 0; g < m->pools.size(); ++g) {
    int longest = R > 0 ? 0 : 1;
    for (int i = 0; i < R; ++i) {
      Request* r = live_request(m, slots[i]);
      if (!r) FAIL(-1, "slot %d holds no live request", slots[i]);
      longest = std::max(longest, (int)r->tables[g].size());
    }
    widths[g] = std::max(width_multiple, (longest + width_multiple - 1) / width_multiple * width_multiple);
  }
  return 0;
}

// For requests slots[0..R) that bring q_len[i] tokens each, rows laid end to end: start[i] (the request's
// length), q_start[i], kv_len[i]; per row its request and position; per group the block tables
// [R, widths[g]] (-1 where no page) and the slot (page * page_size + offset) each row's key and value go to,
// groups one after the other in ``tables`` and ``write_slots`` ([groups][T]).  Returns the number of rows, or
// -(g + 2) if a row has no page in group g (reserve first).
int cm_step_fill(void* h, const int* slots, const int* q_len, int R, const int* widths, int* start, int* q_start,
                 int* kv_len, int* row_req, int* positions, int* tables, int* write_slots) {
  Manager* m = (Manager*)h;
  int T = 0;
  for (int i = 0; i < R; ++i) {
    Request* r = live_request(m, slots[i]);
    if (!r) FAIL(-1, "slot %d holds no live request", slots[i]);
    start[i] = r->length;
    q_start[i] = T;
    kv_len[i] = r->length + q_len[i];
    for (int t = 0; t < q_len[i]; ++t) {
      row_req[T + t] = i;
      positions[T + t] = r->length + t;
    }
    T += q_len[i];
  }
  int* table = tables;
  for (size_t g = 0; g < m->pools.size(); ++g) {
    const int W = widths[g];
    int* ws = write_slots + g * (size_t)T;
    for (int i = 0; i < R; ++i) {
      const std::vector<int>& t = m->requests[slots[i]].tables[g];
      int* row = table + (size_t)i * W;
      const int n = std::min(W, (int)t.size());
      std::copy(t.begin(), t.begin() + n, row);
      std::fill(row + n, row + W, -1);
      for (int k = 0; k < q_len[i]; ++k) {
        const int pos = start[i] + k, b = pos / m->page_size;
        const int page = b < n ? row[b] : -1;
        if (page < 0) FAIL(-(int)g - 2, "cache group %d: a row of this step has no page (reserve before building the step)", (int)g);
        ws[q_start[i] + k] = page * m->page_size + pos % m->page_size;
      }
    }
    table += (size_t)R * W;
  }
  return T;
}

// ---- invariants (tests call this after every operation) ---------------------------------------------------
int cm_check(void* h) {
  Manager* m = (Manager*)h;
  for (size_t g = 0; g < m->pools.size(); ++g) {
    Pool& pool = m->pools[g];
    std::vector<int> held(pool.num_pages, 0), free_n(pool.num_pages, 0);
    for (const Request& r : m->requests)
      if (r.live)
        for (int p : r.tables[g])
          if (p >= 0) {
            if (p >= pool.num_pages) FAIL(-1, "group %d: page %d does not exist", (int)g, p);
            ++held[p];
          }
    for (int p : pool.free_list) {
      if (p < 0 || p >= pool.num_pages) FAIL(-1, "group %d: page %d on the free list does not exist", (int)g, p);
      if (++free_n[p] > 1) FAIL(-1, "group %d: page %d is on the free list twice", (int)g, p);
    }
    int n_held = 0;
    for (int p = 0; p < pool.num_pages; ++p) {
      if (held[p] && free_n[p]) FAIL(-1, "group %d: page %d is both free and held", (int)g, p);
      if (held[p]) ++n_held;
      if (held[p] && pool.refs[p] != held[p]) FAIL(-1, "group %d: page %d held %d times with %d references", (int)g, p, held[p], pool.refs[p]);
      if (free_n[p] && pool.refs[p] != 0) FAIL(-1, "group %d: page %d on the free list is still referenced", (int)g, p);
    }
    // pages taken straight from a pool (tests of the pool alone) are neither free nor in a table
    int loose = 0;
    for (int p = 0; p < pool.num_pages; ++p)
      if (!held[p] && !free_n[p]) ++loose;
    if (loose) FAIL(-1, "group %d: pages lost (%d free + %d held != %d)", (int)g, pool.num_free(), n_held, pool.num_pages);
  }
  std::vector<int> slot_seen(m->max_requests, 0);
  int live = 0;
  for (int s = 0; s < m->max_requests; ++s)
    if (m->requests[s].live) { ++slot_seen[s]; ++live; }
  for (int s : m->free_slots) {
    if (s < 0 || s >= m->max_requests) FAIL(-1, "state slot %d does not exist", s);
    if (++slot_seen[s] > 1) FAIL(-1, "state slot %d is both free and held, or free twice", s);
  }
  if (live + (int)m->free_slots.size() != m->max_requests) FAIL(-1, "state slots lost");
  return 0;
}

}  // extern "C"
