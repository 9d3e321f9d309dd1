// Host-side manager of cache pages and per-request state slots.
//
// The reference keeps one block table on the GPU and edits it element by element
// from C++ (yalis/attention/paged_kv_cache.cpp:12-195), which costs a device
// round trip per row per step (:77, :111, :145).  Here everything lives on the host:
// per request and per cache group a vector of page ids indexed by logical page,
// a FIFO free list per group (pages are taken from the front and given back to the
// back, as the reference's std::deque does, :44, :92-93, :158), and a pool of
// state slots handed out smallest index first (yalis/attention/kv_cache/slot_allocator.py:33-52).
//
// Groups: layers whose mixers need the same kind of pages share a pool.  A group
// with a window gives pages back as soon as no later token can read them.
//
// Plain C interface for ctypes; every function returns a status (0 = ok, <0 = error,
// message from ycm_last_error) or a count.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <deque>
#include <map>
#include <set>
#include <string>
#include <vector>

namespace {

struct Group {
  int32_t num_pages = 0;
  int32_t window = 0;  // 0: keep everything
  std::deque<int32_t> free_pages;
};

struct Request {
  int64_t tokens = 0;  // tokens with pages reserved (>= tokens cached)
  int32_t slot = -1;
  std::vector<std::vector<int32_t>> tables;  // [group][logical page] -> page id or -1
  std::vector<int64_t> first_live;           // [group] first logical page not yet given back
};

struct Manager {
  int32_t page_size = 0;
  std::vector<Group> groups;
  std::map<int64_t, Request> requests;
  std::set<int32_t> free_slots;
  int32_t num_slots = 0;
  std::string error;
};

thread_local std::string g_error;

int fail(Manager* m, const std::string& msg) {
  g_error = msg;
  if (m) m->error = msg;
  return -1;
}

int64_t pages_for(int64_t tokens, int32_t page_size) {
  return (tokens + page_size - 1) / page_size;
}

}  // namespace

extern "C" {

const char* ycm_last_error() { return g_error.c_str(); }

// windows[g] == 0 means the group keeps every token.
void* ycm_create(int32_t page_size, int32_t num_groups, const int32_t* num_pages,
                 const int32_t* windows, int32_t num_slots) {
  if (page_size <= 0 || num_groups < 0 || num_slots <= 0) {
    g_error = "ycm_create: page_size and num_slots must be positive";
    return nullptr;
  }
  auto* m = new Manager();
  m->page_size = page_size;
  m->num_slots = num_slots;
  for (int32_t s = 0; s < num_slots; ++s) m->free_slots.insert(s);
  m->groups.resize(num_groups);
  for (int32_t g = 0; g < num_groups; ++g) {
    if (num_pages[g] <= 0 || windows[g] < 0) {
      g_error = "ycm_create: a group needs pages and a non-negative window";
      delete m;
      return nullptr;
    }
    m->groups[g].num_pages = num_pages[g];
    m->groups[g].window = windows[g];
    for (int32_t p = 0; p < num_pages[g]; ++p) m->groups[g].free_pages.push_back(p);
  }
  return m;
}

void ycm_destroy(void* h) { delete static_cast<Manager*>(h); }

// Admit a request: gives it a state slot (smallest free).  Returns the slot, -2 if
// no slot is free, -1 on error.
int32_t ycm_admit(void* h, int64_t req) {
  auto* m = static_cast<Manager*>(h);
  if (m->requests.count(req)) return fail(m, "admit: request " + std::to_string(req) + " is already live");
  if (m->free_slots.empty()) return -2;
  Request r;
  r.slot = *m->free_slots.begin();
  m->free_slots.erase(m->free_slots.begin());
  r.tables.resize(m->groups.size());
  r.first_live.assign(m->groups.size(), 0);
  m->requests.emplace(req, std::move(r));
  return m->requests[req].slot;
}

// How many pages (summed over groups) growing the request to total_tokens would take.
// Sets per-group counts in need[g] when need is not null.
int64_t ycm_pages_needed(void* h, int64_t req, int64_t total_tokens, int32_t* need) {
  auto* m = static_cast<Manager*>(h);
  auto it = m->requests.find(req);
  if (it == m->requests.end()) return fail(m, "pages_needed: unknown request " + std::to_string(req));
  const Request& r = it->second;
  int64_t want = pages_for(total_tokens, m->page_size);
  int64_t sum = 0;
  for (size_t g = 0; g < m->groups.size(); ++g) {
    int64_t have = static_cast<int64_t>(r.tables[g].size());
    int64_t n = std::max<int64_t>(0, want - have);
    if (need) need[g] = static_cast<int32_t>(n);
    sum += n;
  }
  return sum;
}

// Make sure pages exist for tokens [0, total_tokens) in every group (logical pages
// already given back by a window stay absent).  All or nothing: returns 1 when the
// pages were taken, 0 when some group has too few free pages (nothing changes),
// -1 on error.
int32_t ycm_reserve(void* h, int64_t req, int64_t total_tokens) {
  auto* m = static_cast<Manager*>(h);
  auto it = m->requests.find(req);
  if (it == m->requests.end()) return fail(m, "reserve: unknown request " + std::to_string(req));
  if (total_tokens < 0) return fail(m, "reserve: negative token count");
  Request& r = it->second;
  int64_t want = pages_for(total_tokens, m->page_size);
  for (size_t g = 0; g < m->groups.size(); ++g) {
    int64_t have = static_cast<int64_t>(r.tables[g].size());
    if (want - have > static_cast<int64_t>(m->groups[g].free_pages.size())) return 0;
  }
  for (size_t g = 0; g < m->groups.size(); ++g) {
    while (static_cast<int64_t>(r.tables[g].size()) < want) {
      r.tables[g].push_back(m->groups[g].free_pages.front());
      m->groups[g].free_pages.pop_front();
    }
  }
  r.tokens = std::max(r.tokens, total_tokens);
  return 1;
}

// After a step: cached_tokens of the request are in the cache.  Groups with a
// window give back every page that no later token can read: the next query sits
// at position >= cached_tokens and reads keys j with position - j < window, so
// keys j <= cached_tokens - window are dead.  Returns the number of pages freed.
int32_t ycm_advance(void* h, int64_t req, int64_t cached_tokens) {
  auto* m = static_cast<Manager*>(h);
  auto it = m->requests.find(req);
  if (it == m->requests.end()) return fail(m, "advance: unknown request " + std::to_string(req));
  Request& r = it->second;
  int32_t freed = 0;
  for (size_t g = 0; g < m->groups.size(); ++g) {
    int32_t w = m->groups[g].window;
    if (w <= 0) continue;
    int64_t dead_tokens = cached_tokens - w + 1;  // keys 0 .. dead_tokens-1 are dead
    if (dead_tokens <= 0) continue;
    int64_t dead_pages = dead_tokens / m->page_size;  // whole pages only
    dead_pages = std::min<int64_t>(dead_pages, static_cast<int64_t>(r.tables[g].size()));
    for (int64_t p = r.first_live[g]; p < dead_pages; ++p) {
      int32_t page = r.tables[g][p];
      if (page >= 0) {
        m->groups[g].free_pages.push_back(page);
        r.tables[g][p] = -1;
        ++freed;
      }
    }
    r.first_live[g] = std::max(r.first_live[g], dead_pages);
  }
  return freed;
}

// The request is over (finished, aborted or preempted): all pages and the slot go back.
int32_t ycm_release(void* h, int64_t req) {
  auto* m = static_cast<Manager*>(h);
  auto it = m->requests.find(req);
  if (it == m->requests.end()) return fail(m, "release: unknown request " + std::to_string(req));
  Request& r = it->second;
  int32_t freed = 0;
  for (size_t g = 0; g < m->groups.size(); ++g) {
    for (int32_t page : r.tables[g]) {
      if (page >= 0) {
        m->groups[g].free_pages.push_back(page);
        ++freed;
      }
    }
  }
  m->free_slots.insert(r.slot);
  m->requests.erase(it);
  return freed;
}

int32_t ycm_slot(void* h, int64_t req) {
  auto* m = static_cast<Manager*>(h);
  auto it = m->requests.find(req);
  if (it == m->requests.end()) return fail(m, "slot: unknown request " + std::to_string(req));
  return it->second.slot;
}

int64_t ycm_table_length(void* h, int64_t req, int32_t group) {
  auto* m = static_cast<Manager*>(h);
  auto it = m->requests.find(req);
  if (it == m->requests.end()) return fail(m, "table_length: unknown request " + std::to_string(req));
  if (group < 0 || group >= static_cast<int32_t>(m->groups.size())) return fail(m, "table_length: bad group");
  return static_cast<int64_t>(it->second.tables[group].size());
}

// Copies the request's block table of a group into out[0..capacity); returns its length.
int64_t ycm_table(void* h, int64_t req, int32_t group, int32_t* out, int64_t capacity) {
  auto* m = static_cast<Manager*>(h);
  auto it = m->requests.find(req);
  if (it == m->requests.end()) return fail(m, "table: unknown request " + std::to_string(req));
  if (group < 0 || group >= static_cast<int32_t>(m->groups.size())) return fail(m, "table: bad group");
  const auto& t = it->second.tables[group];
  if (static_cast<int64_t>(t.size()) > capacity) return fail(m, "table: output too small");
  if (!t.empty()) std::memcpy(out, t.data(), t.size() * sizeof(int32_t));
  return static_cast<int64_t>(t.size());
}

int32_t ycm_free_pages(void* h, int32_t group) {
  auto* m = static_cast<Manager*>(h);
  if (group < 0 || group >= static_cast<int32_t>(m->groups.size())) return fail(m, "free_pages: bad group");
  return static_cast<int32_t>(m->groups[group].free_pages.size());
}

int32_t ycm_free_slots(void* h) { return static_cast<int32_t>(static_cast<Manager*>(h)->free_slots.size()); }

int32_t ycm_live_requests(void* h) { return static_cast<int32_t>(static_cast<Manager*>(h)->requests.size()); }

// Copies the free list of a group, front first; returns its length.
int32_t ycm_free_list(void* h, int32_t group, int32_t* out, int32_t capacity) {
  auto* m = static_cast<Manager*>(h);
  if (group < 0 || group >= static_cast<int32_t>(m->groups.size())) return fail(m, "free_list: bad group");
  const auto& f = m->groups[group].free_pages;
  if (static_cast<int32_t>(f.size()) > capacity) return fail(m, "free_list: output too small");
  std::copy(f.begin(), f.end(), out);
  return static_cast<int32_t>(f.size());
}

// Checks that every page of every group is either free exactly once or held by
// exactly one request exactly once, and the same for slots.  0 = consistent.
int32_t ycm_audit(void* h) {
  auto* m = static_cast<Manager*>(h);
  for (size_t g = 0; g < m->groups.size(); ++g) {
    std::vector<int32_t> seen(m->groups[g].num_pages, 0);
    for (int32_t p : m->groups[g].free_pages) {
      if (p < 0 || p >= m->groups[g].num_pages) return fail(m, "audit: free list holds an invalid page");
      if (seen[p]++) return fail(m, "audit: page " + std::to_string(p) + " is in the free list twice");
    }
    for (const auto& kv : m->requests) {
      for (int32_t p : kv.second.tables[g]) {
        if (p < 0) continue;
        if (p >= m->groups[g].num_pages) return fail(m, "audit: a request holds an invalid page");
        if (seen[p]++) return fail(m, "audit: page " + std::to_string(p) + " of group " + std::to_string(g) + " is held twice");
      }
    }
    for (int32_t p = 0; p < m->groups[g].num_pages; ++p)
      if (!seen[p]) return fail(m, "audit: page " + std::to_string(p) + " of group " + std::to_string(g) + " is lost");
  }
  std::vector<int32_t> slots(m->num_slots, 0);
  for (int32_t s : m->free_slots) slots[s]++;
  for (const auto& kv : m->requests) {
    int32_t s = kv.second.slot;
    if (s < 0 || s >= m->num_slots) return fail(m, "audit: a request holds an invalid slot");
    slots[s]++;
  }
  for (int32_t s = 0; s < m->num_slots; ++s)
    if (slots[s] != 1) return fail(m, "audit: slot " + std::to_string(s) + " is lost or held twice");
  return 0;
}

}  // extern "C"
