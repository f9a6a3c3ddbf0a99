// The cache manager: keys and values in pages with a block table per request, one pool of pages
// per group of layers with the same need, and slots for per-request state of fixed size.
//
// The reference keeps one slab `[layer][sequence][K/V][kv head][max_seq][head_dim]` that is
// allocated once for `max_batch x max_seq` tokens and never given back per request
// (/root/reference/src/inference.cu:146-148,174-176).  Here a token at position `pos` of a
// request lives in page `table[pos / P]` at row `pos % P`; pages come from a LIFO free list (a
// page given back is the next one handed out), are given back when the request ends and, in a
// group whose layers read only a window of keys, as soon as the window has passed them.  Page
// contents are never cleared: a request reads only rows it has written itself.
//
// Everything here is host bookkeeping; the device memory behind it belongs to the engine.
#include <algorithm>
#include <random>
#include <set>

#include "../include/inference.h"

namespace tinyinfer {

bool CacheNeed::operator==(const CacheNeed& o) const {
  return kind == o.kind && kv_heads == o.kv_heads && head_dim == o.head_dim && window == o.window &&
         state_shape == o.state_shape && row_shape == o.row_shape && rows_f32 == o.rows_f32;
}

// `scatter_window` > 1: the pages are first handed out in a fixed pseudo-random order within
// windows of that many pages (window after window) instead of 0, 1, 2, ...  Requests that are
// filled one after the other then do not lie at equal distances in memory; at equal distances the
// attention kernels, which walk all requests in step, keep hitting the same memory channels
// (measured on MI355X, a decode step of 64 requests of 2,048 tokens: 5.49 ms in order, 5.03 ms
// shuffled within windows of 512 pages).
PagePool::PagePool(int num_pages, int scatter_window) : num_pages_(num_pages) {
  if (num_pages <= 0) throw CacheError("a page pool needs at least one page, got " + std::to_string(num_pages));
  std::vector<int> order(num_pages);
  for (int i = 0; i < num_pages; ++i) order[i] = i;
  if (scatter_window > 1) {
    uint64_t state = 0x9E3779B97F4A7C15ull ^ (uint64_t)num_pages;
    auto next = [&state]() {
      state += 0x9E3779B97F4A7C15ull;
      uint64_t z = state;
      z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
      z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
      return z ^ (z >> 31);
    };
    for (int i = 0; i < num_pages; i += scatter_window) {
      const int n = std::min(scatter_window, num_pages - i);
      for (int k = n - 1; k > 0; --k) std::swap(order[i + k], order[i + (int)(next() % (uint64_t)(k + 1))]);
    }
  }
  free_.assign(order.rbegin(), order.rend());      // back() is order[0]
  held_.assign(num_pages, 0);
}

int PagePool::take() {
  if (free_.empty()) throw OutOfPages("no free page");
  const int p = free_.back();
  free_.pop_back();
  if (held_[p]) throw CacheError("page " + std::to_string(p) + " handed out twice");
  held_[p] = 1;
  ++taken_total;
  high_water = std::max(high_water, num_pages_ - (int)free_.size());
  return p;
}

void PagePool::give_back(int p) {
  if (p < 0 || p >= num_pages_ || !held_[p]) throw CacheError("page " + std::to_string(p) + " given back but not held");
  held_[p] = 0;
  free_.push_back(p);
}

CacheManager::CacheManager(const std::vector<std::pair<CacheNeed, int>>& groups, int page_size, int num_pages,
                           int max_requests, int max_seq, int scatter_window)
    : page_size(page_size), max_requests(max_requests), max_seq(max_seq),
      table_width(page_size > 0 ? (max_seq + page_size - 1) / page_size : 0) {
  if (page_size <= 0) throw CacheError("page_size must be positive");
  if (max_requests <= 0) throw CacheError("max_requests must be positive");
  for (const auto& g : groups) {
    Group grp;
    grp.need = g.first;
    grp.n_layers = g.second;
    grp.paged = g.first.paged();
    if (grp.paged) {
      grp.pool.reset(new PagePool(num_pages, scatter_window));
      paged_.push_back((int)groups_.size());
    }
    groups_.push_back(std::move(grp));
  }
  for (int s = max_requests - 1; s >= 0; --s) free_slots_.push_back(s);
}

static std::string rq(int64_t r) { return std::to_string(r); }

std::vector<int64_t> CacheManager::live_requests() const {
  std::vector<int64_t> v;
  for (const auto& kv : requests_) v.push_back(kv.first);
  return v;
}
static const char* NOT_ADMITTED = " is not admitted";
int CacheManager::length(int64_t req) const {
  auto it = requests_.find(req);
  if (it == requests_.end()) throw CacheError("request " + rq(req) + NOT_ADMITTED);
  return it->second.length;
}
int CacheManager::reserved(int64_t req) const {
  auto it = requests_.find(req);
  if (it == requests_.end()) throw CacheError("request " + rq(req) + NOT_ADMITTED);
  return it->second.reserved;
}
int CacheManager::slot(int64_t req) const {
  auto it = requests_.find(req);
  if (it == requests_.end()) throw CacheError("request " + rq(req) + NOT_ADMITTED);
  return it->second.slot;
}
int CacheManager::num_free_pages() const {
  int best = 1 << 30;
  for (int g : paged_) best = std::min(best, groups_[g].pool->num_free());
  return best;
}
PagePool& CacheManager::pool(int g) {
  if (g < 0 || g >= (int)groups_.size() || !groups_[g].paged) throw CacheError("cache group " + std::to_string(g) + " has no pages");
  return *groups_[g].pool;
}
const std::vector<int>& CacheManager::table(int g, int64_t req) const {
  if (g < 0 || g >= (int)groups_.size() || !groups_[g].paged) throw CacheError("cache group " + std::to_string(g) + " has no pages");
  auto it = groups_[g].tables.find(req);
  if (it == groups_[g].tables.end()) throw CacheError("request " + rq(req) + NOT_ADMITTED);
  return it->second;
}
const int* CacheManager::table_row(int g, int64_t req) const {
  auto it = groups_[g].rows.find(req);
  if (it == groups_[g].rows.end()) throw CacheError("request " + rq(req) + NOT_ADMITTED);
  return it->second.data();
}

int CacheManager::pages_to_cover(int g, int64_t req, bool admitted, int upto) const {
  int have = 0;
  if (admitted) {
    auto it = groups_[g].tables.find(req);
    if (it != groups_[g].tables.end()) have = (int)it->second.size();
  }
  const int want = (upto + page_size - 1) / page_size;
  return std::max(0, want - have);
}

int CacheManager::pages_needed(int64_t req, bool admitted, int n_tokens, int length) const {
  int base = length;
  if (base < 0) {
    auto it = admitted ? requests_.find(req) : requests_.end();
    base = it != requests_.end() ? it->second.reserved : 0;
  }
  int worst = 0;
  for (int g : paged_) worst = std::max(worst, pages_to_cover(g, req, admitted, base + n_tokens));
  return worst;
}

bool CacheManager::can_reserve(int64_t req, int n_tokens) const {
  auto it = requests_.find(req);
  const bool admitted = it != requests_.end();
  const int base = admitted ? it->second.reserved : 0;
  if (base + n_tokens > max_seq) return false;
  for (int g : paged_)
    if (pages_to_cover(g, req, admitted, base + n_tokens) > groups_[g].pool->num_free()) return false;
  return true;
}

int CacheManager::admit(int64_t req) {
  if (requests_.count(req)) throw CacheError("request " + rq(req) + " is already admitted");
  if (free_slots_.empty()) throw CacheError("no free request slot (max_requests = " + std::to_string(max_requests) + ")");
  const int slot = free_slots_.back();
  free_slots_.pop_back();
  Req r;
  r.slot = slot;
  requests_[req] = r;
  for (int g : paged_) {
    groups_[g].tables[req] = {};
    groups_[g].rows[req].assign(table_width, -1);
  }
  slots_to_clear.push_back(slot);
  return slot;
}

void CacheManager::reserve(int64_t req, int n_tokens) {
  auto it = requests_.find(req);
  if (it == requests_.end()) throw CacheError("request " + rq(req) + NOT_ADMITTED);
  Req& r = it->second;
  const int upto = r.reserved + n_tokens;
  if (upto > max_seq)
    throw CacheError("request " + rq(req) + ": " + std::to_string(upto) + " tokens exceed max_seq = " + std::to_string(max_seq));
  for (int g : paged_) {
    const int need = pages_to_cover(g, req, true, upto);
    if (need > groups_[g].pool->num_free())
      throw OutOfPages("request " + rq(req) + " needs " + std::to_string(need) + " more pages for " +
                       std::to_string(n_tokens) + " tokens, " + std::to_string(groups_[g].pool->num_free()) + " are free");
  }
  for (int g : paged_) {
    Group& grp = groups_[g];
    const int need = pages_to_cover(g, req, true, upto);
    auto& t = grp.tables[req];
    auto& row = grp.rows[req];
    for (int k = 0; k < need; ++k) {
      const int page = grp.pool->take();
      row[t.size()] = page;
      t.push_back(page);
    }
  }
  r.reserved = upto;
}

int CacheManager::first_needed_page(const Group& g, int next_pos) const {
  if (g.need.window <= 0) return 0;
  return std::max(0, next_pos - g.need.window + 1) / page_size;
}

void CacheManager::give_back_page(Group& g, int64_t req, int index) {
  auto& t = g.tables[req];
  g.pool->give_back(t[index]);
  t[index] = -1;
  g.rows[req][index] = -1;
}

void CacheManager::commit(int64_t req, int n_tokens) {
  auto it = requests_.find(req);
  if (it == requests_.end()) throw CacheError("request " + rq(req) + NOT_ADMITTED);
  Req& r = it->second;
  if (r.length + n_tokens > r.reserved)
    throw CacheError("request " + rq(req) + ": committing " + std::to_string(n_tokens) + " tokens beyond its reservation");
  r.length += n_tokens;
  for (int gi : paged_) {
    Group& g = groups_[gi];
    const int first = first_needed_page(g, r.length);
    if (first == 0) continue;
    auto& t = g.tables[req];
    for (int i = 0; i < std::min(first, (int)t.size()); ++i)
      if (t[i] >= 0) give_back_page(g, req, i);
  }
}

// A decode step: one token for each of several admitted requests.  The same as `reserve` (for all
// of them or for none) and `commit` per request.
std::vector<int> CacheManager::reserve_one_each(const std::vector<int64_t>& reqs) {
  std::vector<Req*> rs;
  rs.reserve(reqs.size());
  for (int64_t q : reqs) {
    auto it = requests_.find(q);
    if (it == requests_.end()) throw CacheError("request " + rq(q) + NOT_ADMITTED);
    rs.push_back(&it->second);
  }
  std::vector<int> starts;
  starts.reserve(reqs.size());
  for (size_t i = 0; i < reqs.size(); ++i) {
    const Req& r = *rs[i];
    if (r.reserved != r.length) throw CacheError("request " + rq(reqs[i]) + " has a reservation that was not committed");
    if (r.reserved + 1 > max_seq)
      throw CacheError("request " + rq(reqs[i]) + ": " + std::to_string(r.reserved + 1) + " tokens exceed max_seq = " +
                       std::to_string(max_seq));
    starts.push_back(r.length);
  }
  std::vector<std::pair<int, std::vector<int64_t>>> todo;
  for (int gi : paged_) {
    Group& g = groups_[gi];
    std::vector<int64_t> short_of;
    for (size_t i = 0; i < reqs.size(); ++i)
      if ((int)g.tables[reqs[i]].size() * page_size <= rs[i]->reserved) short_of.push_back(reqs[i]);
    if ((int)short_of.size() > g.pool->num_free())
      throw OutOfPages("the step needs " + std::to_string(short_of.size()) + " new pages, " +
                       std::to_string(g.pool->num_free()) + " are free");
    if (!short_of.empty()) todo.emplace_back(gi, std::move(short_of));
  }
  for (auto& kv : todo) {
    Group& g = groups_[kv.first];
    for (int64_t q : kv.second) {
      auto& t = g.tables[q];
      const int page = g.pool->take();
      g.rows[q][t.size()] = page;
      t.push_back(page);
    }
  }
  for (Req* r : rs) r->reserved += 1;
  return starts;
}

void CacheManager::commit_one_each(const std::vector<int64_t>& reqs) {
  for (int64_t q : reqs) {
    auto it = requests_.find(q);
    if (it == requests_.end()) throw CacheError("request " + rq(q) + NOT_ADMITTED);
    Req& r = it->second;
    if (r.length + 1 > r.reserved) throw CacheError("request " + rq(q) + ": committing a token beyond its reservation");
    r.length += 1;
    for (int gi : paged_) {
      Group& g = groups_[gi];
      if (g.need.window <= 0) continue;
      // a page falls behind the window only when the window's first position enters a new page
      const int lo = r.length - g.need.window + 1;
      if (lo > 0 && lo % page_size == 0) {
        auto& t = g.tables[q];
        for (int i = 0; i < std::min(lo / page_size, (int)t.size()); ++i)
          if (t[i] >= 0) give_back_page(g, q, i);
      }
    }
  }
}

// A step that failed after its reservation: the pages beyond what the committed tokens (and a
// whole page count for them) need go back, so that the next step starts from a clean state.
void CacheManager::rollback(int64_t req) {
  auto it = requests_.find(req);
  if (it == requests_.end()) return;
  Req& r = it->second;
  const int keep = (r.length + page_size - 1) / page_size;
  for (int gi : paged_) {
    Group& g = groups_[gi];
    auto& t = g.tables[req];
    while ((int)t.size() > keep) {
      const int p = t.back();
      if (p >= 0) g.pool->give_back(p);
      g.rows[req][t.size() - 1] = -1;
      t.pop_back();
    }
  }
  r.reserved = r.length;
}

void CacheManager::release(int64_t req) {
  auto it = requests_.find(req);
  if (it == requests_.end()) throw CacheError("request " + rq(req) + " released but not admitted");
  const int slot = it->second.slot;
  requests_.erase(it);
  for (int gi : paged_) {
    Group& g = groups_[gi];
    auto& t = g.tables[req];
    for (auto p = t.rbegin(); p != t.rend(); ++p)      // so the lowest page is handed out next
      if (*p >= 0) g.pool->give_back(*p);
    g.tables.erase(req);
    g.rows.erase(req);
  }
  free_slots_.push_back(slot);
  slots_to_clear.erase(std::remove(slots_to_clear.begin(), slots_to_clear.end(), slot), slots_to_clear.end());
}

// No page lost, held twice or free while held; tables cover what they must.
void CacheManager::check() const {
  auto fail = [](int g, const std::string& what) { throw CacheError("cache group " + std::to_string(g) + ": " + what); };
  for (int gi : paged_) {
    const Group& g = groups_[gi];
    std::vector<int> held;
    for (const auto& kv : g.tables) {
      const auto rit = requests_.find(kv.first);
      if (rit == requests_.end()) fail(gi, "a table without a request");
      const Req& r = rit->second;
      const auto& t = kv.second;
      if ((int)t.size() * page_size < r.reserved) fail(gi, "request " + rq(kv.first) + ": table shorter than its reservation");
      const auto& row = g.rows.at(kv.first);
      for (int i = 0; i < table_width; ++i)
        if (row[i] != (i < (int)t.size() ? t[i] : -1)) fail(gi, "request " + rq(kv.first) + ": the table's row differs");
      const int first = first_needed_page(g, r.length);
      for (int i = 0; i < (int)t.size(); ++i) {
        if (i >= first && t[i] < 0) fail(gi, "request " + rq(kv.first) + ": a page still read was given back");
        if (t[i] >= 0) held.push_back(t[i]);
      }
    }
    std::set<int> held_set(held.begin(), held.end());
    if (held_set.size() != held.size()) fail(gi, "a page is in two places");
    const auto& free_list = g.pool->free_list();
    std::set<int> free_set(free_list.begin(), free_list.end());
    if (free_set.size() != free_list.size()) fail(gi, "a page is free twice");
    for (int p : held)
      if (free_set.count(p)) fail(gi, "a page is free and held");
    if ((int)(free_list.size() + held.size()) != g.pool->num_pages()) fail(gi, "a page is lost");
  }
  std::set<int> slots;
  for (const auto& kv : requests_)
    if (!slots.insert(kv.second.slot).second) throw CacheError("a slot is held twice");
  for (int s : free_slots_)
    if (!slots.insert(s).second) throw CacheError("a slot is free and held, or free twice");
  if ((int)slots.size() != max_requests) throw CacheError("a slot is lost");
}

}  // namespace tinyinfer
