// Host-side runtime core, plain C++ (no GPU calls): the page pool and the block tables of one group of
// layers, and the packing of a step's entries into the int32 arrays that the kernels read.
//
// Behaviour follows the reference's pool (crates/cuda-kernels/src/paged_kv.rs): LIFO free stack that hands
// out page 0 first (:416), the tail page filled before a new page is taken and all-or-nothing allocation
// (:498-533), pages returned when a request ends (:985-1000), truncation that drops whole trailing pages
// (:1004-1037).  Prefix sharing, reference counts and copy-on-write are not part of this engine: a page has
// exactly one owner.  A group may have a window: pages that hold only keys a window has passed are given
// back while the request runs.
//
// Every function is `extern "C"`, takes an opaque handle and returns a count (>= 0) or a negative code;
// nothing throws across the boundary.  The Python classes in arle_amd/cache/pages.py are thin wrappers.
#include <stdint.h>
#include <stdio.h>

#include <algorithm>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace {

constexpr int kFreed = -1;  // block-table entry of a logical page that a window has passed

enum Code : int {
  kUnknownKey = -1,
  kOutOfPages = -2,
  kBufferTooSmall = -3,
  kOutOfRange = -4,
  kNotHeld = -5,
  kKeyExists = -6,
};

struct Pool {
  int num_pages;
  std::vector<int> free_;   // back() is handed out next
  std::vector<char> held;
  explicit Pool(int n) : num_pages(n), held(n, 0) {
    free_.reserve(n);
    for (int p = n - 1; p >= 0; --p) free_.push_back(p);  // pop_back yields 0 first
  }
  bool take(int n, std::vector<int>* out) {
    if (n > static_cast<int>(free_.size())) return false;
    for (int i = 0; i < n; ++i) {
      const int p = free_.back();
      free_.pop_back();
      held[p] = 1;
      out->push_back(p);
    }
    return true;
  }
  bool give_back(int p) {
    if (p < 0 || p >= num_pages || !held[p]) return false;
    held[p] = 0;
    free_.push_back(p);
    return true;
  }
};

struct Table {
  std::vector<int> pages;  // physical ids; kFreed where a window has passed
  int length = 0;          // tokens written so far
  int first_live = 0;      // logical index of the first page still held
};

struct Group {
  int page_size;
  int window;  // 0: none
  Pool pool;
  std::unordered_map<long long, Table> tables;
  Group(int num_pages, int page_size_, int window_) : page_size(page_size_), window(window_), pool(num_pages) {}
  int pages_needed(const Table& t, int n_tokens) const {
    const long long have = static_cast<long long>(t.pages.size()) * page_size;
    const long long need = static_cast<long long>(t.length) + n_tokens;
    return need > have ? static_cast<int>((need - have + page_size - 1) / page_size) : 0;
  }
};

Group* G(void* h) { return static_cast<Group*>(h); }

}  // namespace

extern "C" {

void* arle_group_create(int num_pages, int page_size, int window) {
  if (num_pages < 0 || page_size <= 0 || window < 0) return nullptr;
  return new Group(num_pages, page_size, window);
}
void arle_group_destroy(void* h) { delete G(h); }

int arle_group_num_pages(void* h) { return G(h)->pool.num_pages; }
int arle_group_free_count(void* h) { return static_cast<int>(G(h)->pool.free_.size()); }
int arle_group_held_count(void* h) {
  int n = 0;
  for (char c : G(h)->pool.held) n += c;
  return n;
}

// the pool alone -------------------------------------------------------------------------------------
int arle_group_take(void* h, int n, int* out) {
  std::vector<int> got;
  if (n < 0 || !G(h)->pool.take(n, &got)) return kOutOfPages;
  std::copy(got.begin(), got.end(), out);
  return n;
}
int arle_group_give_back(void* h, const int* pages, int n) {
  for (int i = 0; i < n; ++i)
    if (!G(h)->pool.give_back(pages[i])) return kNotHeld;
  return n;
}

// block tables ---------------------------------------------------------------------------------------
int arle_group_open(void* h, long long key) {
  return G(h)->tables.emplace(key, Table{}).second ? 0 : kKeyExists;
}

int arle_group_pages_needed(void* h, long long key, int n_tokens) {
  auto it = G(h)->tables.find(key);
  if (it == G(h)->tables.end()) return kUnknownKey;
  return G(h)->pages_needed(it->second, n_tokens);
}

// free pages in tokens plus the unused tail room of live requests (paged_kv.rs:1122-1137)
long long arle_group_free_tokens(void* h) {
  Group* g = G(h);
  long long tail = 0;
  for (const auto& kv : g->tables) tail += static_cast<long long>(kv.second.pages.size()) * g->page_size - kv.second.length;
  return static_cast<long long>(g->pool.free_.size()) * g->page_size + tail;
}

// Room for n more tokens; the newly mapped pages go to new_pages, their logical indices start at *first.
// Nothing changes when the pool cannot give all of them.
int arle_group_append(void* h, long long key, int n_tokens, int* first, int* new_pages, int cap) {
  Group* g = G(h);
  auto it = g->tables.find(key);
  if (it == g->tables.end()) return kUnknownKey;
  Table& t = it->second;
  const int need = g->pages_needed(t, n_tokens);
  if (need > cap) return kBufferTooSmall;
  std::vector<int> got;
  if (!g->pool.take(need, &got)) return kOutOfPages;
  *first = static_cast<int>(t.pages.size());
  t.pages.insert(t.pages.end(), got.begin(), got.end());
  t.length += n_tokens;
  std::copy(got.begin(), got.end(), new_pages);
  return need;
}

// Drop tokens beyond new_length and whole trailing pages; returns the dropped (logical, page) pairs.
int arle_group_truncate(void* h, long long key, int new_length, int* logical, int* pages, int cap) {
  Group* g = G(h);
  auto it = g->tables.find(key);
  if (it == g->tables.end()) return kUnknownKey;
  Table& t = it->second;
  if (new_length < 0 || new_length > t.length) return kOutOfRange;
  const int keep = (new_length + g->page_size - 1) / g->page_size;
  const int dropped = static_cast<int>(t.pages.size()) - keep;
  if (dropped > cap) return kBufferTooSmall;
  for (int i = 0; i < dropped; ++i) {
    logical[i] = keep + i;
    pages[i] = t.pages[keep + i];
    if (pages[i] != kFreed && !g->pool.give_back(pages[i])) return kNotHeld;
  }
  t.pages.resize(keep);
  t.length = new_length;
  t.first_live = std::min(t.first_live, keep);
  return dropped;
}

// Give back the pages every key of which the window has passed.  After `length` tokens the next query sits
// at position >= length and reads keys > position - window, so key c is dead once c <= length - window.
int arle_group_trim(void* h, long long key, int* logical, int cap) {
  Group* g = G(h);
  auto it = g->tables.find(key);
  if (it == g->tables.end()) return kUnknownKey;
  if (g->window == 0) return 0;
  Table& t = it->second;
  int dead = std::max(0, t.length - g->window + 1) / g->page_size;
  dead = std::min(dead, static_cast<int>(t.pages.size()));
  int n = 0;
  for (int i = t.first_live; i < dead; ++i) {
    if (n >= cap) return kBufferTooSmall;
    if (!g->pool.give_back(t.pages[i])) return kNotHeld;
    t.pages[i] = kFreed;
    logical[n++] = i;
  }
  t.first_live = std::max(t.first_live, dead);
  return n;
}

int arle_group_close(void* h, long long key) {
  Group* g = G(h);
  auto it = g->tables.find(key);
  if (it == g->tables.end()) return kUnknownKey;
  for (int p : it->second.pages)
    if (p != kFreed && !g->pool.give_back(p)) return kNotHeld;
  g->tables.erase(it);
  return 0;
}

// pages (up to cap), length and first live logical page of a request; returns the number of pages
int arle_group_table(void* h, long long key, int* pages, int cap, int* length, int* first_live) {
  auto it = G(h)->tables.find(key);
  if (it == G(h)->tables.end()) return kUnknownKey;
  const Table& t = it->second;
  *length = t.length;
  *first_live = t.first_live;
  const int n = static_cast<int>(t.pages.size());
  std::copy(t.pages.begin(), t.pages.begin() + std::min(n, cap), pages);
  return n;
}

// No page lost, held twice or freed twice.  0: fine; 1: the message says what is wrong.
int arle_group_check(void* h, char* msg, int cap) {
  Group* g = G(h);
  std::string bad;
  std::vector<int> owned;
  for (const auto& kv : g->tables) {
    for (int p : kv.second.pages)
      if (p != kFreed) owned.push_back(p);
    if (kv.second.length > static_cast<long long>(kv.second.pages.size()) * g->page_size)
      bad = "a request is longer than its pages";
  }
  std::unordered_set<int> owned_set(owned.begin(), owned.end()), free_set(g->pool.free_.begin(), g->pool.free_.end());
  int held = 0;
  for (char c : g->pool.held) held += c;
  if (owned_set.size() != owned.size()) bad = "a page is held by two requests";
  else if (free_set.size() != g->pool.free_.size()) bad = "a page is on the free stack twice";
  else if (std::any_of(owned.begin(), owned.end(), [&](int p) { return free_set.count(p) != 0; }))
    bad = "a page is both held and free";
  else if (static_cast<int>(owned.size() + g->pool.free_.size()) != g->pool.num_pages)
    bad = "pages lost: " + std::to_string(owned.size()) + " held + " + std::to_string(g->pool.free_.size()) +
          " free != " + std::to_string(g->pool.num_pages);
  else if (held != static_cast<int>(owned.size())) bad = "held flags disagree with the block tables";
  if (bad.empty()) return 0;
  snprintf(msg, cap, "%s", bad.c_str());
  return 1;
}

// The int32 arrays of one step, laid out one after the other in `out`:
//   token_ids[T] positions[T] slot_of_token[T] want_rows[R] seg_row0[S+1] seg_slot[S] seg_start[S]
// Entry e brings n_tokens[e] tokens (concatenated in `tokens`) of the request in slot[e] that holds start[e]
// tokens already, and wants n_want[e] places among them (concatenated in `wants`).
// meta (six ints): T, R, max position, longest entry, shortest entry, entries of one token.  Returns 0, or
//   1: a token id outside the vocabulary   2: a wanted place outside its entry   3: an entry without tokens
//   4: `out` has not exactly the size of the step;   where[0..1] = entry and the offending value.
int arle_pack_step(int n_entries, const int* slot, const int* start, const int* n_tokens, const int* tokens,
                   const int* n_want, const int* wants, int vocab_size, int* out, long long out_size, int* meta,
                   int* where) {
  long long T = 0, R = 0;
  for (int e = 0; e < n_entries; ++e) {
    if (n_tokens[e] <= 0) {
      where[0] = e;
      where[1] = n_tokens[e];
      return 3;
    }
    T += n_tokens[e];
    R += n_want[e];
  }
  const long long S = n_entries;
  if (3 * T + R + (S + 1) + 2 * S != out_size) return 4;
  int* ids = out;
  int* pos = ids + T;
  int* slots = pos + T;
  int* want_rows = slots + T;
  int* seg_row0 = want_rows + R;
  int* seg_slot = seg_row0 + S + 1;
  int* seg_start = seg_slot + S;
  int row = 0, w = 0, t = 0, r = 0, max_pos = 0, longest = 0, shortest = INT32_MAX, singles = 0;
  for (int e = 0; e < n_entries; ++e) {
    const int n = n_tokens[e];
    for (int i = 0; i < n; ++i) {
      const int id = tokens[t + i];
      if (id < 0 || id >= vocab_size) {
        where[0] = e;
        where[1] = id;
        return 1;
      }
      ids[row + i] = id;
      pos[row + i] = start[e] + i;
      slots[row + i] = slot[e];
    }
    for (int i = 0; i < n_want[e]; ++i) {
      const int place = wants[w + i];
      if (place < 0 || place >= n) {
        where[0] = e;
        where[1] = place;
        return 2;
      }
      want_rows[r++] = row + place;
    }
    seg_row0[e] = row;
    seg_slot[e] = slot[e];
    seg_start[e] = start[e];
    max_pos = std::max(max_pos, start[e] + n - 1);
    longest = std::max(longest, n);
    shortest = std::min(shortest, n);
    singles += n == 1;
    row += n;
    t += n;
    w += n_want[e];
  }
  seg_row0[n_entries] = row;
  meta[0] = static_cast<int>(T);
  meta[1] = static_cast<int>(R);
  meta[2] = max_pos;
  meta[3] = longest;
  meta[4] = shortest;
  meta[5] = singles;
  return 0;
}

// Which decoding request gives its pages back when they run out: fewest generated tokens first; ties:
// the longest prompt; ties: the first (infer/src/scheduler/cuda/sched/decode.rs:16-21).
int arle_retract_victim(int n, const int* generated, const int* prompt_len) {
  int best = -1;
  for (int i = 0; i < n; ++i)
    if (best < 0 || generated[i] < generated[best] ||
        (generated[i] == generated[best] && prompt_len[i] > prompt_len[best]))
      best = i;
  return best;
}

// How many of the n tokens that a prompt with `remaining` tokens could bring to a step of rows_before rows it brings:
// a portion that is cut anyway gives up the tokens that stand over a multiple of `align` rows, if at least `align`
// tokens stay and the prompt needs no further step for it (the products of a step run in tiles of 128 and 256 rows).
static int aligned_portion(int n, int remaining, int rows_before, int align) {
  if (align <= 0 || n >= remaining) return n;
  const int over = (rows_before + n) % align;
  const int m = n - over;
  if (over == 0 || m < align) return n;
  if ((remaining + m - 1) / m != (remaining + n - 1) / n) return n;
  return m;
}

int arle_aligned_portion(int n, int remaining, int rows_before, int align) {
  return aligned_portion(n, remaining, rows_before, align);
}

// The prompt portions of one step (infer/src/scheduler/cuda/execution.rs:265-317, budget.rs:229-264): the queue is
// walked in order; a request brings min(remaining, chunked_prefill_size) tokens (at most the long-prefill threshold
// beside decoding requests); one that does not fit the tokens left, the requests left or the pages is skipped whole,
// never shrunk, and a later one may still fit.  Pages: on top of what the decoding requests are reserved
// (decode_growth tokens each) and what the portions picked so far take, in every group.
//   groups[n_groups]; decode_keys[n_groups][n_decode], queue_keys[n_groups][n_queue]: a request's key in each group;
//   first_decode[j]: 1 if the request's first decoded token needs a slot when its prompt completes.
// picked[j]: tokens of request j in this step (0: none); page_tokens[j]: tokens its pages were asked for.
// Returns how many were picked, or kUnknownKey.
int arle_plan_prefill(int n_groups, void* const* groups, int n_decode, const long long* decode_keys, const int* decode_growth,
                      int n_queue, const long long* queue_keys, const int* remaining, const int* first_decode,
                      int decode_rows, int max_num_batched_tokens, int max_prefill_tokens, int prefill_max_requests,
                      int chunked_prefill_size, int long_prefill_token_threshold, int step_row_alignment, int* picked,
                      int* page_tokens) {
  std::vector<long long> reserved(n_groups > 0 ? n_groups : 0, 0);
  for (int g = 0; g < n_groups; ++g) {
    Group* grp = G(groups[g]);
    for (int i = 0; i < n_decode; ++i) {
      auto it = grp->tables.find(decode_keys[static_cast<size_t>(g) * n_decode + i]);
      if (it == grp->tables.end()) return kUnknownKey;
      reserved[g] += grp->pages_needed(it->second, decode_growth[i]);
    }
  }
  int tokens_left = std::min(std::max(max_num_batched_tokens - decode_rows, 0), max_prefill_tokens);
  int requests_left = prefill_max_requests >= 0 ? prefill_max_requests : n_queue;
  int cap = chunked_prefill_size;
  if (decode_rows > 0) cap = std::min(cap, long_prefill_token_threshold);
  cap = std::max(cap, 1);
  int count = 0, rows = decode_rows;
  std::vector<int> need(n_groups > 0 ? n_groups : 0, 0);
  for (int j = 0; j < n_queue; ++j) {
    picked[j] = 0;
    page_tokens[j] = 0;
    if (remaining[j] <= 0) continue;
    int n = std::min(remaining[j], cap);
    if (n > tokens_left || requests_left <= 0) continue;  // skipped whole; a later, smaller one may still fit
    n = aligned_portion(n, remaining[j], rows, step_row_alignment);
    const int asked = n + ((n == remaining[j] && first_decode[j]) ? 1 : 0);
    bool fits = true;
    for (int g = 0; g < n_groups && fits; ++g) {
      Group* grp = G(groups[g]);
      auto it = grp->tables.find(queue_keys[static_cast<size_t>(g) * n_queue + j]);
      if (it == grp->tables.end()) return kUnknownKey;
      need[g] = grp->pages_needed(it->second, asked);
      fits = reserved[g] + need[g] <= static_cast<long long>(grp->pool.free_.size());
    }
    if (!fits) continue;
    for (int g = 0; g < n_groups; ++g) reserved[g] += need[g];
    picked[j] = n;
    page_tokens[j] = asked;
    tokens_left -= n;
    requests_left -= 1;
    rows += n;
    count += 1;
  }
  return count;
}

// Which waiting requests are admitted (infer/src/scheduler/cuda/runtime/scheduler_loop.rs:202-315, budget.rs:17-33):
// a request needs a free slot and, in every group, pages for its prompt and one token more, after the pages that the
// running requests still need to reach theirs are set aside; one that does not fit waits, later ones may still go in.
//   page_size[g], free_pages[g]; running_length[i] (tokens cached), running_target[i], waiting_target[j] (tokens).
// admit[j]: 1 or 0.  Returns how many are admitted.
int arle_admit(int n_groups, const int* page_size, const int* free_pages, int free_slots, int n_running,
               const int* running_length, const int* running_target, int n_waiting, const int* waiting_target, int* admit) {
  std::vector<long long> left(n_groups > 0 ? n_groups : 0, 0);
  auto pages = [&](int g, int tokens) { return (static_cast<long long>(tokens) + page_size[g] - 1) / page_size[g]; };
  for (int g = 0; g < n_groups; ++g) {
    left[g] = free_pages[g];
    for (int i = 0; i < n_running; ++i) left[g] -= std::max(0LL, pages(g, running_target[i]) - pages(g, running_length[i]));
  }
  int count = 0;
  for (int j = 0; j < n_waiting; ++j) {
    bool fits = free_slots > 0;
    for (int g = 0; g < n_groups && fits; ++g) fits = pages(g, waiting_target[j]) <= left[g];
    admit[j] = fits ? 1 : 0;
    if (!fits) continue;
    for (int g = 0; g < n_groups; ++g) left[g] -= pages(g, waiting_target[j]);
    free_slots -= 1;
    count += 1;
  }
  return count;
}

}  // extern "C"
