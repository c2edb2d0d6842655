// The host side of the cache and of a step: who holds which slot and which pages, and the
// one int32 array that carries a step's batch to the device.  Plain C++ behind a C
// interface (loaded through ctypes); nothing here touches the GPU.
//
// The reference keeps one cache per sequence and re-uses it by setting pos = 0
// (src/model/mod.rs:235-238); its batching sketch keeps a deque of free blocks
// (src/model/batching.rs:190, 227-234, 549-555).  Here ids come from free lists that refuse
// misuse: an id is never held twice, and giving back an id that is not held is an error.
#include <algorithm>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "../page.h"

namespace {

constexpr int PAGE = TL_PAGE;

// return codes of the interface; the message of the last failure is kept per thread
constexpr int OK = 0, FULL = 1, MISUSE = 2, BAD_VALUE = 3, BAD_STEP = 4;
thread_local std::string g_err;

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_err = buf;
  return code;
}

// Ids 0..n-1.  take() returns the id that was given back last (a freed id is used again at
// once, so re-use is exercised), else the lowest id that was never taken; with `scattered`,
// else the next of a fixed shuffle of the ids.  Pages are handed out scattered: a sequence's
// pages one after the other in memory put the workgroups of a decode step, which start on pages
// a power of two apart, on the same memory channels (attention over 8 x 4,096 keys: 32.1 against
// 30.7 us in a pool that is just large enough, 31.2 against 27.5 in a pool of 3 GB).
struct FreeList {
  int n;
  std::string what;
  std::vector<int> free_;
  std::vector<uint8_t> held;
  FreeList(int n_, const char* what_, bool scattered = false) : n(n_), what(what_), held(n_, 0) {
    free_.reserve(n);
    for (int i = n - 1; i >= 0; --i) free_.push_back(i);
    if (scattered) {                          // Fisher-Yates with a fixed generator: the same order in every run
      uint64_t x = 0x9E3779B97F4A7C15ull;
      for (int i = n - 1; i > 0; --i) {
        x ^= x << 13; x ^= x >> 7; x ^= x << 17;
        std::swap(free_[i], free_[(int)(x % (uint64_t)(i + 1))]);
      }
    }
  }
  int n_free() const { return (int)free_.size(); }
  bool holds(long i) const { return i >= 0 && i < n && held[i]; }
  int take(int* out) {
    if (free_.empty()) return fail(FULL, "no free %s (all %d are held)", what.c_str(), n);
    const int i = free_.back();
    free_.pop_back();
    held[i] = 1;
    *out = i;
    return OK;
  }
  int give_back(long i) {
    if (i < 0 || i >= n) return fail(MISUSE, "%s %ld does not exist (there are %d)", what.c_str(), i, n);
    if (!held[i]) return fail(MISUSE, "%s %ld is given back but is not held", what.c_str(), i);
    held[i] = 0;
    free_.push_back((int)i);
    return OK;
  }
  // every id is either free or held, exactly once
  int check() const {
    std::vector<uint8_t> seen(n, 0);
    for (int i : free_) {
      if (seen[i]) return fail(MISUSE, "%s %d is free twice", what.c_str(), i);
      seen[i] = 1;
      if (held[i]) return fail(MISUSE, "%s %d is both free and held", what.c_str(), i);
    }
    int h = 0;
    for (int i = 0; i < n; ++i) h += held[i];
    if (h + (int)free_.size() != n) return fail(MISUSE, "%s: an id is lost", what.c_str());
    return OK;
  }
};

// Storage of the layers that share one request.  A windowed group gives a sequence a ring
// of ceil(W / PAGE) pages: position p lives in ring page (p / PAGE) % ring, row p % PAGE.
struct Group {
  int ring_pages;
  FreeList pool;
  std::vector<std::vector<int>> pages;      // by slot
  Group(int ring, int n_pages, int max_slots) : ring_pages(ring), pool(n_pages, "page", true), pages(max_slots) {}
  int pages_needed(long length) const { return (int)std::min<long>((length + PAGE - 1) / PAGE, ring_pages); }
};

struct Books {
  FreeList slots;
  std::vector<long> length;                 // by slot; meaningless while the slot is free
  std::vector<Group> groups;
  Books(int max_slots, int n_groups, const int* ring, const int* n_pages)
      : slots(max_slots, "slot"), length(max_slots, 0) {
    for (int g = 0; g < n_groups; ++g) groups.emplace_back(ring[g], n_pages[g], max_slots);
  }

  // Room for n_new more positions in each slot: every sequence gets its pages or none is changed.
  int prepare(int B, const int* slot, const int* n_new) {
    std::vector<long> need(groups.size(), 0);
    std::vector<uint8_t> seen(slots.n, 0);
    for (int b = 0; b < B; ++b) {
      if (!slots.holds(slot[b])) return fail(MISUSE, "slot %d is not held", slot[b]);
      if (seen[slot[b]]) return fail(MISUSE, "slot %d appears twice in one step", slot[b]);
      seen[slot[b]] = 1;
      if (n_new[b] < 1) return fail(BAD_VALUE, "slot %d: a step must bring at least one token", slot[b]);
      for (size_t g = 0; g < groups.size(); ++g)
        need[g] += groups[g].pages_needed(length[slot[b]] + n_new[b]) - (long)groups[g].pages[slot[b]].size();
    }
    for (size_t g = 0; g < groups.size(); ++g)
      if (need[g] > groups[g].pool.n_free())
        return fail(FULL, "the step needs %ld more pages of %d positions, %d of %d are free; raise max_tokens",
                    need[g], PAGE, groups[g].pool.n_free(), groups[g].pool.n);
    for (int b = 0; b < B; ++b)
      for (auto& g : groups) {
        auto& pg = g.pages[slot[b]];
        const int want = g.pages_needed(length[slot[b]] + n_new[b]);
        while ((int)pg.size() < want) {
          int id;
          if (int rc = g.pool.take(&id)) return rc;       // cannot happen: counted above
          pg.push_back(id);
        }
      }
    return OK;
  }
};

// Width of a step's page table: the next power of two, so that it (and what is derived from
// it, like the shape of a captured step) changes rarely while sequences grow.
int table_width(int n_pages, int ring_pages) {
  int w = 1;
  while (w < n_pages) w *= 2;
  return std::max(1, std::min(w, ring_pages));
}

}  // namespace

extern "C" {

const char* tl_host_last_error() { return g_err.c_str(); }
int tl_host_page() { return PAGE; }

// ---- a free list on its own ----------------------------------------------------------
void* tl_freelist_new(int n, const char* what) { return new FreeList(n, what); }
void tl_freelist_delete(void* h) { delete (FreeList*)h; }
int tl_freelist_take(void* h, int* out) { return ((FreeList*)h)->take(out); }
int tl_freelist_give_back(void* h, long i) { return ((FreeList*)h)->give_back(i); }
int tl_freelist_holds(void* h, long i) { return ((FreeList*)h)->holds(i); }
int tl_freelist_n_free(void* h) { return ((FreeList*)h)->n_free(); }
int tl_freelist_check(void* h) { return ((FreeList*)h)->check(); }

// ---- slots, pages, lengths -----------------------------------------------------------
void* tl_books_new(int max_slots, int n_groups, const int* ring_pages, const int* n_pages) {
  return new Books(max_slots, n_groups, ring_pages, n_pages);
}
void tl_books_delete(void* h) { delete (Books*)h; }

int tl_books_alloc_slot(void* h, int* out) {
  Books& k = *(Books*)h;
  if (int rc = k.slots.take(out)) return rc;
  k.length[*out] = 0;
  for (auto& g : k.groups) g.pages[*out].clear();
  return OK;
}

int tl_books_free_slot(void* h, long slot) {
  Books& k = *(Books*)h;
  if (int rc = k.slots.give_back(slot)) return rc;
  for (auto& g : k.groups) {
    for (int p : g.pages[slot])
      if (int rc = g.pool.give_back(p)) return rc;
    g.pages[slot].clear();
  }
  return OK;
}

int tl_books_holds(void* h, long slot) { return ((Books*)h)->slots.holds(slot); }
long tl_books_length(void* h, long slot) {
  Books& k = *(Books*)h;
  return k.slots.holds(slot) ? k.length[slot] : -1;
}
int tl_books_free_slots(void* h) { return ((Books*)h)->slots.n_free(); }
int tl_books_free_pages(void* h, int group) { return ((Books*)h)->groups[group].pool.n_free(); }
int tl_books_page_held(void* h, int group, long page) { return ((Books*)h)->groups[group].pool.holds(page); }

// the slots that are held, in ascending order; returns their number
int tl_books_held_slots(void* h, int* out, int capacity) {
  Books& k = *(Books*)h;
  int n = 0;
  for (int s = 0; s < k.slots.n; ++s)
    if (k.slots.held[s]) {
      if (n < capacity) out[n] = s;
      ++n;
    }
  return n;
}

// the pages of a slot in a group, in the order of the ring; returns their number (-1: not held)
int tl_books_pages(void* h, int group, long slot, int* out, int capacity) {
  Books& k = *(Books*)h;
  if (!k.slots.holds(slot)) return -1;
  const auto& pg = k.groups[group].pages[slot];
  for (int i = 0; i < (int)pg.size() && i < capacity; ++i) out[i] = pg[i];
  return (int)pg.size();
}

int tl_books_prepare(void* h, int B, const int* slot, const int* n_new) { return ((Books*)h)->prepare(B, slot, n_new); }

int tl_books_commit(void* h, int B, const int* slot, const int* n_new) {
  Books& k = *(Books*)h;
  for (int b = 0; b < B; ++b) {
    if (!k.slots.holds(slot[b])) return fail(MISUSE, "slot %d is not held", slot[b]);
    k.length[slot[b]] += n_new[b];
  }
  return OK;
}

// would new sequences of these final lengths find slots and pages now?
int tl_books_fits(void* h, int n, const long* lengths) {
  Books& k = *(Books*)h;
  if (n > k.slots.n_free()) return 0;
  for (auto& g : k.groups) {
    long need = 0;
    for (int i = 0; i < n; ++i) need += g.pages_needed(lengths[i]);
    if (need > g.pool.n_free()) return 0;
  }
  return 1;
}

// invariants: no page or slot lost, held twice, or both free and held
int tl_books_check(void* h) {
  Books& k = *(Books*)h;
  if (int rc = k.slots.check()) return rc;
  for (size_t gi = 0; gi < k.groups.size(); ++gi) {
    Group& g = k.groups[gi];
    if (int rc = g.pool.check()) return rc;
    std::vector<uint8_t> seen(g.pool.n, 0);
    int held = 0;
    for (int s = 0; s < k.slots.n; ++s) {
      if (!k.slots.held[s]) {
        if (!g.pages[s].empty()) return fail(MISUSE, "free slot %d holds pages", s);
        continue;
      }
      for (int p : g.pages[s]) {
        if (!g.pool.holds(p)) return fail(MISUSE, "slot %d lists page %d, which is not held", s, p);
        if (seen[p]) return fail(MISUSE, "page %d is held by two sequences", p);
        seen[p] = 1;
        ++held;
      }
      if ((int)g.pages[s].size() < g.pages_needed(k.length[s]))
        return fail(MISUSE, "slot %d has %zu pages for %ld positions", s, g.pages[s].size(), k.length[s]);
    }
    if (held != g.pool.n - g.pool.n_free()) return fail(MISUSE, "a page is held by no sequence");
  }
  return OK;
}

// Column offsets (and their total) at which sequences lie when each is given room from the
// last multiple of 64 below its cached length up to its end, rounded up to 64: positions that
// are multiples of 64 then lie on columns that are.  The total is the row length of buffers
// laid out so; it avoids multiples of 512, which would put all rows on the same memory channels.
long tl_aligned_columns(int B, const long* n_cached, const long* n_new, int* off) {
  long total = 0;
  for (int b = 0; b < B; ++b) {
    off[b] = (int)total;
    total += ((n_cached[b] % PAGE) + n_new[b] + PAGE - 1) / PAGE * PAGE;
  }
  if (total % 512 == 0) total += PAGE;
  return total;
}

// ---- a step's batch as one int32 array ------------------------------------------------
// Entry b brings n_new[b] tokens (`tokens`, all entries in a row; ignored with token_rows) and
// wants the logits at n_want[b] of them (`want`, indices among the entry's own tokens, all
// entries in a row).  Checks the entries, gets their pages, and writes, one after the other:
// tokens, row positions, row -> sequence, prefix sums [B+1], slots, lengths before, lengths
// after, wanted rows, aligned column offsets, one page table [B, width] per group, and
// token_rows if given.  sizes[] receives the lengths of the pieces (9 + groups (+1)); info[]
// = {rows, wanted, all single, most new tokens, longest length after, aligned columns, pieces,
// width of group 0, width of group 1, ...}.  Returns the number of ints written through *n_out.
int tl_pack_step(void* h, int B, const int* slot, const int* n_new, const int* tokens, const int* n_want,
                 const int* want, int vocab, const int* token_rows, int* out, long capacity, int* sizes,
                 long* info, long* n_out) {
  Books& k = *(Books*)h;
  if (B < 1) return fail(BAD_STEP, "a step needs at least one sequence");
  long N = 0, NW = 0;
  for (int b = 0; b < B; ++b) {
    if (!k.slots.holds(slot[b])) return fail(BAD_STEP, "entry %d: slot %d is not held", b, slot[b]);
    if (n_new[b] < 1) return fail(BAD_STEP, "entry %d: a sequence must bring at least one token", b);
    for (int w = 0; w < n_want[b]; ++w)
      if (want[NW + w] < 0 || want[NW + w] >= n_new[b])
        return fail(BAD_STEP, "entry %d: wanted index %d outside its %d tokens", b, want[NW + w], n_new[b]);
    N += n_new[b];
    NW += n_want[b];
  }
  if (token_rows) {
    if (N != B) return fail(BAD_STEP, "tokens on the device: one row index per entry, and one token per entry");
  } else {
    for (long i = 0; i < N; ++i)
      if (tokens[i] < 0 || tokens[i] >= vocab)
        return fail(BAD_STEP, "token id %d is outside the vocabulary of %d", tokens[i], vocab);
  }
  const int G = (int)k.groups.size();
  std::vector<long> before(B), fresh(B);
  for (int b = 0; b < B; ++b) {
    before[b] = k.length[slot[b]];
    fresh[b] = n_new[b];
  }
  if (int rc = k.prepare(B, slot, n_new)) return rc;          // FULL / MISUSE, nothing changed
  std::vector<int> width(G);
  long table_ints = 0;
  for (int g = 0; g < G; ++g) {
    int most = 0;
    for (int b = 0; b < B; ++b) most = std::max(most, (int)k.groups[g].pages[slot[b]].size());
    width[g] = table_width(most, k.groups[g].ring_pages);
    table_ints += (long)B * width[g];
  }
  const long total = 3 * N + (B + 1) + 3L * B + NW + B + table_ints + (token_rows ? B : 0);
  if (total > capacity) return fail(BAD_VALUE, "the step needs %ld ints, the buffer holds %ld", total, capacity);
  int* p = out;
  int piece = 0;
  auto done = [&](long n) { sizes[piece++] = (int)n; p += n; };
  if (token_rows) std::fill(p, p + N, 0); else std::copy(tokens, tokens + N, p);
  done(N);
  long r = 0;
  for (int b = 0; b < B; ++b)
    for (int i = 0; i < n_new[b]; ++i) p[r++] = (int)(before[b] + i);
  done(N);
  r = 0;
  for (int b = 0; b < B; ++b)
    for (int i = 0; i < n_new[b]; ++i) p[r++] = b;
  done(N);
  p[0] = 0;
  for (int b = 0; b < B; ++b) p[b + 1] = p[b] + n_new[b];
  const int* cu = p;
  done(B + 1);
  std::copy(slot, slot + B, p);
  done(B);
  for (int b = 0; b < B; ++b) p[b] = (int)before[b];
  done(B);
  long longest = 0;
  int most_new = 0;
  bool single = true;
  for (int b = 0; b < B; ++b) {
    p[b] = (int)(before[b] + n_new[b]);
    longest = std::max<long>(longest, p[b]);
    most_new = std::max(most_new, n_new[b]);
    single = single && n_new[b] == 1;
  }
  done(B);
  r = 0;
  {
    long w0 = 0;
    for (int b = 0; b < B; ++b) {
      for (int w = 0; w < n_want[b]; ++w) p[r++] = cu[b] + want[w0 + w];
      w0 += n_want[b];
    }
  }
  done(NW);
  const long cols = tl_aligned_columns(B, before.data(), fresh.data(), p);
  done(B);
  for (int g = 0; g < G; ++g) {
    std::fill(p, p + (long)B * width[g], 0);
    for (int b = 0; b < B; ++b) {
      const auto& pg = k.groups[g].pages[slot[b]];
      std::copy(pg.begin(), pg.end(), p + (long)b * width[g]);
    }
    done((long)B * width[g]);
  }
  if (token_rows) {
    std::copy(token_rows, token_rows + B, p);
    done(B);
  }
  info[0] = N; info[1] = NW; info[2] = single; info[3] = most_new; info[4] = longest; info[5] = cols;
  info[6] = piece;
  for (int g = 0; g < G; ++g) info[7 + g] = width[g];
  *n_out = total;
  return OK;
}

}  // extern "C"
