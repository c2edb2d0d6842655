// Random sequences of operations on the host library's books and packer, for a build with
// the address and undefined-behaviour sanitizers: every step is checked against a model of
// plain containers, and the library's own invariants are asked for all along.
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <vector>

extern "C" {
const char* tl_host_last_error();
void* tl_books_new(int max_slots, int n_groups, const int* ring_pages, const int* n_pages);
void tl_books_delete(void* h);
int tl_books_alloc_slot(void* h, int* out);
int tl_books_free_slot(void* h, long slot);
long tl_books_length(void* h, long slot);
int tl_books_free_pages(void* h, int group);
int tl_books_pages(void* h, int group, long slot, int* out, int capacity);
int tl_books_commit(void* h, int B, const int* slot, const int* n_new);
int tl_books_check(void* h);
int tl_pack_step(void* h, int B, const int* slot, const int* n_new, const int* tokens, const int* n_want,
                 const int* want, int vocab, const int* token_rows, int* out, long capacity, int* sizes,
                 long* info, long* n_out);
}

#define REQUIRE(c)                                                                       \
  do {                                                                                   \
    if (!(c)) {                                                                          \
      std::fprintf(stderr, "line %d: %s failed (%s)\n", __LINE__, #c, tl_host_last_error()); \
      return 1;                                                                          \
    }                                                                                    \
  } while (0)

int main(int argc, char** argv) {
  const unsigned seed = argc > 1 ? std::atoi(argv[1]) : 1;
  std::mt19937 rng(seed);
  const int ring[2] = {3, 1 << 24}, pages[2] = {40, 40};
  const int max_slots = 6, vocab = 97;
  void* h = tl_books_new(max_slots, 2, ring, pages);
  std::map<int, long> length;                      // the model: slot -> positions held
  std::vector<int> out(1 << 16), sizes(32);
  std::vector<long> info(32);
  for (int it = 0; it < 4000; ++it) {
    const int op = rng() % 10;
    if (op < 2 && (int)length.size() < max_slots) {
      int s = -1;
      REQUIRE(tl_books_alloc_slot(h, &s) == 0 && !length.count(s));
      length[s] = 0;
    } else if (op < 3 && !length.empty()) {
      auto itr = length.begin();
      std::advance(itr, rng() % length.size());
      REQUIRE(tl_books_free_slot(h, itr->first) == 0);
      REQUIRE(tl_books_free_slot(h, itr->first) != 0);            // twice: refused
      length.erase(itr);
    } else if (!length.empty()) {
      std::vector<int> slot, n_new, tokens, n_want, want;
      for (auto& kv : length)
        if (rng() % 2) {
          const int n = (rng() % 4 == 0) ? 1 + rng() % 200 : 1;
          slot.push_back(kv.first);
          n_new.push_back(n);
          for (int i = 0; i < n; ++i) tokens.push_back(rng() % vocab);
          const int w = rng() % 3;
          n_want.push_back(w);
          for (int i = 0; i < w; ++i) want.push_back(rng() % n);
        }
      if (slot.empty()) continue;
      const int free0 = tl_books_free_pages(h, 0), free1 = tl_books_free_pages(h, 1);
      long n_out = 0;
      const int rc = tl_pack_step(h, (int)slot.size(), slot.data(), n_new.data(), tokens.data(), n_want.data(),
                                  want.data(), vocab, nullptr, out.data(), (long)out.size(), sizes.data(),
                                  info.data(), &n_out);
      if (rc != 0) {                                               // full: nothing may have changed
        REQUIRE(rc == 1);
        REQUIRE(tl_books_free_pages(h, 0) == free0 && tl_books_free_pages(h, 1) == free1);
        auto itr = length.begin();                                 // make room
        REQUIRE(tl_books_free_slot(h, itr->first) == 0);
        length.erase(itr);
        continue;
      }
      long rows = 0;
      for (int n : n_new) rows += n;
      REQUIRE(info[0] == rows && n_out <= (long)out.size());
      REQUIRE(tl_books_commit(h, (int)slot.size(), slot.data(), n_new.data()) == 0);
      for (size_t b = 0; b < slot.size(); ++b) {
        length[slot[b]] += n_new[b];
        REQUIRE(tl_books_length(h, slot[b]) == length[slot[b]]);
        int pg[64];
        const long need = (length[slot[b]] + 63) / 64;
        REQUIRE(tl_books_pages(h, 0, slot[b], pg, 64) == (need < 3 ? need : 3));      // the ring of the window
        REQUIRE(tl_books_pages(h, 1, slot[b], pg, 64) == need);
      }
    }
    REQUIRE(tl_books_check(h) == 0);
  }
  for (auto& kv : length) REQUIRE(tl_books_free_slot(h, kv.first) == 0);
  REQUIRE(tl_books_free_pages(h, 0) == 40 && tl_books_free_pages(h, 1) == 40 && tl_books_check(h) == 0);
  tl_books_delete(h);
  std::puts("ok");
  return 0;
}
