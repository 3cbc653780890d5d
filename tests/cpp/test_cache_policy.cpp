// Host-only test of the eviction rule shared by a plan's work-list cache and the operator's
// cache of plans (fbgemm_amd/csrc/cache_policy.h). Built with g++ and run by tests/test_cache_policy.py.
#include <cstdio>
#include <map>
#include <random>

#include "../../fbgemm_amd/csrc/cache_policy.h"

struct Entry {
  bool held;
  long last_use;
};

static int failures = 0;
#define CHECK(c, ...) do { if (!(c)) { ++failures; printf("FAIL line %d: ", __LINE__); printf(__VA_ARGS__); printf("\n"); } } while (0)

int main() {
  auto held = [](const Entry& e) { return e.held; };
  auto used = [](const Entry& e) { return e.last_use; };
  std::map<int, Entry> m;
  CHECK(fbgemm_amd::least_recently_used_not_held(m, held, used) == m.end(), "an empty cache has no victim");
  m = {{1, {false, 5}}, {2, {false, 3}}, {3, {false, 9}}};
  CHECK(fbgemm_amd::least_recently_used_not_held(m, held, used)->first == 2, "the least recently used entry goes");
  m[2].held = true; // a captured graph holds entry 2: the next oldest goes instead
  CHECK(fbgemm_amd::least_recently_used_not_held(m, held, used)->first == 1, "a held entry is passed over");
  m[1].held = m[3].held = true;
  CHECK(fbgemm_amd::least_recently_used_not_held(m, held, used) == m.end(), "with every entry held nothing goes");

  // A cache of 16 driven the way a plan drives it: a new key per step, some entries held for
  // good (as a stream capture pins them). Held entries are never dropped, the others never
  // exceed the bound, and what goes is always the oldest of those that may.
  std::mt19937 rng(7);
  std::map<int, Entry> cache;
  const size_t bound = 16;
  long clock = 0;
  int held_count = 0;
  for (int step = 0; step < 2000; ++step) {
    const int key = (int)(rng() % 60);
    auto it = cache.find(key);
    if (it == cache.end()) {
      if (cache.size() >= bound) {
        auto victim = fbgemm_amd::least_recently_used_not_held(cache, held, used);
        if (victim != cache.end()) {
          CHECK(!victim->second.held, "a held entry was chosen");
          for (const auto& kv : cache)
            CHECK(kv.second.held || kv.second.last_use >= victim->second.last_use, "an older entry that may go was passed over");
          cache.erase(victim);
        }
      }
      it = cache.emplace(key, Entry{false, 0}).first;
    }
    it->second.last_use = ++clock;
    if (!it->second.held && rng() % 31 == 0 && held_count < 20) {
      it->second.held = true;
      ++held_count;
    }
    size_t free_entries = 0;
    int still_held = 0;
    for (const auto& kv : cache) {
      if (kv.second.held) ++still_held;
      else ++free_entries;
    }
    CHECK(still_held == held_count, "a held entry was dropped (%d of %d left)", still_held, held_count);
    CHECK(free_entries <= bound, "%zu entries that may go, bound %zu", free_entries, bound);
    CHECK(cache.size() <= bound + (size_t)held_count, "cache of %zu", cache.size());
  }
  CHECK(held_count > 16, "the run should end with more held entries than the bound (%d)", held_count);
  printf("%s: %d failure(s)\n", failures ? "FAILED" : "PASSED", failures);
  return failures ? 1 : 0;
}
