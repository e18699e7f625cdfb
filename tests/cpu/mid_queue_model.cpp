// CPU model of the workgroup's list of mid-size bags (recflex_amd/csrc/include/rfx_mid_queue.h):
// the same function templates the device code runs, with std::atomic-style builtins for the
// list's words.  One thread plays one wavefront of a workgroup: it walks its tiles, now and then
// meets bags that it pushes (summing them itself when the list is full), takes bags from the list
// between tiles, and after its last tile keeps taking until every wavefront has finished and the
// list is empty.  "Summing" a bag reads a plain side value its producer wrote before the push and
// bumps a plain counter of the bag, so that ThreadSanitizer reports a bag handed to two wavefronts
// or handed over without ordering, and the end check finds a bag nobody summed.
//   RELAXED_ENTRY      the entry is stored and loaded without release / acquire
//   NON_ATOMIC_CLAIM   the claim compares and stores in two steps
// (A wavefront that announced its last tile too early would lose nothing -- it takes what it
// pushed itself in its own last round -- only the sharing of those bags.)
#include "rfx_mid_queue.h"

#include <chrono>
#include <cstdio>
#include <random>
#include <thread>
#include <vector>

struct HostMem {
  static int fetch_add(int *p, int v) { return __atomic_fetch_add(p, v, __ATOMIC_RELAXED); }
  static int load(int *p) { return __atomic_load_n(p, __ATOMIC_RELAXED); }
  static bool compare_exchange(int *p, int *expected, int desired) {
#if defined(NON_ATOMIC_CLAIM)
    const int now = __atomic_load_n(p, __ATOMIC_RELAXED);
    if (now != *expected) { *expected = now; return false; }
    std::this_thread::yield();
    __atomic_store_n(p, desired, __ATOMIC_RELAXED);
    return true;
#else
    return __atomic_compare_exchange_n(p, expected, desired, false, __ATOMIC_RELAXED, __ATOMIC_RELAXED);
#endif
  }
#if defined(RELAXED_ENTRY)
  static void store_entry(unsigned long long *p, unsigned long long v) { __atomic_store_n(p, v, __ATOMIC_RELAXED); }
  static unsigned long long load_entry(unsigned long long *p) { return __atomic_load_n(p, __ATOMIC_RELAXED); }
#else
  static void store_entry(unsigned long long *p, unsigned long long v) { __atomic_store_n(p, v, __ATOMIC_RELEASE); }
  static unsigned long long load_entry(unsigned long long *p) { return __atomic_load_n(p, __ATOMIC_ACQUIRE); }
#endif
  static void release_add(int *p, int v) { __atomic_fetch_add(p, v, __ATOMIC_RELEASE); }
  static int acquire_load(int *p) { return __atomic_load_n(p, __ATOMIC_ACQUIRE); }
};

constexpr int CAP = 24;          // small, so that the list also overflows
constexpr int WAVES = 4;
using Queue = rfx::MidQueue<CAP>;

struct Launch {
  Queue q;
  std::vector<int> side;         // plain: written by the producer before the push
  std::vector<int> summed;       // plain: bumped by whoever sums the bag
  std::vector<long long> result; // plain: side value seen by whoever sums the bag
};

static void sum_bag(Launch &l, int feat, int bag) {
  l.result[bag] = static_cast<long long>(feat) * 1000003 + l.side[bag];
  l.summed[bag] += 1;
}

static void drain(Launch &l) {
  unsigned long long v;
  while (rfx::mid_queue_pop_one<HostMem>(&l.q, &v))
    sum_bag(l, static_cast<int>(v >> 32), static_cast<int>(v & 0xffffffffu));
}

static void wavefront(Launch &l, int wave, int tiles, int bags_per_wave, unsigned seed) {
  std::mt19937 rng(seed);
  int next = wave * bags_per_wave, last = next + bags_per_wave;
  for (int t = 0; t < tiles; ++t) {
    const bool final_tile = t == tiles - 1;
    int meet = final_tile ? last - next : static_cast<int>(rng() % 4);
    for (; meet > 0 && next < last; --meet, ++next) {
      l.side[next] = next * 7 + 1;
      if (!rfx::mid_queue_push_one<HostMem>(&l.q, next % 13, next)) sum_bag(l, next % 13, next);
    }
    if (rng() % 3 == 0) std::this_thread::yield();
    if (rfx::mid_queue_pending<HostMem>(&l.q)) drain(l);
  }
  rfx::mid_queue_walk_done_one<HostMem>(&l.q);
  for (;;) {
    const bool open = rfx::mid_queue_open<HostMem>(&l.q);
    if (rfx::mid_queue_pending<HostMem>(&l.q))
      drain(l);
    else if (!open)
      break;
    else
      std::this_thread::yield();
  }
}

int main() {
  const int kLaunches = 400, kTiles = 6, kBagsPerWave = 14;
  long long wrong = 0;
  for (int launch = 0; launch < kLaunches; ++launch) {
    Launch l;
    const int bags = WAVES * kBagsPerWave;
    l.side.assign(bags, 0);
    l.summed.assign(bags, 0);
    l.result.assign(bags, -1);
    for (int i = 0; i < CAP; ++i) l.q.e[i] = Queue::kEmpty;
    l.q.count = 0;
    l.q.taken = 0;
    l.q.walking = WAVES;
    std::vector<std::thread> threads;
    for (int w = 0; w < WAVES; ++w)
      threads.emplace_back(wavefront, std::ref(l), w, kTiles, kBagsPerWave, 977u * launch + w);
    for (auto &t : threads) t.join();
    for (int b = 0; b < bags; ++b)
      if (l.summed[b] != 1 || l.result[b] != static_cast<long long>(b % 13) * 1000003 + b * 7 + 1) ++wrong;
    if (l.q.walking != 0) ++wrong;
  }
  std::printf("%lld bags summed not exactly once or with a wrong value\n", wrong);
  return wrong ? 1 : 0;
}
