// CPU model of the arrival protocol (recflex_amd/csrc/include/rfx_arrival.h): the same function
// templates the device code runs, with plain stores and loads for the slots and a
// release/acquire counter.  One thread plays one part of one bag; tasks are drawn in shuffled
// order by a few worker threads; several "launches" reuse the same slots and counters.  Built
// with -fsanitize=thread: a step moved out of the protocol's order (ARRIVE_BEFORE_STORES,
// COMBINE_BY_ANYONE) is a data race the sanitizer reports, and a wrong sum besides.
#include "rfx_arrival.h"

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <random>
#include <thread>
#include <vector>

struct HostMem {
  static void store_slot(unsigned int *p, const float v) { std::memcpy(p, &v, 4); }      // plain
  static float load_slot(const unsigned int *p) { float v; std::memcpy(&v, p, 4); return v; }
  static void release() {}          // the counter's release ordering carries the slots
  static int arrive(int *c) { return __atomic_fetch_add(c, 1, __ATOMIC_ACQ_REL); }
  static void reset(int *c) { __atomic_store_n(c, 0, __ATOMIC_RELEASE); }
};

constexpr int D = 24;

static float part_value(int launch, int bag, int part, int j) {
  return static_cast<float>((launch * 7 + bag * 3 + part * 5 + j) % 17 - 8);   // small integers: exact sums
}

struct Bag {
  int parts;
  std::vector<unsigned int> slots;   // parts x D
  int counter = 0;
  std::vector<float> out;            // D
};

static void run_part(Bag &b, int launch, int bag, int part) {
  using namespace rfx;
#if defined(ARRIVE_BEFORE_STORES)
  const bool last = arrival_is_last<HostMem>(&b.counter, b.parts);
  for (int j = 0; j < D; ++j) arrival_store<HostMem>(b.slots.data(), part, D, j, part_value(launch, bag, part, j));
#else
  for (int j = 0; j < D; ++j) arrival_store<HostMem>(b.slots.data(), part, D, j, part_value(launch, bag, part, j));
  HostMem::release();
  const bool last = arrival_is_last<HostMem>(&b.counter, b.parts);
#endif
#if defined(COMBINE_BY_ANYONE)
  if (!last && part != 0) return;
#else
  if (!last) return;
#endif
  for (int j = 0; j < D; ++j) b.out[j] = arrival_combine<HostMem>(b.slots.data(), b.parts, D, j);
  if (last) HostMem::reset(&b.counter);
}

int main() {
  const int kBags = 96, kLaunches = 12, kThreads = 8;
  std::vector<Bag> bags(kBags);
  const int part_choices[] = {2, 3, 8, 64};
  std::vector<std::pair<int, int>> tasks;
  for (int b = 0; b < kBags; ++b) {
    bags[b].parts = part_choices[b % 4];
    bags[b].slots.assign(bags[b].parts * D, 0xdeadbeefu);
    bags[b].out.assign(D, -1.f);
    for (int p = 0; p < bags[b].parts; ++p) tasks.emplace_back(b, p);
  }
  std::mt19937 rng(12345);
  int bad = 0;
  for (int launch = 0; launch < kLaunches; ++launch) {
    std::shuffle(tasks.begin(), tasks.end(), rng);
    std::atomic<size_t> next{0};
    std::vector<std::thread> workers;
    for (int t = 0; t < kThreads; ++t)
      workers.emplace_back([&] {
        for (size_t i = next.fetch_add(1); i < tasks.size(); i = next.fetch_add(1))
          run_part(bags[tasks[i].first], launch, tasks[i].first, tasks[i].second);
      });
    for (auto &w : workers) w.join();
    for (int b = 0; b < kBags; ++b) {
      if (bags[b].counter != 0) ++bad;                       // back at zero for the next launch
      for (int j = 0; j < D; ++j) {
        float want = 0.f;
        for (int p = 0; p < bags[b].parts; ++p) want += part_value(launch, b, p, j);
        if (bags[b].out[j] != want) ++bad;
      }
    }
  }
  std::printf("arrival protocol model: %d launches x %d bags, %d wrong values or counters\n", kLaunches,
              kBags, bad);
  return bad ? 1 : 0;
}
