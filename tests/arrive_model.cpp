// A thread model of the hand-over protocol of blok_amd/csrc/kx_arrive.h, for ThreadSanitizer.
//
// Each thread plays a workgroup: in every round it writes its results with plain stores into the slots of the
// (up to two) blocks it contributes to, counts itself in on those blocks' counters, and where it is the last one
// it reads every contributor's slot, checks the values and resets the counter -- exactly what the routed down
// launch (two counters per workgroup), the router GEMV and the q_b GEMV do.  Rounds are separated by a barrier,
// as launches are by the stream.  Built with the protocol's release/acquire ordering the program is race-free
// and every block is finished exactly once per round; built with -DKX_ARRIVE_ORDER=__ATOMIC_RELAXED the same
// program is reported by ThreadSanitizer, which is what shows that the check can fail.
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <atomic>
#include <thread>
#include <vector>
#include "../blok_amd/csrc/kx_arrive.h"

constexpr int GROUPS = 8, BLOCKS = 5, ROUNDS = 400;

static int counter[BLOCKS];
static long slot[BLOCKS][GROUPS];        // plain data: what the groups hand over
static std::atomic<int> finished[BLOCKS];
static std::atomic<int> errors{0};
static pthread_barrier_t round_barrier;

// group g contributes to block g % BLOCKS and, every second group, also to block (g / 2) % BLOCKS
static int block_a(int g) { return g % BLOCKS; }
static int block_b(int g) { return g % 2 ? -1 : (g / 2) % BLOCKS; }
static int contributors(int blk) {
  int n = 0;
  for (int g = 0; g < GROUPS; ++g) n += (block_a(g) == blk) + (block_b(g) == blk && block_b(g) != block_a(g));
  return n;
}

static void finish(int blk, int round) {
  for (int g = 0; g < GROUPS; ++g) {
    const bool in = block_a(g) == blk || block_b(g) == blk;
    if (in && slot[blk][g] != (long)round * 1000 + g) errors.fetch_add(1);
  }
  finished[blk].fetch_add(1);
  kx_arrive_reset(&counter[blk]);
}

static void group(int g) {
  for (int round = 0; round < ROUNDS; ++round) {
    const int blks[2] = {block_a(g), block_b(g) == block_a(g) ? -1 : block_b(g)};
    for (int blk : blks)
      if (blk >= 0) slot[blk][g] = (long)round * 1000 + g;
    if ((g + round) % 3 == 0) std::this_thread::yield();
    for (int blk : blks)
      if (blk >= 0 && kx_arrive_is_last(&counter[blk], contributors(blk))) finish(blk, round);
    pthread_barrier_wait(&round_barrier);
    if (g == 0) {
      for (int b = 0; b < BLOCKS; ++b) {
        const int want = contributors(b) > 0 ? round + 1 : 0;
        if (finished[b].load() != want || __atomic_load_n(&counter[b], __ATOMIC_RELAXED) != 0) errors.fetch_add(1);
      }
    }
    pthread_barrier_wait(&round_barrier);
  }
}

int main() {
  pthread_barrier_init(&round_barrier, nullptr, GROUPS);
  std::vector<std::thread> th;
  for (int g = 0; g < GROUPS; ++g) th.emplace_back(group, g);
  for (auto &t : th) t.join();
  printf("rounds=%d errors=%d\n", ROUNDS, errors.load());
  return errors.load() ? 1 : 0;
}
