// Host test of csrc/wide_schedule.hpp: schedules of the two wave groups of the wide walk kernels.
// Prints one line per case: "<name> <value>".
#include <cstdio>
#include <cstdint>
#include <vector>

#include "wide_schedule.hpp"

using namespace pcm;

static std::vector<int> random_tree(int n, uint32_t seed, int bushiness) {
  // post-order numbering: a node's parent has a larger index; node n - 1 is the root
  std::vector<int> parent(n, -1);
  uint32_t x = seed * 2654435761u + 12345u;
  for (int v = 0; v < n - 1; ++v) {
    x = x * 1664525u + 1013904223u;
    const int span = std::min(n - 1 - v, bushiness);
    parent[v] = v + 1 + (int)((x >> 8) % (uint32_t)span);
  }
  return parent;
}

int main() {
  {   // a chain can only ever use one group: every node needs the tile of the one before, from registers
    std::vector<int> chain = {1, 2, 3, 4, -1};
    const WideSchedule f = wide_two_group_schedule(chain, true), b = wide_two_group_schedule(chain, false);
    std::printf("chain_forward_steps %d\n", f.n_steps);
    std::printf("chain_forward_fault %d\n", wide_schedule_fault(chain, true, f));
    std::printf("chain_backward_steps %d\n", b.n_steps);
    std::printf("chain_backward_fault %d\n", wide_schedule_fault(chain, false, b));
    int one_group = 1;
    for (int v = 0; v < 5; ++v) one_group &= f.group[v] == f.group[0] && b.group[v] == b.group[0];
    std::printf("chain_one_group %d\n", one_group);
  }
  {   // two chains of three under a root: the groups take one chain each
    std::vector<int> par = {1, 2, 6, 4, 5, 6, -1};
    const WideSchedule f = wide_two_group_schedule(par, true);
    std::printf("two_chains_steps %d\n", f.n_steps);
    std::printf("two_chains_fault %d\n", wide_schedule_fault(par, true, f));
    std::printf("two_chains_split %d\n", (int)(f.group[0] != f.group[3] && f.group[0] == f.group[1] && f.group[3] == f.group[4]));
  }
  {   // faults are found: a parent in the slot right after its child of the OTHER group, a slot taken twice
    std::vector<int> par = {2, 2, -1};
    WideSchedule s;
    s.n_steps = 2;
    s.step = {0, 0, 1};
    s.group = {0, 1, 0};   // node 2 (step 1, group 0) needs node 1's tile (group 1, step 0): stored too late
    std::printf("cross_too_early %d\n", wide_schedule_fault(par, true, s));
    s.n_steps = 4;
    s.step = {0, 0, 3};
    std::printf("cross_late_enough %d\n", wide_schedule_fault(par, true, s));
    s.step = {0, 0, 3};
    s.group = {0, 0, 0};
    std::printf("slot_twice %d\n", wide_schedule_fault(par, true, s));
    s.step = {0, 1, 2};
    s.group = {0, 0, 0};   // node 0's tile: neither in registers (two slots back) nor in memory yet at 2*2 - 1 = 3 = 0 + 3: just in time
    std::printf("own_group_two_back %d\n", wide_schedule_fault(par, true, s));
    s.step = {0, 1, 2};
    s.group = {1, 0, 0};   // node 0 in group 1 at step 0: in memory at 1 + 3 = 4 > 3
    std::printf("other_group_two_back %d\n", wide_schedule_fault(par, true, s));
  }
  {   // random trees, both directions: always sound, never longer than one node per step, shorter when bushy
    int faults = 0, too_long = 0, total_nodes = 0, total_steps = 0;
    for (uint32_t seed = 0; seed < 200; ++seed) {
      const int n = 2 + (int)(seed % 61);
      const std::vector<int> par = random_tree(n, seed, 1 + (int)(seed % 7));
      for (int fwd = 0; fwd < 2; ++fwd) {
        const WideSchedule s = wide_two_group_schedule(par, fwd != 0);
        faults += wide_schedule_fault(par, fwd != 0, s) >= 0;
        too_long += s.n_steps > n + 1;
        total_nodes += n;
        total_steps += s.n_steps;
      }
    }
    std::printf("random_faults %d\n", faults);
    std::printf("random_too_long %d\n", too_long);
    std::printf("random_shorter %d\n", (int)(total_steps * 10 < total_nodes * 8));
  }
  return 0;
}
