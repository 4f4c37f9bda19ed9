// Host test of csrc/lean_schedule_check.hpp: hand-made lean schedules, sound and unsound.
// Prints one line per case: "<name> <result>", result = -1 (sound) or step * 16 + wave of a stuck wave.
#include <cstdio>
#include <vector>

#include "lean_schedule_check.hpp"

using namespace pcm;

struct Sched {
  int stride;
  std::vector<int32_t> f;
  explicit Sched(int steps) : stride(steps), f((size_t)kLeanCheckFields * kLeanCheckWaves * steps, 0) {
    for (int w = 0; w < kLeanCheckWaves; ++w)
      for (int s = 0; s < steps; ++s) {
        at(kLeanCheckSlots, w, s) = (int32_t)(0xffffff00u | 99u);   // idle: no children, trash slot 99
        for (int c = 0; c < 3; ++c) at(kLeanCheckA1 + c, w, s) = -1;
      }
  }
  int32_t& at(int field, int w, int s) { return f[((size_t)field * kLeanCheckWaves + w) * stride + s]; }
  // forward item: own slot / turn, up to three (child slot, turn) pairs
  void fwd(int w, int s, int out, int out_turn, std::vector<std::pair<int, int>> kids = {}) {
    uint32_t slots = 0xffffff00u | (uint32_t)out, turns = (uint32_t)out_turn;
    for (size_t c = 0; c < kids.size(); ++c) {
      slots = (slots & ~(0xffu << (8 * (c + 1)))) | ((uint32_t)kids[c].first << (8 * (c + 1)));
      turns |= (uint32_t)kids[c].second << (8 * (c + 1));
    }
    at(kLeanCheckSlots, w, s) = (int32_t)slots;
    at(kLeanCheckTurns, w, s) = (int32_t)turns;
  }
  // backward item: the slot its ratio tile comes in (99: the root), inner children's (slot, turn)
  void bwd(int w, int s, int in, int in_turn, std::vector<std::pair<int, int>> kids = {}) {
    fwd(w, s, in, in_turn, kids);
    for (size_t c = 0; c < kids.size(); ++c) at(kLeanCheckA1 + (int)c, w, s) = (int32_t)(c << 3);   // inner child: even
  }
};

int main() {
  {   // a chain of three nodes handing tiles up through two slots
    Sched q(3);
    q.fwd(0, 0, 0, 0);
    q.fwd(5, 1, 1, 0, {{0, 0}});
    q.fwd(2, 2, 99, 0, {{1, 0}});
    std::printf("forward_chain %d\n", lean_schedule_stuck_at(q.f.data(), q.stride, 3, true, 99));
  }
  {   // producer and consumer in the same step on different waves: no barrier, so this is sound
    Sched q(1);
    q.fwd(0, 0, 0, 0);
    q.fwd(1, 0, 99, 0, {{0, 0}});
    std::printf("forward_same_step %d\n", lean_schedule_stuck_at(q.f.data(), q.stride, 1, true, 99));
  }
  {   // a slot reused: second tile is turn 1, its writer waits for the first reader
    Sched q(4);
    q.fwd(0, 0, 0, 0);
    q.fwd(1, 1, 99, 0, {{0, 0}});
    q.fwd(0, 2, 0, 1);
    q.fwd(1, 3, 99, 0, {{0, 1}});
    std::printf("forward_reuse %d\n", lean_schedule_stuck_at(q.f.data(), q.stride, 4, true, 99));
  }
  {   // the consumer names a turn nobody posts
    Sched q(2);
    q.fwd(0, 0, 0, 0);
    q.fwd(1, 1, 99, 0, {{0, 1}});
    std::printf("forward_wrong_turn %d\n", lean_schedule_stuck_at(q.f.data(), q.stride, 2, true, 99));
  }
  {   // one wave is to read a tile it only writes in its next step
    Sched q(2);
    q.fwd(3, 0, 99, 0, {{0, 0}});
    q.fwd(3, 1, 0, 0);
    std::printf("forward_own_future %d\n", lean_schedule_stuck_at(q.f.data(), q.stride, 2, true, 99));
  }
  {   // a slot taken again while its first tile was never read
    Sched q(2);
    q.fwd(0, 0, 0, 0);
    q.fwd(4, 1, 0, 1);
    std::printf("forward_overwrite %d\n", lean_schedule_stuck_at(q.f.data(), q.stride, 2, true, 99));
  }
  {   // backward: the root fills two children's slots, they read them, one hands on to a grandchild
    Sched q(3);
    q.bwd(0, 0, 99, 0, {{0, 0}, {1, 0}});
    q.bwd(0, 1, 0, 0, {{2, 0}});
    q.bwd(1, 1, 1, 0);
    q.bwd(7, 2, 2, 0);
    std::printf("backward_tree %d\n", lean_schedule_stuck_at(q.f.data(), q.stride, 3, false, 99));
  }
  {   // backward: a child scheduled on its parent's wave before the parent
    Sched q(2);
    q.bwd(0, 0, 0, 0);
    q.bwd(0, 1, 99, 0, {{0, 0}});
    std::printf("backward_child_first %d\n", lean_schedule_stuck_at(q.f.data(), q.stride, 2, false, 99));
  }
  return 0;
}
