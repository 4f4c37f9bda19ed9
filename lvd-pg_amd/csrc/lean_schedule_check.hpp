// Host-side proof that a lean walk schedule cannot leave a wave waiting for ever.
//
// The lean walk kernels have no barrier between steps: tiles pass from wave to wave through LDS slots whose
// state words go 2t (free for the slot's t-th tile) -> 2t + 1 (tile there) -> 2t + 2 (read, free again), all
// modulo 256; a producer waits for 2t, the one consumer for 2t + 1, and every wave works through its steps in
// order.  Whether that terminates depends on the schedule alone, so it is checked when the schedule is built:
// the waits and posts of every wave are replayed on the host, each wave advancing whenever the state it waits
// for is there.  A slot's state is only ever changed by the one operation that is next in the slot's chain, so
// the replay's order does not matter: either every wave reaches its end, or the waves that are left wait for
// states nobody will post -- on the device they would run into their poll limit and void the pass.
//
// Plain C++ (no HIP): also compiled into a host test.
#pragma once

#include <cstdint>
#include <vector>

namespace pcm {

// field rows of a lean schedule, [field][wave][stride]; the names are those of hclt_walk_lean.hip.hpp
constexpr int kLeanCheckA1 = 2, kLeanCheckSlots = 6, kLeanCheckTurns = 8, kLeanCheckFields = 9, kLeanCheckWaves = 16;

struct LeanSlotOp {
  uint8_t slot, value;
  bool wait;   // wait until the slot's state equals value / set the slot's state to value
};

// the slot operations of wave w in step s, in the order the kernels issue them
inline void lean_step_ops(const int32_t* f, int stride, int w, int s, bool forward, int trash_slot, std::vector<LeanSlotOp>& ops) {
  auto get = [&](int field) { return (uint32_t)f[((size_t)field * kLeanCheckWaves + w) * stride + s]; };
  const uint32_t slots = get(kLeanCheckSlots), turns = get(kLeanCheckTurns);
  auto sl = [&](int c) { return (uint8_t)((slots >> (8 * c)) & 0xffu); };
  auto st = [&](int c, int add) { return (uint8_t)((2u * ((turns >> (8 * c)) & 0x7fu) + (uint32_t)add) & 0xffu); };
  if (forward) {
    for (int c = 1; c <= 3; ++c)
      if (sl(c) != 0xffu) {   // a child's tile: wait for it, read it, free the slot
        ops.push_back({sl(c), st(c, 1), true});
        ops.push_back({sl(c), st(c, 2), false});
      }
    if (sl(0) != (uint8_t)trash_slot) {   // the node's own tile goes into its slot once that is free
      ops.push_back({sl(0), st(0, 0), true});
      ops.push_back({sl(0), st(0, 1), false});
    }
    return;
  }
  bool inner[4] = {false, false, false, false};
  for (int c = 1; c <= 3; ++c) {
    const int32_t a = (int32_t)get(kLeanCheckA1 + c - 1);
    inner[c] = a >= 0 && !(a & 1);
  }
  for (int c = 1; c <= 3; ++c)
    if (inner[c]) ops.push_back({sl(c), st(c, 0), true});   // the children's slots must be free
  if (sl(0) != (uint8_t)trash_slot) {                       // the node's ratio tile, left by its parent
    ops.push_back({sl(0), st(0, 1), true});
    ops.push_back({sl(0), st(0, 2), false});
  }
  if (inner[1])
    for (int c = 1; c <= 3; ++c)
      if (inner[c]) ops.push_back({sl(c), st(c, 1), false});
}

// -1 if every wave gets through its `n_steps` steps; otherwise step * 16 + wave of the first wave found stuck.
inline int lean_schedule_stuck_at(const int32_t* f, int stride, int n_steps, bool forward, int trash_slot) {
  std::vector<std::vector<LeanSlotOp>> ops(kLeanCheckWaves);
  std::vector<std::vector<int>> step_of(kLeanCheckWaves);
  for (int w = 0; w < kLeanCheckWaves; ++w)
    for (int s = 0; s < n_steps; ++s) {
      const size_t before = ops[w].size();
      lean_step_ops(f, stride, w, s, forward, trash_slot, ops[w]);
      step_of[w].resize(ops[w].size(), s);
      (void)before;
    }
  uint8_t state[256] = {0};
  std::vector<size_t> pos(kLeanCheckWaves, 0);
  for (bool moved = true; moved;) {
    moved = false;
    for (int w = 0; w < kLeanCheckWaves; ++w)
      while (pos[w] < ops[w].size()) {
        const LeanSlotOp& o = ops[w][pos[w]];
        if (o.wait && state[o.slot] != o.value) break;
        if (!o.wait) state[o.slot] = o.value;
        ++pos[w];
        moved = true;
      }
  }
  for (int w = 0; w < kLeanCheckWaves; ++w)
    if (pos[w] < ops[w].size()) return step_of[w][pos[w]] * kLeanCheckWaves + w;
  return -1;
}

}  // namespace pcm
