// Schedule of the wide walk kernels (hclt_wide.hip): pure host code, no device types, so that it can be
// compiled and tested without a GPU.
//
// A workgroup of the wide walks has two groups of waves that work half a step apart: while one group runs a
// node's matrix instructions, the other sums, exponentiates and exchanges the operands of ITS node, and the
// two swap roles at every barrier.  In units of half a step, the slot (step t, group g) starts at 2t + g; its
// tile is stored at the end of the slot, and the group waits for its stores at the barrier in the middle of its
// next slot, so the tile is in memory for the other group at 2t + g + 3.  The tiles a node needs are requested
// during the second half of the same group's slot before, at 2t + g - 1, so they must be in memory by then --
// unless it is the tile of that very slot before, which is still in the group's registers.  Going up the tree (forward) a node needs
// the tiles of its non-leaf children; going down (backward) the flow tile of its parent.
#pragma once

#include <algorithm>
#include <vector>

namespace pcm {

struct WideSchedule {
  int n_steps = 0;
  std::vector<int> step, group;   // per node
};

// may node n, with the tiles of `deps` as operands, take slot (t, g)?
inline bool wide_slot_ok(const WideSchedule& s, const std::vector<int>& deps, int t, int g) {
  int in_registers = 0;
  for (int x : deps) {
    if (s.step[x] < 0) return false;
    const int done = 2 * s.step[x] + s.group[x] + 3;
    if (done <= 2 * t + g - 1) continue;
    if (s.group[x] == g && s.step[x] == t - 1 && ++in_registers == 1) continue;
    return false;
  }
  return true;
}

// parent[n] = parent node or -1; greedy list scheduling, the node with the longest way still to go first
inline WideSchedule wide_two_group_schedule(const std::vector<int>& parent, bool forward) {
  const int n = (int)parent.size();
  std::vector<std::vector<int>> deps(n);
  std::vector<int> depth(n, 0), height(n, 1);
  for (int v = 0; v < n; ++v) {
    if (forward) { if (parent[v] >= 0) deps[parent[v]].push_back(v); }
    else if (parent[v] >= 0) deps[v].push_back(parent[v]);
    int d = 0;
    for (int u = v; parent[u] >= 0; u = parent[u]) ++d;
    depth[v] = d;
  }
  for (int d = n; d >= 0; --d)   // heights, deepest nodes first
    for (int v = 0; v < n; ++v)
      if (depth[v] == d && parent[v] >= 0) height[parent[v]] = std::max(height[parent[v]], height[v] + 1);
  const std::vector<int>& priority = forward ? depth : height;
  WideSchedule s;
  s.step.assign(n, -1);
  s.group.assign(n, -1);
  int placed = 0;
  for (int time = 0; placed < n; ++time) {
    const int t = time / 2, g = time % 2;
    int best = -1;
    for (int v = 0; v < n; ++v) {
      if (s.step[v] >= 0 || !wide_slot_ok(s, deps[v], t, g)) continue;
      if (best < 0 || priority[v] > priority[best]) best = v;
    }
    if (best < 0) continue;   // (the root of the remaining work is always placeable two half-steps later at most)
    s.step[best] = t;
    s.group[best] = g;
    s.n_steps = t + 1;
    ++placed;
  }
  return s;
}

// -1 when every node's operands are where its slot expects them and no slot is taken twice, else the first node at fault
inline int wide_schedule_fault(const std::vector<int>& parent, bool forward, const WideSchedule& s) {
  const int n = (int)parent.size();
  std::vector<int> taken((size_t)std::max(s.n_steps, 0) * 2, -1);
  for (int v = 0; v < n; ++v) {
    if (s.step[v] < 0 || s.step[v] >= s.n_steps || s.group[v] < 0 || s.group[v] > 1) return v;
    int& owner = taken[(size_t)s.step[v] * 2 + s.group[v]];
    if (owner >= 0) return v;
    owner = v;
    std::vector<int> deps;
    if (forward) { for (int c = 0; c < n; ++c) if (parent[c] == v) deps.push_back(c); }
    else if (parent[v] >= 0) deps.push_back(parent[v]);
    if (!wide_slot_ok(s, deps, s.step[v], s.group[v])) return v;
  }
  return -1;
}

}  // namespace pcm
