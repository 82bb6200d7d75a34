// smem.cpp — static planning of a workgroup's shared memory (LDS) and the check for the barriers a
// sequence of accesses to it needs.  Host code only.
//
// kapy_smem_plan follows the reference's allocator (lib/Analysis/AllocAnalysis.cpp:187-270): every
// buffer starts at offset 0; two buffers interfere when their live ranges and their byte ranges both
// intersect; the interference graph is coloured first-fit in buffer order; a buffer of colour 0 goes to
// offset 0, any other one behind the farthest end of its neighbours, rounded up to the alignment; graph
// and placement are rebuilt until nothing interferes.  As written the reference sends colour-0 buffers
// back to offset 0 on every pass, which can undo an earlier bump and cycle (three buffers A, B, C with B
// overlapping both in time and size(C) > size(A) do); when a placement repeats, this planner continues
// with the rule of the allocator the reference derives from (colour-0 buffers keep their offset), under
// which offsets only grow, and as a last resort lays the buffers end to end.
//
// kapy_smem_barriers follows lib/Analysis/BlockAnalysis.cpp:37-88 (fixed point over the blocks of a
// control-flow graph) and :114-169 (per op): a barrier op clears the pending reads and writes; a
// cp_async_wait_group that no barrier follows gets one after it; any other op whose byte ranges meet the
// pending ones as read-after-write, write-after-read or write-after-write gets a barrier before it, and its
// own ranges become pending.
#include <algorithm>
#include <deque>
#include <set>
#include <utility>
#include <vector>

#include "common.hpp"

namespace kapy {
namespace {

inline bool meets(int64_t a0, int64_t a1, int64_t b0, int64_t b1) { return a0 < b1 && b0 < a1; }

struct Pending {
  std::set<std::pair<int64_t, int64_t>> reads, writes;
  void join(const Pending &o) {
    reads.insert(o.reads.begin(), o.reads.end());
    writes.insert(o.writes.begin(), o.writes.end());
  }
  void sync() { reads.clear(); writes.clear(); }
  static bool meet(const std::set<std::pair<int64_t, int64_t>> &x, const std::set<std::pair<int64_t, int64_t>> &y) {
    for (auto &a : x)
      for (auto &b : y)
        if (meets(a.first, a.second, b.first, b.second)) return true;
    return false;
  }
  bool hazard(const Pending &op) const { return meet(writes, op.reads) || meet(reads, op.writes) || meet(writes, op.writes); }
  bool covers(const Pending &o) const {
    return std::includes(reads.begin(), reads.end(), o.reads.begin(), o.reads.end()) &&
           std::includes(writes.begin(), writes.end(), o.writes.begin(), o.writes.end());
  }
};

}  // namespace
}  // namespace kapy

using namespace kapy;

extern "C" int64_t kapy_smem_plan(kapy_smem_buffer *buffers, int32_t n, int64_t alignment) {
  if (n < 0 || (n > 0 && !buffers)) return fail(KAPY_ERR_INVALID, "smem_plan: null buffers");
  if (alignment == 0) alignment = 128;
  if (alignment < 0 || (alignment & (alignment - 1))) return fail(KAPY_ERR_INVALID, "smem_plan: alignment must be a power of two");
  for (int i = 0; i < n; ++i) {
    if (buffers[i].size < 0 || buffers[i].live_end < buffers[i].live_start) return fail(KAPY_ERR_INVALID, "smem_plan: buffer %d has a negative size or live range", i);
    buffers[i].offset = 0;
  }
  auto align_up = [&](int64_t x) { return (x + alignment - 1) & ~(alignment - 1); };
  std::vector<std::vector<int>> graph(n);
  auto build_graph = [&]() {
    bool any = false;
    for (int i = 0; i < n; ++i) {
      graph[i].clear();
      for (int j = 0; j < n; ++j) {
        if (i == j) continue;
        const kapy_smem_buffer &a = buffers[i], &b = buffers[j];
        if (meets(a.live_start, a.live_end, b.live_start, b.live_end) && meets(a.offset, a.offset + a.size, b.offset, b.offset + b.size)) {
          graph[i].push_back(j);
          any = true;
        }
      }
    }
    return any;
  };
  int64_t total = 0;
  auto place = [&](bool colour0_returns_to_zero) {
    std::vector<int> colour(n, -1);
    std::vector<char> available(std::max(n, 1));
    for (int i = 0; i < n; ++i) {
      std::fill(available.begin(), available.end(), 1);
      for (int j : graph[i])
        if (colour[j] >= 0) available[colour[j]] = 0;
      colour[i] = int(std::find(available.begin(), available.end(), 1) - available.begin());
    }
    total = 0;
    for (int i = 0; i < n; ++i) {
      if (colour[i] == 0) {
        if (colour0_returns_to_zero) buffers[i].offset = 0;
      } else {
        int64_t off = 0;
        for (int j : graph[i]) off = std::max(off, buffers[j].offset + buffers[j].size);
        buffers[i].offset = align_up(off);
      }
      total = std::max(total, buffers[i].offset + buffers[i].size);
    }
  };
  std::set<std::vector<int64_t>> seen;
  bool as_reference = true;
  int64_t passes = 0;
  bool busy = build_graph();
  do {
    place(as_reference);
    busy = build_graph();
    if (busy && as_reference) {
      std::vector<int64_t> state(n);
      for (int i = 0; i < n; ++i) state[i] = buffers[i].offset;
      if (!seen.insert(state).second) as_reference = false;  // the placement repeats: offsets may only grow from here
    }
    if (busy && ++passes > 64 + 8 * int64_t(n)) {  // last resort: end to end
      int64_t off = 0;
      for (int i = 0; i < n; ++i) { buffers[i].offset = off; off = align_up(off + buffers[i].size); }
      total = 0;
      for (int i = 0; i < n; ++i) total = std::max(total, buffers[i].offset + buffers[i].size);
      busy = false;
    }
  } while (busy);
  return total;
}

extern "C" int kapy_smem_barriers(const kapy_smem_op *ops, int32_t n_ops, const kapy_smem_access *accesses, int32_t n_accesses,
                                  const int32_t *succ_begin, const int32_t *succ, int32_t n_blocks, int32_t *barrier) {
  if (n_ops < 0 || n_blocks <= 0 || (n_ops > 0 && (!ops || !barrier)) || !succ_begin) return fail(KAPY_ERR_INVALID, "smem_barriers: null argument");
  std::vector<std::pair<int, int>> block_ops(n_blocks, {0, 0});  // [first, last) op of each block
  for (int b = 0, i = 0; b < n_blocks; ++b) {
    block_ops[b].first = i;
    while (i < n_ops && ops[i].block == b) ++i;
    block_ops[b].second = i;
    if (b == n_blocks - 1 && i != n_ops) return fail(KAPY_ERR_INVALID, "smem_barriers: ops must be grouped by ascending block");
  }
  for (int i = 0; i < n_ops; ++i) {
    barrier[i] = 0;
    if (ops[i].kind < 0 || ops[i].kind > 2) return fail(KAPY_ERR_INVALID, "smem_barriers: op %d has an unknown kind", i);
    if (ops[i].n_accesses < 0 || ops[i].first_access < 0 || ops[i].first_access + ops[i].n_accesses > n_accesses ||
        (ops[i].n_accesses > 0 && !accesses))
      return fail(KAPY_ERR_INVALID, "smem_barriers: op %d names accesses outside the array", i);
  }
  for (int b = 0; b < n_blocks; ++b) {
    if (succ_begin[b] > succ_begin[b + 1] || succ_begin[b] < 0) return fail(KAPY_ERR_INVALID, "smem_barriers: successor ranges must ascend");
    for (int s = succ_begin[b]; s < succ_begin[b + 1]; ++s)
      if (!succ || succ[s] < 0 || succ[s] >= n_blocks) return fail(KAPY_ERR_INVALID, "smem_barriers: successor out of range");
  }
  std::vector<Pending> incoming(n_blocks), outgoing(n_blocks);
  std::vector<char> visited(n_blocks, 0);
  std::deque<int> list{0};
  while (!list.empty()) {
    const int b = list.front();
    list.pop_front();
    Pending cur = incoming[b];
    for (int i = block_ops[b].first; i < block_ops[b].second; ++i) {
      if (barrier[i] & 1) cur.sync();  // a barrier placed before this op by an earlier visit is part of the block now
      if (ops[i].kind == 1) { cur.sync(); continue; }
      if (ops[i].kind == 2) {
        const bool followed = (barrier[i] & 2) || (i + 1 < block_ops[b].second && ops[i + 1].kind == 1);
        if (!followed) barrier[i] |= 2;
        cur.sync();
        continue;
      }
      Pending mine;
      for (int k = ops[i].first_access; k < ops[i].first_access + ops[i].n_accesses; ++k) {
        if (accesses[k].end <= accesses[k].begin) continue;
        (accesses[k].is_write ? mine.writes : mine.reads).insert({accesses[k].begin, accesses[k].end});
      }
      if (cur.hazard(mine)) {
        barrier[i] |= 1;
        cur.sync();
      }
      cur.join(mine);
    }
    // The reference stops at a block whose state equals the joined one; a state the joined one already covers
    // adds nothing to any successor either, and stopping there also ends the case where a barrier placed on an
    // earlier visit has made the state smaller for good.
    if (visited[b] && outgoing[b].covers(cur)) continue;
    visited[b] = 1;
    outgoing[b].join(cur);
    for (int s = succ_begin[b]; s < succ_begin[b + 1]; ++s) {
      incoming[succ[s]].join(outgoing[b]);
      list.push_back(succ[s]);
    }
  }
  int count = 0;
  for (int i = 0; i < n_ops; ++i) count += (barrier[i] & 1) + ((barrier[i] >> 1) & 1);
  return count;
}
