// Static GEMM plan: order families, block assignment with farthest-next-use eviction, dependency edges, and
// the three-resource pipeline simulation used to choose among orders (and, by the autotuner, among tile sizes).
#include "gemm_plan.hpp"

#include <algorithm>
#include <atomic>
#include <cfloat>
#include <climits>
#include <cmath>
#include <condition_variable>
#include <cstdlib>
#include <deque>
#include <functional>
#include <mutex>
#include <stdexcept>
#include <string>
#include <thread>

namespace paralia {

std::vector<int> gemm_task_order(const GemmProblem& p, int order_id) {
  const int Mg = p.Mg(), Ng = p.Ng(), Kg = p.Kg();   // p.k_split is the caller's business (build_gemm_plan sets it)
  order_id %= ORDER_STRIP_END;             // strips change launches, not the order
  order_id %= ORDER_K_SPLIT;
  order_id %= ORDER_MERGE_CHAINS;          // merging launches does not change the order
  order_id %= 40000;                       // nor does the eviction policy
  const bool repeat = order_id >= 20000;  // every panel k-outer, not only the first
  const int orient = (order_id % 20000) / 10000;
  int w = order_id % 10000;
  if (w == ORDER_FULL_PANEL) w = orient == 0 ? Ng : Mg;   // may now exceed 99: the block test below is on the id's own w
  const bool block = order_id % 10000 >= ORDER_BLOCK_ROWS;
  std::vector<int> order;
  order.reserve((size_t)Mg * Ng * Kg);
  auto id = [&](int mi, int ni, int ki) { return (mi * Ng + ni) * Kg + ki; };
  // One panel of C tiles, rows [m0, m1) x columns [n0, n1), in k-outer order.  Every k-step walks the tiles in
  // growing squares (shell d = max(row, column) inside the panel).  In the first steps, while the link is still behind,
  // every newly fetched A or B tile then at once enables a whole row or column of subkernels (column by column the
  // first fetches would enable one subkernel each while the compute streams starve).  Later the walk keeps the streams
  // level: the K chains are dealt to the exec queues in first-fire order, which is this walk, so its consecutive
  // subkernels sit on different queues in every step (column by column, a column whose tiles all drew the same queue
  // runs on one stream while the other waits for the next column's B tile).
  auto panel = [&](int m0, int m1, int n0, int n1) {
    const int rows = m1 - m0, cols = n1 - n0;
    if (rows <= 0 || cols <= 0 || Kg <= 0) return;
    for (int ki = 0; ki < Kg; ++ki)
      for (int d = 0; d < std::max(rows, cols); ++d) {
        if (d < cols)
          for (int mi = 0; mi < std::min(d, rows); ++mi) order.push_back(id(m0 + mi, n0 + d, ki));
        if (d < rows)
          for (int ni = 0; ni <= std::min(d, cols - 1); ++ni) order.push_back(id(m0 + d, n0 + ni, ki));
      }
  };
  if (block) {
    // Block orders (w = rows * 100 + columns): a block of rows x columns C tiles at the top left as one k-outer panel.
    // orient 0: then the other rows of the block's columns, then the other columns, tile by tile; orient 1: the other
    // columns of the block's rows first, then the other rows.  Against a panel over all rows the block needs fewer
    // tiles before its C tiles are complete, so the write-backs start earlier: the order for shapes the link bounds.
    const int wm = std::min(w / ORDER_BLOCK_ROWS, Mg), wn = std::min(w % ORDER_BLOCK_ROWS, Ng);
    if (repeat || wn < 1) throw std::runtime_error("gemm plan: unknown order id");
    panel(0, wm, 0, wn);
    auto chains = [&](int m0, int m1, int n0, int n1, bool rows_outer) {
      if (rows_outer) {
        for (int mi = m0; mi < m1; ++mi)
          for (int ni = n0; ni < n1; ++ni)
            for (int ki = 0; ki < Kg; ++ki) order.push_back(id(mi, ni, ki));
      } else {
        for (int ni = n0; ni < n1; ++ni)
          for (int mi = m0; mi < m1; ++mi)
            for (int ki = 0; ki < Kg; ++ki) order.push_back(id(mi, ni, ki));
      }
    };
    if (orient == 0) {
      chains(wm, Mg, 0, wn, true);    // a fetched row of A serves the block's columns
      chains(0, Mg, wn, Ng, false);   // a fetched column of B serves every row
    } else {
      chains(0, wm, wn, Ng, false);
      chains(wm, Mg, 0, Ng, true);
    }
    return order;
  }
  if (orient == 0) {
    w = std::min(w, Ng);
    if (repeat) {
      for (int n0 = 0; n0 < Ng; n0 += std::max(w, 1)) panel(0, Mg, n0, std::min(Ng, n0 + std::max(w, 1)));
    } else {
      panel(0, Mg, 0, w);
      for (int ni = w; ni < Ng; ++ni)
        for (int mi = 0; mi < Mg; ++mi)
          for (int ki = 0; ki < Kg; ++ki) order.push_back(id(mi, ni, ki));
    }
  } else {
    w = std::min(w, Mg);
    if (repeat) {
      for (int m0 = 0; m0 < Mg; m0 += std::max(w, 1)) panel(m0, std::min(Mg, m0 + std::max(w, 1)), 0, Ng);
    } else {
      panel(0, w, 0, Ng);
      for (int mi = w; mi < Mg; ++mi)
        for (int ni = 0; ni < Ng; ++ni)
          for (int ki = 0; ki < Kg; ++ki) order.push_back(id(mi, ni, ki));
    }
  }
  return order;
}

std::vector<int> gemm_candidate_orders(const GemmProblem& p, bool probe, bool merge) {
  std::vector<int> ids;
  ids.push_back(order_id_of(1, 0));  // the reference's index order; needs the fewest blocks
  if (!(p.a_remote || p.b_remote || p.c_remote)) return ids;
  GemmProblem unsplit = p;
  unsplit.k_split = 1;
  const bool limited = p.pool_blocks < gemm_full_block_num(unsplit);
  static const int widths[] = {1, 2, 3, 4, 5, 6, 8, 10, 12, 16, 20, 24, 32, 48, 64};
  static const int probe_widths[] = {2, 4};
  for (int orient = 0; orient < 2; ++orient) {
    const int g = orient == 0 ? p.Ng() : p.Mg();
    if (orient == 0 && !probe) ids.push_back(order_id_of(0, 0));
    if (probe) {
      // two narrow panels and one three quarters of the grid wide: compute-bound shapes want the wide one (16384^3: five
      // or six of eight), and a probe without it misjudged 2048-tiles by 8 % (16384 x 8192 x 16384)
      const int wide = std::min((3 * g + 2) / 4, ORDER_FULL_PANEL - 1);
      for (int w : probe_widths)
        if (w < g) ids.push_back(order_id_of(orient, w));
      if (wide < g && wide != probe_widths[0] && wide != probe_widths[1]) ids.push_back(order_id_of(orient, wide));
    } else {
      for (int w : widths)
        if (w < g) ids.push_back(order_id_of(orient, w));
    }
    ids.push_back(order_id_of(orient, std::min(g, ORDER_FULL_PANEL)));   // the whole grid as one k-outer panel
  }
  // blocks one or two tiles short of the grid in each direction (full pool only: a block order re-reads nothing)
  if (!limited && p.Mg() > 1 && p.Ng() > 1)
    for (int orient = 0; orient < 2; ++orient)
      for (int dm = 1; dm <= (probe ? 1 : 2); ++dm)
        for (int dn = 1; dn <= (probe ? 1 : 2); ++dn) {
          const int wm = p.Mg() - dm, wn = p.Ng() - dn;
          if (wm < 1 || wn < 1 || wm >= ORDER_BLOCK_ROWS || wn >= ORDER_BLOCK_ROWS) continue;
          if (probe && orient == 1) continue;
          ids.push_back(order_id_of(orient, wm * ORDER_BLOCK_ROWS + wn));
        }
  // every panel k-outer: what a block pool smaller than the working set needs (each fetched tile is used by a whole
  // row or column of the panel before it is evicted); a panel as wide as the grid is already listed above
  if (!probe || limited)
    for (int orient = 0; orient < 2; ++orient) {
      const int g = orient == 0 ? p.Ng() : p.Mg();
      if (probe) {
        // besides the two standard widths, the widest panel whose accumulators plus one k-step of A and B tiles fit the
        // pool, and the next wider one: the best width of a limited pool sits there, and a probe without it can misjudge
        // the tile size by 15 %
        const int other = orient == 0 ? p.Mg() : p.Ng();
        const int fit = (int)std::min<long>(ORDER_FULL_PANEL - 2, std::max<long>(1, (p.pool_blocks - other) / (other + 1)));
        int ws[4] = {probe_widths[0], probe_widths[1], fit, fit + 1};
        for (int i = 0; i < 4; ++i) {
          bool seen = false;
          for (int j = 0; j < i; ++j) seen |= ws[j] == ws[i];
          if (!seen && ws[i] < g) ids.push_back(20000 + order_id_of(orient, ws[i]));
        }
      } else {
        for (int w : widths)
          if (w < g) ids.push_back(20000 + order_id_of(orient, w));
      }
    }
  // with evictions in sight, every order also with the eviction policy that favours long-untouched tiles
  if (limited) {
    const size_t n = ids.size();
    for (size_t i = 0; i < n; ++i) ids.push_back(40000 + ids[i]);
  } else if (merge && p.Kg() > 1) {
    // the whole working set fits: the orders that run K chains back to back also with those chains as one launch
    const size_t n = ids.size();
    for (size_t i = 0; i < n; ++i)
      if (ids[i] < 20000) ids.push_back(ORDER_MERGE_CHAINS + ids[i]);
  }
  return ids;
}

long gemm_full_block_num(const GemmProblem& p) {
  const long a = (long)p.Mg() * p.Kg(), b = (long)p.Kg() * p.Ng(), c = (long)p.Mg() * p.Ng();
  // dgemm.cpp:80-82: one spare block plus every tile of A, B and C, plus C once more for the lazy write-back.
  return 1 + a + b + 2 * c;
}

long gemm_max_block_num(const GemmProblem& p) {
  GemmProblem q = p;
  q.k_split = 4;
  return gemm_full_block_num(q);
}

namespace {

struct Block {
  int kind = -1;  // -1 free, 0 A tile, 1 B tile, 2 accumulator, 3 source C
  int idx = -1;
  int content_cmd = -1;        // command after which the content is valid (the fetch)
  int last_touch = -1;         // latest command that wrote or read the content
  // commands that must complete before the block may be overwritten: at most one per stream (streams run their
  // commands in order, so the latest of a stream covers the earlier ones)
  int pending[MAX_WAITS];
  int npending = 0;
  bool ever_used = false;
};

// What each stream is already known to be behind: covered[s][r] = the latest command of stream r that some earlier
// command of stream s waited for.  Streams run their commands in order, so a later command of s need not wait for
// that command of r, or any before it, again.  In a k-outer panel most subkernels read tiles their stream's earlier
// subkernels already waited for.
constexpr int PLAN_STREAMS = STREAM_EXEC0 + MAX_EXEC_QUEUES;
struct Covered {
  int at[PLAN_STREAMS][PLAN_STREAMS];
  Covered() { for (auto& row : at) for (int& x : row) x = -1; }
};

void add_wait(std::vector<Cmd>& cmds, Cmd& c, int w, Covered& cov) {
  if (w < 0) return;
  if (cmds[w].stream == c.stream) return;  // stream order already covers it
  if (w <= cov.at[c.stream][cmds[w].stream]) return;  // an earlier command of this stream waited for it, or for a later one
  for (int i = 0; i < c.nwait; ++i) {
    if (c.wait[i] == w) return;
    if (cmds[c.wait[i]].stream == cmds[w].stream) {
      // streams run their commands in order: the later of two commands of one stream covers the earlier
      if (w > c.wait[i]) { c.wait[i] = w; cmds[w].signals = true; cov.at[c.stream][cmds[w].stream] = w; }
      return;
    }
  }
  if (c.nwait >= MAX_WAITS) throw std::runtime_error("gemm plan: too many dependencies on one command");
  c.wait[c.nwait++] = w;
  cmds[w].signals = true;
  cov.at[c.stream][cmds[w].stream] = w;
}

// Row strips for the call's last launch (ORDER_STRIP_END), which multiplies launch_k of k into the C tile (mi, ni): rows
// per strip, 0 when the tile is too small to cut, and how many ways a strip's launch splits K.  Up to four strips of at
// least 256 rows, in whole 128-row tiles of the kernel; a strip's workgroups are to fill every compute unit twice (512
// places) as long as a workgroup keeps 512 of k.
int strip_rows(const GemmProblem& p, int mi, int ni, long launch_k, int* splits) {
  const long tm = p.tm(mi), tn = p.tn(ni);
  const long n = std::min(4L, tm / 256);
  *splits = 0;
  if (n < 2) return 0;
  const long rows = ((tm + n - 1) / n + 127) / 128 * 128;
  const long tiles = ((rows + 127) / 128) * ((tn + 127) / 128);
  const long want = (512 + tiles - 1) / tiles;
  *splits = (int)std::max(1L, std::min(want, launch_k / 512));
  return (int)rows;
}

}  // namespace

GemmPlan build_gemm_plan(const GemmProblem& p_in, int order_id) {
  if (p_in.T <= 0 || p_in.M <= 0 || p_in.N <= 0) throw std::runtime_error("gemm plan: invalid dimensions");
  GemmPlan plan;
  plan.p = p_in;
  if (order_id < 0 || order_id / ORDER_STRIP_END > 1) throw std::runtime_error("gemm plan: unknown order id");
  const bool strip_end = order_id >= ORDER_STRIP_END;
  order_id %= ORDER_STRIP_END;
  plan.p.k_split = 1 << (order_id / ORDER_K_SPLIT);
  const GemmProblem& p = plan.p;
  if (order_id >= ORDER_K_SPLIT && p.slabs() == 1) throw std::runtime_error("gemm plan: this problem has no thin start");
  plan.order_id = order_id + (strip_end ? ORDER_STRIP_END : 0);
  plan.task_order = gemm_task_order(p, order_id);
  order_id %= ORDER_K_SPLIT;
  const bool merge = order_id >= ORDER_MERGE_CHAINS;
  order_id %= ORDER_MERGE_CHAINS;
  const int Mg = p.Mg(), Ng = p.Ng(), Kg = p.Kg();
  const int NQ = std::max(1, std::min(p.exec_queues, MAX_EXEC_QUEUES));
  const bool any_remote = p.a_remote || p.b_remote || p.c_remote;
  if (any_remote && p.pool_blocks < 3)
    throw std::runtime_error("PARALiA gemm: Not able to run with < 3 blocks per cache");

  // positions at which every A / B tile is used, for farthest-next-use eviction
  // (every A tile is used by Ng subkernels, every B tile by Mg: two dense tables, rows filled in order of use)
  struct Uses {
    int per = 0;
    std::vector<int> pos, fill;
    Uses(size_t tiles, int per_tile) : per(per_tile), pos(tiles * (size_t)per_tile), fill(tiles, 0) {}
    void add(size_t tile, int p) { pos[tile * per + fill[tile]++] = p; }
    int size(size_t tile) const { return fill[tile]; }
    int at(size_t tile, int i) const { return pos[tile * per + i]; }
  } a_uses((size_t)Mg * Kg, Ng), b_uses((size_t)Kg * Ng, Mg);
  for (int pos = 0; pos < (int)plan.task_order.size(); ++pos) {
    const int t = plan.task_order[pos];
    const int ki = t % Kg, ni = (t / Kg) % Ng, mi = t / (Kg * Ng);
    a_uses.add((size_t)mi * Kg + ki, pos);
    b_uses.add((size_t)ki * Ng + ni, pos);
  }
  std::vector<int> a_ptr((size_t)Mg * Kg, 0), b_ptr((size_t)Kg * Ng, 0);
  std::vector<int> a_blk((size_t)Mg * Kg, -1), b_blk((size_t)Kg * Ng, -1), c_blk((size_t)Mg * Ng, -1);
  std::vector<int> fired((size_t)Mg * Ng, 0), queue_of((size_t)Mg * Ng, 0);
  std::vector<Block> blocks((size_t)(any_remote ? p.pool_blocks : 0));
  // FIFO: never-used blocks first, then released blocks oldest first, so a recycled block's previous users
  // (a write-back still in flight, say) have had the longest time to finish before its new writer waits on them
  std::deque<int> free_list;
  int first_dynamic = 0;
  if (merge) {
    // panel layout: every tile of A and B has its own block for the whole call, the k tiles of a panel side by side
    plan.panels = true;
    if (p.a_remote) { plan.a_first = first_dynamic; first_dynamic += Mg * Kg; }
    if (p.b_remote) { plan.b_first = first_dynamic; first_dynamic += Kg * Ng; }
    const int c_min = p.c_remote ? (p.beta_zero ? 1 : 2) : 0;
    if (any_remote && (long)first_dynamic + c_min > p.pool_blocks)
      throw std::runtime_error("PARALiA gemm: device block pool too small for the panel layout of merged K chains");
  }
  for (int b = first_dynamic; b < (int)blocks.size(); ++b) free_list.push_back(b);
  int c_seq = 0;
  const bool slack_policy = order_id >= 40000;
  int cur_pos = 0;
  std::vector<Cmd>& cmds = plan.cmds;
  cmds.reserve(plan.task_order.size() * 2 + 16);
  Covered covered;

  auto release = [&](int b, int after_cmd) {
    blocks[b].kind = -1;
    blocks[b].idx = -1;
    blocks[b].pending[0] = after_cmd;
    blocks[b].npending = 1;
    blocks[b].last_touch = after_cmd;
    free_list.push_back(b);
  };

  // Returns a block whose previous content may be dropped; "waits" receives what a writer must wait for.
  auto alloc = [&](int pin1, int pin2, std::vector<int>& waits) -> int {
    // Policy 0 recycles a free block if there is one, else evicts the tile whose next use is farthest away: the fewest
    // fetches, but the block is often one read a moment ago (a tile that has just died, or in a k-outer panel the most
    // recent tiles, which the next panel needs last), so the fetch waits for that subkernel and the copy stream never
    // gets ahead.  Policy 1 also looks at the tiles not needed within the next pool-size subkernels and takes, among
    // them and the oldest free block, the one untouched for longest: its readers finished long ago, so the fetch
    // can start at once.  Which policy wins depends on whether copies or subkernels bound the schedule; the
    // simulation decides.
    int b = -1;
    int best_next = -1, best_touch = INT_MAX;
    if (plan.panels && free_list.empty())  // the tiles of A and B keep their blocks for the whole call: nothing to evict
      throw std::runtime_error("PARALiA gemm: device block pool too small for the panel layout of merged K chains");
    if (free_list.empty() || slack_policy) {
      for (int i = 0; i < (int)blocks.size(); ++i) {
        if (i == pin1 || i == pin2) continue;
        int next;
        if (blocks[i].kind == 0) {
          const int t = blocks[i].idx;
          next = a_ptr[t] < a_uses.size(t) ? a_uses.at(t, a_ptr[t]) : INT_MAX;
        } else if (blocks[i].kind == 1) {
          const int t = blocks[i].idx;
          next = b_ptr[t] < b_uses.size(t) ? b_uses.at(t, b_ptr[t]) : INT_MAX;
        } else {
          continue;  // free blocks; accumulators and source-C blocks are exclusive: never evicted
        }
        if (slack_policy && next - cur_pos > (int)blocks.size()) {
          if (blocks[i].last_touch < best_touch) {
            best_touch = blocks[i].last_touch;
            b = i;
          }
        } else if (best_touch == INT_MAX && next > best_next) {
          best_next = next;
          b = i;
        }
      }
    }
    if (!free_list.empty() && !(best_touch < blocks[free_list.front()].last_touch)) {
      b = free_list.front();
      free_list.pop_front();
    } else {
      if (b < 0) throw std::runtime_error("PARALiA gemm: device block pool too small for this subkernel order");
      if (blocks[b].kind == 0) a_blk[blocks[b].idx] = -1;
      else b_blk[blocks[b].idx] = -1;
      ++plan.n_evictions;
    }
    waits.insert(waits.end(), blocks[b].pending, blocks[b].pending + blocks[b].npending);
    blocks[b].npending = 0;
    blocks[b].ever_used = true;
    return b;
  };

  auto note_reader = [&](int b, int cmd_idx) {
    // one pending reader per stream is enough: streams run their commands in order
    blocks[b].last_touch = cmd_idx;
    Block& blk = blocks[b];
    for (int i = 0; i < blk.npending; ++i)
      if (cmds[blk.pending[i]].stream == cmds[cmd_idx].stream) {
        blk.pending[i] = cmd_idx;
        return;
      }
    if (blk.npending >= MAX_WAITS) throw std::runtime_error("gemm plan: too many streams read one block");
    blk.pending[blk.npending++] = cmd_idx;
  };

  struct OpenChain {
    bool active = false;
    int ci = -1, mi = -1, ni = -1, ki0 = -1, kn = 0, ablk = -1, bblk = -1, beta_mode = BETA_ONE;
    std::vector<int> waits;
  } open;
  auto close_chain = [&]() -> int {
    Cmd c;
    c.kind = CMD_GEMM; c.mi = open.mi; c.ni = open.ni; c.ki = open.ki0; c.kn = open.kn; c.stream = STREAM_EXEC0 + queue_of[open.ci];
    c.block = p.c_remote ? c_blk[open.ci] : -1; c.a_block = open.ablk; c.b_block = open.bblk; c.beta_mode = open.beta_mode;
    cmds.push_back(c);
    for (int x : open.waits) add_wait(cmds, cmds.back(), x, covered);
    open.active = false;
    return (int)cmds.size() - 1;
  };

  std::vector<int> gemm_waits, w;   // scratch, reused by every subkernel
  int strip_splits = 0;
  for (int pos = 0; pos < (int)plan.task_order.size(); ++pos) {
    const int t = plan.task_order[pos];
    const int ki = t % Kg, ni = (t / Kg) % Ng, mi = t / (Kg * Ng);
    const int ai = mi * Kg + ki, bi = ki * Ng + ni, ci = mi * Ng + ni;
    cur_pos = pos;
    ++a_ptr[ai];
    ++b_ptr[bi];
    int ablk = -1, bblk = -1;
    gemm_waits.clear();

    if (p.a_remote) {
      if (a_blk[ai] < 0) {
        w.clear();
        const int b = plan.panels ? plan.a_first + mi * Kg + ki : alloc(p.b_remote ? b_blk[bi] : -1, -1, w);
        blocks[b].ever_used = true;
        Cmd c;
        c.kind = CMD_FETCH_A; c.mi = mi; c.ki = ki; c.stream = STREAM_H2D; c.block = b;
        cmds.push_back(c);
        for (int x : w) add_wait(cmds, cmds.back(), x, covered);
        blocks[b].kind = 0; blocks[b].idx = ai; blocks[b].content_cmd = blocks[b].last_touch = (int)cmds.size() - 1;
        a_blk[ai] = b;
        ++plan.n_fetch[0];
      }
      ablk = a_blk[ai];
      gemm_waits.push_back(blocks[ablk].content_cmd);
    }
    if (p.b_remote) {
      if (b_blk[bi] < 0) {
        w.clear();
        const int b = plan.panels ? plan.b_first + ni * Kg + ki : alloc(ablk, -1, w);
        blocks[b].ever_used = true;
        Cmd c;
        c.kind = CMD_FETCH_B; c.ki = ki; c.ni = ni; c.stream = STREAM_H2D; c.block = b;
        cmds.push_back(c);
        for (int x : w) add_wait(cmds, cmds.back(), x, covered);
        blocks[b].kind = 1; blocks[b].idx = bi; blocks[b].content_cmd = blocks[b].last_touch = (int)cmds.size() - 1;
        b_blk[bi] = b;
        ++plan.n_fetch[1];
      }
      bblk = b_blk[bi];
      gemm_waits.push_back(blocks[bblk].content_cmd);
    }

    int beta_mode = BETA_ONE;
    if (fired[ci] == 0) {
      // reference: each C tile's K-chain is pinned to one exec queue, handed out round-robin (Subkernel.cpp:18-22)
      queue_of[ci] = c_seq++ % NQ;
      if (p.c_remote) {
        const int b = alloc(ablk, bblk, gemm_waits);
        blocks[b].kind = 2; blocks[b].idx = ci;
        c_blk[ci] = b;
        beta_mode = BETA_ZERO;  // lazy write-back: accumulate locally first (dgemm.cpp:273-279)
      } else {
        beta_mode = BETA_USER;  // resident C: plain read-modify-write (dgemm.cpp:259-260)
      }
    }
    // The launch of this subkernel.  With merged K chains a subkernel that continues the chain of the previous one in
    // the order (same C tile, next k tile) joins its launch, which is only written out when the chain ends: by then
    // every fetch it depends on is already in the command list.
    if (merge && open.active && open.ci == ci && open.ki0 + open.kn == ki) {
      ++open.kn;
      open.waits.insert(open.waits.end(), gemm_waits.begin(), gemm_waits.end());
    } else {
      if (open.active) close_chain();
      open.active = true;
      open.ci = ci; open.mi = mi; open.ni = ni; open.ki0 = ki; open.kn = 1;
      open.ablk = ablk; open.bblk = bblk; open.beta_mode = beta_mode;
      open.waits = gemm_waits;
    }
    // The call's last launch on a C tile that goes back to the host (ORDER_STRIP_END): row strips, see below.
    int rows_per = 0;
    if (strip_end && p.c_remote && fired[ci] + 1 == Kg && pos + 1 == (int)plan.task_order.size()) {
      long launch_k = 0;
      for (int kt = open.ki0; kt < open.ki0 + open.kn; ++kt) launch_k += p.tk(kt);
      rows_per = strip_rows(p, mi, ni, launch_k, &strip_splits);
    }
    int gemm_idx = -1;
    auto after_launch = [&](int launch) {
      if (ablk >= 0) note_reader(ablk, launch);
      if (bblk >= 0) note_reader(bblk, launch);
      // A tile that no later subkernel reads gives its block back at once (its readers stay pending on the block): the
      // FIFO then hands out the longest-dead block first, so the fetch that reuses it rarely waits and the copy stream
      // can run a whole k-step ahead of the subkernels even when the pool is much smaller than the operands.
      if (ablk >= 0 && a_ptr[ai] == a_uses.size(ai)) {
        blocks[ablk].kind = -1; blocks[ablk].idx = -1;
        a_blk[ai] = -1;
        free_list.push_back(ablk);
      }
      if (bblk >= 0 && b_ptr[bi] == b_uses.size(bi)) {
        blocks[bblk].kind = -1; blocks[bblk].idx = -1;
        b_blk[bi] = -1;
        free_list.push_back(bblk);
      }
    };
    if (!merge && rows_per == 0) {
      gemm_idx = close_chain();
      after_launch(gemm_idx);
    }

    if (++fired[ci] == Kg && p.c_remote && rows_per > 0) {
      // The last launch of the call in row strips, one launch each on the tile's stream, and with it everything that
      // follows on those rows: the fetch of the caller's C and the lazy reduce (beta != 0), and the write-back.  The
      // strips' copies and kernels pipeline, so what is left when the last kernel ends is a strip's write-back.
      const int accb = c_blk[ci];
      const int tm = (int)p.tm(mi), stream = STREAM_EXEC0 + queue_of[ci];
      std::vector<int> strip_last;   // per strip: the command its write-back waits for
      for (int r0 = 0; r0 < tm; r0 += rows_per) {
        Cmd c;
        c.kind = CMD_GEMM; c.mi = mi; c.ni = ni; c.ki = open.ki0; c.kn = open.kn; c.stream = stream;
        c.block = accb; c.a_block = open.ablk; c.b_block = open.bblk; c.beta_mode = open.beta_mode;
        c.row0 = r0; c.rows = std::min(rows_per, tm - r0); c.splits = strip_splits;
        cmds.push_back(c);
        for (int x : open.waits) add_wait(cmds, cmds.back(), x, covered);
        strip_last.push_back((int)cmds.size() - 1);
      }
      open.active = false;
      if (!merge) after_launch(strip_last.back());   // (the stream's last strip covers the earlier ones)
      if (!p.beta_zero) {
        w.clear();
        const int sb = alloc(accb, -1, w);
        blocks[sb].kind = 3; blocks[sb].idx = ci;
        std::vector<int> fetches;
        for (int r0 = 0; r0 < tm; r0 += rows_per) {
          Cmd f;
          f.kind = CMD_FETCH_C; f.mi = mi; f.ni = ni; f.stream = STREAM_H2D; f.block = sb; f.row0 = r0; f.rows = std::min(rows_per, tm - r0);
          cmds.push_back(f);
          for (int x : w) add_wait(cmds, cmds.back(), x, covered);
          fetches.push_back((int)cmds.size() - 1);
        }
        blocks[sb].content_cmd = fetches.back();
        ++plan.n_fetch[2];
        for (size_t i = 0; i < strip_last.size(); ++i) {
          Cmd r;
          r.kind = CMD_REDUCE; r.mi = mi; r.ni = ni; r.stream = stream; r.block = accb; r.a_block = sb;
          r.row0 = cmds[strip_last[i]].row0; r.rows = cmds[strip_last[i]].rows;
          cmds.push_back(r);
          add_wait(cmds, cmds.back(), fetches[i], covered);
          strip_last[i] = (int)cmds.size() - 1;
        }
        release(sb, strip_last.back());
      }
      for (size_t i = 0; i < strip_last.size(); ++i) {
        Cmd wb;
        wb.kind = CMD_WRITEBACK; wb.mi = mi; wb.ni = ni; wb.stream = STREAM_D2H; wb.block = accb;
        wb.row0 = cmds[strip_last[i]].row0; wb.rows = cmds[strip_last[i]].rows;
        cmds.push_back(wb);
        add_wait(cmds, cmds.back(), strip_last[i], covered);
      }
      release(accb, (int)cmds.size() - 1);
      c_blk[ci] = -1;
    } else if (fired[ci] == Kg && p.c_remote) {
      if (open.active) gemm_idx = close_chain();
      const int accb = c_blk[ci];
      int last = gemm_idx;
      if (!p.beta_zero) {
        // lazy reduce: fetch the caller's tile now, out = beta * src + acc (dgemm.cpp:173-179)
        w.clear();
        const int sb = alloc(accb, -1, w);
        Cmd f;
        f.kind = CMD_FETCH_C; f.mi = mi; f.ni = ni; f.stream = STREAM_H2D; f.block = sb;
        cmds.push_back(f);
        for (int x : w) add_wait(cmds, cmds.back(), x, covered);
        const int fetch_idx = (int)cmds.size() - 1;
        blocks[sb].kind = 3; blocks[sb].idx = ci; blocks[sb].content_cmd = fetch_idx;
        ++plan.n_fetch[2];
        Cmd r;
        r.kind = CMD_REDUCE; r.mi = mi; r.ni = ni; r.stream = STREAM_EXEC0 + queue_of[ci]; r.block = accb; r.a_block = sb;
        cmds.push_back(r);
        add_wait(cmds, cmds.back(), fetch_idx, covered);
        last = (int)cmds.size() - 1;
        release(sb, last);
      }
      Cmd wb;
      wb.kind = CMD_WRITEBACK; wb.mi = mi; wb.ni = ni; wb.stream = STREAM_D2H; wb.block = accb;
      cmds.push_back(wb);
      add_wait(cmds, cmds.back(), last, covered);
      release(accb, (int)cmds.size() - 1);
      c_blk[ci] = -1;
    }
  }
  if (open.active) close_chain();
  // with panels the pool is addressed by block number up to the last one in use
  if (plan.panels) {
    for (int b = 0; b < (int)blocks.size(); ++b)
      if (blocks[b].ever_used) plan.blocks_used = b + 1;
  } else {
    for (const Block& b : blocks) plan.blocks_used += b.ever_used ? 1 : 0;
  }
  return plan;
}

double StageTimes::exec_time(long T, long m, long n, long k) const {
  const double vol = (double)m * n * (double)(k > 0 ? k : 1);
  const double T3 = (double)T * T * T;
  if (exec_table.empty() || vol >= T3) return t_exec * vol / T3;
  // seconds per unit volume at the cube of equal volume, interpolated between the neighbouring table entries
  const double edge = std::cbrt(vol);
  auto rate = [](const std::pair<long, double>& e) { return e.second / ((double)e.first * e.first * e.first); };
  if (edge <= exec_table.front().first) return rate(exec_table.front()) * vol * (exec_table.front().first / edge);
  for (size_t i = 1; i < exec_table.size(); ++i)
    if (edge <= exec_table[i].first) {
      const double f = (edge - exec_table[i - 1].first) / (double)(exec_table[i].first - exec_table[i - 1].first);
      return ((1 - f) * rate(exec_table[i - 1]) + f * rate(exec_table[i])) * vol;
    }
  return rate(exec_table.back()) * vol;
}

namespace {

using Intervals = std::vector<std::pair<double, double>>;

// Completion time of a copy that needs `work` seconds on an otherwise idle link and starts at s, when it runs sl
// times slower while the opposite direction is busy.  `busy` is sorted and disjoint; `cursor` only moves forward
// because the copies of one direction start in non-decreasing time order.
double stretched_end(double s, double work, double sl, const Intervals& busy, size_t& cursor) {
  if (sl <= 1.0 || busy.empty()) return s + work;
  while (cursor < busy.size() && busy[cursor].second <= s) ++cursor;
  double t = s;
  for (size_t c = cursor; work > 0; ++c) {
    if (c >= busy.size()) return t + work;
    if (t < busy[c].first) {
      const double idle = busy[c].first - t;
      if (work <= idle) return t + work;
      work -= idle;
      t = busy[c].first;
    }
    const double span = busy[c].second - t;
    if (work * sl <= span) return t + work * sl;
    work -= span / sl;
    t = busy[c].second;
  }
  return t;
}

void add_interval(Intervals& v, double a, double b) {
  if (b <= a) return;
  if (!v.empty() && a <= v.back().second) v.back().second = std::max(v.back().second, b);
  else v.emplace_back(a, b);
}

}  // namespace

std::atomic<long> plan_simulations{0};

PipelineResult simulate_plan(const GemmPlan& plan, const StageTimes& st) {
  ++plan_simulations;
  const GemmProblem& p = plan.p;
  const double T2 = (double)p.T * p.T;
  std::vector<double> finish(plan.cmds.size(), 0.0);
  // The two copy directions share the host link: a copy is slower while the opposite direction is busy
  // (the sl factor of the link model, CoModel.cpp:143-162).  The commands are walked in plan order, not in time
  // order, so the opposite direction's busy intervals are taken from the previous pass; the first pass runs
  // without slowdown and two more settle the schedule.
  const bool contended = st.h2d_sl > 1.0 || st.d2h_sl > 1.0;
  Intervals busy_h2d, busy_d2h;
  PipelineResult r;
  for (int pass = 0; pass < (contended ? 3 : 1); ++pass) {
    Intervals now_h2d, now_d2h;
    size_t cur_h2d = 0, cur_d2h = 0;
    double h2d = 0, d2h = 0, exec = 0;
    double qclock[MAX_EXEC_QUEUES] = {0};
    double deficit = st.tr_amp > 0 ? 1.0 - std::exp(-st.tr_gap0 / st.tr_idle) : 0.0;
    r = PipelineResult();
    for (size_t i = 0; i < plan.cmds.size(); ++i) {
      const Cmd& c = plan.cmds[i];
      double ready = 0;
      for (int w = 0; w < c.nwait; ++w) ready = std::max(ready, finish[c.wait[w]]);
      double dur = 0;
      switch (c.kind) {
        case CMD_FETCH_A: dur = st.h2d_ti + st.h2d_tb * (double)p.tm(c.mi) * p.tk(c.ki) * p.elem; break;
        case CMD_FETCH_B: dur = st.h2d_ti + st.h2d_tb * (double)p.tk(c.ki) * p.tn(c.ni) * p.elem; break;
        case CMD_FETCH_C: dur = st.h2d_ti + st.h2d_tb * (double)(c.rows > 0 ? c.rows : p.tm(c.mi)) * p.tn(c.ni) * p.elem; break;
        case CMD_GEMM:
          for (int k = c.ki; k < c.ki + c.kn; ++k) {
            if (k < p.slabs() && p.slabs() > 1)
              dur += st.exec_time(p.T, p.tm(c.mi), p.tn(c.ni), p.T) * (double)p.tk(k) / (double)p.T + st.slab_fixed * std::max(1.0, 1024.0 / (double)p.tk(k));
            else dur += st.exec_time(p.T, p.tm(c.mi), p.tn(c.ni), p.tk(k));
          }
          if (c.kn > 1) dur = std::max(0.5 * dur, dur - (c.kn - 1) * st.merge_saving * ((double)p.tm(c.mi) * p.tn(c.ni)) / T2);
          if (c.rows > 0) {
            // a row strip: its share of the tile's launch, and what splitting K adds
            dur *= (double)c.rows / (double)p.tm(c.mi);
            if (c.splits > 1) dur += st.split_fixed + st.split_pass_tb * (2.0 * c.splits + 1.0) * (double)c.rows * p.tn(c.ni) * p.elem;
          }
          break;
        case CMD_REDUCE: dur = st.t_reduce * ((double)(c.rows > 0 ? c.rows : p.tm(c.mi)) * p.tn(c.ni)) / T2; break;
        case CMD_WRITEBACK: dur = st.d2h_ti + st.d2h_tb * (double)(c.rows > 0 ? c.rows : p.tm(c.mi)) * p.tn(c.ni) * p.elem; break;
      }
      if (c.stream == STREAM_H2D) {
        const double s = std::max(ready, h2d);
        finish[i] = h2d = stretched_end(s, dur, st.h2d_sl, busy_d2h, cur_d2h);
        add_interval(now_h2d, s, h2d);
        r.t_h2d += h2d - s;
      } else if (c.stream == STREAM_D2H) {
        const double s = std::max(ready, d2h);
        finish[i] = d2h = stretched_end(s, dur, st.d2h_sl, busy_h2d, cur_h2d);
        add_interval(now_d2h, s, d2h);
        r.t_d2h += d2h - s;
      } else {
        // exec queues are in-order each and share the one compute resource
        const int q = c.stream - STREAM_EXEC0;
        const double s = std::max(std::max(ready, qclock[q]), exec);
        if (st.tr_amp > 0) {
          if (s > exec) deficit = 1.0 - (1.0 - deficit) * std::exp(-(s - exec) / st.tr_idle);
          if (c.kind == CMD_GEMM) dur *= 1.0 + st.tr_amp * deficit;
          deficit *= std::exp(-dur / st.tr_recover);
        }
        finish[i] = qclock[q] = exec = s + dur;
        r.t_exec += dur;
      }
      r.t_total = std::max(r.t_total, finish[i]);
    }
    busy_h2d.swap(now_h2d);
    busy_d2h.swap(now_d2h);
  }
  return r;
}

namespace {

// Worker threads of the order search.  The candidates of one search are independent (build a plan, simulate it), so
// they are dealt to a few threads through a shared counter and their results are gathered per candidate; which order
// wins is then decided by one thread walking the results in candidate order, so the outcome does not depend on timing.
// The pool lives as long as the process; PARALIA_PLAN_THREADS sets its size (1: everything on the calling thread).
class SearchThreads {
 public:
  static SearchThreads& get() {
    static SearchThreads* pool = new SearchThreads();   // never destroyed: joining at exit could wait on a thread that is gone
    return *pool;
  }
  // runs fn(i) for i in [0, n), on the calling thread and the workers
  // (small = true: the items are too cheap to be worth waking anybody)
  void run(int n, const std::function<void(int)>& fn, bool small = false) {
    if (n <= 0) return;
    if (workers_.empty() || n == 1 || small) {
      for (int i = 0; i < n; ++i) fn(i);
      return;
    }
    std::lock_guard<std::mutex> one_search_at_a_time(run_mu_);
    std::unique_lock<std::mutex> lk(mu_);
    fn_ = &fn; n_ = n; next_ = 0; done_ = 0; ++generation_;
    cv_.notify_all();
    lk.unlock();
    work();
    lk.lock();
    done_cv_.wait(lk, [&] { return done_ == n_ && active_ == 0; });
    fn_ = nullptr;
  }

 private:
  SearchThreads() {
    // more than four gain nothing: a search has a few dozen plans of some tens of microseconds each
    unsigned want = std::min(4u, std::max(1u, std::thread::hardware_concurrency()));
    if (const char* env = getenv("PARALIA_PLAN_THREADS")) want = (unsigned)std::max(1, std::min(64, atoi(env)));
    for (unsigned t = 1; t < want; ++t) workers_.emplace_back([this] { loop(); });
    for (auto& w : workers_) w.detach();
  }
  void work() {
    for (;;) {
      int i;
      {
        std::lock_guard<std::mutex> lk(mu_);
        if (!fn_ || next_ >= n_) return;
        i = next_++;
      }
      (*fn_)(i);
      std::lock_guard<std::mutex> lk(mu_);
      if (++done_ == n_) done_cv_.notify_all();
    }
  }
  void loop() {
    long seen = 0;
    std::unique_lock<std::mutex> lk(mu_);
    for (;;) {
      cv_.wait(lk, [&] { return generation_ != seen; });
      seen = generation_;
      ++active_;
      lk.unlock();
      work();
      lk.lock();
      if (--active_ == 0) done_cv_.notify_all();
    }
  }
  std::vector<std::thread> workers_;
  std::mutex mu_, run_mu_;
  std::condition_variable cv_, done_cv_;
  const std::function<void(int)>* fn_ = nullptr;
  int n_ = 0, next_ = 0, done_ = 0, active_ = 0;
  long generation_ = 0;
};

struct Evaluated {
  bool ok = false;
  PipelineResult r;
  long evictions = 0;
  std::string err;
};

// build + simulate every id of the list, in parallel
std::vector<Evaluated> evaluate_orders(const GemmProblem& p, const StageTimes& st, const std::vector<int>& ids) {
  std::vector<Evaluated> out(ids.size());
  const std::function<void(int)> one = [&](int i) {
    try {
      GemmPlan plan = build_gemm_plan(p, ids[i]);
      out[i].r = simulate_plan(plan, st);
      out[i].evictions = plan.n_evictions;
      out[i].ok = true;
    } catch (const std::runtime_error& e) {
      out[i].err = e.what();  // this order does not fit the pool; others may
    }
  };
  SearchThreads::get().run((int)ids.size(), one, /*small=*/p.subkernels() * (long)ids.size() < 6000);
  return out;
}

}  // namespace

int pick_gemm_order(const GemmProblem& p, const StageTimes& st, PipelineResult* best_out, bool probe) {
  // Two groups of orders, each with its own best: the panel orders, and the block orders (w >= ORDER_BLOCK_ROWS), which
  // end in two tile-by-tile phases and are taken only when they win by more than a percent (12288^3: simulated 0.6 %
  // faster than the best panel order, measured 1 % slower; 8192^3: simulated 3.9 %, measured 5.6 % faster).
  struct Group {
    int id = -1;
    PipelineResult r;
    std::vector<std::pair<double, int>> ranked;  // (makespan, id) of every feasible order, in candidate order
  } grp[2];
  auto is_block = [](int id) { return id % 10000 >= ORDER_BLOCK_ROWS; };
  std::string last_err;
  // The variants with merged K chains come second: merging takes at most (launches saved) x (saving per launch) off an
  // order's makespan -- it removes that much compute and otherwise only delays launches -- so a merged variant is built
  // only where its plain order, less that bound, gets under the best plain order.
  std::vector<int> ids, merged_ids;
  for (int id : gemm_candidate_orders(p, probe, st.merge_saving > 0))
    if (!is_block(id) || st.block_orders) (id % ORDER_K_SPLIT >= ORDER_MERGE_CHAINS ? merged_ids : ids).push_back(id);
  auto gather = [&](const std::vector<int>& list, const std::vector<Evaluated>& evals) {
    for (size_t i = 0; i < list.size(); ++i) {
      const int id = list[i];
      if (!evals[i].ok) { last_err = evals[i].err; continue; }
      const PipelineResult& r = evals[i].r;
      Group& g = grp[is_block(id) ? 1 : 0];
      g.ranked.emplace_back(r.t_total, id);
      if (g.id < 0 || r.t_total < g.r.t_total * (1.0 - 1e-9)) {
        g.r = r;
        g.id = id;
      }
    }
  };
  const std::vector<Evaluated> evals = evaluate_orders(p, st, ids);
  gather(ids, evals);
  if (!merged_ids.empty()) {
    double best_plain = DBL_MAX;
    for (const Evaluated& e : evals)
      if (e.ok) best_plain = std::min(best_plain, e.r.t_total);
    const double most_saved = (double)(p.subkernels() - (long)p.Mg() * p.Ng()) * st.merge_saving;
    std::vector<int> worth;
    for (int id : merged_ids) {
      const auto plain = std::find(ids.begin(), ids.end(), id - ORDER_MERGE_CHAINS);
      if (plain == ids.end()) { worth.push_back(id); continue; }
      const Evaluated& e = evals[plain - ids.begin()];
      if (st.exhaustive || (e.ok && e.r.t_total - most_saved <= best_plain)) worth.push_back(id);
    }
    // the ranking keeps candidate order: merged variants behind the plain ones, as the candidate list has them
    gather(worth, evaluate_orders(p, st, worth));
  }
  if (grp[0].id < 0 && grp[1].id < 0) throw std::runtime_error(last_err.empty() ? "gemm plan: no feasible order" : last_err);
  // the best orders also with a thin start (first k tile in 2 or 4 slabs), where the operands cross the link; the
  // three best of a group, because the order that wins with a thin start is often the runner-up without one (a wider
  // panel, whose longer wait for its first tiles the slabs take away)
  GemmProblem unsplit = p;
  unsplit.k_split = 1;
  if (st.thin_start && (p.a_remote || p.b_remote) && !probe && p.pool_blocks >= gemm_full_block_num(unsplit))
    for (Group& g : grp) {
      if (g.id < 0) continue;
      // a thin start takes at most seven eighths of the first A and B tiles' fetch off a call: a group that would
      // still trail the other group's plain best by more than that is not worth the nine plans
      const Group& other = grp[&g == &grp[0] ? 1 : 0];
      const double thin_gain = ((p.a_remote ? 1 : 0) + (p.b_remote ? 1 : 0)) * 0.875 * st.h2d_tb * (double)p.T * std::min(p.T, p.K) * p.elem;
      if (!st.exhaustive && other.id >= 0 && g.r.t_total - thin_gain > other.r.t_total) continue;
      // makespans that differ only in the last bits are ties (compared in single precision), and ties keep the
      // candidate order, as the choice above does
      std::stable_sort(g.ranked.begin(), g.ranked.end(),
                       [](const std::pair<double, int>& a, const std::pair<double, int>& b) { return (float)a.first < (float)b.first; });
      const double unsplit_best = g.r.t_total;
      std::vector<int> thin_ids;
      for (size_t b = 0; b < std::min<size_t>(3, g.ranked.size()); ++b)
        for (int s = 1; s <= 3; ++s) thin_ids.push_back(g.ranked[b].second + s * ORDER_K_SPLIT);
      const std::vector<Evaluated> thin = evaluate_orders(p, st, thin_ids);
      for (size_t i = 0; i < thin_ids.size(); ++i)
        if (thin[i].ok && thin[i].evictions == 0 && thin[i].r.t_total < unsplit_best * (1.0 - 1e-3) && thin[i].r.t_total < g.r.t_total) {
          g.r = thin[i].r;
          g.id = thin_ids[i];
        }
    }
  const Group& pick = (grp[0].id < 0 || (grp[1].id >= 0 && grp[1].r.t_total < 0.99 * grp[0].r.t_total)) ? grp[1] : grp[0];
  PipelineResult chosen = pick.r;
  const int id = (st.strip_end && !probe) ? with_strip_end(p, st, pick.id, &chosen) : pick.id;
  if (best_out) *best_out = chosen;
  return id;
}

int with_strip_end(const GemmProblem& p, const StageTimes& st, int order_id, PipelineResult* r) {
  // With C on the device nothing is written back and the flag builds the same plan.  Offered to merged K chains only:
  // there the last launch is long and its strips cost little beside it; the strips of a last k-step took as long as
  // they saved or longer (dgemm 8192^3: 23.28 -> 23.32 ms, 12288^3: 56.12 -> 56.16 ms, simulated 0.1 ms shorter).
  if (!p.c_remote || order_id >= ORDER_STRIP_END || order_id % ORDER_K_SPLIT < ORDER_MERGE_CHAINS) return order_id;
  const std::vector<int> strip_id = {order_id + ORDER_STRIP_END};
  const std::vector<Evaluated> strip = evaluate_orders(p, st, strip_id);
  if (strip[0].ok && r && strip[0].r.t_total < r->t_total * (1.0 - 1e-3)) {
    *r = strip[0].r;
    return strip_id[0];
  }
  return order_id;
}

}  // namespace paralia
