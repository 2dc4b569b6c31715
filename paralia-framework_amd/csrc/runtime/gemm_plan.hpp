// Static plan of one tiled GEMM call on one GPU: subkernel order, device-block assignment (with eviction when
// the pool is smaller than the working set) and the cross-stream dependencies, all decided on the host before
// anything is enqueued.  Pure host logic -- no HIP types -- so it is unit-tested without a GPU.
//
// Where the reference does this work: subkernel creation and beta schedule in
// Library_scheduler/src/Functions/dgemm.cpp:123-205,273-279; block grabbing and tile fetch in
// Subkernel.cpp:90-135; readiness polling and launch in Subkernel.cpp:192-247 and dgemm.cpp:290-314;
// subkernel choice in Subkernel.cpp:384-448; write-back in Subkernel_backup.cpp:1128-1260.
// The reference decides these dynamically with a manager thread polling events every 100 us; here the order
// is fixed up front from a simulated H2D / compute / D2H pipeline and the dependencies are handed to the HIP
// streams as event waits, so the host never polls.
#ifndef PARALIA_GEMM_PLAN_HPP
#define PARALIA_GEMM_PLAN_HPP

#include <atomic>
#include <utility>
#include <vector>

namespace paralia {

constexpr int MAX_EXEC_QUEUES = 8;  // MAX_BACKEND_L of the reference (CMakeLists.txt:69)
constexpr int MAX_WAITS = 2 + MAX_EXEC_QUEUES + 2;

struct GemmProblem {
  long M = 0, N = 0, K = 0, T = 0;
  bool a_remote = true, b_remote = true, c_remote = true;  // operand lives off the device
  bool beta_zero = false;                                    // caller's beta == 0: C is never fetched
  int elem = 8;                                              // bytes per element
  int exec_queues = 2;
  long pool_blocks = 0;                                      // device blocks available (>= 3 when anything is remote)
  // Thin start: the first k tile is cut into slabs (each its own k tile, fetched and multiplied separately), so the
  // first subkernels can start after a fraction of the first tiles has crossed the link.  k_split = 2 or 4: that many
  // equal slabs; k_split = 8: a graded start, four slabs of T/8, T/8, T/4 and T/2 -- the first kernels start after an
  // eighth of a tile, and the slabs grow as the link gets ahead, so the later ones pay less per launch.  Taken as 1
  // when it does not apply (K < T, T not divisible, slabs under 16).
  int k_split = 1;
  int slabs() const {
    if (k_split == 8) return (K >= T && T % 8 == 0 && T / 8 >= 16) ? 4 : 1;
    return (k_split > 1 && K >= T && T % k_split == 0 && T / k_split >= 16) ? k_split : 1;
  }
  long slab_k0(int i) const {  // first k of slab i of the first tile (i == slabs(): T)
    if (k_split != 8) return (long)i * (T / slabs());
    return i == 0 ? 0 : i == 1 ? T / 8 : i == 2 ? T / 4 : i == 3 ? T / 2 : T;
  }
  int Mg() const { return (int)((M + T - 1) / T); }
  int Ng() const { return (int)((N + T - 1) / T); }
  int Kg() const { return K > 0 ? (int)((K + T - 1) / T) + slabs() - 1 : 1; }
  long tm(int mi) const { return mi == Mg() - 1 ? M - (long)mi * T : T; }
  long tn(int ni) const { return ni == Ng() - 1 ? N - (long)ni * T : T; }
  long k0(int ki) const { const int s = slabs(); return ki < s ? slab_k0(ki) : (long)(ki - s + 1) * T; }  // first k of tile ki
  long tk(int ki) const {
    if (K <= 0) return 0;
    if (ki < slabs() && slabs() > 1) return slab_k0(ki + 1) - slab_k0(ki);
    return ki == Kg() - 1 ? K - k0(ki) : T;
  }
  long subkernels() const { return (long)Mg() * Ng() * Kg(); }
};

enum CmdKind : int { CMD_FETCH_A = 0, CMD_FETCH_B = 1, CMD_FETCH_C = 2, CMD_GEMM = 3, CMD_REDUCE = 4, CMD_WRITEBACK = 5 };
enum : int { STREAM_H2D = 0, STREAM_D2H = 1, STREAM_EXEC0 = 2 };
enum : int { BETA_ZERO = 0, BETA_ONE = 1, BETA_USER = 2 };

struct Cmd {
  int kind = 0;
  int mi = -1, ni = -1, ki = -1;  // FETCH_A: (mi, ki); FETCH_B: (ki, ni); everything on C: (mi, ni)
  int stream = 0;
  int block = -1;     // block written by a FETCH; accumulator block of GEMM / REDUCE / WRITEBACK (-1: caller's C)
  int a_block = -1;   // GEMM: block of the A tile (-1: caller's memory); REDUCE: block holding the fetched source C
  int b_block = -1;   // GEMM: block of the B tile (-1: caller's memory)
  int kn = 1;         // GEMM: number of consecutive k tiles ki .. ki + kn - 1 multiplied by this one launch
  // FETCH_C / GEMM / REDUCE / WRITEBACK on a row strip of the C tile: rows row0 .. row0 + rows - 1 of it (rows == 0: the
  // whole tile)
  int row0 = 0, rows = 0;
  int splits = 0;     // GEMM: ways the launch is to split K over workgroups (0: the kernel launcher's own choice)
  int beta_mode = BETA_ONE;
  int nwait = 0;
  int wait[MAX_WAITS];  // earlier commands on other streams that must have completed
  bool signals = false; // some later command on another stream waits on this one
};

struct GemmPlan {
  GemmProblem p;
  int order_id = 0;
  // Panel layout: the k tiles of an A row panel (and of a B column panel) sit in consecutive blocks, block
  // a_first + mi * Kg + ki for A(mi, ki) and b_first + ni * Kg + ki for B(ki, ni), and inside a panel the tiles are
  // placed so that the panel is ONE matrix with one leading dimension (for an operand that is contiguous along m or
  // n: dense tiles one after the other; for an operand contiguous along k: the tiles stacked in a K x tile matrix).
  // A launch can then multiply several k tiles at once.  Only when the pool holds every tile of A and B.
  bool panels = false;
  int a_first = -1, b_first = -1;
  std::vector<int> task_order;  // subkernel ids mi*Ng*Kg + ni*Kg + ki in firing order
  std::vector<Cmd> cmds;
  long blocks_used = 0;
  long n_fetch[3] = {0, 0, 0};  // A, B, C tile fetches issued (re-fetches after eviction included)
  long n_evictions = 0;
};

// Order families.  id = orient * 10000 + w.  orient 0: the first w column-tiles of C are processed as one
// panel in k-outer (outer-product) order, the remaining columns tile by tile (ni, mi, ki);
// orient 1: the same with row-tiles (remaining rows in the reference's index order mi, ni, ki).
// w = 0 with orient 1 is exactly the reference's subkernel index order (dgemm.cpp:139-142).
// id = 20000 + orient * 10000 + w: every group of w column-tiles (row-tiles) is processed as such a k-outer panel,
// one after the other; this is the family for block pools smaller than the working set.
// + 40000: same order, but evictions prefer the tile untouched for longest among those not needed soon (instead of
// the one needed farthest in the future), which lets fetches run ahead of the subkernels.
// + 80000: panel layout (GemmPlan::panels) and merged K chains: wherever the order runs consecutive k-steps of one C
// tile back to back, they become one launch over the joined k range.  That saves the launch's fixed cost -- for the
// large fp32 tiles, whose workgroups hold a compute unit alone, the prologue and epilogue nothing else overlaps -- at
// the price of starting only when all its tiles have arrived.  Needs a pool that holds the whole working set.
constexpr int ORDER_MERGE_CHAINS = 80000;
// w = rows * 100 + columns (rows >= 1): block orders.  That block of C tiles at the top left is the k-outer panel; the
// other rows of its columns and then the other columns follow tile by tile (orient 1: the other columns of its rows,
// then the other rows).  Its C tiles are complete after (rows + columns) * Kg fetched tiles instead of (Mg + w) * Kg,
// so write-backs start earlier: for shapes bounded by the link (dgemm 8192^3 from the host: 24.7 -> 23.3 ms).
constexpr int ORDER_BLOCK_ROWS = 100;
// Panel widths therefore stay below 100, and w = 99 stands for "the whole grid", however many tiles that is (a grid of
// 128 column tiles would otherwise read as the block 1 x 28).
constexpr int ORDER_FULL_PANEL = 99;
// + 160000 * s: thin start (GemmProblem::k_split = 2^s): s = 1 or 2: 2^s equal slabs; s = 3: the graded start.
constexpr int ORDER_K_SPLIT = 160000;
// + 640000: strip end.  The last launch of the call -- the last k-step, or the whole merged K chain, of the C tile the
// order completes last -- is made in row strips of that tile, one launch after the other, and what follows it on those
// rows (with beta != 0 the fetch of the caller's C and the lazy reduce; the write-back) strip by strip behind them, so
// that the copies left over when the last kernel ends are a strip's, not a tile's.  A strip alone has too few
// 128 x 128 tiles for the device, so its launch splits K (Cmd::splits).  Only where C goes back to the host; elsewhere,
// and for a last tile under 512 rows, the id builds the same plan as without it.
constexpr int ORDER_STRIP_END = 640000;
inline int order_id_of(int orient, int w) { return orient * 10000 + w; }
std::vector<int> gemm_task_order(const GemmProblem& p, int order_id);
// probe = true: a handful of representative orders, enough to rank tile sizes before the full search
// merge = true: also the variants with merged K chains (when the pool holds the whole working set)
std::vector<int> gemm_candidate_orders(const GemmProblem& p, bool probe = false, bool merge = false);

// Throws std::runtime_error when pool_blocks cannot hold the minimum working set (3 blocks, dgemm.cpp:90-93).
GemmPlan build_gemm_plan(const GemmProblem& p, int order_id);

// Block pool size the reference would ask for (dgemm.cpp:23-36,80-82).
long gemm_full_block_num(const GemmProblem& p);
// The same with the most slabs a thin start may add: what a caller may offer as pool_blocks at most (the pool is
// allocated for the blocks the chosen plan uses, not for this number).
long gemm_max_block_num(const GemmProblem& p);

// Stage costs of a full T x T (x T) tile; edge tiles scale with their area / volume.
struct StageTimes {
  double t_exec = 0;                 // one T^3 subkernel
  // Optional lookup (cube edge, seconds) sorted by edge: an m x n x k subkernel is priced at the flop rate of the
  // cube of equal volume, so ragged edge tiles cost their (lower) small-kernel rate instead of a pro-rata share.
  std::vector<std::pair<long, double>> exec_table;
  double exec_time(long T, long m, long n, long k) const;
  double h2d_ti = 0, h2d_tb = 0;     // seconds, seconds per byte
  double d2h_ti = 0, d2h_tb = 0;
  double h2d_sl = 1, d2h_sl = 1;     // how much slower a copy runs while the opposite direction is busy (>= 1)
  double t_reduce = 0;               // one T^2 scale-add
  // seconds a launch over kn k tiles of a full T x T C tile takes less than kn separate launches, per launch saved
  // (0: merging K chains is not worth considering for this kernel)
  double merge_saving = 0;
  bool thin_start = true;            // offer the thin start (order ids of 160000 and above) to the order search
  // Power-state transient of the device: after the compute units sat idle, tile kernels start slower and recover while
  // they run.  deficit in [0, 1] grows towards 1 with time constant tr_idle while no kernel runs and decays with
  // tr_recover while one does; a tile kernel takes (1 + tr_amp * deficit) times its steady time.  tr_amp = 0: not modelled.
  double tr_amp = 0, tr_idle = 6e-3, tr_recover = 8e-3;
  double tr_gap0 = 1e-3;             // idle time assumed in front of the call (calls made back to back)
  bool block_orders = true;          // offer the block orders (w >= ORDER_BLOCK_ROWS) to the order search
  // simulate every candidate, also those a bound shows cannot win (merged variants, thin starts of a trailing group):
  // the slow search the pruned one is tested against
  bool exhaustive = false;
  // a slab of the thin start: the full tile's time in proportion to its k, plus this much per launch for slabs 1024 deep
  // or deeper, in inverse proportion to the depth below that (measured inside streamed calls, two launches sharing the
  // device: 2048 x 2048 x 1024 slabs +2 us, x 512 slabs +4.5 us against a quarter of the whole tile's 231.5 us)
  double slab_fixed = 2e-6;
  // a launch that splits K s ways (Cmd::splits): one more round's fixed cost and the reduction's launch, and the
  // reduction's pass over 2 s + 1 copies of the strip
  double split_fixed = 10.6e-6, split_pass_tb = 1.0 / 6.15e12;
  bool strip_end = true;             // offer the strip end (order ids of 640000 and above) to the order search
};
struct PipelineResult {
  double t_total = 0, t_h2d = 0, t_exec = 0, t_d2h = 0;  // makespan and busy time per resource
};
PipelineResult simulate_plan(const GemmPlan& plan, const StageTimes& st);
extern std::atomic<long> plan_simulations;   // plans simulated by this process so far (the order search's unit of work)
// Builds every candidate order, simulates it, returns the id with the smallest makespan.
// (with StageTimes::strip_end, and not for a probe, the winner goes through with_strip_end)
int pick_gemm_order(const GemmProblem& p, const StageTimes& st, PipelineResult* best, bool probe = false);
// The order also with its last C tile in row strips (ORDER_STRIP_END): that id, and its result in *r, when the simulated
// call gets shorter than *r by more than a thousandth; else the id as it came.
int with_strip_end(const GemmProblem& p, const StageTimes& st, int order_id, PipelineResult* r);

}  // namespace paralia
#endif
