// Autotuning controller: picks the tile size T (and, for GEMM, the subkernel order) for one call on one GPU.
//
// Three selectors, all available at run time (PARALIA_T_SELECT = pipeline | reuse | heuristic):
//   heuristic  the reference's main-branch scan of every integer T under penalty terms
//              (Autotuner/src/Autotuner.cpp:571-655);
//   reuse      the reference's model-driven search, argmin of the CoCoPeLia data-reuse model over the
//              benchmarked T values (Model_functions.cpp:195-244 with ModelLvl3.cpp:476-551);
//   pipeline   (default) the same search, but each T is priced by simulating this runtime's actual H2D /
//              compute / D2H command streams for the best subkernel order (runtime/gemm_plan.cpp).
// Without a database only the heuristic is possible.
#include <cfloat>
#include <climits>
#include <cmath>
#include <cstdlib>
#include <algorithm>
#include <cstring>

#include "Autotuner.hpp"
#include "backend_wrappers.hpp"
#include "paralia_hip.h"
#include "runtime/gemm_plan.hpp"

ATC::ATC() {
  active_unit_id_list = (int*)malloc(LOC_NUM * sizeof(int));
  active_unit_score = (double*)malloc(LOC_NUM * sizeof(double));
  Subkernels_per_unit_num = (int*)malloc(LOC_NUM * sizeof(int));
  Subkernels_per_unit_list = (int**)malloc(LOC_NUM * sizeof(int*));
  for (int d = 0; d < LOC_NUM; d++) {
    active_unit_id_list[d] = -42;
    active_unit_score[d] = -42.0;
    Subkernels_per_unit_list[d] = NULL;
    Subkernels_per_unit_num[d] = 0;
  }
  T = active_unit_num = subkernel_num = -1;
  pred_t = pred_J = power_delay = energy_delay = -1.0;
  pred_t_pesimistic = pred_J_pesimistic = power_delay_pesimistic = energy_delay_pesimistic = -1.0;
  T_aggregate_sl = T_imbalance_sl = T_remainder_sl = T_small_sl = T_sknum_sl = T_big_sl = 0.0;
  cache_limit = 0;
  unit_modeler_list = (MD_p*)calloc(LOC_NUM, sizeof(MD_p));
  has_db = false;
  owns_modelers = true;
  order_id = 10000;
  exec_queues = 2;
  T_selected_by = "unset";
}

ATC::~ATC() {
  free(active_unit_id_list);
  free(active_unit_score);
  free(Subkernels_per_unit_num);
  for (int d = 0; d < LOC_NUM; d++) free(Subkernels_per_unit_list[d]);
  free(Subkernels_per_unit_list);
  if (owns_modelers)
    for (int d = 0; d < LOC_NUM; d++) delete unit_modeler_list[d];
  free(unit_modeler_list);
}

void ATC::reset() {
  for (int d = 0; d < LOC_NUM; d++) {
    free(Subkernels_per_unit_list[d]);
    Subkernels_per_unit_list[d] = NULL;
    Subkernels_per_unit_num[d] = 0;
  }
  T = active_unit_num = subkernel_num = -1;
  pred_t = -1.0;
  cache_limit = 0;
}

int ATC::diff_intialized_params_ATC(ATC_p other) {
  int result = 0;
  if (other->T != -1 && other->T != T) result++;
  if (other->active_unit_num != -1 && other->active_unit_num != active_unit_num) result++;
  else if (other->active_unit_num != -1 && other->active_unit_num == active_unit_num) {
    for (int ctr = 0; ctr < active_unit_num; ctr++)
      if (other->active_unit_id_list[ctr] != active_unit_id_list[ctr]) { result++; break; }
  }
  if (other->cache_limit != 0 && other->cache_limit != cache_limit) result++;
  return result;
}

void ATC::mimic_ATC(ATC_p other) {
  T = other->T;
  T_aggregate_sl = other->T_aggregate_sl; T_imbalance_sl = other->T_imbalance_sl; T_remainder_sl = other->T_remainder_sl;
  T_small_sl = other->T_small_sl; T_sknum_sl = other->T_sknum_sl; T_big_sl = other->T_big_sl;
  active_unit_num = other->active_unit_num;
  for (int d = 0; d < LOC_NUM; d++) {
    active_unit_id_list[d] = other->active_unit_id_list[d];
    active_unit_score[d] = other->active_unit_score[d];
    Subkernels_per_unit_num[d] = other->Subkernels_per_unit_num[d];
    free(Subkernels_per_unit_list[d]);
    Subkernels_per_unit_list[d] = NULL;
    if (other->Subkernels_per_unit_list[d] && other->subkernel_num > 0) {
      Subkernels_per_unit_list[d] = (int*)malloc(other->subkernel_num * sizeof(int));
      memcpy(Subkernels_per_unit_list[d], other->Subkernels_per_unit_list[d], other->subkernel_num * sizeof(int));
    }
  }
  split_homogeneously = other->split_homogeneously;
  pred_t = other->pred_t; pred_J = other->pred_J; power_delay = other->power_delay; energy_delay = other->energy_delay;
  pred_t_pesimistic = other->pred_t_pesimistic; pred_J_pesimistic = other->pred_J_pesimistic;
  power_delay_pesimistic = other->power_delay_pesimistic; energy_delay_pesimistic = other->energy_delay_pesimistic;
  subkernel_num = other->subkernel_num;
  cache_limit = other->cache_limit;
  if (owns_modelers)
    for (int d = 0; d < LOC_NUM; d++) delete unit_modeler_list[d];
  owns_modelers = false;  // the original keeps them alive (it sits in the problem-metadata cache)
  for (int d = 0; d < LOC_NUM; d++) unit_modeler_list[d] = other->unit_modeler_list[d];
  problem = other->problem;
  has_db = other->has_db;
  order_id = other->order_id;
  exec_queues = other->exec_queues;
  T_selected_by = other->T_selected_by;
  pipeline = other->pipeline;
}

void ATC::update_sk_num(long long subkernel_num_in) {
  const long prev = subkernel_num;
  subkernel_num = (long)subkernel_num_in;
  if (prev != subkernel_num)
    for (int d = 0; d < LOC_NUM; d++) {
      free(Subkernels_per_unit_list[d]);
      Subkernels_per_unit_list[d] = (int*)malloc(subkernel_num * sizeof(int));
      for (long s = 0; s < subkernel_num; s++) Subkernels_per_unit_list[d][s] = -1;
    }
}

// One unit owns every subkernel: all distributions of the reference (Subkernel_distributions.cpp) collapse
// to the identity list 0 .. n-1 on unit 0.
void ATC::distribute_subkernels(int D1GridSz, int D2GridSz, int D3GridSz) {
  (void)D1GridSz; (void)D2GridSz; (void)D3GridSz;
  for (int d = 0; d < LOC_NUM; d++) Subkernels_per_unit_num[d] = 0;
  Subkernels_per_unit_num[0] = (int)subkernel_num;
  for (long s = 0; s < subkernel_num; s++) Subkernels_per_unit_list[0][s] = (int)s;
}

void ATC::init_modelers(const char* routine_name, const ProblemDesc& desc) {
  (void)routine_name;
  const std::string db = paralia_db_dir();
  if (owns_modelers)
    for (int d = 0; d < LOC_NUM; d++) { delete unit_modeler_list[d]; unit_modeler_list[d] = nullptr; }
  owns_modelers = true;
  // only the GPU unit executes; the host "unit" of the reference (CPU workload) is not used on this path
  unit_modeler_list[0] = new Modeler(db, 0, desc);
}

void ATC::set_T_slowdowns(double* sl) {
  T_aggregate_sl = sl[0]; T_imbalance_sl = sl[1]; T_remainder_sl = sl[2];
  T_small_sl = sl[3]; T_sknum_sl = sl[4]; T_big_sl = sl[5];
}

static long sk_num_of(const ProblemDesc& P, long T) {
  auto cdiv = [](long a, long b) { return a / b + ((a % b) ? 1 : 0); };
  if (P.problem == BLAS3) return cdiv(P.D1, T) * cdiv(P.D2, T) * cdiv(P.D3, T);
  if (P.problem == BLAS2) return cdiv(P.D1, T) * cdiv(P.D2, T);
  return cdiv(P.D1, T);
}

void ATC::get_T_slowdowns(double* slowdown, int candidate_T) {
  // int arithmetic and conversion order as in Autotuner.cpp:571-603
  const int D1 = (int)problem.D1, D2 = (problem.D2 == -1) ? D1 : (int)problem.D2, D3 = (problem.D3 == -1) ? D1 : (int)problem.D3;
  for (int idx = 0; idx < 6; idx++) slowdown[idx] = 0.0;
  ProblemDesc cube = problem;
  cube.problem = BLAS3; cube.D1 = D1; cube.D2 = D2; cube.D3 = D3;
  const long sk = sk_num_of(cube, candidate_T);
  int bucket_num = (int)(sk / (D3 / candidate_T + ((D3 % candidate_T) ? 1 : 0)));
  slowdown[1] = (bucket_num / active_unit_num)
                    ? 1.0 * (bucket_num % active_unit_num) / (bucket_num / active_unit_num) * active_unit_num
                    : 1.0 * bucket_num / active_unit_num;
  if (D1 % candidate_T) slowdown[2] += 1.0 / (D1 / candidate_T);
  if (D2 % candidate_T) slowdown[2] += 1.0 / (D2 / candidate_T);
  if (D3 % candidate_T) slowdown[2] += 1.0 / (D3 / candidate_T);
  if (candidate_T < TILE_MIN) slowdown[3] += 1.0 * TILE_MIN / candidate_T * TILE_MIN_SLOWDOWN;
  long dev_sks = (long)((1.0 * sk) / active_unit_num);
  slowdown[4] += 2.0 / (dev_sks);
  if (dev_sks > MAX_DESIRED_SK_DEV) slowdown[4] += (1.0 * dev_sks / MAX_DESIRED_SK_DEV) * MAX_DESIRED_SK_DEV_SLOWDOWN;
  if (candidate_T > TILE_MAX) slowdown[5] += candidate_T / TILE_MAX * TILE_MAX_SLOWDOWN;
  slowdown[0] = slowdown[1] + slowdown[2] + slowdown[3] + slowdown[4] + slowdown[5];
}

double ATC::optimize_tile() {
  double timer = csecond();
  if (active_unit_num <= 0) error("ATC::optimize_tile: Called with active_unit_num = %d\n", active_unit_num);
  const int D1 = (int)problem.D1, D2 = (problem.D2 == -1) ? D1 : (int)problem.D2, D3 = (problem.D3 == -1) ? D1 : (int)problem.D3;
  const int max_allowed_T = std::min(D1, std::min(D2, D3));
  int best_T = -1;
  double best_sl[6], cur[6];
  for (int i = 0; i < 6; i++) best_sl[i] = DBL_MAX;
  for (int cand = max_allowed_T; cand > 0; cand--) {
    get_T_slowdowns(cur, cand);
    if (cur[0] < best_sl[0]) {
      for (int i = 0; i < 6; i++) best_sl[i] = cur[i];
      best_T = cand;
    }
  }
  T = best_T;
  set_T_slowdowns(best_sl);
  return csecond() - timer;
}

double ATC::optimize_tile_CoCoPeLia(int model_idx, ModelType mode) {
  double timer = csecond();
  MD_p model = unit_modeler_list[model_idx];
  if (!model) error("ATC::optimize_tile_CoCoPeLia: no modeler for unit index %d (database missing?)\n", model_idx);
  long min_T = model->getMinT();
  const long max_allowed_T = model->getMaxT();
  if (min_T > max_allowed_T) {
    T = max_allowed_T;
    pred_t = 0;  // undefined performance below the smallest benchmarked tile
    return csecond() - timer;
  }
  double min_t = model->predict(mode, model->exec->T[0]);
  if (min_t < 0) error("CoCoPeLiaModelOptimizeTile: First value in DM results in negative prediction");
  long prev_trial_T = 0;
  for (long ctr = 1; ctr < model->exec->lines(); ctr++) {
    const long trial_T = model->exec->T[ctr];
    if (trial_T > max_allowed_T) break;
    if (trial_T == prev_trial_T) continue;
    const double temp_t = model->predict(mode, trial_T);
    if (temp_t >= 0 && temp_t < min_t) {
      min_t = temp_t;
      min_T = trial_T;
    }
    prev_trial_T = trial_T;
  }
  T = min_T;
  pred_t = min_t;
  return csecond() - timer;
}

namespace {

paralia::GemmProblem gemm_problem_of(const ProblemDesc& d, long T, int exec_queues) {
  paralia::GemmProblem gp;
  gp.M = d.D1; gp.N = d.D2; gp.K = d.D3; gp.T = T;
  gp.a_remote = remote(d.loc[0], 0); gp.b_remote = remote(d.loc[1], 0); gp.c_remote = remote(d.loc[2], 0);
  gp.beta_zero = d.beta_is_zero;
  gp.elem = d.dtype_sz;
  gp.exec_queues = exec_queues;
  const long full = paralia::gemm_max_block_num(gp);
  gp.pool_blocks = full;
  if (d.pool_budget_bytes > 0) {
    const long long blk = (long long)T * T * d.dtype_sz;
    gp.pool_blocks = (long)std::min<long long>(full, d.pool_budget_bytes / blk);
  }
  return gp;
}

// Nominal MI355X stage costs, used only when no database has been deployed.
paralia::StageTimes nominal_stage_times(const ProblemDesc& d, long T) {
  paralia::StageTimes st;
  const double flops = d.dtype_sz == 8 ? 60e12 : 120e12;
  st.t_exec = 2.0 * T * T * T / flops;
  st.h2d_ti = st.d2h_ti = 10e-6;
  st.h2d_tb = st.d2h_tb = 1.0 / 50e9;
  st.t_reduce = 3.0 * T * T * d.dtype_sz / 3e12;
  return st;
}

}  // namespace

// What one launch over several k tiles of a C tile saves against one launch per k tile, per launch saved.  The fp32
// kernel's larger macro tiles leave no room for a second workgroup on a compute unit, so nothing overlaps a
// workgroup's prologue (first panels) and epilogue (the read-modify-write of its part of C): measured on sgemm
// 32768^3 N/T at T = 4096, 336 launches fewer took 13.5 ms less = 40 us each, for one round of 256 tiles of 256 x 256
// per launch.  The fp64 kernel runs two workgroups per compute unit that cover each other's ends; there a launch saved
// is worth the gap between two launches of a stream: dgemm 16384^3 at T = 2048 with 128 launches fewer (448 instead of
// 576) took 0.55 ms less (123.3 / 123.7 against 123.9 / 124.2 ms), 4 us each.
// Both figures are KernelFit's (merge_saving_us_f64 / _f32): the deploy tool derives them from the launch gap and the
// large tile's fixed cost it measures.
static double paralia_merge_saving(const ProblemDesc& d, long T, const KernelFit& fit) {
  const char* env = getenv("PARALIA_MERGE_CHAINS");  // "0": never merge
  if (env && *env && atoi(env) == 0) return 0.0;
  // measured for tiles that fill the device by themselves; smaller ones run split-K kernels whose time a joined k range
  // changes in ways this term does not describe
  if (d.dtype_sz != 4) return T >= 1792 ? fit.merge_saving_us_f64 * 1e-6 : 0.0;
  // a launch with fewer workgroups than compute units wastes that much less of the device: scale by the rounds of 256
  // workgroups it amounts to, as a fraction
  const double rounds = (double)((T + 255) / 256) * (double)((T + 255) / 256) / 256.0;
  const int tr = d.TransA == 'N' ? (d.TransB == 'N' ? 0 : 1) : (d.TransB == 'N' ? 2 : 3);
  return fit.merge_saving_us_f32[tr] * 1e-6 * rounds;
}

paralia::StageTimes paralia_stage_times(const ATC* atc, long T) {
  const ProblemDesc& d = atc->problem;
  if (!atc->has_db || !atc->unit_modeler_list[0]) return nominal_stage_times(d, T);
  const Modeler* m = atc->unit_modeler_list[0];
  paralia::StageTimes st;
  st.t_exec = m->exec->predict(T, d.TransA, d.TransB);
  for (long i = 0; i < m->exec->lines(); ++i)
    if (m->exec->TransA.empty() || (m->exec->TransA[i] == d.TransA && m->exec->TransB[i] == d.TransB))
      if (st.exec_table.empty() || st.exec_table.back().first < m->exec->T[i])
        st.exec_table.emplace_back(m->exec->T[i], m->exec->av_time[i]);
  // The table holds the time per launch while two compute streams keep the device filled.  In a streamed call a launch
  // also runs without a partner -- on the ramp, at the tail, whenever the other stream waits for a tile -- and then
  // takes its lone time, which for tiles whose workgroups do not fill whole rounds of the device is a third longer.
  // Measured streamed calls behave as if that were the case for about 7 % of a launch (12288^3: T = 3072 predicted
  // 0.3 % faster than T = 2048 without this term, measured 2.3 % slower; 14336^3 and 20000 x 20000 x 4096 alike).
  const double lone_share = m->fit.lone_share;
  st.t_exec *= 1 + lone_share * (m->exec->lone_ratio(T, d.TransA, d.TransB) - 1);
  for (auto& e : st.exec_table) e.second *= 1 + lone_share * (m->exec->lone_ratio(e.first, d.TransA, d.TransB) - 1);
  const comm_data* h2d = m->link[idxize(-1)];
  const comm_data* d2h = m->revlink[idxize(-1)];
  st.h2d_ti = h2d->ti; st.h2d_tb = h2d->tb;
  st.d2h_ti = d2h->ti; st.d2h_tb = d2h->tb;
  st.h2d_sl = std::max(1.0, h2d->sl); st.d2h_sl = std::max(1.0, d2h->sl);
  st.t_reduce = 3.0 * T * T * d.dtype_sz / m->fit.geadd_bytes_per_s;
  st.merge_saving = paralia_merge_saving(d, T, m->fit);
  st.slab_fixed = m->fit.slab_fixed_us * 1e-6;
  const char* thin = getenv("PARALIA_THIN_START");  // "0": never cut the first k tile into slabs
  st.thin_start = !(thin && *thin && atoi(thin) == 0);
  // a strip of the call's last C tile splits K: one more round of workgroups with its fixed cost, the reduction's
  // launch, and the reduction's pass over the slices
  st.split_fixed = (m->fit.launcher.f32_small_fixed_us + m->fit.launcher.splitk_launch_us) * 1e-6;
  st.split_pass_tb = 1e-6 / m->fit.launcher.pass_bytes_per_us;
  const char* strip = getenv("PARALIA_STRIP_END");  // "0": the last C tile is never cut into row strips
  st.strip_end = !(strip && *strip && atoi(strip) == 0);
  if (d.problem == BLAS3 && m->transient_amplitude > 0) {
    st.tr_amp = m->transient_amplitude;
    st.tr_idle = m->transient_idle_s;
    st.tr_recover = m->transient_recover_s;
  }
  const char* search = getenv("PARALIA_PLAN_SEARCH");  // "exhaustive": no candidate is dismissed by a bound
  st.exhaustive = search && !strcmp(search, "exhaustive");
  const char* blk = getenv("PARALIA_BLOCK_ORDERS");  // "0": never start with a block of C tiles smaller than a full panel
  st.block_orders = !(blk && *blk && atoi(blk) == 0);
  return st;
}

double ATC::autotune_problem(const char* routine_name, const ProblemDesc& desc) {
  double timer = csecond();
  problem = desc;
  problem.func = routine_name;
  if (!strcmp(routine_name, "Dgemm") || !strcmp(routine_name, "Sgemm")) problem.problem = BLAS3;
  else if (!strcmp(routine_name, "Dgemv")) problem.problem = BLAS2;
  else if (!strcmp(routine_name, "Daxpy") || !strcmp(routine_name, "Ddot")) problem.problem = BLAS1;
  else error("ATC::autotune_problem: routine %s not integrated\n", routine_name);

  // one GPU: the unit list is {0} whatever was asked for (predefined lists naming other units are an error)
  if (active_unit_num > 1) error("ATC::autotune_problem: %d units requested, this build drives one GPU\n", active_unit_num);
  if (active_unit_num == 1 && active_unit_id_list[0] != 0)
    error("ATC::autotune_problem: unit id %d requested, only device 0 is driven\n", active_unit_id_list[0]);
  active_unit_num = 1;
  active_unit_id_list[0] = 0;
  active_unit_score[0] = 1.0;

  const char* sel_env = getenv("PARALIA_T_SELECT");
  std::string selector = sel_env ? sel_env : "pipeline";
  has_db = false;
  try {
    init_modelers(routine_name, problem);
    has_db = true;
  } catch (const paralia_error& e) {
    static bool warned = false;
    if (!warned) warning("autotuner database not usable (%s); falling back to the tile heuristic\n", e.what());
    warned = true;
    if (owns_modelers)
      for (int d = 0; d < LOC_NUM; d++) { delete unit_modeler_list[d]; unit_modeler_list[d] = nullptr; }
  }

  bool any_remote = false;
  for (int i = 0; i < problem.numT; i++) any_remote |= remote(problem.loc[i], 0) != 0;
  const char* q_env = getenv("PARALIA_EXEC_QUEUES");
  if (q_env && atoi(q_env) > 0) exec_queues = std::min(atoi(q_env), (int)paralia::MAX_EXEC_QUEUES);
  pipeline = PipelineEstimate();

  if (problem.problem == BLAS3) {
    int searched_order = -1;            // order search result of the tile size the pipeline model chose, if it ran
    paralia::PipelineResult searched_r;
    const long min_dim = std::min(problem.D1, std::min(problem.D2, problem.D3));
    const long max_dim = std::max(problem.D1, std::max(problem.D2, problem.D3));
    if (T > 0) {
      if (T > max_dim) T = max_dim;  // a tile larger than every dimension is the whole problem
      T_selected_by = "user";
    } else if (!any_remote) {
      // nothing to stream: one launch over the caller's matrices, T only labels the call
      T = max_dim;
      T_selected_by = "resident";
    } else if (!has_db || selector == "heuristic") {
      optimize_tile();
      T_selected_by = "heuristic";
    } else if (selector == "reuse" || selector == "cocopelia") {
      optimize_tile_CoCoPeLia(0, COCOPELIA_REUSE);
      T_selected_by = "cocopelia-reuse";
    } else {
      const Modeler* m = unit_modeler_list[0];
      // Two passes over the benchmarked tile sizes.  The first prices each T with a handful of representative
      // subkernel orders (largest tiles first: they have few subkernels and are cheap to simulate, and once a good
      // makespan is known the small tiles, whose kernels alone already take longer than that, are dismissed without
      // building a plan).  The second runs the full order search for the (at most three) T whose penalised probe is
      // within 10 % of the best, best probe first, and skips a T whose floor is above a result already in hand.
      struct Cand { long T; double probe_t, floor_t; };
      // The tile size is chosen without the strip end: row strips take most of the last write-back off every tile size,
      // and the larger the tile the more -- but a grid of few large tiles also ends with one compute stream idle for
      // longer, which the simulated device (kernels one at a time) does not see (16384^3: T = 4096 with strips simulated
      // 0.2 % faster than T = 2048 with strips, measured 1.3 % slower).  The chosen tile's order gets its strips below.
      auto search_times = [&](long cand) {
        paralia::StageTimes st = paralia_stage_times(this, cand);
        st.strip_end = false;
        return st;
      };
      constexpr long PROBE_ABOVE_SUBKERNELS = 48;
      const char* verbose_env = getenv("PARALIA_VERBOSE");
      const bool chatty = verbose_env && atoi(verbose_env) > 1;
      const char* search_env = getenv("PARALIA_PLAN_SEARCH");
      const bool exhaustive = search_env && !strcmp(search_env, "exhaustive");
      // predictions of neighbouring T differ by less than the model's accuracy: the reference's penalty terms
      // (ragged edges, too few or too many subkernels, Autotuner.cpp:571-603) break such near-ties
      auto penalty = [&](long cand) {
        if (cand > min_dim) return 1.0;
        double sl[6];
        get_T_slowdowns(sl, (int)cand);
        return 1.0 + 0.02 * sl[0];
      };
      // What no order of a tile size can beat: the tile kernels run one at a time on the simulated device, so a call
      // takes at least the sum of its subkernels' times, less what merged K chains can save at most (one saving per
      // k-step after a C tile's first).  A tile size whose floor is above a makespan already found is dismissed without
      // building a single plan -- for the small tiles, whose plans have thousands of commands, that is most of the
      // search's time.
      auto compute_floor = [&](const paralia::GemmProblem& gp, const paralia::StageTimes& st) {
        double total = 0;
        const long kfull = problem.D3 / gp.T, krem = problem.D3 % gp.T;
        for (int mi = 0; mi < gp.Mg(); ++mi)
          for (int ni = 0; ni < gp.Ng(); ++ni) {
            const long m = gp.tm(mi), n = gp.tn(ni);
            total += kfull * st.exec_time(gp.T, m, n, gp.T) + (krem ? st.exec_time(gp.T, m, n, krem) : 0.0);
          }
        const double saved = (double)(gp.subkernels() - (long)gp.Mg() * gp.Ng()) * st.merge_saving;
        return std::max(0.5 * total, total - saved);
      };
      // ... and at both ends nothing overlaps: no kernel starts before the first pair of A and B tiles has crossed the
      // link (an eighth of each, if the graded thin start applies), and the C tile of the last kernel goes
      // back (after its lazy reduce) when every kernel has finished.
      auto call_floor = [&](const paralia::GemmProblem& gp, const paralia::StageTimes& st) {
        double t = compute_floor(gp, st);
        const double eighth = (double)gp.T * std::min<long>(gp.T, problem.D3) / 8.0 * problem.dtype_sz;
        if (gp.a_remote) t += st.h2d_ti + st.h2d_tb * std::min<double>(eighth, (double)gp.tm(gp.Mg() - 1) * std::min<long>(gp.T, problem.D3) / 8.0 * problem.dtype_sz);
        if (gp.b_remote) t += st.h2d_ti + st.h2d_tb * std::min<double>(eighth, (double)gp.tn(gp.Ng() - 1) * std::min<long>(gp.T, problem.D3) / 8.0 * problem.dtype_sz);
        if (gp.c_remote) {
          const double smallest = (double)std::min(gp.tm(0), gp.tm(gp.Mg() - 1)) * std::min(gp.tn(0), gp.tn(gp.Ng() - 1));
          // (of a last tile cut into row strips, one strip: no thinner than a 128-row tile of the kernel)
          const bool strips = st.strip_end && st.merge_saving > 0;
          const double last_rows = (double)std::min(std::min(gp.tm(0), gp.tm(gp.Mg() - 1)), strips ? 128L : LONG_MAX);
          t += st.d2h_ti + st.d2h_tb * last_rows * std::min(gp.tn(0), gp.tn(gp.Ng() - 1)) * problem.dtype_sz;
          if (!gp.beta_zero) t += st.t_reduce * smallest / ((double)gp.T * gp.T);
        }
        return t;
      };
      // the tile sizes in the order of their floors: a good makespan early dismisses the most
      struct Entry { long T; double floor_t; paralia::GemmProblem gp; };
      std::vector<Entry> entries;
      long prev = -1;
      for (long i = m->exec->lines() - 1; i >= 0; i--) {
        const long cand = m->exec->T[i];
        if (cand == prev) continue;
        prev = cand;
        // tiles may be shallower than T in K (depth min(T, K)), so only M and N bound the candidates
        if (cand > std::min(problem.D1, problem.D2)) continue;
        // MinAllowedTBLAS3 (ModelLvl3.cpp): tiles below 1024 are not considered when the problem is larger than that
        if (cand < m->getMinT() && std::min(problem.D1, problem.D2) >= m->getMinT()) continue;
        paralia::GemmProblem gp = gemm_problem_of(problem, cand, exec_queues);
        if (gp.pool_blocks < 3 || gp.subkernels() > 20000) continue;
        entries.push_back({cand, call_floor(gp, search_times(cand)) * penalty(cand), gp});
      }
      std::stable_sort(entries.begin(), entries.end(), [](const Entry& x, const Entry& y) { return x.floor_t < y.floor_t; });
      std::vector<Cand> cands;
      double best_probe = DBL_MAX, best_probe_score = DBL_MAX;
      for (const Entry& e : entries) {
        const long cand = e.T;
        if (e.floor_t > best_probe_score && !exhaustive) break;   // and so is every floor behind it
        paralia::PipelineResult r;
        try {
          // a grid of a few dozen subkernels gets the full order search at once: its plans cost microseconds, and the
          // handful of orders of a probe misses the block orders that win there (sgemm 4096^3 from the host: T = 1536
          // probed at 3.24 ms, searched at 3.08, and left out of the finalists)
          paralia::pick_gemm_order(e.gp, search_times(cand), &r, /*probe=*/e.gp.subkernels() > PROBE_ABOVE_SUBKERNELS);
        } catch (const std::runtime_error&) { continue; }
        cands.push_back({cand, r.t_total * penalty(cand), e.floor_t});
        best_probe = std::min(best_probe, r.t_total);
        best_probe_score = std::min(best_probe_score, r.t_total * penalty(cand));
        if (chatty) fprintf(stderr, "  probe T = %ld: %.3lf ms (floor %.3lf), %ld plans simulated so far\n", cand, r.t_total * 1e3, e.floor_t * 1e3, paralia::plan_simulations.load());
      }
      // back to table order (largest T first): what the selection below was written for
      std::sort(cands.begin(), cands.end(), [](const Cand& x, const Cand& y) { return x.T > y.T; });
      long best_T = -1;
      double best_t = DBL_MAX;
      int best_order = -1;
      paralia::PipelineResult best_r;
      // at most the three best probes go on (kept in table order, largest T first, so that ties still go to the
      // smaller tile below)
      double cut = DBL_MAX;
      if (cands.size() > 3) {
        std::vector<double> ts;
        for (const Cand& c : cands) ts.push_back(c.probe_t);
        std::nth_element(ts.begin(), ts.begin() + 2, ts.end());
        cut = ts[2];
      }
      // the full search of the best probe first: its result dismisses the others by their floors
      std::vector<const Cand*> finalists;
      for (const Cand& c : cands)
        if (!(c.probe_t > 1.1 * best_probe || c.probe_t > cut)) finalists.push_back(&c);
      std::stable_sort(finalists.begin(), finalists.end(), [](const Cand* x, const Cand* y) { return x->probe_t < y->probe_t; });
      // A tile size that cuts the problem into thousands of subkernels costs its full search 10 - 20 ms and the call as
      // many launches and copies; it goes on only when its probe is 2 % ahead of the best finalist with fewer (the
      // full search moves a probe by 1 - 2 %, so anything closer is a tie the lighter plan should win)
      constexpr long HEAVY_SUBKERNELS = 2048;
      auto subkernels_of = [&](long cand) { return gemm_problem_of(problem, cand, exec_queues).subkernels(); };
      double best_light_probe = DBL_MAX;
      for (const Cand* c : finalists)
        if (subkernels_of(c->T) <= HEAVY_SUBKERNELS) best_light_probe = std::min(best_light_probe, c->probe_t);
      for (const Cand* c : finalists) {
        if (c->floor_t > best_t && !exhaustive) continue;
        const long cand = c->T;
        if (!exhaustive && best_light_probe < DBL_MAX && subkernels_of(cand) > HEAVY_SUBKERNELS && c->probe_t > 0.98 * best_light_probe) continue;
        paralia::GemmProblem gp = gemm_problem_of(problem, cand, exec_queues);
        paralia::PipelineResult r;
        int oid = -1;
        try {
          oid = paralia::pick_gemm_order(gp, search_times(cand), &r);
        } catch (const std::runtime_error&) { continue; }
        const double score = r.t_total * penalty(cand);
        if (chatty) fprintf(stderr, "  full search T = %ld: %.3lf ms, order %d, %ld plans simulated so far\n", cand, r.t_total * 1e3, oid, paralia::plan_simulations.load());
        if (score < best_t || (score == best_t && cand < best_T)) {  // ties go to the smaller tile
          best_t = score; best_T = cand; best_order = oid; best_r = r;
        }
      }
      if (best_T >= 0) {
        const paralia::StageTimes st = paralia_stage_times(this, best_T);
        if (st.strip_end) best_order = paralia::with_strip_end(gemm_problem_of(problem, best_T, exec_queues), st, best_order, &best_r);
        searched_order = best_order; searched_r = best_r;
      }
      if (best_T < 0) {
        // C narrower than every benchmarked tile: one tile across the short side, as square as that allows
        T = std::max(std::min(problem.D1, problem.D2), std::min(max_dim, m->exec->MinT()));
        T_selected_by = "heuristic";
      } else {
        T = best_T;
        T_selected_by = "pipeline-model";
      }
    }
    if (T <= 0) error("ATC::autotune_problem: T = %ld after tuning\n", T);
    if (T <= min_dim) {
      double sl[6];
      get_T_slowdowns(sl, (int)T);
      set_T_slowdowns(sl);
    }
    // order + predicted time for the chosen T
    paralia::GemmProblem gp = gemm_problem_of(problem, T, exec_queues);
    if (any_remote && gp.pool_blocks < 3)
      error("PARALiA gemm: Problem cannot run with less memory than %lld\n", 3LL * T * T * problem.dtype_sz);
    paralia::PipelineResult r;
    try {
      // the tile search has already run the order search of the tile it chose
      if (searched_order >= 0) { order_id = searched_order; r = searched_r; }
      else order_id = paralia::pick_gemm_order(gp, paralia_stage_times(this, T), &r);
      // PARALIA_GEMM_ORDER pins the subkernel order family (gemm_plan.hpp) when that order fits the block pool
      const char* o_env = getenv("PARALIA_GEMM_ORDER");
      if (o_env && *o_env) {
        try {
          r = paralia::simulate_plan(paralia::build_gemm_plan(gp, atoi(o_env)), paralia_stage_times(this, T));
          order_id = atoi(o_env);
        } catch (const std::runtime_error&) {}
      }
    } catch (const std::runtime_error& e) { error("%s\n", e.what()); }
    pipeline.t_total = r.t_total; pipeline.t_h2d_busy = r.t_h2d; pipeline.t_exec_busy = r.t_exec;
    pipeline.t_d2h_busy = r.t_d2h; pipeline.order_id = order_id;
    pred_t = r.t_total;
    pred_t_pesimistic = r.t_h2d + r.t_exec + r.t_d2h;
    if (!any_remote && T >= max_dim) {
      // One product alone on the device: the launcher's own model of it (whole rounds of workgroups, split K, the head /
      // tail cut, the fp32 macro tiles) instead of the tile table stretched to the product's size, plus the launch and
      // the synchronisation of the call.  Over 124 device-resident shapes (M, N up to 8192, K 512 .. 16384, both
      // precisions) the median error went from 4.6 % to 2.5 %, the largest from 42 % to 22 %.
      const double us = pl_gemm_tile_alone_us(problem.dtype_sz, problem.TransA, problem.TransB, problem.D1, problem.D2, problem.D3,
                                              problem.beta_is_zero ? 1 : 0, 1L << 30);
      if (us > 0) pred_t = pred_t_pesimistic = us * 1e-6 + 8e-6;
    }
    gp.k_split = 1 << (order_id % paralia::ORDER_STRIP_END / paralia::ORDER_K_SPLIT);  // a thin start adds k tiles
    update_sk_num(gp.subkernels());
    distribute_subkernels(gp.Mg(), gp.Ng(), gp.Kg());
  } else if (problem.problem == BLAS2) {
    // dgemv streams every A tile over the link exactly once and the kernels are three orders of magnitude faster
    // than the copies, so the call is a two-stage pipeline (tile copies, tile kernels) with the vectors riding
    // along.  Each benchmarked T is priced by walking that pipeline in the subkernel order mi * Ng + ni
    // (dgemv.cpp:57-60); the reference's own BLAS-2 model (ModelLvl2.cpp:194-259) is available as
    // PARALIA_T_SELECT=cocopelia.
    const long M = problem.D1, N = problem.D2;
    const long max_dim = std::max(M, N);
    const bool a_remote = remote(problem.loc[0], 0) != 0;
    const bool is_n = problem.TransA == 'N';
    auto cdiv = [](long a, long b) { return a / b + ((a % b) ? 1 : 0); };
    auto estimate = [&](long cand) -> double {
      const Modeler* m = unit_modeler_list[0];
      const comm_data* h2d = m->link[idxize(-1)];
      const comm_data* d2h = m->revlink[idxize(-1)];
      const double t_exec = m->exec->predict(cand, problem.TransA);
      const long len_x = is_n ? N : M, len_y = is_n ? M : N;
      double copy_end = 0, exec_end = 0;
      if (remote(problem.loc[1], 0)) copy_end += t_com_predict(h2d, (double)len_x * problem.dtype_sz);
      if (remote(problem.loc[2], 0) && !problem.beta_is_zero) copy_end += t_com_predict(h2d, (double)len_y * problem.dtype_sz);
      exec_end = copy_end;
      for (long mi = 0; mi < cdiv(M, cand); ++mi)
        for (long ni = 0; ni < cdiv(N, cand); ++ni) {
          const double tm = (double)std::min(cand, M - mi * cand), tn = (double)std::min(cand, N - ni * cand);
          if (a_remote) copy_end += t_com_predict(h2d, tm * tn * problem.dtype_sz);
          exec_end = std::max(exec_end, copy_end) + t_exec * (tm * tn) / ((double)cand * cand);
        }
      if (remote(problem.loc[2], 0)) exec_end += t_com_predict(d2h, (double)len_y * problem.dtype_sz);
      return exec_end;
    };
    if (T > 0) {
      if (T > max_dim) T = max_dim;
      T_selected_by = "user";
    } else if (!a_remote) {
      T = max_dim;  // A already in HBM: one launch over the caller's matrix
      T_selected_by = "resident";
    } else if (!has_db) {
      T = std::min(max_dim, 4096L);  // 128 MiB tiles: the link runs at its asymptotic rate
      T_selected_by = "heuristic";
    } else if (selector == "cocopelia" || selector == "reuse") {
      optimize_tile_CoCoPeLia(0, COCOPELIA_BIDIRECTIONAL);
      T_selected_by = "cocopelia-bidirectional";
    } else {
      const Modeler* m = unit_modeler_list[0];
      long best_T = -1, prev = -1;
      double best_t = DBL_MAX;
      for (long i = 0; i < m->exec->lines(); i++) {
        const long cand = m->exec->T[i];
        if (cand == prev || cand > max_dim) continue;
        prev = cand;
        if (problem.pool_budget_bytes > 0 && 4LL * cand * cand * problem.dtype_sz > problem.pool_budget_bytes) continue;
        const double t = estimate(cand);
        if (t < best_t) { best_t = t; best_T = cand; }
      }
      if (best_T < 0) {
        T = std::min(max_dim, m->exec->MinT());
        T_selected_by = "heuristic";
      } else {
        T = best_T;
        T_selected_by = "pipeline-model";
      }
    }
    if (T <= 0) error("ATC::autotune_problem: T = %ld after tuning\n", T);
    if (has_db) pred_t = estimate(T);
    update_sk_num(sk_num_of(problem, T));
    distribute_subkernels((int)cdiv(M, T), (int)cdiv(N, T), 1);
  } else {
    const long N = problem.D1;
    if (T > 0) {
      if (T > N) T = N;
      T_selected_by = "user";
    } else if (!any_remote) {
      T = N;
      T_selected_by = "resident";
    } else if (has_db) {
      optimize_tile_CoCoPeLia(0, COCOPELIA_BIDIRECTIONAL);
      T_selected_by = "cocopelia-bidirectional";
    } else {
      T = std::min(N, 1L << 22);  // 32 MiB tiles: large enough to run the link at its asymptotic rate
      T_selected_by = "heuristic";
    }
    if (T <= 0) T = std::max(1L, N);
    if (has_db && any_remote) pred_t = unit_modeler_list[0]->predict(COCOPELIA_BIDIRECTIONAL, T);
    else if (has_db) pred_t = unit_modeler_list[0]->exec->predict(T);
    update_sk_num(sk_num_of(problem, T));
    distribute_subkernels((int)subkernel_num, 1, 1);
  }
  pred_J = -1.0;  // no power sampling on this platform
  const char* verbose = getenv("PARALIA_VERBOSE");
  if (verbose && atoi(verbose) > 1)
    fprintf(stderr, "ATC::autotune_problem: %ld plans simulated so far in this process, this search took %.2lf ms\n",
            paralia::plan_simulations.load(), (csecond() - timer) * 1000);
  if (verbose && atoi(verbose) > 0) {
    fprintf(stderr, "====================================\n");
    fprintf(stderr, "ATC::autotune_problem: %s (%ld,%ld,%ld) -> T = %ld [%s], order %d, %ld subkernels, "
            "predicted %.3lf ms (h2d %.3lf, exec %.3lf, d2h %.3lf busy)\n", routine_name, problem.D1, problem.D2, problem.D3,
            T, T_selected_by, order_id, subkernel_num, pred_t * 1000, pipeline.t_h2d_busy * 1000,
            pipeline.t_exec_busy * 1000, pipeline.t_d2h_busy * 1000);
    fprintf(stderr, "====================================\n");
  }
  return csecond() - timer;
}

void ATC::print() {
  fprintf(stderr, "Autotune controller:\n->T = %ld\n->active_unit_num = %d\n->pred_t = %lf\n->subkernel_num = %ld\n"
          "->cache_limit = %lld\n->order_id = %d\n->T_selected_by = %s\n\n", T, active_unit_num, pred_t, subkernel_num,
          cache_limit, order_id, T_selected_by);
}

// "T,active_unit_num,dev_ids_token,cache_limit" -- the first four columns of a runner log row
// (Autotuner.cpp:839-846; testing.cpp:420-428).
const char* ATC::print_csv() {
  char* outstring = (char*)malloc(256 * sizeof(char));
  int dev_ids_token = 0;
  if (active_unit_num > 0)
    for (int i = 0; i < active_unit_num; i++) dev_ids_token += (int)pow(10, idxize(active_unit_id_list[i]));
  snprintf(outstring, 256, "%ld,%d,%d,%lld", T, active_unit_num, dev_ids_token, cache_limit);
  return outstring;
}
