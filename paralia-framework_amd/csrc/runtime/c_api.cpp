// extern "C" faces of the routines, the helper surface and a few read-only probes of the host logic
// (autotuner, planner) so that tests and foreign-language hosts can reach them without C++ linkage.
// Errors become status codes here; the message of the last one is kept per thread.
#include <cstring>
#include <memory>
#include <string>

#include "PARALiA.hpp"
#include "backend_wrappers.hpp"
#include "gemm_plan.hpp"
#include "host_staging.hpp"
#include "paralia_hip.h"

namespace paralia {
ATC_p dgemm_impl(char, char, long, long, long, double, double*, long, double*, long, double, double*, long, ATC_p);
ATC_p sgemm_impl(char, char, long, long, long, float, float*, long, float*, long, float, float*, long, ATC_p);
ATC_p dgemv_impl(char, long, long, double, double*, long, double*, long, double, double*, long, ATC_p);
ATC_p daxpy_impl(long, double, double*, long, double*, long, ATC_p);
ATC_p ddot_impl(long, double*, long, double*, long, double*, ATC_p);
void cache_free_impl(short);
void runtime_stats(long*, long*, long long*, long*);
void runtime_reset();
void stream_queues(int*, int*);
void last_call_phases(double*);
void runtime_shutdown();
void trace_enable(int);
long trace_read(double*, long);
}  // namespace paralia
paralia::StageTimes paralia_stage_times(const ATC* atc, long T);

namespace {
thread_local std::string g_msg = "no error";

void fill_info(pl_atc_info* info, ATC_p atc) {
  if (!info || !atc) return;
  memset(info, 0, sizeof(*info));
  info->T = atc->T;
  info->pred_t = atc->pred_t;
  info->subkernel_num = atc->subkernel_num;
  info->order_id = atc->order_id;
  info->exec_queues = atc->exec_queues;
  info->cache_limit = atc->cache_limit;
  info->has_db = atc->has_db ? 1 : 0;
  strncpy(info->selected_by, atc->T_selected_by ? atc->T_selected_by : "", sizeof(info->selected_by) - 1);
  info->slowdowns[0] = atc->T_aggregate_sl; info->slowdowns[1] = atc->T_imbalance_sl; info->slowdowns[2] = atc->T_remainder_sl;
  info->slowdowns[3] = atc->T_small_sl; info->slowdowns[4] = atc->T_sknum_sl; info->slowdowns[5] = atc->T_big_sl;
  info->pipe_total = atc->pipeline.t_total; info->pipe_h2d = atc->pipeline.t_h2d_busy;
  info->pipe_exec = atc->pipeline.t_exec_busy; info->pipe_d2h = atc->pipeline.t_d2h_busy;
}

template <typename F> int guarded(F&& f) {
  try {
    f();
    return PL_OK;
  } catch (const paralia_error& e) {
    g_msg = e.what();
    return e.code ? e.code : PL_ERR_ARG;
  } catch (const std::exception& e) {
    g_msg = e.what();
    return PL_ERR_ARG;
  }
}

ATC* make_predef(long T, long long cache_limit) {
  if (T <= 0 && cache_limit <= 0) return nullptr;
  ATC* p = new ATC();
  p->T = T > 0 ? T : -1;
  p->cache_limit = cache_limit > 0 ? cache_limit : 0;
  return p;
}
}  // namespace

extern "C" {

const char* PARALiA_last_error(void) { return g_msg.c_str(); }

int PARALiA_dgemm(char TransA, char TransB, long M, long N, long K, double alpha, double* A, long ldA, double* B, long ldB,
                  double beta, double* C, long ldC, long T, long long cache_limit, pl_atc_info* info) {
  return guarded([&] {
    std::unique_ptr<ATC> predef(make_predef(T, cache_limit));
    std::unique_ptr<ATC> out(paralia::dgemm_impl(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, predef.get()));
    fill_info(info, out.get());
  });
}
int PARALiA_sgemm(char TransA, char TransB, long M, long N, long K, float alpha, float* A, long ldA, float* B, long ldB,
                  float beta, float* C, long ldC, long T, long long cache_limit, pl_atc_info* info) {
  return guarded([&] {
    std::unique_ptr<ATC> predef(make_predef(T, cache_limit));
    std::unique_ptr<ATC> out(paralia::sgemm_impl(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, predef.get()));
    fill_info(info, out.get());
  });
}
int PARALiA_dgemv(char TransA, long M, long N, double alpha, double* A, long ldA, double* x, long incx, double beta, double* y,
                  long incy, long T, long long cache_limit, pl_atc_info* info) {
  return guarded([&] {
    std::unique_ptr<ATC> predef(make_predef(T, cache_limit));
    std::unique_ptr<ATC> out(paralia::dgemv_impl(TransA, M, N, alpha, A, ldA, x, incx, beta, y, incy, predef.get()));
    fill_info(info, out.get());
  });
}
int PARALiA_daxpy(long N, double alpha, double* x, long incx, double* y, long incy, long T, pl_atc_info* info) {
  return guarded([&] {
    std::unique_ptr<ATC> predef(make_predef(T, 0));
    std::unique_ptr<ATC> out(paralia::daxpy_impl(N, alpha, x, incx, y, incy, predef.get()));
    fill_info(info, out.get());
  });
}
int PARALiA_ddot(long N, double* x, long incx, double* y, long incy, double* result, long T, pl_atc_info* info) {
  return guarded([&] {
    std::unique_ptr<ATC> predef(make_predef(T, 0));
    std::unique_ptr<ATC> out(paralia::ddot_impl(N, x, incx, y, incy, result, predef.get()));
    fill_info(info, out.get());
  });
}
// The multi-threaded strided host copy that gathers / scatters tiles of pageable operands (host_staging.hpp).
int PARALiA_host_copy2d(void* dst, long dst_pitch, const void* src, long src_pitch, long width_bytes, long cols, int threads) {
  return guarded([&] {
    if (!dst || !src || dst_pitch < width_bytes || src_pitch < width_bytes || width_bytes < 0 || cols < 0 || threads < 1)
      throw paralia_error(PL_ERR_ARG, "PARALiA_host_copy2d: invalid argument\n");
    paralia::CopyThreads pool(threads);
    pool.copy2d(dst, (size_t)dst_pitch, src, (size_t)src_pitch, (size_t)width_bytes, cols);
  });
}
int PARALiA_dev_cache_free(int dev_id) {
  return guarded([&] { paralia::cache_free_impl((short)dev_id); });
}
int PARALiA_runtime_stats(long* pmd_hits, long* pmd_misses, long long* pool_bytes, long* pmd_entries) {
  return guarded([&] { paralia::runtime_stats(pmd_hits, pmd_misses, pool_bytes, pmd_entries); });
}
int PARALiA_runtime_reset(void) {
  return guarded([&] { paralia::runtime_reset(); });
}
int PARALiA_runtime_shutdown(void) {
  return guarded([&] { paralia::runtime_shutdown(); });
}
int PARALiA_trace_enable(int on) {
  return guarded([&] { paralia::trace_enable(on); });
}
long PARALiA_trace_read(double* rows, long max_rows) {
  long n = -1;
  guarded([&] { n = paralia::trace_read(rows, max_rows); });
  return n;
}
int PARALiA_last_call_phases(double seconds[6]) {
  return guarded([&] {
    if (!seconds) throw paralia_error(PL_ERR_NULL, "PARALiA_last_call_phases: null output\n");
    paralia::last_call_phases(seconds);
  });
}
int PARALiA_stream_queues(int* independent, int* created) {
  return guarded([&] { paralia::stream_queues(independent, created); });
}
int PARALiA_set_db_dir(const char* dir) {
  paralia_set_db_dir(dir);
  return PL_OK;
}

// ---- helper surface ----
int PARALiA_malloc(void** ptr, long long bytes, int loc) {
  return guarded([&] { *ptr = CoCoMalloc(bytes, (short)loc, 1); });
}
int PARALiA_free(void* ptr, int loc) {
  return guarded([&] { CoCoFree(ptr, (short)loc); });
}
int PARALiA_vec_init_f64(double* p, long long n, int seed, int loc) {
  return guarded([&] { CoCoVecInit<double>(p, n, seed, (short)loc); });
}
int PARALiA_vec_init_f32(float* p, long long n, int seed, int loc) {
  return guarded([&] { CoCoVecInit<float>(p, n, seed, (short)loc); });
}
int PARALiA_test_equality_f64(double* ref, double* x, long long n) { return Dtest_equality(ref, x, n); }
int PARALiA_test_equality_f32(float* ref, float* x, long long n) { return Stest_equality(ref, x, n); }

// ---- host-logic probes (no GPU needed) ----
long PARALiA_heuristic_tile(long D1, long D2, long D3, double slowdowns[6]) {
  long T = -1;
  int rc = guarded([&] {
    ATC atc;
    atc.problem.problem = BLAS3; atc.problem.D1 = D1; atc.problem.D2 = D2; atc.problem.D3 = D3;
    atc.active_unit_num = 1; atc.active_unit_id_list[0] = 0;
    atc.optimize_tile();
    T = atc.T;
    if (slowdowns) {
      slowdowns[0] = atc.T_aggregate_sl; slowdowns[1] = atc.T_imbalance_sl; slowdowns[2] = atc.T_remainder_sl;
      slowdowns[3] = atc.T_small_sl; slowdowns[4] = atc.T_sknum_sl; slowdowns[5] = atc.T_big_sl;
    }
  });
  return rc == PL_OK ? T : -1;
}

int PARALiA_T_slowdowns(long D1, long D2, long D3, long T, double slowdowns[6]) {
  return guarded([&] {
    ATC atc;
    atc.problem.problem = BLAS3; atc.problem.D1 = D1; atc.problem.D2 = D2; atc.problem.D3 = D3;
    atc.active_unit_num = 1; atc.active_unit_id_list[0] = 0;
    atc.get_T_slowdowns(slowdowns, (int)T);
  });
}

static ProblemDesc desc_of(const char* func, long D1, long D2, long D3, char ta, char tb, const int loc[3], int beta_zero) {
  ProblemDesc d;
  d.func = func;
  const bool l1 = !strcmp(func, "Daxpy") || !strcmp(func, "Ddot");
  const bool l2 = !strcmp(func, "Dgemv");
  d.problem = l1 ? BLAS1 : l2 ? BLAS2 : BLAS3;
  d.D1 = D1; d.D2 = l1 ? 1 : D2; d.D3 = (l1 || l2) ? 1 : D3;
  d.TransA = ta; d.TransB = tb;
  d.dtype_sz = !strcmp(func, "Sgemm") ? 4 : 8;
  d.numT = l1 ? 2 : 3;
  if (l1) { d.in[2] = 0; d.out[0] = 0; d.out[1] = !strcmp(func, "Daxpy") ? 1 : 0; d.out[2] = 0; }
  for (int i = 0; i < 3; ++i) d.loc[i] = d.out_loc[i] = (i < d.numT) ? loc[i] : 0;
  d.beta_is_zero = beta_zero != 0;
  return d;
}

// Prediction of one model for one T from the database under db_dir; negative on error.
double PARALiA_model_predict(const char* db_dir, const char* func, int mode, long D1, long D2, long D3, char ta, char tb,
                             const int loc[3], long T) {
  double out = -1;
  guarded([&] {
    Modeler m(db_dir, 0, desc_of(func, D1, D2, D3, ta, tb, loc, 0));
    out = m.predict((ModelType)mode, T);
  });
  return out;
}

// Full autotune (no GPU calls): selector as in PARALIA_T_SELECT; T_in > 0 presets the tile.
int PARALiA_autotune(const char* db_dir, const char* func, long D1, long D2, long D3, char ta, char tb, const int loc[3],
                     int beta_zero, long T_in, long long pool_budget_bytes, pl_atc_info* info) {
  return guarded([&] {
    if (db_dir) paralia_set_db_dir(db_dir);
    ATC atc;
    if (T_in > 0) atc.T = T_in;
    ProblemDesc d = desc_of(func, D1, D2, D3, ta, tb, loc, beta_zero);
    d.pool_budget_bytes = pool_budget_bytes;
    atc.autotune_problem(func, d);
    fill_info(info, &atc);
  });
}

static paralia::GemmProblem gp_of(long M, long N, long K, long T, int a_remote, int b_remote, int c_remote, int beta_zero,
                                  int elem, int exec_queues, long pool_blocks) {
  paralia::GemmProblem gp;
  gp.M = M; gp.N = N; gp.K = K; gp.T = T;
  gp.a_remote = a_remote; gp.b_remote = b_remote; gp.c_remote = c_remote; gp.beta_zero = beta_zero;
  gp.elem = elem; gp.exec_queues = exec_queues;
  gp.pool_blocks = pool_blocks > 0 ? pool_blocks : paralia::gemm_max_block_num(gp);
  return gp;
}

// Builds the static plan and writes it as rows of PL_PLAN_ROW ints:
// kind, mi, ni, ki, stream, block, a_block, b_block, beta_mode, nwait, wait[0..PL_PLAN_MAX_WAITS-1], kn (k tiles of a
// GEMM launch; more than 1 only for order ids of 80000 and above, the merged K chains), row0, rows (a GEMM or
// WRITEBACK on a row strip of its C tile; rows = 0: the whole tile), splits (ways a strip's launch splits K).
// stats: [blocks_used, fetch_A, fetch_B, fetch_C, evictions, subkernels].  Returns the number of commands.
long PARALiA_gemm_plan(long M, long N, long K, long T, int a_remote, int b_remote, int c_remote, int beta_zero, int elem,
                       int exec_queues, long pool_blocks, int order_id, int* rows, long max_rows, long stats[6]) {
  long n = -1;
  guarded([&] {
    paralia::GemmPlan plan = paralia::build_gemm_plan(gp_of(M, N, K, T, a_remote, b_remote, c_remote, beta_zero, elem, exec_queues, pool_blocks), order_id);
    n = (long)plan.cmds.size();
    if (stats) {
      stats[0] = plan.blocks_used; stats[1] = plan.n_fetch[0]; stats[2] = plan.n_fetch[1]; stats[3] = plan.n_fetch[2];
      stats[4] = plan.n_evictions; stats[5] = plan.p.subkernels();
    }
    if (rows)
      for (long i = 0; i < n && i < max_rows; ++i) {
        const paralia::Cmd& c = plan.cmds[i];
        int* r = rows + i * PL_PLAN_ROW;
        r[0] = c.kind; r[1] = c.mi; r[2] = c.ni; r[3] = c.ki; r[4] = c.stream; r[5] = c.block; r[6] = c.a_block; r[7] = c.b_block;
        r[8] = c.beta_mode; r[9] = c.nwait;
        for (int w = 0; w < PL_PLAN_MAX_WAITS; ++w) r[10 + w] = w < c.nwait ? c.wait[w] : -1;
        r[10 + PL_PLAN_MAX_WAITS] = c.kn;
        r[11 + PL_PLAN_MAX_WAITS] = c.row0; r[12 + PL_PLAN_MAX_WAITS] = c.rows; r[13 + PL_PLAN_MAX_WAITS] = c.splits;
      }
  });
  return n;
}

// Simulated makespan of one order (order_id >= 0) or of the best candidate (order_id < 0; *picked receives it).
double PARALiA_gemm_plan_simulate(long M, long N, long K, long T, int a_remote, int b_remote, int c_remote, int beta_zero,
                                  int elem, int exec_queues, long pool_blocks, int order_id, double t_exec, double h2d_ti,
                                  double h2d_tb, double d2h_ti, double d2h_tb, double t_reduce, double h2d_sl, double d2h_sl, int* picked,
                                  double busy[3]) {
  double out = -1;
  guarded([&] {
    paralia::GemmProblem gp = gp_of(M, N, K, T, a_remote, b_remote, c_remote, beta_zero, elem, exec_queues, pool_blocks);
    paralia::StageTimes st;
    st.t_exec = t_exec; st.h2d_ti = h2d_ti; st.h2d_tb = h2d_tb; st.d2h_ti = d2h_ti; st.d2h_tb = d2h_tb; st.t_reduce = t_reduce;
    st.h2d_sl = h2d_sl; st.d2h_sl = d2h_sl;
    st.strip_end = false;   // its price comes with the kernel fit of a database: a pinned id is simulated, the search does not offer it
    paralia::PipelineResult r;
    if (order_id >= 0) {
      r = paralia::simulate_plan(paralia::build_gemm_plan(gp, order_id), st);
      if (picked) *picked = order_id;
    } else {
      const int id = paralia::pick_gemm_order(gp, st, &r);
      if (picked) *picked = id;
    }
    if (busy) { busy[0] = r.t_h2d; busy[1] = r.t_exec; busy[2] = r.t_d2h; }
    out = r.t_total;
  });
  return out;
}

}  // extern "C"
