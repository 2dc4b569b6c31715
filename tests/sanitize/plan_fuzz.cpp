// Random GEMM problems through the host-side planner: plan building for every order family and eviction policy, pools from
// three blocks to the full working set, the order search and the three-resource simulation.  Built with
// -fsanitize=address,undefined by tests/test_host_sanitizers.py; pure host code, no GPU.
// usage: plan_fuzz [iterations]
#include <cstdio>
#include <cstdlib>
#include <random>
#include <stdexcept>
#include "runtime/gemm_plan.hpp"
using namespace paralia;
int main(int argc, char** argv) {
  const int iterations = argc > 1 ? atoi(argv[1]) : 6000;
  std::mt19937_64 rng(12345);
  long built = 0, refused = 0;
  for (int it = 0; it < iterations; ++it) {
    GemmProblem p;
    p.M = 1 + rng() % 3000; p.N = 1 + rng() % 3000; p.K = rng() % 3000;
    const long Ts[] = {64, 100, 128, 256, 300, 512, 1000};
    p.T = Ts[rng() % 7];
    p.a_remote = rng() % 2; p.b_remote = rng() % 2; p.c_remote = rng() % 2;
    p.beta_zero = rng() % 2; p.elem = (rng() % 2) ? 8 : 4; p.exec_queues = 1 + rng() % 4;
    const long full = gemm_full_block_num(p);
    const long pools[] = {gemm_max_block_num(p), full, 3, 4, 5, 8, std::max(3L, full / 2), std::max(3L, full / 3), std::max(3L, full / 8)};
    p.pool_blocks = pools[rng() % 9];
    if (p.subkernels() > 6000) continue;
    StageTimes st; st.t_exec = 1e-4; st.h2d_ti = 1e-5; st.h2d_tb = 2e-11; st.d2h_ti = 1e-5; st.d2h_tb = 2e-11; st.t_reduce = 1e-5; st.h2d_sl = 1.01; st.d2h_sl = 1.2;
    st.merge_saving = (rng() % 2) ? 4e-6 : 0.0;
    try {
      if (rng() % 4 == 0) {
        PipelineResult r; pick_gemm_order(p, st, &r, rng() % 2);
      } else {
        const int orient = rng() % 2;
        // panel widths, and now and then a block order (rows * 100 + columns; zero columns and repeated panels are refused)
        const int w = (rng() % 4 == 0) ? (int)((1 + rng() % 30) * ORDER_BLOCK_ROWS + rng() % 30) : (int)(rng() % 40);
        int id = orient * 10000 + w + ((w > 0 && rng() % 2) ? 20000 : 0) + ((rng() % 2) ? 40000 : 0);
        if (rng() % 3 == 0) id = ORDER_MERGE_CHAINS + orient * 10000 + w;  // merged K chains (refused unless the pool holds everything)
        if (rng() % 3 == 0) id += ORDER_K_SPLIT * (1 + rng() % 3);  // thin start: first k tile in 2 or 4 equal slabs or graded (refused when it does not apply)
        if (rng() % 3 == 0) id += ORDER_STRIP_END;  // the last launch in row strips (the same plan where the last tile is too small or stays on the device)
        GemmPlan plan = build_gemm_plan(p, id);
        PipelineResult r = simulate_plan(plan, st);
        if (!(r.t_total >= 0)) { printf("bad makespan\n"); return 1; }
      }
      ++built;
    } catch (const std::runtime_error&) { ++refused; }
  }
  printf("built %ld refused %ld\n", built, refused);
  return 0;
}
