///
/// Autotuner of the MI355X PARALiA runtime: link models, exec-time lookup tables, overlap models and the
/// autotuning controller (ATC) the routines return.
///
/// Mirrors the public surface of the reference's Autotuner/include/Autotuner.hpp:121-174 (class ATC),
/// CoModel.hpp:10-37 and GPUexec_lookup.hpp for one GPU plus the host (LOC_NUM = 2).  Multi-unit members
/// (LinkMap, per-unit subkernel lists, workload split) are kept only as far as one unit needs them.
///
#ifndef PARALIA_AUTOTUNER_HPP
#define PARALIA_AUTOTUNER_HPP

#include <string>
#include <vector>

#include "paralia_hip.h"

#ifndef LOC_NUM
#define LOC_NUM 2  // one GPU (index 0) + host (last index), as in the reference's idxize(-1) = LOC_NUM - 1
#endif

// constants of the tile heuristic (reference CMakeLists.txt:157-165) and the pool sizing (:34, :69)
#define TILE_MIN 2048
#define TILE_MIN_SLOWDOWN 0.2
#define MIN_DESIRED_SK_DEV 64
#define MAX_DESIRED_SK_DEV 512
#define MAX_DESIRED_SK_DEV_SLOWDOWN 0.1
#define TILE_MAX 4096
#define TILE_MAX_SLOWDOWN 0.1
#define PROBLEM_GPU_PERCENTAGE 70
#define MAX_BACKEND_L 8
#define NORMALIZE_NEAR_SPLIT_LIMIT 0.05
#define PROBLEM_MD_CACHE 100

inline int idxize(int loc) { return loc < 0 ? LOC_NUM - 1 : loc; }
inline int deidxize(int idx) { return idx == LOC_NUM - 1 ? -1 : idx; }
inline int remote(int loc, int unit_id) { return idxize(loc) != idxize(unit_id) ? 1 : 0; }

enum ModelType {
  COCOPELIA_BASELINE = 3,
  COCOPELIA_DATALOC = 4,
  COCOPELIA_BIDIRECTIONAL = 5,
  COCOPELIA_REUSE = 6,
  // 7 is the reference's COCOPELIA_PIPELINE_EMULATE (ModelLvl3.cpp:554-650), left out on purpose: it multiplies its
  // transfer times by the operands' location codes, which were 0 / 1 when it was written and are -1 for the host
  // now, so its copy terms come out negative; the plan simulator of this runtime (runtime/gemm_plan.hpp) does that
  // job, with both copy directions.
  FULL_OVERLAP = 9,
  NO_OVERLAP = 10
};
const char* printModel(ModelType mode);

enum ProblemType { BLAS1 = 0, BLAS2 = 1, BLAS3 = 2 };

/// Latency/bandwidth model of one direction of the host link: t = ti + tb * bytes, and the slowdown sl
/// (clamped to [1, 2]) it suffers while the opposite direction is busy (CoModel.cpp:14-66,107-162).
typedef struct comm_data {
  double ti = 0, tb = 0, sl = 1;
  int from = 0, to = 0;
}* CoModel_p;

CoModel_p CoModel_init(const std::string& db_dir, int to, int from);  // reads Processed/Link-Stats_loc_dest-<to>_loc_src-<from>.log
CoModel_p CoModel_init_local(int dev_id);
double t_com_predict(const comm_data* model, double bytes);
double t_com_sl(const comm_data* model, double bytes);
double t_com_bid_predict(const comm_data* model1, const comm_data* model2, double bytes1, double bytes2);

/// Exec-time lookup table of one routine on one device (GPUexec_lookup.cpp:41-129, 275-359).
struct GPUexecModel {
  std::string func;
  ProblemType problem = BLAS3;
  std::vector<long> T;
  std::vector<double> av_time;
  std::vector<char> TransA, TransB;  // empty for BLAS-1
  // BLAS-3 only, optional (<func>_lone-launch_dev-<id>.log, rows TransA,TransB,T,seconds): time of a tile launch that has
  // the device to itself; av_time is the time per launch when the compute streams keep it filled.  -1 where not measured.
  std::vector<double> lone_time;
  double lone_ratio(long T, char TransA, char TransB) const;  // lone / filled time of that row, 1 when unknown
  long lines() const { return (long)T.size(); }
  long MinT() const;
  long MaxT() const;
  long NearestT(long Tin) const;
  double predict(long T, char TransA = 'N', char TransB = 'N') const;  // exact hit, else cubic scaling from NearestT
};
GPUexecModel* GPUexecModel_init(const std::string& db_dir, int dev_id, const char* func);

/// Fitted constants of this device's kernels that are not table rows: the tile-GEMM launcher's cost model (handed to
/// the launcher with pl_gemm_set_fit when a Modeler is built) and the terms the plan simulator adds to the table times.
/// Read from Processed/Kernel-fit_dev-<id>.log ("name: value" lines, written by the deploy tool; not a file of the
/// reference, whose kernels are cuBLAS's); a missing file or a missing line leaves the built-in value (measured on an
/// MI355X).
struct KernelFit {
  pl_gemm_fit launcher;
  double merge_saving_us_f64 = 3.0;    // a launch saved by merging K chains, fp64: the gap between two launches of a stream
  // fp32, per round of 256 large tiles and per transpose (NN, NT, TN, TT): the fixed cost of a launch that accumulates,
  // less the launch gap
  double merge_saving_us_f32[4] = {8.0, 11.0, 6.0, 7.0};
  double lone_share = 0.07;            // share of a streamed call's launches that run without a partner on the device
  double geadd_bytes_per_s = 5e12;     // rate of the lazy-reduce kernel over its 3 T^2 elements
  double slab_fixed_us = 2.0;          // extra time of a thin-start slab launch 1024 deep (deeper: the same, shallower: in inverse proportion)
  bool from_file = false;
  KernelFit() { pl_gemm_fit_defaults(&launcher); }
};
KernelFit KernelFit_load(const std::string& db_dir, int dev_id);

/// What the models need to know about one call (the reference's Vdata + Modeler fields, Autotuner.hpp:22-36,70-84).
struct ProblemDesc {
  const char* func = "Dgemm";
  ProblemType problem = BLAS3;
  long D1 = -1, D2 = -1, D3 = -1;  // M, N, K  (BLAS-1: N, 1, 1)
  char TransA = 'N', TransB = 'N';
  int dtype_sz = 8;
  int numT = 3;
  int in[3] = {1, 1, 1}, out[3] = {0, 0, 1};
  int loc[3] = {-1, -1, -1}, out_loc[3] = {-1, -1, -1};
  bool beta_is_zero = false;        // C is not fetched when beta == 0
  long long pool_budget_bytes = 0;  // device memory the block pool may take (0: unknown, assume everything fits)
  int exec_queues = 2;              // compute streams the executor will use
};

typedef class Modeler {
 public:
  ProblemDesc P;
  comm_data* link[LOC_NUM];     // transfers from location idx into this unit  (Modeler.cpp:26)
  comm_data* revlink[LOC_NUM];  // transfers from this unit to location idx     (Modeler.cpp:27)
  GPUexecModel* exec = nullptr;
  int unit_id = 0;
  // Power-state transient of the unit (Processed/Power-transient_dev-<id>.log, optional, not a table of the reference):
  // after its compute units sat idle a tile kernel takes up to (1 + amplitude) times its steady time; the deficit grows
  // with time constant idle_s while nothing runs and decays with recover_s while kernels do.  amplitude 0: not measured.
  double transient_amplitude = 0, transient_idle_s = 0, transient_recover_s = 0;
  KernelFit fit;                // Processed/Kernel-fit_dev-<id>.log, optional
  Modeler(const std::string& db_dir, int dev_id, const ProblemDesc& desc);
  ~Modeler();
  long getMinT() const;
  long getMaxT() const;
  long getSKNum(long T) const;
  long getFlops() const;
  double predict(ModelType mode, long T) const;
}* MD_p;

/// Simulated three-stream pipeline (H2D, compute, D2H) of a concrete subkernel order: the model this runtime
/// uses to pick both T and the order; see gemm_plan.hpp.  Declared here because ATC reports its result.
struct PipelineEstimate {
  double t_total = -1, t_h2d_busy = 0, t_exec_busy = 0, t_d2h_busy = 0;
  int order_id = 0;
};

typedef class ATC {
 public:
  long T;
  double T_aggregate_sl, T_imbalance_sl, T_remainder_sl, T_small_sl, T_sknum_sl, T_big_sl;
  int active_unit_num;
  int* active_unit_id_list;
  double* active_unit_score;
  short split_homogeneously = 0;
  double pred_t, pred_J, power_delay, energy_delay;
  double pred_t_pesimistic, pred_J_pesimistic, power_delay_pesimistic, energy_delay_pesimistic;
  long subkernel_num;
  int* Subkernels_per_unit_num;
  int** Subkernels_per_unit_list;
  long long cache_limit;
  MD_p* unit_modeler_list;
  // --- additions of this runtime ---
  ProblemDesc problem;       ///< the call being tuned (dims drive the heuristic even without a database)
  bool has_db;               ///< Processed/*.log files were found and loaded
  bool owns_modelers;        ///< copies made by mimic_ATC share the modelers of the original
  int order_id;              ///< subkernel order family picked by the pipeline model (gemm_plan.hpp)
  int exec_queues;           ///< compute streams used
  const char* T_selected_by; ///< "user", "pipeline-model", "cocopelia-reuse", "cocopelia-bidirectional", "heuristic", "resident"
  PipelineEstimate pipeline; ///< simulated H2D / compute / D2H pipeline of the chosen (T, order)

  ATC();
  ~ATC();
  void reset();
  int diff_intialized_params_ATC(class ATC* other_ATC);
  void mimic_ATC(class ATC* other_ATC);
  void update_sk_num(long long subkernel_num_in);
  void distribute_subkernels(int D1GridSz, int D2GridSz, int D3GridSz);
  /// Tunes T (unless preset), fills pred_t and the subkernel list; returns the seconds it took
  /// (reference Autotuner.cpp:279-559, single-unit path).
  double autotune_problem(const char* routine_name, const ProblemDesc& desc);
  void init_modelers(const char* routine_name, const ProblemDesc& desc);
  double optimize_tile();                                              // heuristic scan (Autotuner.cpp:605-655)
  void get_T_slowdowns(double* slowdowns, int candidate_T);            // (Autotuner.cpp:571-603)
  void set_T_slowdowns(double* slowdowns);
  double optimize_tile_CoCoPeLia(int model_idx, ModelType mode);       // argmin over benchmarked T (Model_functions.cpp:195-244)
  void print();
  const char* print_csv();
}* ATC_p;

/// Directory holding Processed/*.log: $PARALIA_DEPLOYDB, else the database shipped beside the library.
std::string paralia_db_dir();
void paralia_set_db_dir(const char* dir);

#endif
