// Modeler: per-unit bundle of link models + exec lookup, and the CoCoPeLia overlap predictions.
// Arithmetic follows the reference's Autotuner/src/ModelLvl3.cpp:20-73 (full overlap), :239-284 (no overlap),
// :287-346 (baseline), :348-408 (data location), :410-474 (bidirectional), :476-551 (reuse) and
// ModelLvl1.cpp:262-326 (BLAS-1 bidirectional), ModelLvl2.cpp:89-259 (BLAS-2: full / zero overlap and bidirectional),
// reduced to one GPU plus the host.
#include <cstdio>
#include <cmath>
#include <cstring>

#include "Autotuner.hpp"
#include "backend_wrappers.hpp"

// "name: value" lines; names this build does not know are ignored, so are values that do not parse.
KernelFit KernelFit_load(const std::string& db_dir, int dev_id) {
  KernelFit k;
  char filename[1024];
  snprintf(filename, sizeof filename, "%s/Processed/Kernel-fit_dev-%d.log", db_dir.c_str(), dev_id);
  FILE* fp = fopen(filename, "r");
  if (!fp) return k;
  k.from_file = true;
  static const char* const trans[4] = {"NN", "NT", "TN", "TT"};
  char line[512];
  while (fgets(line, sizeof line, fp)) {
    char name[128];
    double v = 0;
    if (line[0] == '#' || sscanf(line, " %127[^:]: %lf", name, &v) != 2) continue;
    const std::string n(name);
    pl_gemm_fit& f = k.launcher;
    if (n == "lone_us_per_k_f64") f.lone_us_per_k[0] = v;
    else if (n == "lone_us_per_k_f32") f.lone_us_per_k[1] = v;
    else if (n == "lone_fixed_k") f.lone_fixed_k = v;
    else if (n == "splitk_launch_us") f.splitk_launch_us = v;
    else if (n == "pass_bytes_per_us") f.pass_bytes_per_us = v;
    else if (n == "f32_small_us_per_k") f.f32_small_us_per_k = v;
    else if (n == "f32_small_fixed_us") f.f32_small_fixed_us = v;
    else if (n == "f32_wide_gain") f.f32_wide_gain = v;
    else if (n == "f32_wide_fixed_us_beta0") f.f32_wide_fixed_us[0] = v;
    else if (n == "f32_wide_fixed_us_beta1") f.f32_wide_fixed_us[1] = v;
    else if (n == "edge_rounds_small") f.edge_rounds[0] = v;
    else if (n == "edge_rounds_large") f.edge_rounds[1] = v;
    else if (n == "merge_saving_us_f64") k.merge_saving_us_f64 = v;
    else if (n == "merge_saving_us_f32") { for (double& x : k.merge_saving_us_f32) x = v; }
    else if (n == "lone_share") k.lone_share = v;
    else if (n == "geadd_bytes_per_s") k.geadd_bytes_per_s = v;
    else if (n == "slab_fixed_us") k.slab_fixed_us = v;
    else
      for (int t = 0; t < 4; ++t) {
        if (n == std::string("f32_large_gain_") + trans[t]) f.f32_large_gain[t] = v;
        else if (n == std::string("f32_large_fixed_us_beta0_") + trans[t]) f.f32_large_fixed_us[t][0] = v;
        else if (n == std::string("f32_large_fixed_us_beta1_") + trans[t]) f.f32_large_fixed_us[t][1] = v;
        else if (n == std::string("merge_saving_us_f32_") + trans[t]) k.merge_saving_us_f32[t] = v;
      }
  }
  fclose(fp);
  bool merge_ok = k.merge_saving_us_f64 >= 0;
  for (double x : k.merge_saving_us_f32) merge_ok = merge_ok && x >= 0;
  if (!(merge_ok && k.lone_share >= 0 && k.lone_share <= 1 && k.geadd_bytes_per_s > 0 && k.slab_fixed_us >= 0))
    error("KernelFit_load: %s holds a value out of range\n", filename);
  return k;
}

Modeler::Modeler(const std::string& db_dir, int dev_id, const ProblemDesc& desc) : P(desc), unit_id(dev_id) {
  for (int idx = 0; idx < LOC_NUM; ++idx) {
    const int other = deidxize(idx);
    if (other != dev_id) {
      link[idx] = CoModel_init(db_dir, dev_id, other);     // into this unit (Modeler.cpp:26)
      revlink[idx] = CoModel_init(db_dir, other, dev_id);  // out of this unit (Modeler.cpp:27)
    } else {
      link[idx] = revlink[idx] = CoModel_init_local(dev_id);
    }
  }
  exec = GPUexecModel_init(db_dir, dev_id, desc.func);
  // the launcher prices its macro tiles and split counts with the constants of the database in use
  fit = KernelFit_load(db_dir, dev_id);
  if (pl_gemm_set_fit(&fit.launcher) != 0) error("Modeler: Processed/Kernel-fit_dev-%d.log of %s holds a launcher constant out of range\n", dev_id, db_dir.c_str());
  char filename[1024];
  snprintf(filename, sizeof filename, "%s/Processed/Power-transient_dev-%d.log", db_dir.c_str(), dev_id);
  if (FILE* fp = fopen(filename, "r")) {
    double a = 0, rec = 0, idle = 0;
    if (fscanf(fp, "Amplitude: %lf\nRecovery: %lf\nIdle: %lf", &a, &rec, &idle) == 3 && a > 0 && a < 1 && rec > 0 && idle > 0) {
      transient_amplitude = a;
      transient_recover_s = rec;
      transient_idle_s = idle;
    }
    fclose(fp);
  }
}

Modeler::~Modeler() {
  for (int idx = 0; idx < LOC_NUM; ++idx) {
    if (revlink[idx] != link[idx]) delete revlink[idx];
    delete link[idx];
  }
  delete exec;
}

long Modeler::getMinT() const {
  if (P.problem == BLAS3 || P.problem == BLAS2) return std::max(exec->MinT(), 1024L);  // MinAllowedTBLAS3 / BLAS2
  return exec->MinT();
}
long Modeler::getMaxT() const {
  if (P.problem == BLAS3) return std::min(std::min(P.D1, P.D2), P.D3);
  if (P.problem == BLAS2) return std::min(P.D1, P.D2);  // MaxAllowedTBLAS2
  return P.D1;
}
long Modeler::getSKNum(long T) const {
  auto cdiv = [](long a, long b) { return a / b + ((a % b) ? 1 : 0); };
  if (P.problem == BLAS3) return cdiv(P.D1, T) * cdiv(P.D2, T) * cdiv(P.D3, T);
  if (P.problem == BLAS2) return cdiv(P.D1, T) * cdiv(P.D2, T);  // GetSKNumBLAS2
  return cdiv(P.D1, T);
}
long Modeler::getFlops() const {
  if (P.problem == BLAS3) return gemm_flops(P.D1, P.D2, P.D3);
  if (P.problem == BLAS2) return gemv_flops(P.D1, P.D2);
  return axpy_flops(P.D1);
}

namespace {
// Dim1 x Dim2 of operand i: A is D1 x D3, B is D3 x D2, C is D1 x D2 (CoCoModel_gemm_init); vectors are D1 x 1.
void dims_of(const ProblemDesc& P, int i, double* d1, double* d2) {
  if (P.problem == BLAS2) {
    // CoCoModel_gemv_init (ModelLvl2.cpp:66-71): A is D1 x D2, "x" D1 x 1, "y" D2 x 1 whatever TransA says
    *d1 = (i == 2) ? (double)P.D2 : (double)P.D1;
    *d2 = (i == 0) ? (double)P.D2 : 1;
    return;
  }
  if (P.problem != BLAS3) { *d1 = (double)P.D1; *d2 = 1; return; }
  *d1 = (i == 1) ? (double)P.D3 : (double)P.D1;
  *d2 = (i == 0) ? (double)P.D3 : (double)P.D2;
}
}  // namespace

double Modeler::predict(ModelType mode, long T) const {
  // The location that prices a tile transfer is the one holding the most operands, the host winning ties
  // (ModelLvl3.cpp:306-312): with one GPU that is the host unless the device holds strictly more.
  int on_host = 0;
  for (int i = 0; i < P.numT; ++i) on_host += remote(P.loc[i], unit_id);
  const int mv_idx = (on_host >= P.numT - on_host) ? idxize(-1) : idxize(unit_id);
  const comm_data* recv_m = link[mv_idx];
  const comm_data* send_m = revlink[mv_idx];

  if (P.problem == BLAS1) {
    if (mode != COCOPELIA_BIDIRECTIONAL) error("Modeler::predict: BLAS-1 supports only COCOPELIA_BIDIRECTIONAL\n");
    const double t_exec = exec->predict(T);
    if (t_exec < 0) return -1.0;
    const double bytes = (double)T * P.dtype_sz;
    const double t_recv = t_com_predict(recv_m, bytes), t_send = t_com_predict(send_m, bytes);
    int numTin = 0, numTout = 0;
    for (int i = 0; i < P.numT; ++i) {
      numTin += P.in[i] * remote(P.loc[i], unit_id);
      numTout += P.out[i] * remote(P.loc[i], unit_id);
    }
    const double ker_over = (1.0 * P.D1 / T) - 1;
    const double t_over = t_com_bid_predict(recv_m, send_m, bytes * numTin, bytes * numTout);
    return fmax(t_exec, t_over) * ker_over + fmax(t_exec, numTout * t_send) + numTin * t_recv + numTout * t_send;
  }

  if (P.problem == BLAS2) {
    if (mode == FULL_OVERLAP || mode == NO_OVERLAP) {
      const long Tbig = exec->NearestT((long)fmin((double)exec->MaxT(), fmin((double)P.D1, (double)P.D2)));
      const double t_exec = (P.D1 * 1.0 / Tbig * P.D2 * 1.0 / Tbig) * exec->predict(Tbig, P.TransA);
      if (t_exec < 0) return -1.0;
      double t_recv = 0, t_send = 0;
      for (int i = 0; i < P.numT; ++i) {
        double d1, d2;
        dims_of(P, i, &d1, &d2);
        t_recv += P.in[i] * t_com_predict(link[idxize(P.loc[i])], d1 * d2 * P.dtype_sz);
        t_send += P.out[i] * t_com_predict(link[idxize(P.out_loc[i])], d1 * d2 * P.dtype_sz);
      }
      return mode == FULL_OVERLAP ? fmax(t_exec, fmax(t_recv, t_send)) : t_exec + t_recv + t_send;
    }
    if (mode != COCOPELIA_BIDIRECTIONAL) error("Modeler::predict: BLAS-2 supports FULL_OVERLAP, NO_OVERLAP and COCOPELIA_BIDIRECTIONAL\n");
    // ModelLvl2.cpp:194-259.  The reference prices a BLAS-2 tile transfer as T elements (a vector tile), not the
    // T x T matrix tile that actually moves, and counts D1/T kernels; kept as it is, which is why this runtime
    // picks T for dgemv with its own streaming estimate (ATC::autotune_problem) and reports this one on request.
    const double t_exec = exec->predict(T, P.TransA);
    if (t_exec < 0) return -1.0;
    const double bytes = (double)T * P.dtype_sz;
    const double t_recv = t_com_predict(recv_m, bytes), t_send = t_com_predict(send_m, bytes);
    int numTin = 0, numTout = 0;
    for (int i = 0; i < P.numT; ++i) {
      numTin += P.in[i] * remote(P.loc[i], unit_id);
      numTout += P.out[i] * remote(P.loc[i], unit_id);
    }
    const double ker_over = (1.0 * P.D1 / T) - 1;
    const double t_over = t_com_bid_predict(recv_m, send_m, bytes * numTin, bytes * numTout);
    return fmax(t_exec, t_over) * ker_over + fmax(t_exec, numTout * t_send) + numTin * t_recv + numTout * t_send;
  }

  if (mode == FULL_OVERLAP || mode == NO_OVERLAP) {
    const long maxT = exec->MaxT();
    const long Tbig = exec->NearestT((long)fmin((double)maxT, fmin(fmin((double)P.D1, (double)P.D2), (double)P.D3)));
    const double t_exec = (P.D1 * 1.0 / Tbig * P.D2 * 1.0 / Tbig * P.D3 * 1.0 / Tbig) * exec->predict(Tbig, P.TransA, P.TransB);
    if (t_exec < 0) return -1.0;
    double t_recv = 0, t_send = 0;
    for (int i = 0; i < P.numT; ++i) {
      double d1, d2;
      dims_of(P, i, &d1, &d2);
      // the reference prices both directions with the same (receive-side) link model here
      t_recv += P.in[i] * t_com_predict(link[idxize(P.loc[i])], d1 * d2 * P.dtype_sz);
      t_send += P.out[i] * t_com_predict(link[idxize(P.out_loc[i])], d1 * d2 * P.dtype_sz);
    }
    return mode == FULL_OVERLAP ? fmax(t_exec, fmax(t_recv, t_send)) : t_exec + t_recv + t_send;
  }

  const double t_exec = exec->predict(T, P.TransA, P.TransB);
  if (t_exec < 0) return -1.0;
  const double tile_bytes = (double)T * T * P.dtype_sz;
  const double t_recv = t_com_predict(recv_m, tile_bytes), t_send = t_com_predict(send_m, tile_bytes);
  const double ker_over = (1.0 * P.D1 / T) * (1.0 * P.D2 / T) * (1.0 * P.D3 / T) - 1;
  int numTin = 0, numTout = 0;

  switch (mode) {
    case COCOPELIA_BASELINE: {
      for (int i = 0; i < P.numT; ++i) { numTin += P.in[i]; numTout += P.out[i]; }
      const double t_over = fmax(numTin * t_recv, t_send * numTout);
      return fmax(t_exec, t_over) * ker_over + t_exec + numTin * t_recv + numTout * t_send;
    }
    case COCOPELIA_DATALOC:
    case COCOPELIA_BIDIRECTIONAL: {
      for (int i = 0; i < P.numT; ++i) {
        numTin += P.in[i] * remote(P.loc[i], unit_id);
        numTout += P.out[i] * remote(P.loc[i], unit_id);
      }
      const double t_over = (mode == COCOPELIA_DATALOC)
                                ? fmax(numTin * t_recv, t_send * numTout)
                                : t_com_bid_predict(recv_m, send_m, tile_bytes * numTin, tile_bytes * numTout);
      return fmax(t_exec, t_over) * ker_over + t_exec + numTin * t_recv + numTout * t_send;
    }
    case COCOPELIA_REUSE: {
      double zero_over = ker_over, one_over = 0, two_over = 0;
      for (int i = 0; i < P.numT; ++i) {
        double d1, d2;
        dims_of(P, i, &d1, &d2);
        const int rin = P.in[i] * remote(P.loc[i], unit_id);
        numTin += rin;
        numTout += P.out[i] * remote(P.out_loc[i], unit_id);
        one_over += rin * (d1 / T) * (d2 / T);
        if (t_recv > t_exec)
          for (int j = i + 1; j < P.numT; ++j)
            if (rin != 0 && (P.in[j] * remote(P.loc[j], unit_id)) != 0) {
              // tiles of operands i and j that can be fetched under one kernel share a dimension:
              // A-C share D1 (= Dim1 of A); A-B share D3 and B-C share D2 (= Dim2 of the first)
              two_over += ((i == 0 && j == 2) ? d1 : d2) / T - 1;
            }
      }
      if (2 * t_recv > t_exec && t_exec > t_recv) two_over += (1.0 * P.D3 / T);
      one_over -= (2 * two_over + numTin);
      zero_over -= (one_over + two_over);
      return t_exec * (1 + zero_over) + fmax(t_exec, t_recv) * one_over + fmax(t_exec, t_recv * 2) * two_over +
             numTin * t_recv + numTout * t_send;
    }
    default:
      error("Modeler::predict: mode %s not available\n", printModel(mode));
  }
}
