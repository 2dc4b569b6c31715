// Link models and exec-time lookup tables: file parsing and prediction.
// Formats and arithmetic follow the reference's Autotuner/src/CoModel.cpp:14-66,107-162 and
// GPUexec_lookup.cpp:15-129,250-359 so that database files are interchangeable.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "Autotuner.hpp"
#include "backend_wrappers.hpp"

namespace {
std::string g_db_dir;
std::mutex g_db_mu;
}  // namespace

void paralia_set_db_dir(const char* dir) {
  std::lock_guard<std::mutex> lk(g_db_mu);
  g_db_dir = dir ? dir : "";
}

// Set by the library at load time to <directory of libparalia.so>/../db/<device>, see runtime/helpers.cpp.
std::string paralia_default_db_dir();

std::string paralia_db_dir() {
  {
    std::lock_guard<std::mutex> lk(g_db_mu);
    if (!g_db_dir.empty()) return g_db_dir;
  }
  const char* env = getenv("PARALIA_DEPLOYDB");
  if (env && *env) return env;
  return paralia_default_db_dir();
}

const char* printModel(ModelType mode) {
  switch (mode) {
    case COCOPELIA_BASELINE: return "COCOPELIA_BASELINE";
    case COCOPELIA_DATALOC: return "COCOPELIA_DATALOC";
    case COCOPELIA_BIDIRECTIONAL: return "COCOPELIA_BIDIRECTIONAL";
    case COCOPELIA_REUSE: return "COCOPELIA_REUSE";
    case FULL_OVERLAP: return "FULL_OVERLAP";
    case NO_OVERLAP: return "NO_OVERLAP";
  }
  return "UNKNOWN";
}

// File: "Intercept: <ti>\nCoefficient: <tb>\n" then any number of "Slowdown([src]->[dst]): <sl>\n" lines
// (written by LinkPreprocessing.py.in:55-60).  On one GPU the only other link is the opposite direction,
// whose slowdown entry is the one kept.
CoModel_p CoModel_init(const std::string& db_dir, int to, int from) {
  char filename[1024];
  snprintf(filename, sizeof filename, "%s/Processed/Link-Stats_loc_dest-%d_loc_src-%d.log", db_dir.c_str(), to, from);
  FILE* fp = fopen(filename, "r");
  if (!fp) error("CoModel_init(%d,%d): t_comm LogFile =%s not generated\n", to, from, filename);
  CoModel_p m = new comm_data();
  long double ti, tb;
  int items = fscanf(fp, "Intercept: %Le\nCoefficient: %Le\n", &ti, &tb);
  if (items != 2) {
    fclose(fp);
    delete m;
    error("CoModel_init: Problem in reading model Inter/Coef from %s\n", filename);
  }
  m->ti = (double)ti;
  m->tb = (double)tb;
  m->sl = 1;
  m->to = to;
  m->from = from;
  int loc_src, loc_dest;
  long double sl;
  while (!feof(fp)) {
    items = fscanf(fp, "Slowdown([%d]->[%d]): %Le\n", &loc_src, &loc_dest, &sl);
    if (items != 3) {
      fclose(fp);
      delete m;
      error("CoModel_init(%d,%d): Problem in reading model Slowdown\n", to, from);
    }
    if (sl < 1 - NORMALIZE_NEAR_SPLIT_LIMIT) sl = 1;
    else if (sl > 2) sl = 2.0;
    // keep the slowdown caused by the opposite direction of this link (sl[from][to] in the reference's matrix)
    if (!(fabsl(sl - 1) < NORMALIZE_NEAR_SPLIT_LIMIT) && idxize(loc_src) == idxize(to) && idxize(loc_dest) == idxize(from))
      m->sl = (double)sl;
  }
  fclose(fp);
  return m;
}

CoModel_p CoModel_init_local(int dev_id) {
  CoModel_p m = new comm_data();
  m->to = m->from = dev_id;
  return m;
}

double t_com_predict(const comm_data* model, double bytes) {
  if (bytes < 0) return -1;
  if (bytes == 0) return 0;
  return model->ti + model->tb * bytes;
}

double t_com_sl(const comm_data* model, double bytes) {
  if (bytes < 0) return -1;
  if (bytes == 0) return 0;
  return model->ti + model->tb * bytes * model->sl;
}

double t_com_bid_predict(const comm_data* model1, const comm_data* model2, double bytes1, double bytes2) {
  if (bytes1 < 0 || bytes2 < 0) return -1;
  if (bytes1 == 0) return t_com_predict(model2, bytes2);
  if (bytes2 == 0) return t_com_predict(model1, bytes1);
  const double t_sl1 = t_com_sl(model1, bytes1), t_sl2 = t_com_sl(model2, bytes2);
  if (t_sl1 < t_sl2) return t_sl1 * (1.0 - 1 / model2->sl) + bytes2 * model2->tb + model2->ti / model2->sl;
  return t_sl2 * (1.0 - 1 / model1->sl) + bytes1 * model1->tb + model1->ti / model1->sl;
}

// ------------------------------------------------------------------------------------------ exec lookup

long GPUexecModel::MinT() const {
  long r = T[0];
  for (long v : T) if (v < r) r = v;
  return r;
}
long GPUexecModel::MaxT() const {
  long r = T[0];
  for (long v : T) if (v > r) r = v;
  return r;
}
// Largest benchmarked T not above Tin (the table is sorted by T); the smallest one when Tin is below all.
long GPUexecModel::NearestT(long Tin) const {
  if (Tin < T[0]) return T[0];
  long prev = T[0];
  for (long v : T) {
    if (v == Tin) return v;
    if (v > Tin) break;
    prev = v;
  }
  return prev;
}
double GPUexecModel::predict(long Tq, char ta, char tb) const {
  const bool flags = !TransA.empty();
  for (size_t i = 0; i < T.size(); ++i)
    if (T[i] == Tq && (!flags || (TransA[i] == ta && TransB[i] == tb))) return av_time[i];
  const long nearest = NearestT(Tq);
  long double reg_t = 0;
  for (size_t i = 0; i < T.size(); ++i)
    if (T[i] == nearest && (!flags || (TransA[i] == ta && TransB[i] == tb))) {
      reg_t = av_time[i];
      break;
    }
  if (reg_t == 0) error("Failed to find nearest_T = %ld for regression\n", nearest);
  // cubic scaling from the nearest benchmarked size, for every routine (GPUexec_lookup.cpp:127, :357)
  return (double)(reg_t * pow((double)Tq, 3) / pow((double)nearest, 3));
}

// BLAS-3 line: TransA,TransB,M,N,K,t,W,J,err,n,bench   (GPUexec_lookup.cpp:79-82)
// BLAS-2 line: TransA,M,N,t,W,J,err,n,bench            (GPUexec_lookup.cpp:196-198)
// BLAS-1 line: T,t,W,J,err,n,bench                     (GPUexec_lookup.cpp:311)
GPUexecModel* GPUexecModel_init(const std::string& db_dir, int dev_id, const char* func) {
  ProblemType problem;
  if (!strcmp(func, "Dgemm") || !strcmp(func, "Sgemm")) problem = BLAS3;
  else if (!strcmp(func, "Dgemv")) problem = BLAS2;
  else if (!strcmp(func, "Daxpy") || !strcmp(func, "Ddot")) problem = BLAS1;
  else error("GPUexecModel_init: Invalid/Not implemented func %s\n", func);
  char filename[1024];
  snprintf(filename, sizeof filename, "%s/Processed/%s_lookup-table_dev-%d.log", db_dir.c_str(), func, dev_id);
  FILE* fp = fopen(filename, "r");
  if (!fp) error("GPUexecModel_init: t_exec LogFile %s not generated\n", filename);
  GPUexecModel* m = new GPUexecModel();
  m->func = func;
  m->problem = problem;
  char line[512];
  int lineno = 0;
  while (fgets(line, sizeof line, fp)) {
    ++lineno;
    if (line[0] == '\n' || line[0] == '\0') continue;
    long Tv, d2, d3, n;
    double t, W, J, err, bench;
    if (problem == BLAS3) {
      char ta, tb;
      if (sscanf(line, "%c,%c,%ld,%ld,%ld,%lf,%lf,%lf,%lf,%ld,%lf", &ta, &tb, &Tv, &d2, &d3, &t, &W, &J, &err, &n, &bench) != 11) {
        fclose(fp);
        delete m;
        error("GPUexecModel_init: Problem in reading model (%s line %d)\n", filename, lineno);
      }
      m->TransA.push_back(ta);
      m->TransB.push_back(tb);
    } else if (problem == BLAS2) {
      char ta;
      if (sscanf(line, "%c,%ld,%ld,%lf,%lf,%lf,%lf,%ld,%lf", &ta, &Tv, &d2, &t, &W, &J, &err, &n, &bench) != 9) {
        fclose(fp);
        delete m;
        error("GPUexecModel_init: Problem in reading model (%s line %d)\n", filename, lineno);
      }
      m->TransA.push_back(ta);
      m->TransB.push_back('N');  // no second flag: lookups pass the default
    } else {
      if (sscanf(line, "%ld,%lf,%lf,%lf,%lf,%ld,%lf", &Tv, &t, &W, &J, &err, &n, &bench) != 7) {
        fclose(fp);
        delete m;
        error("GPUexecModel_init: Problem in reading model (%s line %d)\n", filename, lineno);
      }
    }
    m->T.push_back(Tv);
    m->av_time.push_back(t);
  }
  fclose(fp);
  if (m->T.empty()) {
    delete m;
    error("GPUexecModel_init: empty lookup table %s\n", filename);
  }
  m->lone_time.assign(m->T.size(), -1.0);
  if (problem == BLAS3) {
    snprintf(filename, sizeof filename, "%s/Processed/%s_lone-launch_dev-%d.log", db_dir.c_str(), func, dev_id);
    fp = fopen(filename, "r");  // optional: databases without it price every launch at its filled-device time
    if (fp) {
      while (fgets(line, sizeof line, fp)) {
        char ta, tb;
        long Tv;
        double t;
        if (sscanf(line, "%c,%c,%ld,%lf", &ta, &tb, &Tv, &t) != 4) continue;
        for (size_t i = 0; i < m->T.size(); ++i)
          if (m->T[i] == Tv && m->TransA[i] == ta && m->TransB[i] == tb) m->lone_time[i] = t;
      }
      fclose(fp);
    }
  }
  return m;
}

double GPUexecModel::lone_ratio(long Tin, char ta, char tb) const {
  for (size_t i = 0; i < T.size(); ++i)
    if (T[i] == Tin && (TransA.empty() || (TransA[i] == ta && TransB[i] == tb)))
      return (i < lone_time.size() && lone_time[i] > 0 && av_time[i] > 0) ? std::max(1.0, lone_time[i] / av_time[i]) : 1.0;
  return 1.0;
}
