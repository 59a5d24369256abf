// planner.cpp -- which activations to move off the device, and how, under a memory target.
//
// The reference's planner is c10::PolicyMaker in a patched PyTorch that is not
// part of its tree.  What the tree shows is how it is driven: during one
// profiled iteration the model's forward records, per op, its compute time
// (add_comptime), its output tensor and size (add_tensor(index, nbytes)) and
// which tensor it consumed (add_stepdep({pre.tensor_id, index}));
// add_omitid(id) excludes a tensor (CSWAP+/inception-v3-cifar100.cpp:207-214).
// After the iteration init(ratio) fixes the target and make_policy(time_)
// returns one action code per tensor (0 keep, 2 raw swap, 3 ZVC, 6 ZFP --
// CSWAP+/Execution.h:70,86,107) plus the predicted iteration time;
// capuchin(time_) is the raw-swap baseline it is compared with
// (CSWAP+/vgg16-cifar10.cpp:474-497), and read_lastvisit(path, begin_stage)
// fills Execution::begin_stage with the op at which each tensor is last used
// (CSWAP+/resnet-cifar10.cpp:330).
//
// This file is an own design behind those calls.  Model of one iteration:
// forward ops 0..N-1 with times c[i], backward in reverse with bwd_factor*c[i].
// Tensor t is produced by op t and last consumed in forward by op u(t); it can
// leave the device when op u(t) starts (that is begin_stage[t]) and is needed
// again when the backward of op u(t) starts.  Swapping it out costs the
// compression kernels on the compute stream plus whatever part of the copy the
// compute of op u(t) does not cover (Execution::post waits at the end of that
// op); swapping it in costs the decompression plus whatever part of the inbound
// copy the backward of op u(t)+1 does not cover (one tensor of look-ahead).
// make_policy takes, per tensor, the cheapest action the cost model allows and
// then tensors in order of overhead per byte until the target is met.
#include <algorithm>
#include <map>
#include <mutex>
#include <vector>

#include "common.h"

namespace {

struct TensorRec {
  size_t bytes = 0;
  size_t nx = 0, ny = 0, nz = 0;
  long long nnz = -1;  // unknown
  int last_use = -1;   // op index of the last forward consumer
  bool omit = false;
  bool present = false;
};

struct Option {
  int code = 0;  // 0 keep, 2 raw, 3 ZVC, 6 ZFP
  double overhead_us = 0;
  size_t bytes_out = 0;
};

}  // namespace

struct cswap_planner {
  std::mutex mu;
  cswap_costs costs;
  unsigned maxbits = 512;
  double bwd_factor = 2.0;
  double ratio = 0.0;
  std::vector<double> comptime;  // forward time of op i, microseconds
  std::map<int, TensorRec> tensors;
  cswap_plan_summary last;
};

static int code_of(int policy) { return policy == CSWAP_POLICY_SPARSE ? 3 : policy == CSWAP_POLICY_ZFP ? 6 : 2; }

// cost of moving tensor r out at op u and back in before the backward of op u
static Option price(const cswap_planner* p, const TensorRec& r, int policy)
{
  const cswap_costs& c = p->costs;
  Option o;
  o.code = code_of(policy);
  const size_t n = r.bytes / 4;
  const double in_bytes = (double)r.bytes;
  double t_comp = 0, t_decomp = 0;
  if (policy == CSWAP_POLICY_NONE) {
    o.bytes_out = r.bytes;
  } else if (policy == CSWAP_POLICY_SPARSE) {
    o.bytes_out = cswap_policy_bytes(CSWAP_POLICY_SPARSE, n, (size_t)r.nnz, 0, c.process, 0, 0, 0);
    t_comp = c.probe_latency_us + 3.0 * c.kernel_latency_us + in_bytes / (c.zvc_compress_gbs * 1e3);
    t_decomp = c.kernel_latency_us + in_bytes / (c.zvc_expand_gbs * 1e3);
  } else {
    o.bytes_out = r.nx ? cswap_zfp_stream_capacity(r.nx, r.ny, r.nz, p->maxbits)
                       : cswap_policy_bytes(CSWAP_POLICY_ZFP, n, 0, p->maxbits, 0, 0, 0, 0);
    t_comp = c.zfp_latency_us + in_bytes / (c.zfp_compress_gbs * 1e3);
    t_decomp = c.zfp_latency_us + in_bytes / (c.zfp_decompress_gbs * 1e3);
  }
  const double t_out = c.copy_latency_us + (double)o.bytes_out / (c.bw_d2h_gbs * 1e3);
  const double t_in = c.copy_latency_us + (double)o.bytes_out / (c.bw_h2d_gbs * 1e3);
  const int u = r.last_use;
  const int nops = (int)p->comptime.size();
  const double cover_fwd = u >= 0 && u < nops ? p->comptime[(size_t)u] : 0.0;
  const double cover_bwd = u + 1 < nops ? p->bwd_factor * p->comptime[(size_t)u + 1] : 0.0;
  o.overhead_us = t_comp + std::max(0.0, t_out - cover_fwd) + t_decomp + std::max(0.0, t_in - cover_bwd);
  return o;
}

static bool eligible(const cswap_planner* p, const TensorRec& r, int id)
{
  const int nops = (int)p->comptime.size();
  if (!r.present || r.omit || r.bytes < p->costs.size_floor_bytes || (r.bytes & 3)) return false;
  // consumed by a later op, and not by the very last one (backward starts right after it)
  return r.last_use > id && r.last_use < nops - 1;
}

static double base_time(const cswap_planner* p)
{
  double t = 0;
  for (double c : p->comptime) t += c * (1.0 + p->bwd_factor);
  return t;
}

static int plan(cswap_planner* p, bool raw_only, int* policy, int* begin_stage, int n, cswap_plan_summary* out)
{
  if (!p || !policy || n <= 0) return CSWAP_E_ARG;
  std::lock_guard<std::mutex> lock(p->mu);
  for (int i = 0; i < n; i++) {
    policy[i] = 0;
    if (begin_stage) begin_stage[i] = i + 1;  // Execution::init_ default (Execution.h:61)
  }
  struct Cand {
    int id;
    Option opt;
    double key;
  };
  std::vector<Cand> cands;
  size_t total = 0;
  const cswap_costs& c = p->costs;
  const int nops = (int)p->comptime.size();
  for (const auto& kv : p->tensors) {
    const int id = kv.first;
    const TensorRec& r = kv.second;
    if (!r.present) continue;
    total += r.bytes;
    if (id < 0 || id >= n) continue;
    if (begin_stage && r.last_use > id) begin_stage[id] = r.last_use;
    if (!eligible(p, r, id)) continue;
    Option best = price(p, r, CSWAP_POLICY_NONE);
    if (!raw_only) {
      const size_t nelem = r.bytes / 4;
      if (r.nnz >= 0 && (size_t)r.nnz <= nelem && nelem <= 0x7fffffffull && c.zvc_compress_gbs > 0 &&
          c.zvc_expand_gbs > 0) {
        Option s = price(p, r, CSWAP_POLICY_SPARSE);
        if ((double)s.bytes_out < c.sparse_max_ratio * (double)r.bytes && s.overhead_us < best.overhead_us) best = s;
      }
      if (c.allow_lossy && c.zfp_compress_gbs > 0 && c.zfp_decompress_gbs > 0) {
        Option z = price(p, r, CSWAP_POLICY_ZFP);
        // a lossy option has to beat the best lossless one by the configured margin
        if (z.bytes_out < r.bytes && z.overhead_us < c.lossy_min_gain * best.overhead_us) best = z;
      }
    }
    Cand cd;
    cd.id = id;
    cd.opt = best;
    if (raw_only) {
      // baseline rule: longest absence first (time between the last forward use and the backward of that op)
      double away = 0;
      for (int i = r.last_use + 1; i < nops; i++) away += p->comptime[(size_t)i] * (1.0 + p->bwd_factor);
      cd.key = -away;
    } else {
      cd.key = best.overhead_us / (double)r.bytes;
    }
    cands.push_back(cd);
  }
  std::stable_sort(cands.begin(), cands.end(), [](const Cand& a, const Cand& b) {
    return a.key != b.key ? a.key < b.key : a.id < b.id;
  });
  const double target = p->ratio * (double)total;
  cswap_plan_summary s;
  s.base_time_us = base_time(p);
  s.time_us = s.base_time_us;
  s.bytes_total = total;
  s.bytes_target = (size_t)target;
  s.bytes_moved = 0;
  s.bytes_on_link = 0;
  s.n_selected = 0;
  for (const Cand& cd : cands) {
    if ((double)s.bytes_moved >= target) break;
    policy[cd.id] = cd.opt.code;
    s.bytes_moved += p->tensors[cd.id].bytes;
    s.bytes_on_link += cd.opt.bytes_out;
    s.time_us += cd.opt.overhead_us;
    s.n_selected++;
  }
  s.target_met = (double)s.bytes_moved >= target ? 1 : 0;
  p->last = s;
  if (out) *out = s;
  return CSWAP_OK;
}

extern "C" cswap_planner* cswap_planner_create(const cswap_costs* costs, unsigned zfp_maxbits)
{
  cswap_planner* p = new (std::nothrow) cswap_planner;
  if (!p) return nullptr;
  if (costs && costs->bw_d2h_gbs > 0 && costs->bw_h2d_gbs > 0) p->costs = *costs;
  else cswap_costs_default(&p->costs);
  p->maxbits = zfp_maxbits >= 16 && zfp_maxbits <= 4096 ? zfp_maxbits : 512;
  p->last = cswap_plan_summary();
  return p;
}

extern "C" void cswap_planner_destroy(cswap_planner* p) { delete p; }

extern "C" int cswap_planner_reset(cswap_planner* p)
{
  if (!p) return CSWAP_E_ARG;
  std::lock_guard<std::mutex> lock(p->mu);
  p->comptime.clear();
  p->tensors.clear();
  p->ratio = 0;
  return CSWAP_OK;
}

extern "C" int cswap_planner_set_backward_factor(cswap_planner* p, double f)
{
  if (!p || !(f >= 0)) return CSWAP_E_ARG;
  std::lock_guard<std::mutex> lock(p->mu);
  p->bwd_factor = f;
  return CSWAP_OK;
}

extern "C" int cswap_planner_add_comptime(cswap_planner* p, double microseconds)
{
  if (!p || !(microseconds >= 0)) return CSWAP_E_ARG;
  std::lock_guard<std::mutex> lock(p->mu);
  p->comptime.push_back(microseconds);
  return CSWAP_OK;
}

extern "C" int cswap_planner_add_tensor(cswap_planner* p, int id, size_t nbytes)
{
  if (!p || id < 0) return CSWAP_E_ARG;
  std::lock_guard<std::mutex> lock(p->mu);
  TensorRec& r = p->tensors[id];
  r.bytes = nbytes;
  r.present = true;
  return CSWAP_OK;
}

extern "C" int cswap_planner_add_stepdep(cswap_planner* p, int from_id, int to_id)
{
  if (!p || to_id < 0) return CSWAP_E_ARG;
  if (from_id < 0) return CSWAP_OK;  // the model input is not a tracked tensor (tensor_id -1)
  std::lock_guard<std::mutex> lock(p->mu);
  TensorRec& r = p->tensors[from_id];
  r.last_use = std::max(r.last_use, to_id);
  return CSWAP_OK;
}

extern "C" int cswap_planner_add_omitid(cswap_planner* p, int id)
{
  if (!p || id < 0) return CSWAP_E_ARG;
  std::lock_guard<std::mutex> lock(p->mu);
  p->tensors[id].omit = true;
  return CSWAP_OK;
}

extern "C" int cswap_planner_set_field(cswap_planner* p, int id, size_t nx, size_t ny, size_t nz)
{
  if (!p || id < 0 || !nx || !ny || !nz) return CSWAP_E_ARG;
  std::lock_guard<std::mutex> lock(p->mu);
  TensorRec& r = p->tensors[id];
  r.nx = nx; r.ny = ny; r.nz = nz;
  return CSWAP_OK;
}

extern "C" int cswap_planner_set_nnz(cswap_planner* p, int id, size_t nnz)
{
  if (!p || id < 0) return CSWAP_E_ARG;
  std::lock_guard<std::mutex> lock(p->mu);
  p->tensors[id].nnz = (long long)nnz;
  return CSWAP_OK;
}

extern "C" int cswap_planner_init(cswap_planner* p, double ratio)
{
  if (!p || !(ratio >= 0) || ratio > 1.0) return CSWAP_E_ARG;
  std::lock_guard<std::mutex> lock(p->mu);
  p->ratio = ratio;
  return CSWAP_OK;
}

extern "C" int cswap_planner_make_policy(cswap_planner* p, int* policy, int* begin_stage, int n,
                                         cswap_plan_summary* summary)
{
  return plan(p, false, policy, begin_stage, n, summary);
}

extern "C" int cswap_planner_capuchin(cswap_planner* p, int* policy, int* begin_stage, int n,
                                      cswap_plan_summary* summary)
{
  return plan(p, true, policy, begin_stage, n, summary);
}
