// cswap_policy_maker.hpp -- header-only C++ face of the planner (cswap_planner_* in
// cswap_hip.h) with the method names the reference's model drivers call on
// c10::GetPolicyMaker() (CSWAP+/inception-v3-cifar100.cpp:207-214,
// CSWAP+/vgg16-cifar10.cpp:474-497, CSWAP+/resnet-cifar10.cpp:330).  The
// reference's class is part of a patched PyTorch that its tree does not hold;
// the planning itself is this library's own cost model.
#ifndef CSWAP_POLICY_MAKER_HPP
#define CSWAP_POLICY_MAKER_HPP

#include <vector>

#include "cswap_hip.h"

namespace cswap {

class PolicyMaker {
 public:
  explicit PolicyMaker(const cswap_costs* costs = nullptr, unsigned zfp_maxbits = 0)
      : p_(cswap_planner_create(costs, zfp_maxbits)) {}
  ~PolicyMaker() { cswap_planner_destroy(p_); }
  PolicyMaker(const PolicyMaker&) = delete;
  PolicyMaker& operator=(const PolicyMaker&) = delete;

  // one profiled iteration
  void add_comptime(double microseconds) { cswap_planner_add_comptime(p_, microseconds); }
  void add_tensor(int index, size_t nbytes) { cswap_planner_add_tensor(p_, index, nbytes); }
  void add_stepdep(const std::vector<int>& dep)  // {pre.tensor_id, index}
  {
    if (dep.size() == 2) cswap_planner_add_stepdep(p_, dep[0], dep[1]);
  }
  void add_omitid(int index) { cswap_planner_add_omitid(p_, index); }
  void set_field(int index, size_t nx, size_t ny, size_t nz) { cswap_planner_set_field(p_, index, nx, ny, nz); }
  void set_nnz(int index, size_t nnz) { cswap_planner_set_nnz(p_, index, nnz); }
  void reset() { cswap_planner_reset(p_); }

  // share of the recorded activation bytes to move off the device
  void init(double ratio) { cswap_planner_init(p_, ratio); }

  // One action per tensor for Execution::policy (0 keep, 2 raw, 3 ZVC, 6 ZFP);
  // time_ receives the predicted iteration time in microseconds, as in the
  // reference's  policy1 = GetPolicyMaker()->make_policy(time_).
  std::vector<int> make_policy(int& time_, int n_tensors) { return plan(false, time_, n_tensors); }
  std::vector<int> capuchin(int& time_, int n_tensors) { return plan(true, time_, n_tensors); }

  // begin_stage of the last plan: the op at which each tensor is last used in
  // forward (what read_lastvisit(path, exe.begin_stage) supplies in the reference)
  const std::vector<int>& begin_stage() const { return begin_stage_; }
  const cswap_plan_summary& summary() const { return summary_; }

 private:
  std::vector<int> plan(bool raw_only, int& time_, int n)
  {
    std::vector<int> policy((size_t)(n > 0 ? n : 0), 0);
    begin_stage_.assign(policy.size(), 0);
    time_ = 0;
    if (n <= 0) return policy;
    int rc = raw_only ? cswap_planner_capuchin(p_, policy.data(), begin_stage_.data(), n, &summary_)
                      : cswap_planner_make_policy(p_, policy.data(), begin_stage_.data(), n, &summary_);
    if (rc != CSWAP_OK) return std::vector<int>();  // the reference's drivers stop on an empty policy
    time_ = (int)summary_.time_us;
    return policy;
  }

  cswap_planner* p_;
  std::vector<int> begin_stage_;
  cswap_plan_summary summary_ = {};
};

}  // namespace cswap
#endif
