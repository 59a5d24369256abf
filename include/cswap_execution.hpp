// cswap_execution.hpp -- header-only C++ mirror of the reference's swap scheduler
// `class Execution` (CSWAP+/Execution.h:38-446) over the C ABI of cswap_hip.h.
//
// The reference walks a model's forward pass as  preforward(); for each op:
// pre(input) -> op -> post(input, output);  postforward()  and identifies tensors
// by the index of the op that produced them (`tensor_id`, Execution.h:219).  A
// tensor is swapped out when the running op index reaches begin_stage[id]
// (Execution.h:69: by default id+1, the op that consumes it) with the action
// policy[id]: 0 keep, 2 raw swap, 3 ZVC, 6 ZFP (Execution.h:70,86,107), and -1 here
// for "let the selector decide".  The reference works on torch::Tensor and a
// patched autograd; this mirror takes raw device pointers and field extents, and
// offers the backward-side `fetch` the reference hides in its autograd engine.
#ifndef CSWAP_EXECUTION_HPP
#define CSWAP_EXECUTION_HPP

#include <map>
#include <vector>

#include "cswap_hip.h"

namespace cswap {

enum Layer_type { CONV, POOL, ACT, BN, FC, MASKFILL };  // Execution.h:28-35

class Execution {
 public:
  explicit Execution(cswap_engine* engine) : engine_(engine) {}

  // Execution::init_(n): room for n tensors, nothing swapped by default
  void init_(int n)
  {
    policy.assign((size_t)n, 0);
    begin_stage.assign((size_t)n, 0);
    for (int i = 0; i < n; i++) begin_stage[(size_t)i] = i + 1;
  }
  void init() { index = -1; }
  void preforward() { init(); }
  void postforward() {}

  // One input of an op: its tensor id (-1: not a tracked tensor), device pointer and field extents.
  struct Input {
    int tensor_id;
    const float* d_tensor;
    size_t nx, ny, nz;
  };

  // Call before op `index+1` runs on `compute`.  `tensor_id` is the id of the
  // op's input (-1: not a tracked tensor).  Returns a CSWAP_* status.
  int pre(int tensor_id, const float* d_tensor, size_t nx, size_t ny, size_t nz, cswap_stream_t compute,
          Layer_type layer_type = ACT)
  {
    const Input one = {tensor_id, d_tensor, nx, ny, nz};
    return pre(std::vector<Input>(1, one), compute, layer_type);
  }

  // The same for an op with several inputs (concatenation, residual add;
  // Execution.h:135-212): the op index advances once, every input whose
  // begin_stage is this op goes out under its own policy, and the copies queue
  // on the engine's copy stream in input order (the reference opens one stream
  // per input, Execution.h:165,195,200; one link carries them either way).
  // On an error the inputs already started stay pending for post().
  int pre(const std::vector<Input>& inputs, cswap_stream_t compute, Layer_type = ACT)
  {
    index++;
    pending_.clear();
    for (const Input& in : inputs) {
      if (in.tensor_id < 0 || (size_t)in.tensor_id >= policy.size()) continue;
      const int pol = policy[(size_t)in.tensor_id];
      if (index != begin_stage[(size_t)in.tensor_id] || pol == 0 || pol == 1) continue;
      if (tickets_.count(in.tensor_id)) continue;  // the same tensor fed twice to one op
      int ticket = -1;
      int rc = cswap_swap_out(engine_, in.d_tensor, in.nx, in.ny, in.nz, pol, compute, &ticket);
      if (rc) return rc;
      tickets_[in.tensor_id] = ticket;
      pending_.push_back(in.tensor_id);
    }
    return CSWAP_OK;
  }

  // Call after the op has been launched: waits for the copies started by the
  // matching pre() (Execution.h:248-299, 311-401); afterwards the caller may
  // release the device storage of the inputs.  Returns the id of the op's output tensor.
  int post(int* status = nullptr)
  {
    int rc = CSWAP_OK;
    for (int id : pending_) {
      int r = cswap_swap_wait(engine_, tickets_[id]);
      if (r && !rc) rc = r;
    }
    pending_.clear();
    if (status) *status = rc;
    return index;
  }

  bool swapped(int tensor_id) const { return tickets_.count(tensor_id) != 0; }

  // what happened to the tensor (the reference's com_and_tran tag): 0 if it was kept
  int com_and_tran(int tensor_id) const
  {
    auto it = tickets_.find(tensor_id);
    if (it == tickets_.end()) return 0;
    cswap_ticket_info info;
    return cswap_swap_info(engine_, it->second, &info) == CSWAP_OK ? info.policy : 0;
  }

  // Backward side, ahead of time: start the inbound copy of a tensor that a later
  // fetch() will ask for, so that it overlaps the backward kernels before it.
  int prefetch(int tensor_id)
  {
    auto it = tickets_.find(tensor_id);
    if (it == tickets_.end()) return CSWAP_E_STATE;
    return cswap_swap_prefetch(engine_, it->second);
  }

  // Backward side: bring the tensor back into d_out on `compute` and forget it.
  int fetch(int tensor_id, float* d_out, cswap_stream_t compute)
  {
    auto it = tickets_.find(tensor_id);
    if (it == tickets_.end()) return CSWAP_E_STATE;
    int rc = cswap_swap_in(engine_, it->second, d_out, compute);
    if (rc) return rc;
    rc = cswap_swap_release(engine_, it->second);  // waits for the decompression
    tickets_.erase(it);
    return rc;
  }

  int index = -1;
  std::vector<int> policy;
  std::vector<int> begin_stage;

 private:
  cswap_engine* engine_;
  std::map<int, int> tickets_;
  std::vector<int> pending_;
};

}  // namespace cswap
#endif
