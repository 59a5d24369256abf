// cswap_execution.hpp -- header-only C++ mirror of the reference's swap scheduler
// `class Execution` (CSWAP+/Execution.h:38-446) over the C ABI of cswap_hip.h.
//
// The reference walks a model's forward pass as  preforward(); for each op:
// pre(input, layer_type) -> op -> post(input, output, layer_type);  postforward()
// and identifies tensors by the index of the op that produced them (`tensor_id`,
// Execution.h:219).  A tensor is dealt with when the running op index reaches
// begin_stage[id] (Execution.h:69: by default id+1, the op that consumes it).
// What happens to it follows the reference's branch order:
//   post, Execution.h:243:  policy[id] == 1, or policy_ == 4 and the consuming op is
//        not a convolution -> the tensor is dropped (to be recomputed in backward),
//        tag 1 -- whatever pre() would have done with it;
//   pre,  Execution.h:70:   policy[id] == 2, or the consuming op is a convolution and
//        policy_ > 2 (the vDNN and SuperNeurons modes) -> raw swap, tag 2;
//   pre,  Execution.h:86:   policy[id] == 3 -> ZVC, tag 3;
//   pre,  Execution.h:107:  policy[id] == 6 -> ZFP, tag 6;
//   anything else (0) -> kept.
// policy_ (Execution.h:420): 1 this scheme, 2 Capuchin, 3 vDNN, 4 SuperNeurons.
// Added here: policy[id] == -1 lets the selector decide per tensor, and its
// decisions are remembered from one iteration to the next (see `recheck`).
// The reference works on torch::Tensor and a patched autograd; this mirror takes
// raw device pointers and field extents, and offers the backward-side `fetch` the
// reference hides in its autograd engine.
#ifndef CSWAP_EXECUTION_HPP
#define CSWAP_EXECUTION_HPP

#include <map>
#include <set>
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
  // setRatio (Execution.h:63, called again from the training loop): 4 * ratio bits per 4x4x4
  // block for the ZFP swap-outs from now on; 128 = a quarter of the fp32 size.
  int setRatio(int ratio) { return ratio > 0 ? cswap_engine_set_zfp_maxbits(engine_, 4u * (unsigned)ratio) : CSWAP_E_ARG; }
  // also forgets what the previous iteration dropped (the caller recomputed it)
  void preforward()
  {
    init();
    dropped_.clear();
  }
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
  int pre(const std::vector<Input>& inputs, cswap_stream_t compute, Layer_type layer_type = ACT)
  {
    index++;
    pending_.clear();
    for (const Input& in : inputs) {
      if (in.tensor_id < 0 || (size_t)in.tensor_id >= policy.size()) continue;
      if (index != begin_stage[(size_t)in.tensor_id]) continue;
      if (tickets_.count(in.tensor_id) || dropped_.count(in.tensor_id)) continue;  // fed twice to one op
      int act = action(policy[(size_t)in.tensor_id], policy_, layer_type);
      if (act == 0) continue;
      if (act == 1) {  // nothing to move: post() reports it as dropped
        dropped_.insert(in.tensor_id);
        continue;
      }
      const size_t n = in.nx * in.ny * in.nz;
      Memo* memo = nullptr;
      if (act == CSWAP_POLICY_AUTO && recheck > 0) {
        memo = &memo_[in.tensor_id];
        if (memo->n == n && memo->uses < recheck &&
            (memo->policy == CSWAP_POLICY_ZFP || memo->policy == CSWAP_POLICY_NONE)) {
          act = memo->policy;  // remembered: no counting pass, no host round trip
          memo->uses++;
          memo_hits++;
          memo = nullptr;
        } else if (memo->n == n && memo->policy == CSWAP_POLICY_SPARSE) {
          // remembered as sparse: still the selector's call, with the compaction itself as its
          // probe (the payload is made by the time the count is known; the count confirms or
          // overturns the choice every time, so this memory never goes stale)
          act = CSWAP_POLICY_AUTO_SPARSE;
        }
      }
      int ticket = -1;
      int rc = cswap_swap_out(engine_, in.d_tensor, in.nx, in.ny, in.nz, act, compute, &ticket);
      if (rc) return rc;
      if (memo) {  // the selector decided: remember what
        cswap_ticket_info info;
        if (cswap_swap_info(engine_, ticket, &info) == CSWAP_OK) {
          memo->n = n;
          memo->policy = info.policy;
          memo->uses = 0;
        }
      }
      tickets_[in.tensor_id] = ticket;
      pending_.push_back(in.tensor_id);
    }
    return CSWAP_OK;
  }

  // What the reference does with a tensor whose entry in policy[] is `entry`, under
  // the global mode `mode`, when the op that consumes it is of type `layer_type`:
  // 0 keep, 1 drop, 2 raw swap, 3 ZVC, 6 ZFP, -1 selector (Execution.h:70,86,107,243).
  static int action(int entry, int mode, Layer_type layer_type)
  {
    if (entry == 1 || (mode == 4 && layer_type != CONV)) return 1;
    if (entry == 2 || (layer_type == CONV && mode > 2)) return CSWAP_POLICY_NONE;
    if (entry == CSWAP_POLICY_SPARSE || entry == CSWAP_POLICY_ZFP || entry == CSWAP_POLICY_AUTO) return entry;
    return 0;
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
  // true from the pre() that dropped the tensor until the next preforward()
  bool dropped(int tensor_id) const { return dropped_.count(tensor_id) != 0; }

  // what happened to the tensor (the reference's com_and_tran tag, Execution.h:247,262,
  // 280,299): 1 dropped, 2 raw, 3 ZVC, 6 ZFP; 0 if it was kept
  int com_and_tran(int tensor_id) const
  {
    if (dropped_.count(tensor_id)) return 1;
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
  int policy_ = 1;  // 1 this scheme, 2 Capuchin, 3 vDNN, 4 SuperNeurons (Execution.h:420)
  // Selector memo.  A tensor whose entry is -1 is probed (a counting pass and a small
  // host round trip, the one the reference pays at Execution.h:92) and priced by the
  // selector.  When that ends in ZFP or in the raw swap, the next `recheck` iterations
  // take the same action for the tensor at this position, as long as its size is the
  // same, without probing; then it is probed again.  A ZVC decision is never reused:
  // its payload needs the count anyway.  recheck = 0 switches the memo off.
  int recheck = 16;
  long memo_hits = 0;  // swaps that went out on a remembered decision
  void forget() { memo_.clear(); }

 private:
  struct Memo {
    size_t n = 0;
    int policy = 0;
    int uses = 0;
  };
  cswap_engine* engine_;
  std::map<int, int> tickets_;
  std::set<int> dropped_;
  std::map<int, Memo> memo_;
  std::vector<int> pending_;
};

}  // namespace cswap
#endif
