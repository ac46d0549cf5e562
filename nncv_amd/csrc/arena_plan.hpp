// Offsets of the intermediate tensors of one forward pass inside a single device allocation.
//
// "Greedy by Size for Offset Calculation" of Pisarchyk & Lee, Efficient Memory Management for Deep
// Neural Net Inference (arXiv 2001.03288, section 5.2) — the algorithm of the reference's
// MemSolver::solve (src/nncv/compiler/Optimizer/MemSolver.cpp:15-47), which the reference has but
// never wires into a pipeline.  Tensors are placed in non-increasing order of size; each goes into
// the smallest gap, between already placed tensors whose lifetimes overlap its own, that holds
// it, or behind the last of them.  Unlike the reference, the list of placed tensors is kept
// sorted by offset, as the paper requires for the gap scan to be meaningful.
#pragma once
#include <cstddef>
#include <vector>

namespace nncv_hip {

struct TensorLife {
  int first_op, last_op;  // inclusive range of operator indices during which the tensor is live
  size_t bytes;
  size_t offset;          // out
};

// Fills `offset` of every record (input order is kept) and returns the arena size.  Offsets and
// sizes are rounded up to `align` bytes (a power of two; 1 = none).
size_t plan_offsets(std::vector<TensorLife>& tensors, size_t align);

// Operator steps a tensor's memory is kept after its last reader before the planners of the forward passes hand it to
// another tensor (they add this to every last_op).  Measured on ResNet-18 at batch 32 (rocprofv3, median per launch): a
// launch whose output lies where the previous launch's INPUT lay runs 2-4.4 us longer (16.4 against 12.0 us for the first
// stride-1 convolution after a down-sampling one, 14.0 against 11.8 one stage deeper), one launch further back it is
// still 2.3 us (13.4 against 11.1), from three launches on nothing; the whole pass gains 9 us of 256 for 20 % more
// workspace.  NNCV_HIP_ARENA_LINGER overrides (0 = hand memory on at once); arena_linger_forced() says that it did.
int arena_linger();
bool arena_linger_forced();

// How many forward passes the caller says it keeps in flight on different streams (nncv_hip_set_overlap_hint; 1 unless
// told otherwise, NNCV_HIP_OVERLAP sets the initial value).  From three up the planners pick the forms that measured
// faster when launches of different passes share the chip -- what counts then is how long a launch's workgroups hold
// their LDS and register slots, not how soon the launch ends: the 128-filter form of the 3x3 stream kernel wherever
// the filter count allows it (half the workgroups of the 64-filter form, no exchange between K groups), for one-slab
// layers the 64-filter form with resident weights on half the places, and the patch kernel where neither fits; in
// ResNet-18 from batch 16 up also no lingering in the arena (the penalty
// it avoids belongs to launches that have the chip to themselves; four smaller working sets share the caches better:
// 0.165 against 0.168 ms -- MobileNetV3's small tensors measured the other way, 0.169 against 0.162, and keep
// lingering) and average pool and FC as two small launches instead of the fused head's 1024 workgroups that each pool
// their image again.  ResNet-18 at batch 32 with four passes in flight: 0.160 against 0.174 ms per pass; one pass at a
// time the same choices cost 7 % (0.275 against 0.256).
// The value belongs to the network handle (nncv_hip_resnet18_create_ex; clones inherit it): while an entry point serves a
// handle that has one, OverlapScope makes it the answer of overlap_hint() on that thread, so two handles with different
// values plan, capture and replay side by side.  Handles without a value, the single-layer entry points and the operator-
// list executor follow the process-wide default (overlap_default).
int overlap_hint();
int overlap_default();
void set_overlap_hint(int passes);
class OverlapScope {
 public:
  explicit OverlapScope(int passes);  // passes <= 0: leaves the thread's current value alone
  ~OverlapScope();
  OverlapScope(const OverlapScope&) = delete;
  OverlapScope& operator=(const OverlapScope&) = delete;

 private:
  int prev_;
};

}  // namespace nncv_hip
