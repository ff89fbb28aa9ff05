// KNCustomizedOp: a kernel-level operator whose body is a thread-block graph
// (reference include/mirage/kernel/customized.h:28-45).
#pragma once

#include "mirage/kernel/operator.h"
#include "mirage/threadblock/graph.h"

namespace mirage {
namespace kernel {

class KNCustomizedOp : public KNOperator {
public:
  // Builds the thread-block graph from a plan: one input loader per tensor, the
  // plan's operators in order, then one accumulating output per tile that no
  // later operator consumes (reference src/kernel/customized.cc:65-186).
  KNCustomizedOp(std::vector<DTensor> const &inputs,
                 mirage::threadblock::ExecutionPlan const &plan);
  // Rebuilds an existing thread-block graph over new inputs and recovers its plan.
  KNCustomizedOp(std::vector<DTensor> const &inputs, mirage::threadblock::Graph const &_graph);
  virtual ~KNCustomizedOp();
  bool profile(ProfileResult &profile) override;
  void run(void);  // one fp16 launch on the backend stream, no synchronisation
  bool fingerprint(void) override;
  operator json() const override;  // adds bgraph and plan (src/kernel/customized.cc:315-321)

  mirage::threadblock::ExecutionPlan plan;
  mirage::threadblock::Graph bgraph;

private:
  void add_output(mirage::threadblock::STensor const &stensor, int3 output_map);
};

}  // namespace kernel
}  // namespace mirage
