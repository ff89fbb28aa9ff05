// mirage::kernel::Graph — the kernel-level graph builder (reference
// include/mirage/kernel/graph.h:28-85).  `create_*` return nullptr when an
// operator is infeasible (shape mismatch, arena exhausted); the value- and
// pointer-returning wrappers abort on that and append the operator.
#pragma once

#include "mirage/kernel/customized.h"
#include "mirage/kernel/device_tensor.h"
#include "mirage/kernel/operator.h"
#include "mirage/threadblock/graph.h"
#include <vector>

namespace mirage {
namespace kernel {

class Graph {
public:
  Graph(void);
  ~Graph();
  Graph(Graph const &) = delete;
  Graph &operator=(Graph const &) = delete;

  DTensor new_input(std::vector<int> const &dims, mirage::type::DataType data_type,
                    mirage::layout::DmemLayout layout);
  DTensor *new_input_ptr(std::vector<int> const &dims, mirage::type::DataType data_type,
                         mirage::layout::DmemLayout layout);
  KNOperator *create_input_op(std::vector<int> const &dims, mirage::type::DataType data_type,
                              mirage::layout::DmemLayout layout);

  DTensor matmul(DTensor const &A, DTensor const &B);
  DTensor *matmul(DTensor const *A, DTensor const *B);
  KNOperator *create_matmul_op(DTensor const &A, DTensor const &B);

  DTensor exp(DTensor const &input);
  DTensor *exp(DTensor const *input);
  DTensor silu(DTensor const &input);  // extension
  KNOperator *create_elementunary_op(DTensor const &input, mirage::type::KNOperatorType _type);

  DTensor add(DTensor const &input1, DTensor const &input2);
  DTensor mul(DTensor const &input1, DTensor const &input2);
  DTensor div(DTensor const &input1, DTensor const &input2);
  DTensor *add(DTensor const *input1, DTensor const *input2);
  DTensor *mul(DTensor const *input1, DTensor const *input2);
  DTensor *div(DTensor const *input1, DTensor const *input2);
  KNOperator *create_elementbinary_op(DTensor const &input1, DTensor const &input2,
                                      mirage::type::KNOperatorType _type);

  DTensor reduction(DTensor const &input, int dim, int size = 1);
  DTensor *reduction(DTensor const *input, int dim, int size = 1);
  KNOperator *create_reduction_op(DTensor const &input, int dim, int factor);

  std::vector<DTensor> customized(std::vector<DTensor> const &inputs,
                                  mirage::threadblock::ExecutionPlan const &plan);
  KNOperator *create_customized_op(std::vector<DTensor> const &inputs,
                                   mirage::threadblock::ExecutionPlan const &plan);
  std::vector<DTensor> customized(std::vector<DTensor> const &inputs,
                                  mirage::threadblock::Graph const &_graph);
  KNOperator *create_customized_op(std::vector<DTensor> const &inputs,
                                   mirage::threadblock::Graph const &_graph);

  // Writes a self-contained HIP program for gfx950: one specialised kernel per
  // customized operator, a launcher over all of them and a main() that fills the
  // tensors with random values and times the launcher (the role of the reference's
  // generate_triton_program, include/mirage/kernel/graph.h:79 and
  // src/kernel/triton_code_gen.cc:354-450; other kernel-level operators are skipped,
  // as there).
  void generate_hip_program(char const *filepath);

  // the graph as the array of its operators' JSON entries (what to_json(json &, Graph
  // const &) writes, src/kernel/graph.cc:33-37), so that `json(g)` reads as in the
  // reference's cpp_examples/profile.cc:22
  operator json() const;

  // Operators in creation order.  The graph deletes them newest-first on
  // destruction (the arena is LIFO); callers that pop an operator delete it
  // themselves, as the reference's search does.
  std::vector<mirage::kernel::KNOperator *> operators;
};

}  // namespace kernel
}  // namespace mirage
