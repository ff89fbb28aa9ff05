// mirage::threadblock::Graph — the thread-block-level graph builder — and
// ExecutionPlan, the serialisable recipe a customized op is built from
// (reference include/mirage/threadblock/graph.h:28-117).
#pragma once

#include "mirage/kernel/device_tensor.h"
#include "mirage/threadblock/operator.h"
#include "mirage/threadblock/serializer/kernel_params.h"
#include "mirage/threadblock/smem_tensor.h"
#include "mirage/utils/hip_types.h"
#include <sys/types.h>
#include <utility>
#include <vector>

namespace mirage {
namespace threadblock {

class ExecutionPlan {
public:
  // (operator, operands); an operand is (index of the producing operator inside
  // the thread-block graph, index of its output tensor)
  std::vector<std::pair<mirage::type::TBOperatorType, std::vector<std::pair<int, int>>>> ops;
  std::vector<int3> input_map;   // per input: tensor dim split by grid x / y / z (-1: none)
  std::vector<int> forloop_dim;  // per input: tensor dim split by the for-loop (-1: none)
  std::vector<mirage::layout::SmemLayout> input_smem_layouts;
  int3 output_map;               // shared by all outputs
  int forloop_range;
  int reduction_dimx = mirage::type::TB_REDUCTION_DIMX;
  dim3 grid_dim, block_dim;
};

class Graph {
public:
  Graph(dim3 grid_dim, dim3 block_dim, int forloop_range, int reduction_dimx);

  STensor new_input(mirage::kernel::DTensor const &dtensor, int3 input_map, int forloop_dim,
                    mirage::layout::SmemLayout layout);
  TBOperator *create_input_op(mirage::kernel::DTensor const &dtensor, int3 input_map,
                              int forloop_dim, mirage::layout::SmemLayout layout);
  mirage::kernel::DTensor new_output(STensor const &stensor, int3 output_map);
  TBOperator *create_output_op(STensor const &stensor, int3 output_map);
  STensor matmul(STensor const &A, STensor const &B);
  TBOperator *create_matmul_op(STensor const &A, STensor const &B);
  STensor exp(STensor const &A);
  STensor silu(STensor const &A);  // extension
  TBOperator *create_elementunary_op(STensor const &A, mirage::type::TBOperatorType _type);
  STensor add(STensor const &A, STensor const &B);
  STensor mul(STensor const &A, STensor const &B);
  STensor div(STensor const &A, STensor const &B);
  TBOperator *create_elementbinary_op(STensor const &A, STensor const &B,
                                      mirage::type::TBOperatorType _type);
  STensor reduction(STensor const &A, int dim);
  TBOperator *create_reduction_op(STensor const &A, int dim);
  STensor reduction_to_dimx(STensor const &A, int dim);
  TBOperator *create_reduction_to_dimx_op(STensor const &A, int dim);
  STensor concat(STensor const &A, STensor const &B, int dim);
  TBOperator *create_concat_op(STensor const &A, STensor const &B, int dim);

  off_t allocate(STensor const &tensor);
  void free(STensor const &tensor);
  void free(std::vector<STensor> const &tensors);

  // Lowers the graph to the flat program; `fingerprint` selects fp_ptr or
  // data_ptr of the device tensors (reference src/threadblock/graph.cc:68-432).
  NewKernelParams get_new_kernel_params(bool fingerprint) const;

  // Upper bound of smem_offset for graphs built afterwards.  Defaults to the
  // reference's MAX_SMEM_SIZE (or environment MIRAGE_SMEM_BUDGET).  Tiles are
  // re-placed by the backend from their live ranges, so the budget limits the
  // graph's address space, not the LDS a launch requests.
  static void set_smem_budget(size_t bytes);
  static size_t smem_budget();

  // {graph_level, grid_dim, block_dim, forloop_range, reduction_dimx, operators,
  // smem_offset} (reference threadblock/graph.h:107, src/threadblock/graph.cc:476-489)
  operator json() const;

  dim3 grid_dim, block_dim;
  int forloop_range;
  int reduction_dimx;
  std::vector<mirage::threadblock::TBOperator *> operators;
  off_t smem_offset;
  std::vector<std::pair<off_t, size_t>> allocated_tensors;
};

}  // namespace threadblock
}  // namespace mirage
