// NewKernelParams: the flat program a thread-block graph is lowered to (reference
// include/mirage/threadblock/serializer/kernel_params.h:25-35).  Per operator, in
// order, `parameters` holds
//   input loader (19): row block strides x,y,z; column block strides x,y,z; row and
//       column for-loop strides; batch-offset block strides x,y,z and for-loop
//       stride; device matrix rows, cols; tile rows, cols; dmem layout; smem
//       layout; tile offset
//   output saver (17): row block strides; column block strides; batch-offset block
//       strides; device matrix rows, cols; tile rows, cols; dmem layout; smem
//       layout; input tile offset; accumulator offset
//   matmul (6): m, n, k, A, B, C offsets        unary (2): offset, element count
//   binary (9): shape1 x,y,z; shape2 x,y,z; in1, in2, out offsets
//   reduction (5): output elements, degree, inner range, in, out offsets
//   concat (7): output elements, A extent, B extent, inner size, A, B, out offsets
#pragma once

#include "mirage/type.h"

namespace mirage {
namespace threadblock {

struct alignas(16) NewKernelParams {
  static int const MAX_NUM_OPERATORS = 16;
  static int const MAX_NUM_PARAMETERS = 120;
  static int const MAX_NUM_DMEM_INPUTS = 4;
  static int const MAX_NUM_DMEM_OUTPUTS = 4;
  int num_operators, num_parameters, num_dmem_inputs, num_dmem_outputs;
  int parameters[MAX_NUM_PARAMETERS];
  mirage::type::TBOperatorType operator_types[MAX_NUM_OPERATORS];
  void *dmem_input_ptrs[MAX_NUM_DMEM_INPUTS];
  void *dmem_output_ptrs[MAX_NUM_DMEM_OUTPUTS];
};

}  // namespace threadblock
}  // namespace mirage
