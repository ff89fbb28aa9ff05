// Thread-block-level operators (reference include/mirage/threadblock/{operator,
// matmul,element_unary,element_binary,reduction,concat}.h).  Each owns the
// STensor(s) it defines; constructing one allocates from the graph's address
// space, destroying it releases (LIFO).
#pragma once

#include "mirage/kernel/device_tensor.h"
#include "mirage/threadblock/smem_tensor.h"
#include "mirage/type.h"
#include "mirage/utils/hip_types.h"
#include "mirage/utils/json_value.h"
#include <vector>

namespace mirage {
namespace threadblock {

class Graph;

class TBOperator {
public:
  TBOperator(Graph *graph, mirage::type::TBOperatorType);
  TBOperator(Graph *graph, mirage::type::TBOperatorType, STensor const &input1);
  TBOperator(Graph *graph, mirage::type::TBOperatorType, STensor const &input1,
             STensor const &input2);
  TBOperator(Graph *graph, mirage::type::TBOperatorType, std::vector<STensor> const &inputs);
  virtual ~TBOperator();
  // the operator's entry in the JSON form of its thread-block graph (reference
  // threadblock/operator.h:41, src/threadblock/graph.cc:485 `json(*op)`)
  virtual operator json() const = 0;

  Graph *bgraph;
  mirage::type::TBOperatorType op_type;
  std::vector<STensor> input_tensors;
  std::vector<STensor> output_tensors;
};

// Loads this block's / this iteration's tile of a device tensor.
class TBInputOp : public TBOperator {
public:
  TBInputOp(Graph *_graph, mirage::kernel::DTensor const &dtensor, int3 input_map,
            int forloop_dim, mirage::layout::SmemLayout layout);
  ~TBInputOp();
  operator json() const override;

  mirage::kernel::DTensor dtensor;
  int3 input_map;
  int forloop_dim;
};

// Accumulates its input tile over the for-loop (the "forloop_accum" of a
// mugraph) and stores the sum into this block's tile of a new device tensor.
class TBOutputOp : public TBOperator {
public:
  TBOutputOp(Graph *_graph, STensor const &stensor, int3 output_map);
  ~TBOutputOp();
  operator json() const override;

  mirage::kernel::DTensor dtensor;
  int3 output_map;
};

class TBMatmulOp : public TBOperator {
public:
  TBMatmulOp(Graph *_graph, STensor const &A, STensor const &B);
  ~TBMatmulOp();
  operator json() const override;
};

class TBElementUnaryOp : public TBOperator {  // in place
public:
  TBElementUnaryOp(Graph *_graph, STensor const &A, mirage::type::TBOperatorType _type);
  ~TBElementUnaryOp();
  operator json() const override;
};

class TBElementBinaryOp : public TBOperator {
public:
  TBElementBinaryOp(Graph *_graph, STensor const &A, STensor const &B,
                    mirage::type::TBOperatorType _type);
  ~TBElementBinaryOp();
  operator json() const override;
};

class TBReductionOp : public TBOperator {
public:
  TBReductionOp(Graph *graph, STensor const &input, int dim, int size);
  ~TBReductionOp();
  operator json() const override;

  int reduce_dim, reduce_size;
};

class TBConcatOp : public TBOperator {
public:
  TBConcatOp(Graph *graph, STensor const &A, STensor const &B, int dim);
  ~TBConcatOp();
  operator json() const override;

  int concat_dim;
};

}  // namespace threadblock
}  // namespace mirage
