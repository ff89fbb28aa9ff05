// Kernel-level graph construction: shape inference, feasibility checks and arena
// allocation of every operator's outputs.  Behaviour follows the reference's
// src/kernel/{operator,matmul,element_unary,element_binary,reduction,customized}.cc:
// `create_*` returns nullptr for an infeasible operator, the wrappers abort.
#include "mirage/kernel/device_memory_manager.h"
#include "mirage/kernel/graph.h"
#include "mirage/utils/hip_types.h"

#include <algorithm>

namespace mirage {
namespace kernel {

using mirage::threadblock::ExecutionPlan;
using mirage::threadblock::STensor;
using namespace mirage::type;

// ---- operator base -----------------------------------------------------------
KNOperator::KNOperator(KNOperatorType _type) : op_type(_type) {}
KNOperator::KNOperator(KNOperatorType _type, DTensor const &a) : op_type(_type) {
  input_tensors.push_back(a);
}
KNOperator::KNOperator(KNOperatorType _type, DTensor const &a, DTensor const &b)
    : op_type(_type) {
  input_tensors.push_back(a);
  input_tensors.push_back(b);
}
KNOperator::KNOperator(KNOperatorType _type, std::vector<DTensor> const &inputs)
    : op_type(_type), input_tensors(inputs) {}
KNOperator::~KNOperator() {}

void KNOperator::release_outputs() {
  DeviceMemoryManager *dmm = DeviceMemoryManager::get_instance();
  for (int i = (int)output_tensors.size() - 1; i >= 0; i--) {
    dmm->free(output_tensors[i]);
  }
}

static bool arena_has_room(size_t bytes) {
  DeviceMemoryManager *dmm = DeviceMemoryManager::get_instance();
  return (size_t)dmm->offset + bytes <= dmm->total_size;
}

static void adopt_output(KNOperator *op, DTensor &t) {
  t.owner_op = op;
  t.owner_ts_idx = (int)op->output_tensors.size();
  t.guid = DTensor::next_guid++;
  DeviceMemoryManager::get_instance()->allocate(t);
  op->output_tensors.push_back(t);
}

// ---- graph ---------------------------------------------------------------------
Graph::Graph() {}

Graph::~Graph() {
  while (!operators.empty()) {
    delete operators.back();
    operators.pop_back();
  }
}

// input (reference src/kernel/operator.cc:48-113)
DTensor Graph::new_input(std::vector<int> const &dims, DataType data_type,
                         mirage::layout::DmemLayout layout) {
  KNOperator *op = create_input_op(dims, data_type, layout);
  MIRAGE_CHECK(op != nullptr, "input does not fit the device arena");
  operators.push_back(op);
  return op->output_tensors[0];
}

DTensor *Graph::new_input_ptr(std::vector<int> const &dims, DataType data_type,
                              mirage::layout::DmemLayout layout) {
  new_input(dims, data_type, layout);
  return &operators.back()->output_tensors[0];
}

KNOperator *Graph::create_input_op(std::vector<int> const &dims, DataType data_type,
                                   mirage::layout::DmemLayout layout) {
  if (dims.empty() || dims.size() > MAX_TENSOR_DIMS) {
    return nullptr;
  }
  DTensor probe;
  probe.num_dims = (int)dims.size();
  probe.data_type = data_type;
  for (int i = 0; i < probe.num_dims; i++) {
    probe.dim[i] = dims[i];
  }
  if (!arena_has_room(probe.data_size())) {
    return nullptr;
  }
  return new KNInputOp(dims, data_type, layout);
}

KNInputOp::KNInputOp(std::vector<int> const &dims, DataType data_type,
                     mirage::layout::DmemLayout layout)
    : KNOperator(KN_INPUT_OP) {
  DTensor t;
  t.num_dims = (int)dims.size();
  for (int i = 0; i < t.num_dims; i++) {
    t.dim[i] = dims[i];
  }
  t.data_type = data_type;
  t.layout = layout;
  adopt_output(this, t);
}
KNInputOp::~KNInputOp() { release_outputs(); }

// matmul (reference src/kernel/matmul.cc:28-103)
DTensor Graph::matmul(DTensor const &A, DTensor const &B) {
  KNOperator *op = create_matmul_op(A, B);
  MIRAGE_CHECK(op != nullptr, "infeasible matmul");
  operators.push_back(op);
  return op->output_tensors[0];
}

DTensor *Graph::matmul(DTensor const *A, DTensor const *B) {
  matmul(*A, *B);
  return &operators.back()->output_tensors[0];
}

static bool matmul_shapes_ok(DTensor const &A, DTensor const &B) {
  if (A.num_dims != B.num_dims || A.num_dims < 2) {
    return false;
  }
  if (A.dim[A.num_dims - 1] != B.dim[B.num_dims - 2]) {
    return false;
  }
  for (int i = 0; i < A.num_dims - 2; i++) {
    if (A.dim[i] != B.dim[i]) {
      return false;
    }
  }
  return true;
}

KNOperator *Graph::create_matmul_op(DTensor const &A, DTensor const &B) {
  if (!matmul_shapes_ok(A, B)) {
    return nullptr;
  }
  DTensor C = A;
  C.dim[C.num_dims - 1] = B.dim[C.num_dims - 1];
  if (!arena_has_room(C.data_size())) {
    return nullptr;
  }
  return new KNMatmulOp(A, B);
}

KNMatmulOp::KNMatmulOp(DTensor const &A, DTensor const &B) : KNOperator(KN_MATMUL_OP, A, B) {
  MIRAGE_CHECK(matmul_shapes_ok(A, B), "matmul shapes do not agree");
  DTensor C;
  C.num_dims = A.num_dims;
  for (int i = 0; i < C.num_dims; i++) {
    C.dim[i] = A.dim[i];
  }
  C.dim[C.num_dims - 1] = B.dim[C.num_dims - 1];
  C.layout = mirage::layout::DmemRowMajor;  // outputs are always row-major
  C.data_type = A.data_type;
  adopt_output(this, C);
}
KNMatmulOp::~KNMatmulOp() { release_outputs(); }

// element-wise unary (reference src/kernel/element_unary.cc:25-71)
DTensor Graph::exp(DTensor const &input) {
  KNOperator *op = create_elementunary_op(input, KN_EXP_OP);
  MIRAGE_CHECK(op != nullptr, "infeasible exp");
  operators.push_back(op);
  return op->output_tensors[0];
}

DTensor *Graph::exp(DTensor const *input) {
  exp(*input);
  return &operators.back()->output_tensors[0];
}

DTensor Graph::silu(DTensor const &input) {
  KNOperator *op = create_elementunary_op(input, KN_SILU_OP);
  MIRAGE_CHECK(op != nullptr, "infeasible silu");
  operators.push_back(op);
  return op->output_tensors[0];
}

KNOperator *Graph::create_elementunary_op(DTensor const &input, KNOperatorType type) {
  if (type != KN_EXP_OP && type != KN_SILU_OP) {
    return nullptr;
  }
  if (!arena_has_room(input.data_size())) {
    return nullptr;
  }
  return new KNElementUnaryOp(input, type);
}

KNElementUnaryOp::KNElementUnaryOp(DTensor const &input, KNOperatorType type)
    : KNOperator(type, input) {
  DTensor out = input;
  adopt_output(this, out);
}
KNElementUnaryOp::~KNElementUnaryOp() { release_outputs(); }

// element-wise binary (reference src/kernel/element_binary.cc:25-124)
static bool broadcastable(DTensor const &a, DTensor const &b) {
  if (a.num_dims != b.num_dims) {
    return false;
  }
  for (int i = 0; i < a.num_dims; i++) {
    if (a.dim[i] != b.dim[i] && a.dim[i] > 1 && b.dim[i] > 1) {
      return false;
    }
  }
  return true;
}

static DTensor binary_result(Graph *g, std::vector<KNOperator *> &ops, DTensor const &a,
                             DTensor const &b, KNOperatorType t, char const *what) {
  KNOperator *op = g->create_elementbinary_op(a, b, t);
  MIRAGE_CHECK(op != nullptr, what);
  ops.push_back(op);
  return op->output_tensors[0];
}

DTensor Graph::add(DTensor const &a, DTensor const &b) {
  return binary_result(this, operators, a, b, KN_ADD_OP, "infeasible add");
}
DTensor Graph::mul(DTensor const &a, DTensor const &b) {
  return binary_result(this, operators, a, b, KN_MUL_OP, "infeasible mul");
}
DTensor Graph::div(DTensor const &a, DTensor const &b) {
  return binary_result(this, operators, a, b, KN_DIV_OP, "infeasible div");
}
DTensor *Graph::add(DTensor const *a, DTensor const *b) {
  add(*a, *b);
  return &operators.back()->output_tensors[0];
}
DTensor *Graph::mul(DTensor const *a, DTensor const *b) {
  mul(*a, *b);
  return &operators.back()->output_tensors[0];
}
DTensor *Graph::div(DTensor const *a, DTensor const *b) {
  div(*a, *b);
  return &operators.back()->output_tensors[0];
}

KNOperator *Graph::create_elementbinary_op(DTensor const &a, DTensor const &b,
                                           KNOperatorType type) {
  if (!broadcastable(a, b)) {
    return nullptr;
  }
  DTensor out = a;
  for (int i = 0; i < out.num_dims; i++) {
    out.dim[i] = std::max(a.dim[i], b.dim[i]);
  }
  if (!arena_has_room(out.data_size())) {
    return nullptr;
  }
  return new KNElementBinaryOp(a, b, type);
}

KNElementBinaryOp::KNElementBinaryOp(DTensor const &a, DTensor const &b, KNOperatorType type)
    : KNOperator(type, a, b) {
  MIRAGE_CHECK(broadcastable(a, b), "binary operands are not broadcastable");
  DTensor out = a;
  for (int i = 0; i < out.num_dims; i++) {
    out.dim[i] = std::max(a.dim[i], b.dim[i]);
  }
  adopt_output(this, out);
}
KNElementBinaryOp::~KNElementBinaryOp() { release_outputs(); }

// reduction (reference src/kernel/reduction.cc:27-82)
DTensor Graph::reduction(DTensor const &input, int dim, int size) {
  KNOperator *op = create_reduction_op(input, dim, size);
  MIRAGE_CHECK(op != nullptr, "infeasible reduction");
  operators.push_back(op);
  return op->output_tensors[0];
}

DTensor *Graph::reduction(DTensor const *input, int dim, int size) {
  reduction(*input, dim, size);
  return &operators.back()->output_tensors[0];
}

KNOperator *Graph::create_reduction_op(DTensor const &input, int dim, int size) {
  if (dim < 0 || input.num_dims <= dim || size <= 0 || input.dim[dim] % size != 0) {
    return nullptr;
  }
  if (!arena_has_room(input.data_size())) {
    return nullptr;
  }
  return new KNReductionOp(input, dim, size);
}

KNReductionOp::KNReductionOp(DTensor const &input, int dim, int size)
    : KNOperator((KNOperatorType)(KN_REDUCTION_0_OP + dim), input), reduction_dim_idx(dim),
      reduction_dim_size(size) {
  MIRAGE_CHECK(dim < input.num_dims && input.dim[dim] % size == 0, "bad reduction");
  DTensor out = input;
  out.dim[dim] = size;
  adopt_output(this, out);
}
KNReductionOp::~KNReductionOp() { release_outputs(); }

// customized (reference src/kernel/customized.cc:32-312)
std::vector<DTensor> Graph::customized(std::vector<DTensor> const &inputs,
                                       ExecutionPlan const &plan) {
  KNOperator *op = create_customized_op(inputs, plan);
  MIRAGE_CHECK(op != nullptr, "infeasible customized op");
  operators.push_back(op);
  return op->output_tensors;
}

KNOperator *Graph::create_customized_op(std::vector<DTensor> const &inputs,
                                        ExecutionPlan const &plan) {
  return new KNCustomizedOp(inputs, plan);
}

std::vector<DTensor> Graph::customized(std::vector<DTensor> const &inputs,
                                       mirage::threadblock::Graph const &_graph) {
  KNOperator *op = create_customized_op(inputs, _graph);
  MIRAGE_CHECK(op != nullptr, "infeasible customized op");
  operators.push_back(op);
  return op->output_tensors;
}

KNOperator *Graph::create_customized_op(std::vector<DTensor> const &inputs,
                                        mirage::threadblock::Graph const &_graph) {
  size_t out_bytes = 0;
  for (mirage::threadblock::TBOperator *op : _graph.operators) {
    if (op->op_type == TB_OUTPUT_OP) {
      out_bytes += static_cast<mirage::threadblock::TBOutputOp *>(op)->dtensor.data_size();
    }
  }
  if (!arena_has_room(out_bytes)) {
    return nullptr;
  }
  return new KNCustomizedOp(inputs, _graph);
}

// Appends one thread-block operator of kind `t` over `ins` to `bg`.
static void append_tb_op(mirage::threadblock::Graph &bg, TBOperatorType t,
                         std::vector<STensor> const &ins) {
  auto arity = [&](size_t n) { MIRAGE_CHECK(ins.size() == n, "wrong operand count in plan"); };
  if (t == TB_MATMUL_OP) {
    arity(2);
    bg.matmul(ins[0], ins[1]);
  } else if (t == TB_EXP_OP) {
    arity(1);
    bg.exp(ins[0]);
  } else if (t == TB_SILU_OP) {
    arity(1);
    bg.silu(ins[0]);
  } else if (t == TB_ADD_OP) {
    arity(2);
    bg.add(ins[0], ins[1]);
  } else if (t == TB_MUL_OP) {
    arity(2);
    bg.mul(ins[0], ins[1]);
  } else if (t == TB_DIV_OP) {
    arity(2);
    bg.div(ins[0], ins[1]);
  } else if (t >= TB_REDUCTION_0_OP && t <= TB_REDUCTION_2_OP) {
    arity(1);
    bg.reduction(ins[0], t - TB_REDUCTION_0_OP);
  } else if (t >= TB_REDUCTION_0_TO_DIMX_OP && t <= TB_REDUCTION_2_TO_DIMX_OP) {
    arity(1);
    bg.reduction_to_dimx(ins[0], t - TB_REDUCTION_0_TO_DIMX_OP);
  } else if (t >= TB_CONCAT_0_OP && t <= TB_CONCAT_2_OP) {
    arity(2);
    bg.concat(ins[0], ins[1], t - TB_CONCAT_0_OP);
  } else {
    MIRAGE_CHECK(false, "unsupported thread-block operator in plan");
  }
}

void KNCustomizedOp::add_output(STensor const &stensor, int3 output_map) {
  DTensor dt = bgraph.new_output(stensor, output_map);
  adopt_output(this, dt);
  // the output operator keeps the allocated tensor (pointers included)
  auto *out = static_cast<mirage::threadblock::TBOutputOp *>(bgraph.operators.back());
  out->dtensor = output_tensors.back();
}

KNCustomizedOp::KNCustomizedOp(std::vector<DTensor> const &_inputs, ExecutionPlan const &_plan)
    : KNOperator(KN_CUSTOMIZED_OP, _inputs), plan(_plan),
      bgraph(_plan.grid_dim, _plan.block_dim, _plan.forloop_range, _plan.reduction_dimx) {
  size_t const n = _inputs.size();
  MIRAGE_CHECK(plan.input_map.size() == n && plan.forloop_dim.size() == n &&
                   plan.input_smem_layouts.size() == n,
               "plan does not describe every input");
  for (size_t i = 0; i < n; i++) {
    bgraph.new_input(input_tensors[i], plan.input_map[i], plan.forloop_dim[i],
                     plan.input_smem_layouts[i]);
  }
  for (auto const &entry : plan.ops) {
    std::vector<STensor> ins;
    for (auto const &idx : entry.second) {
      MIRAGE_CHECK(idx.first >= 0 && idx.first < (int)bgraph.operators.size(),
                   "plan operand names a missing operator");
      auto const &outs = bgraph.operators[idx.first]->output_tensors;
      MIRAGE_CHECK(idx.second >= 0 && idx.second < (int)outs.size(),
                   "plan operand names a missing tensor");
      ins.push_back(outs[idx.second]);
    }
    append_tb_op(bgraph, entry.first, ins);
  }
  // every tile of a non-input operator that no later operator reads is an output
  size_t const num_ops = bgraph.operators.size();
  for (size_t i = 0; i < num_ops; i++) {
    mirage::threadblock::TBOperator const *op = bgraph.operators[i];
    if (op->op_type == TB_INPUT_OP) {
      continue;
    }
    for (STensor const &t : op->output_tensors) {
      bool consumed = false;
      for (size_t j = i + 1; j < num_ops && !consumed; j++) {
        for (STensor const &u : bgraph.operators[j]->input_tensors) {
          if (u == t) {
            consumed = true;
            break;
          }
        }
      }
      if (!consumed) {
        add_output(t, plan.output_map);
      }
    }
  }
}

KNCustomizedOp::KNCustomizedOp(std::vector<DTensor> const &_inputs,
                               mirage::threadblock::Graph const &_graph)
    : KNOperator(KN_CUSTOMIZED_OP, _inputs),
      bgraph(_graph.grid_dim, _graph.block_dim, _graph.forloop_range, _graph.reduction_dimx) {
  plan.grid_dim = _graph.grid_dim;
  plan.block_dim = _graph.block_dim;
  plan.forloop_range = _graph.forloop_range;
  plan.reduction_dimx = _graph.reduction_dimx;
  size_t next_input = 0;
  for (mirage::threadblock::TBOperator *op : _graph.operators) {
    std::vector<STensor> ins;
    std::vector<std::pair<int, int>> indices;
    for (STensor const &t : op->input_tensors) {
      int op_idx = -1;
      for (size_t l = 0; l < _graph.operators.size(); l++) {
        if (_graph.operators[l] == t.owner_op) {
          op_idx = (int)l;
          break;
        }
      }
      MIRAGE_CHECK(op_idx >= 0, "tile produced outside the graph");
      ins.push_back(bgraph.operators[op_idx]->output_tensors[t.owner_ts_idx]);
      indices.push_back({op_idx, t.owner_ts_idx});
    }
    if (op->op_type == TB_INPUT_OP) {
      auto *in = static_cast<mirage::threadblock::TBInputOp *>(op);
      // the loader keeps the device tensor it was created over (as the reference does)
      MIRAGE_CHECK(next_input++ < input_tensors.size(), "more input loaders than inputs");
      bgraph.new_input(in->dtensor, in->input_map, in->forloop_dim,
                       in->output_tensors[0].layout);
      plan.input_map.push_back(in->input_map);
      plan.forloop_dim.push_back(in->forloop_dim);
      plan.input_smem_layouts.push_back(in->output_tensors[0].layout);
    } else if (op->op_type == TB_OUTPUT_OP) {
      auto *out = static_cast<mirage::threadblock::TBOutputOp *>(op);
      MIRAGE_CHECK(ins.size() == 1, "output operator takes one tile");
      add_output(ins[0], out->output_map);
      plan.output_map = out->output_map;
    } else {
      plan.ops.push_back({op->op_type, indices});
      append_tb_op(bgraph, op->op_type, ins);
    }
  }
}

KNCustomizedOp::~KNCustomizedOp() {
  while (!bgraph.operators.empty()) {
    delete bgraph.operators.back();
    bgraph.operators.pop_back();
  }
  release_outputs();
}

}  // namespace kernel
}  // namespace mirage
