// Thread-block-level graph construction and lowering to the flat program.
// Shape rules, the bump allocation of tile addresses and the stride arithmetic of
// get_new_kernel_params follow the reference's src/threadblock/*.cc.
#include "mirage/threadblock/graph.h"
#include "mirage/utils/hip_types.h"

#include <algorithm>
#include <cstdlib>

namespace mirage {
namespace threadblock {

using namespace mirage::type;
using mirage::kernel::DTensor;

// ---- operator base --------------------------------------------------------------
TBOperator::TBOperator(Graph *g, TBOperatorType t) : bgraph(g), op_type(t) {}
TBOperator::TBOperator(Graph *g, TBOperatorType t, STensor const &a) : bgraph(g), op_type(t) {
  input_tensors.push_back(a);
}
TBOperator::TBOperator(Graph *g, TBOperatorType t, STensor const &a, STensor const &b)
    : bgraph(g), op_type(t) {
  input_tensors.push_back(a);
  input_tensors.push_back(b);
}
TBOperator::TBOperator(Graph *g, TBOperatorType t, std::vector<STensor> const &ins)
    : bgraph(g), op_type(t), input_tensors(ins) {}
TBOperator::~TBOperator() {}

// ---- graph, address space ---------------------------------------------------------
static size_t g_smem_budget = 0;

void Graph::set_smem_budget(size_t bytes) { g_smem_budget = bytes; }

size_t Graph::smem_budget() {
  if (g_smem_budget == 0) {
    g_smem_budget = MAX_SMEM_SIZE;
    if (char const *env = std::getenv("MIRAGE_SMEM_BUDGET")) {
      g_smem_budget = std::strtoull(env, nullptr, 10);
    }
  }
  return g_smem_budget;
}

Graph::Graph(dim3 _grid_dim, dim3 _block_dim, int _forloop_range, int _reduction_dimx)
    : grid_dim(_grid_dim), block_dim(_block_dim), forloop_range(_forloop_range),
      reduction_dimx(_reduction_dimx), smem_offset(0) {
  MIRAGE_CHECK(reduction_dimx > 0, "reduction_dimx must be positive");
  MIRAGE_CHECK(forloop_range > 0, "forloop_range must be positive");
}

static off_t granules(size_t bytes) { return (off_t)((bytes + 15) & ~(size_t)15); }

// reference src/threadblock/graph.cc:43-66
off_t Graph::allocate(STensor const &tensor) {
  off_t at = smem_offset;
  off_t bytes = granules(tensor.size());
  smem_offset += bytes;
  MIRAGE_CHECK((size_t)smem_offset <= smem_budget(), "thread-block graph exceeds its smem budget");
  allocated_tensors.push_back({at, (size_t)bytes});
  return at;
}

void Graph::free(STensor const &tensor) {
  MIRAGE_CHECK(!allocated_tensors.empty() &&
                   allocated_tensors.back().first == tensor.smem_offset &&
                   allocated_tensors.back().second == (size_t)granules(tensor.size()),
               "tiles must be freed in reverse allocation order");
  smem_offset -= allocated_tensors.back().second;
  allocated_tensors.pop_back();
}

void Graph::free(std::vector<STensor> const &tensors) {
  for (int i = (int)tensors.size() - 1; i >= 0; i--) {
    free(tensors[i]);
  }
}

static bool fits(Graph const *g, size_t bytes) {
  return (size_t)g->smem_offset + bytes <= Graph::smem_budget();
}

static void own(TBOperator *op, STensor &t, bool allocate) {
  t.owner_op = op;
  t.owner_ts_idx = (int)op->output_tensors.size();
  t.guid = STensor::next_guid++;
  if (allocate) {
    t.smem_offset = (int)op->bgraph->allocate(t);
  }
  op->output_tensors.push_back(t);
}

// ---- input loader (reference src/threadblock/input_loader.cc:22-140) ---------------
// tile = device tensor with dim[imap.g] divided by grid.g (where grid.g > 1) and
// dim[forloop_dim] divided by forloop_range; false when something does not divide
static bool input_tile_shape(Graph const *g, DTensor const &dt, int3 imap, int forloop_dim,
                             STensor &tile) {
  tile.num_dims = dt.num_dims;
  tile.data_type = dt.data_type;
  for (int i = 0; i < dt.num_dims; i++) {
    tile.dim[i] = dt.dim[i];
  }
  int const map[3] = {imap.x, imap.y, imap.z};
  unsigned const grid[3] = {g->grid_dim.x, g->grid_dim.y, g->grid_dim.z};
  for (int d = 0; d < 3; d++) {
    if (grid[d] > 1 && map[d] >= 0) {
      if (map[d] >= dt.num_dims || tile.dim[map[d]] <= 0 || tile.dim[map[d]] % grid[d] != 0) {
        return false;
      }
      tile.dim[map[d]] /= grid[d];
    }
  }
  if (forloop_dim >= 0) {
    if (forloop_dim >= dt.num_dims || tile.dim[forloop_dim] <= 0 ||
        tile.dim[forloop_dim] % g->forloop_range != 0) {
      return false;
    }
    tile.dim[forloop_dim] /= g->forloop_range;
  }
  return true;
}

STensor Graph::new_input(DTensor const &dtensor, int3 input_map, int forloop_dim,
                         mirage::layout::SmemLayout layout) {
  TBOperator *op = create_input_op(dtensor, input_map, forloop_dim, layout);
  MIRAGE_CHECK(op != nullptr, "infeasible input loader");
  operators.push_back(op);
  return op->output_tensors[0];
}

TBOperator *Graph::create_input_op(DTensor const &dtensor, int3 input_map, int forloop_dim,
                                   mirage::layout::SmemLayout layout) {
  STensor tile;
  MIRAGE_CHECK(input_tile_shape(this, dtensor, input_map, forloop_dim, tile),
               "grid or for-loop does not divide the input");
  for (int i = 0; i < tile.num_dims - 2; i++) {
    if (tile.dim[i] != 1) {
      return nullptr;  // the loader moves 2-D tiles only
    }
  }
  if (!fits(this, tile.size())) {
    return nullptr;
  }
  return new TBInputOp(this, dtensor, input_map, forloop_dim, layout);
}

TBInputOp::TBInputOp(Graph *_graph, DTensor const &_dtensor, int3 _input_map, int _forloop_dim,
                     mirage::layout::SmemLayout _layout)
    : TBOperator(_graph, TB_INPUT_OP), dtensor(_dtensor), input_map(_input_map),
      forloop_dim(_forloop_dim) {
  STensor tile;
  MIRAGE_CHECK(input_tile_shape(bgraph, dtensor, input_map, forloop_dim, tile),
               "grid or for-loop does not divide the input");
  for (int i = 0; i < tile.num_dims - 2; i++) {
    MIRAGE_CHECK(tile.dim[i] == 1, "input tile has a leading dim larger than 1");
  }
  tile.layout = _layout;
  own(this, tile, true);
}
TBInputOp::~TBInputOp() { bgraph->free(output_tensors[0]); }

// ---- output / for-loop accumulator (reference src/threadblock/output.cc:22-79) -----
DTensor Graph::new_output(STensor const &stensor, int3 output_map) {
  TBOperator *op = create_output_op(stensor, output_map);
  MIRAGE_CHECK(op != nullptr, "infeasible output");
  operators.push_back(op);
  return static_cast<TBOutputOp *>(op)->dtensor;
}

TBOperator *Graph::create_output_op(STensor const &stensor, int3 output_map) {
  if ((size_t)smem_offset + stensor.size() >= smem_budget()) {
    return nullptr;
  }
  return new TBOutputOp(this, stensor, output_map);
}

TBOutputOp::TBOutputOp(Graph *_graph, STensor const &input, int3 _output_map)
    : TBOperator(_graph, TB_OUTPUT_OP, input), output_map(_output_map) {
  STensor accum = input;  // the accumulator tile
  own(this, accum, true);
  dtensor.num_dims = accum.num_dims;
  dtensor.data_type = accum.data_type;
  dtensor.layout = mirage::layout::DmemRowMajor;
  for (int i = 0; i < dtensor.num_dims; i++) {
    dtensor.dim[i] = accum.dim[i];
  }
  int const map[3] = {output_map.x, output_map.y, output_map.z};
  unsigned const grid[3] = {bgraph->grid_dim.x, bgraph->grid_dim.y, bgraph->grid_dim.z};
  for (int d = 0; d < 3; d++) {
    if (grid[d] > 1 && map[d] >= 0) {
      MIRAGE_CHECK(map[d] < dtensor.num_dims, "output_map names a missing dim");
      dtensor.dim[map[d]] *= grid[d];
    }
  }
}
TBOutputOp::~TBOutputOp() { bgraph->free(output_tensors); }

// ---- matmul (reference src/threadblock/matmul.cc:22-86) ------------------------------
STensor Graph::matmul(STensor const &A, STensor const &B) {
  TBOperator *op = create_matmul_op(A, B);
  MIRAGE_CHECK(op != nullptr, "infeasible thread-block matmul");
  operators.push_back(op);
  return op->output_tensors[0];
}

TBOperator *Graph::create_matmul_op(STensor const &A, STensor const &B) {
  if (A.num_dims != B.num_dims || A.num_dims < 2 ||
      A.dim[A.num_dims - 1] != B.dim[B.num_dims - 2]) {
    return nullptr;
  }
  for (int i = 0; i < A.num_dims - 2; i++) {
    if (A.dim[i] != 1 || B.dim[i] != 1) {
      return nullptr;  // no batched matmul inside a thread block
    }
  }
  STensor C = A;
  C.dim[C.num_dims - 1] = B.dim[C.num_dims - 1];
  if (!fits(this, C.size())) {
    return nullptr;
  }
  return new TBMatmulOp(this, A, B);
}

TBMatmulOp::TBMatmulOp(Graph *_graph, STensor const &A, STensor const &B)
    : TBOperator(_graph, TB_MATMUL_OP, A, B) {
  STensor C;
  C.layout = mirage::layout::SmemRowMajor;
  C.num_dims = A.num_dims;
  for (int i = 0; i < C.num_dims; i++) {
    C.dim[i] = A.dim[i];
  }
  C.dim[C.num_dims - 1] = B.dim[C.num_dims - 1];
  C.data_type = A.data_type;
  own(this, C, true);
}
TBMatmulOp::~TBMatmulOp() { bgraph->free(output_tensors); }

// ---- element-wise unary, in place (reference src/threadblock/element_unary.cc) -------
STensor Graph::exp(STensor const &A) {
  TBOperator *op = create_elementunary_op(A, TB_EXP_OP);
  MIRAGE_CHECK(op != nullptr, "infeasible exp");
  operators.push_back(op);
  return op->output_tensors[0];
}

STensor Graph::silu(STensor const &A) {
  TBOperator *op = create_elementunary_op(A, TB_SILU_OP);
  MIRAGE_CHECK(op != nullptr, "infeasible silu");
  operators.push_back(op);
  return op->output_tensors[0];
}

TBOperator *Graph::create_elementunary_op(STensor const &A, TBOperatorType _type) {
  if (_type != TB_EXP_OP && _type != TB_SILU_OP) {
    return nullptr;
  }
  return new TBElementUnaryOp(this, A, _type);
}

TBElementUnaryOp::TBElementUnaryOp(Graph *_graph, STensor const &A, TBOperatorType _type)
    : TBOperator(_graph, _type, A) {
  STensor out = A;  // same address: the result overwrites the operand
  own(this, out, false);
}
TBElementUnaryOp::~TBElementUnaryOp() {}

// ---- element-wise binary (reference src/threadblock/element_binary.cc) ----------------
static STensor binary_op(Graph *g, STensor const &A, STensor const &B, TBOperatorType t,
                         char const *what) {
  TBOperator *op = g->create_elementbinary_op(A, B, t);
  MIRAGE_CHECK(op != nullptr, what);
  g->operators.push_back(op);
  return op->output_tensors[0];
}
STensor Graph::add(STensor const &A, STensor const &B) {
  return binary_op(this, A, B, TB_ADD_OP, "infeasible add");
}
STensor Graph::mul(STensor const &A, STensor const &B) {
  return binary_op(this, A, B, TB_MUL_OP, "infeasible mul");
}
STensor Graph::div(STensor const &A, STensor const &B) {
  return binary_op(this, A, B, TB_DIV_OP, "infeasible div");
}

static bool broadcast_shape(STensor const &A, STensor const &B, STensor &out) {
  if (A.num_dims != B.num_dims) {
    return false;
  }
  out = A;
  for (int i = 0; i < A.num_dims; i++) {
    if (A.dim[i] != B.dim[i] && A.dim[i] > 1 && B.dim[i] > 1) {
      return false;
    }
    out.dim[i] = std::max(A.dim[i], B.dim[i]);
  }
  return true;
}

TBOperator *Graph::create_elementbinary_op(STensor const &A, STensor const &B,
                                           TBOperatorType _type) {
  STensor out;
  if (!broadcast_shape(A, B, out) || !fits(this, out.size())) {
    return nullptr;
  }
  return new TBElementBinaryOp(this, A, B, _type);
}

TBElementBinaryOp::TBElementBinaryOp(Graph *_graph, STensor const &A, STensor const &B,
                                     TBOperatorType _type)
    : TBOperator(_graph, _type, A, B) {
  STensor out;
  MIRAGE_CHECK(broadcast_shape(A, B, out), "binary operands are not broadcastable");
  own(this, out, true);
}
TBElementBinaryOp::~TBElementBinaryOp() { bgraph->free(output_tensors); }

// ---- reductions (reference src/threadblock/reduction.cc:22-98) --------------------------
STensor Graph::reduction(STensor const &A, int dim) {
  TBOperator *op = create_reduction_op(A, dim);
  MIRAGE_CHECK(op != nullptr, "infeasible reduction");
  operators.push_back(op);
  return op->output_tensors[0];
}

TBOperator *Graph::create_reduction_op(STensor const &A, int dim) {
  MIRAGE_CHECK(dim >= 0 && dim < A.num_dims, "reduction dim out of range");
  if (dim < A.num_dims - 2) {
    return nullptr;
  }
  STensor out = A;
  out.dim[dim] = 1;
  if (!fits(this, out.size())) {
    return nullptr;
  }
  return new TBReductionOp(this, A, dim, 1);
}

STensor Graph::reduction_to_dimx(STensor const &A, int dim) {
  TBOperator *op = create_reduction_to_dimx_op(A, dim);
  MIRAGE_CHECK(op != nullptr, "infeasible reduction_to_dimx");
  operators.push_back(op);
  return op->output_tensors[0];
}

TBOperator *Graph::create_reduction_to_dimx_op(STensor const &A, int dim) {
  MIRAGE_CHECK(dim >= 0 && dim < A.num_dims, "reduction dim out of range");
  STensor out = A;
  out.dim[dim] = reduction_dimx;
  if (!fits(this, out.size())) {
    return nullptr;
  }
  return new TBReductionOp(this, A, dim, reduction_dimx);
}

TBReductionOp::TBReductionOp(Graph *g, STensor const &input, int dim, int size)
    : TBOperator(g,
                 (TBOperatorType)((size == 1 ? TB_REDUCTION_0_OP : TB_REDUCTION_0_TO_DIMX_OP) + dim),
                 input),
      reduce_dim(dim), reduce_size(size) {
  STensor out = input;
  out.dim[dim] = size;
  own(this, out, true);
}
TBReductionOp::~TBReductionOp() { bgraph->free(output_tensors[0]); }

// ---- concat (reference src/threadblock/concat.cc:22-75) -----------------------------------
STensor Graph::concat(STensor const &A, STensor const &B, int dim) {
  TBOperator *op = create_concat_op(A, B, dim);
  MIRAGE_CHECK(op != nullptr, "infeasible concat");
  operators.push_back(op);
  return op->output_tensors[0];
}

TBOperator *Graph::create_concat_op(STensor const &A, STensor const &B, int dim) {
  if (A.num_dims != B.num_dims || dim < 0 || A.num_dims <= dim) {
    return nullptr;
  }
  for (int i = 0; i < A.num_dims; i++) {
    if (i != dim && A.dim[i] != B.dim[i]) {
      return nullptr;
    }
  }
  if (!fits(this, A.size() + B.size())) {
    return nullptr;
  }
  return new TBConcatOp(this, A, B, dim);
}

TBConcatOp::TBConcatOp(Graph *g, STensor const &A, STensor const &B, int dim)
    : TBOperator(g, (TBOperatorType)(TB_CONCAT_0_OP + dim), A, B), concat_dim(dim) {
  MIRAGE_CHECK(A.layout == B.layout, "concat operands must share a layout");
  STensor out = A;
  out.dim[dim] = A.dim[dim] + B.dim[dim];
  own(this, out, true);
}
TBConcatOp::~TBConcatOp() { bgraph->free(output_tensors[0]); }

// ---- lowering (reference src/threadblock/graph.cc:68-432) ------------------------------------
namespace {

struct Emitter {
  NewKernelParams &p;
  void put(int v) {
    MIRAGE_CHECK(p.num_parameters < NewKernelParams::MAX_NUM_PARAMETERS,
                 "thread-block graph has too many parameters");
    p.parameters[p.num_parameters++] = v;
  }
  void put3(int const v[3]) {
    put(v[0]);
    put(v[1]);
    put(v[2]);
  }
};

// element strides of the leading (batch) dims of a row-major tensor whose last
// two dims form the matrix
void batch_strides(DTensor const &dt, int strides[MAX_TENSOR_DIMS]) {
  int const nd = dt.num_dims;
  for (int i = 0; i < MAX_TENSOR_DIMS; i++) {
    strides[i] = 0;
  }
  if (nd > 2) {
    strides[nd - 3] = dt.dim[nd - 2] * dt.dim[nd - 1];
    for (int j = nd - 4; j >= 0; j--) {
      strides[j] = strides[j + 1] * dt.dim[j + 1];
    }
  }
}

void shape3(STensor const &t, int out[3]) {
  for (int i = 0; i < t.num_dims - 3; i++) {
    MIRAGE_CHECK(t.dim[i] == 1, "binary operand has more than three non-unit dims");
  }
  out[2] = t.num_dims > 0 ? t.dim[t.num_dims - 1] : 1;
  out[1] = t.num_dims > 1 ? t.dim[t.num_dims - 2] : 1;
  out[0] = t.num_dims > 2 ? t.dim[t.num_dims - 3] : 1;
}

}  // namespace

NewKernelParams Graph::get_new_kernel_params(bool fingerprint) const {
  NewKernelParams params;
  params.num_operators = (int)operators.size();
  params.num_parameters = 0;
  params.num_dmem_inputs = 0;
  params.num_dmem_outputs = 0;
  MIRAGE_CHECK(params.num_operators <= NewKernelParams::MAX_NUM_OPERATORS,
               "thread-block graph has too many operators");
  Emitter em{params};
  int const F = forloop_range;
  for (size_t i = 0; i < operators.size(); i++) {
    TBOperator const *op = operators[i];
    params.operator_types[i] = op->op_type;
    TBOperatorType const t = op->op_type;
    if (t == TB_INPUT_OP) {
      auto const *in = static_cast<TBInputOp const *>(op);
      MIRAGE_CHECK(params.num_dmem_inputs < NewKernelParams::MAX_NUM_DMEM_INPUTS,
                   "too many device inputs");
      params.dmem_input_ptrs[params.num_dmem_inputs++] =
          fingerprint ? (void *)in->dtensor.fp_ptr : in->dtensor.data_ptr;
      STensor const &tile = op->output_tensors[0];
      DTensor const &dt = in->dtensor;
      int const nd = tile.num_dims, R = nd - 2, C = nd - 1;
      MIRAGE_CHECK(nd == dt.num_dims && nd >= 2, "input tile and tensor ranks differ");
      int const map[3] = {in->input_map.x, in->input_map.y, in->input_map.z};
      int const fd = in->forloop_dim;
      int row_bs[3], col_bs[3], g_bs[3] = {0, 0, 0};
      for (int g = 0; g < 3; g++) {
        // a block's tiles are contiguous: when the for-loop walks the same dim, the
        // block stride spans all of its iterations
        row_bs[g] = (map[g] == R ? tile.dim[R] : 0) * (fd == R ? F : 1);
        col_bs[g] = (map[g] == C ? tile.dim[C] : 0) * (fd == C ? F : 1);
      }
      int strides[MAX_TENSOR_DIMS];
      batch_strides(dt, strides);
      int g_fs = 0;
      if (nd > 2) {
        for (int g = 0; g < 3; g++) {
          if (map[g] >= 0 && map[g] < nd - 2) {
            g_bs[g] = strides[map[g]];
          }
        }
        if (fd >= 0 && fd < nd - 2) {
          g_fs = tile.dim[fd] * strides[fd];
        }
      }
      em.put3(row_bs);
      em.put3(col_bs);
      em.put(fd == R ? tile.dim[R] : 0);
      em.put(fd == C ? tile.dim[C] : 0);
      em.put3(g_bs);
      em.put(g_fs);
      em.put(dt.dim[R]);
      em.put(dt.dim[C]);
      em.put(tile.dim[R]);
      em.put(tile.dim[C]);
      em.put(dt.layout);
      em.put(tile.layout);
      em.put(tile.smem_offset);
    } else if (t == TB_OUTPUT_OP) {
      auto const *out = static_cast<TBOutputOp const *>(op);
      MIRAGE_CHECK(params.num_dmem_outputs < NewKernelParams::MAX_NUM_DMEM_OUTPUTS,
                   "too many device outputs");
      params.dmem_output_ptrs[params.num_dmem_outputs++] =
          fingerprint ? (void *)out->dtensor.fp_ptr : out->dtensor.data_ptr;
      STensor const &src = op->input_tensors[0];
      STensor const &acc = op->output_tensors[0];
      DTensor const &dt = out->dtensor;
      int const nd = src.num_dims, R = nd - 2, C = nd - 1;
      MIRAGE_CHECK(nd == acc.num_dims && nd == dt.num_dims && nd >= 2, "output ranks differ");
      int const map[3] = {out->output_map.x, out->output_map.y, out->output_map.z};
      int row_bs[3], col_bs[3], g_bs[3] = {0, 0, 0};
      for (int g = 0; g < 3; g++) {
        row_bs[g] = map[g] == R ? src.dim[R] : 0;
        col_bs[g] = map[g] == C ? src.dim[C] : 0;
      }
      int strides[MAX_TENSOR_DIMS];
      batch_strides(dt, strides);
      if (nd > 2) {
        for (int g = 0; g < 3; g++) {
          if (map[g] >= 0 && map[g] < nd - 2) {
            g_bs[g] = strides[map[g]];
          }
        }
      }
      em.put3(row_bs);
      em.put3(col_bs);
      em.put3(g_bs);
      em.put(dt.dim[R]);
      em.put(dt.dim[C]);
      em.put(src.dim[R]);
      em.put(src.dim[C]);
      em.put(dt.layout);
      em.put(src.layout);
      em.put(src.smem_offset);
      em.put(acc.smem_offset);
    } else if (t == TB_MATMUL_OP) {
      STensor const &A = op->input_tensors[0], &B = op->input_tensors[1];
      STensor const &C = op->output_tensors[0];
      int const nd = A.num_dims;
      em.put(A.dim[nd - 2]);
      em.put(B.dim[nd - 1]);
      em.put(A.dim[nd - 1]);
      em.put(A.smem_offset);
      em.put(B.smem_offset);
      em.put(C.smem_offset);
    } else if (t == TB_EXP_OP || t == TB_SILU_OP) {
      STensor const &x = op->input_tensors[0];
      MIRAGE_CHECK(x.smem_offset == op->output_tensors[0].smem_offset, "unary must be in place");
      em.put(x.smem_offset);
      em.put((int)x.num_elements());
    } else if (t == TB_ADD_OP || t == TB_MUL_OP || t == TB_DIV_OP) {
      // TB_MUL_OP is serialised like add / div; the reference has no case for it
      int s1[3], s2[3];
      shape3(op->input_tensors[0], s1);
      shape3(op->input_tensors[1], s2);
      em.put3(s1);
      em.put3(s2);
      em.put(op->input_tensors[0].smem_offset);
      em.put(op->input_tensors[1].smem_offset);
      em.put(op->output_tensors[0].smem_offset);
    } else if (t > TB_REDUCTION_FIRST_OP_ID && t <= TB_REDUCTION_2_TO_DIMX_OP) {
      STensor const &x = op->input_tensors[0], &y = op->output_tensors[0];
      int const dim = t >= TB_REDUCTION_0_TO_DIMX_OP ? t - TB_REDUCTION_0_TO_DIMX_OP
                                                     : t - TB_REDUCTION_0_OP;
      int const degree = (int)(x.num_elements() / y.num_elements());
      int inner = 1;
      for (int d = dim; d < y.num_dims; d++) {
        inner *= y.dim[d];
      }
      em.put((int)y.num_elements());
      em.put(degree);
      em.put(inner);
      em.put(x.smem_offset);
      em.put(y.smem_offset);
    } else if (t >= TB_CONCAT_0_OP && t <= TB_CONCAT_2_OP) {
      STensor const &A = op->input_tensors[0], &B = op->input_tensors[1];
      STensor const &y = op->output_tensors[0];
      int const dim = t - TB_CONCAT_0_OP;
      int inner = 1;
      for (int d = dim + 1; d < y.num_dims; d++) {
        inner *= y.dim[d];
      }
      em.put((int)y.num_elements());
      em.put(A.dim[dim]);
      em.put(B.dim[dim]);
      em.put(inner);
      em.put(A.smem_offset);
      em.put(B.smem_offset);
      em.put(y.smem_offset);
    } else {
      MIRAGE_CHECK(false, "thread-block operator cannot be lowered");
    }
  }
  // loaders lead, savers trail: the interpreters rely on it
  for (int i = 0; i < params.num_dmem_inputs; i++) {
    MIRAGE_CHECK(params.operator_types[i] == TB_INPUT_OP, "input loaders must come first");
  }
  for (int i = params.num_operators - params.num_dmem_outputs; i < params.num_operators; i++) {
    MIRAGE_CHECK(params.operator_types[i] == TB_OUTPUT_OP, "output savers must come last");
  }
  return params;
}

}  // namespace threadblock
}  // namespace mirage
