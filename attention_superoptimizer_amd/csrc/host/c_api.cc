// C facade over the mirage:: host API, for bindings that cannot speak C++ (the
// package's ctypes layer; the reference binds the same classes through Cython,
// python/mirage/_cython/CCore.pxd:52-84).  Tensor handles are DTensor* into the
// owning operator's output list and stay valid until that operator is deleted.
// Graph-building calls return NULL / -1 for an infeasible operator instead of
// aborting (they go through the create_* functions).
#include "mi355_abi.h"
#include "mirage/kernel/device_memory_manager.h"
#include "mirage/kernel/graph.h"
#include "mirage/utils/hip_types.h"

#include <cstring>

using namespace mirage;
using kernel::DTensor;
using kernel::KNOperator;

namespace mirage {
namespace kernel {
void execute_once(KNOperator *op);
}
}  // namespace mirage

extern "C" {

typedef struct mirage_c_plan {
  int grid_dim[3];
  int block_dim[3];
  int forloop_range;
  int reduction_dimx;
  int num_inputs;
  int input_map[4][3];
  int forloop_dim[4];
  int input_smem_layout[4];
  int output_map[3];
  int num_ops;
  int op_type[16];
  int op_num_operands[16];
  int op_operands[16][2][2];
} mirage_c_plan;

void *mirage_graph_create(void) { return new kernel::Graph(); }

void mirage_graph_destroy(void *g) { delete static_cast<kernel::Graph *>(g); }

int mirage_graph_num_operators(void *g) {
  return (int)static_cast<kernel::Graph *>(g)->operators.size();
}

static void *push(kernel::Graph *g, KNOperator *op) {
  if (op == nullptr) {
    return nullptr;
  }
  g->operators.push_back(op);
  return &op->output_tensors[0];
}

void *mirage_graph_new_input(void *g, int const *dims, int nd, int dtype, int layout) {
  auto *G = static_cast<kernel::Graph *>(g);
  std::vector<int> d(dims, dims + nd);
  return push(G, G->create_input_op(d, (type::DataType)dtype, (layout::DmemLayout)layout));
}

void *mirage_graph_matmul(void *g, void *a, void *b) {
  auto *G = static_cast<kernel::Graph *>(g);
  return push(G, G->create_matmul_op(*static_cast<DTensor *>(a), *static_cast<DTensor *>(b)));
}

void *mirage_graph_unary(void *g, int op, void *a) {
  auto *G = static_cast<kernel::Graph *>(g);
  return push(G, G->create_elementunary_op(*static_cast<DTensor *>(a), (type::KNOperatorType)op));
}

void *mirage_graph_binary(void *g, int op, void *a, void *b) {
  auto *G = static_cast<kernel::Graph *>(g);
  return push(G, G->create_elementbinary_op(*static_cast<DTensor *>(a), *static_cast<DTensor *>(b),
                                            (type::KNOperatorType)op));
}

void *mirage_graph_reduction(void *g, void *a, int dim, int size) {
  auto *G = static_cast<kernel::Graph *>(g);
  return push(G, G->create_reduction_op(*static_cast<DTensor *>(a), dim, size));
}

int mirage_graph_customized(void *g, void *const *inputs, int num_inputs, mirage_c_plan const *p,
                            void **outputs, int max_outputs) {
  auto *G = static_cast<kernel::Graph *>(g);
  if (p == nullptr || num_inputs != p->num_inputs || num_inputs > 4 || p->num_ops > 16) {
    return -1;
  }
  threadblock::ExecutionPlan plan;
  plan.grid_dim = dim3(p->grid_dim[0], p->grid_dim[1], p->grid_dim[2]);
  plan.block_dim = dim3(p->block_dim[0], p->block_dim[1], p->block_dim[2]);
  plan.forloop_range = p->forloop_range;
  plan.reduction_dimx = p->reduction_dimx;
  plan.output_map = {p->output_map[0], p->output_map[1], p->output_map[2]};
  std::vector<DTensor> ins;
  for (int i = 0; i < num_inputs; i++) {
    ins.push_back(*static_cast<DTensor *>(inputs[i]));
    plan.input_map.push_back({p->input_map[i][0], p->input_map[i][1], p->input_map[i][2]});
    plan.forloop_dim.push_back(p->forloop_dim[i]);
    plan.input_smem_layouts.push_back((layout::SmemLayout)p->input_smem_layout[i]);
  }
  for (int i = 0; i < p->num_ops; i++) {
    std::vector<std::pair<int, int>> operands;
    for (int j = 0; j < p->op_num_operands[i]; j++) {
      operands.push_back({p->op_operands[i][j][0], p->op_operands[i][j][1]});
    }
    plan.ops.push_back({(type::TBOperatorType)p->op_type[i], operands});
  }
  KNOperator *op = G->create_customized_op(ins, plan);
  if (op == nullptr) {
    return -1;
  }
  G->operators.push_back(op);
  int n = (int)op->output_tensors.size();
  for (int i = 0; i < n && i < max_outputs; i++) {
    outputs[i] = &op->output_tensors[i];
  }
  return n;
}

// deletes the newest operator (the arena is LIFO)
int mirage_graph_pop_operator(void *g) {
  auto *G = static_cast<kernel::Graph *>(g);
  if (G->operators.empty()) {
    return -1;
  }
  delete G->operators.back();
  G->operators.pop_back();
  return 0;
}

int mirage_op_type(void *g, int idx) {
  return static_cast<kernel::Graph *>(g)->operators.at(idx)->op_type;
}

int mirage_op_num_outputs(void *g, int idx) {
  return (int)static_cast<kernel::Graph *>(g)->operators.at(idx)->output_tensors.size();
}

void *mirage_op_output(void *g, int idx, int ts) {
  return &static_cast<kernel::Graph *>(g)->operators.at(idx)->output_tensors.at(ts);
}

int mirage_op_fingerprint(void *g, int idx) {
  return static_cast<kernel::Graph *>(g)->operators.at(idx)->fingerprint() ? 0 : -1;
}

// mean milliseconds per launch, by the reference's profile() protocol
float mirage_op_profile(void *g, int idx) {
  ProfileResult r;
  static_cast<kernel::Graph *>(g)->operators.at(idx)->profile(r);
  return r.run_time;
}

int mirage_op_execute(void *g, int idx) {
  kernel::execute_once(static_cast<kernel::Graph *>(g)->operators.at(idx));
  return 0;
}

// the lowered program of a customized op, as handed to the backend
int mirage_op_lowered(void *g, int idx, int fingerprint, mi355_plan *out, int *smem_offset) {
  KNOperator *op = static_cast<kernel::Graph *>(g)->operators.at(idx);
  if (op->op_type != type::KN_CUSTOMIZED_OP || out == nullptr) {
    return -1;
  }
  auto *c = static_cast<kernel::KNCustomizedOp *>(op);
  threadblock::NewKernelParams p = c->bgraph.get_new_kernel_params(fingerprint != 0);
  std::memset(out, 0, sizeof(*out));
  out->grid_dim[0] = c->bgraph.grid_dim.x;
  out->grid_dim[1] = c->bgraph.grid_dim.y;
  out->grid_dim[2] = c->bgraph.grid_dim.z;
  out->block_dim[0] = c->bgraph.block_dim.x;
  out->block_dim[1] = c->bgraph.block_dim.y;
  out->block_dim[2] = c->bgraph.block_dim.z;
  out->forloop_range = c->bgraph.forloop_range;
  out->reduction_dimx = c->bgraph.reduction_dimx;
  out->smem_bytes = (int)c->bgraph.smem_offset;
  out->num_operators = p.num_operators;
  out->num_parameters = p.num_parameters;
  out->num_dmem_inputs = p.num_dmem_inputs;
  out->num_dmem_outputs = p.num_dmem_outputs;
  for (int i = 0; i < p.num_operators; i++) {
    out->operator_types[i] = p.operator_types[i];
  }
  std::memcpy(out->parameters, p.parameters, sizeof(int) * p.num_parameters);
  if (smem_offset != nullptr) {
    *smem_offset = (int)c->bgraph.smem_offset;
  }
  return 0;
}

int mirage_tensor_info(void *t, int *num_dims, int *dims, int *dtype, int *layout,
                       long long *guid) {
  auto *T = static_cast<DTensor *>(t);
  *num_dims = T->num_dims;
  for (int i = 0; i < T->num_dims; i++) {
    dims[i] = T->dim[i];
  }
  *dtype = T->data_type;
  *layout = T->layout;
  *guid = (long long)T->guid;
  return 0;
}

void *mirage_tensor_ptr(void *t, int fingerprint) {
  auto *T = static_cast<DTensor *>(t);
  return fingerprint ? (void *)T->fp_ptr : T->data_ptr;
}

int mirage_tensor_write(void *t, int fingerprint, void const *host, size_t bytes) {
  auto *T = static_cast<DTensor *>(t);
  size_t want = fingerprint ? T->fingerprint_size() : T->data_size();
  if (bytes != want) {
    return -1;
  }
  kernel::require_device("tensor write");
  return mi355_memcpy_h2d(fingerprint ? (void *)T->fp_ptr : T->data_ptr, host, bytes);
}

int mirage_tensor_read(void *t, int fingerprint, void *host, size_t bytes) {
  auto *T = static_cast<DTensor *>(t);
  size_t want = fingerprint ? T->fingerprint_size() : T->data_size();
  if (bytes != want) {
    return -1;
  }
  kernel::require_device("tensor read");
  return mi355_memcpy_d2h(host, fingerprint ? (void const *)T->fp_ptr : T->data_ptr, bytes);
}

int mirage_tensor_same_fingerprint(void *a, void *b) {
  return static_cast<DTensor *>(a)->has_same_fingerprint(*static_cast<DTensor *>(b)) ? 1 : 0;
}

// Graph::generate_hip_program
int mirage_graph_generate_hip_program(void *g, char const *path) {
  static_cast<kernel::Graph *>(g)->generate_hip_program(path);
  return 0;
}

void mirage_set_smem_budget(size_t bytes) { threadblock::Graph::set_smem_budget(bytes); }
size_t mirage_get_smem_budget(void) { return threadblock::Graph::smem_budget(); }

int mirage_device_ready(void) {
  return kernel::DeviceMemoryManager::get_instance()->device_ready ? 1 : 0;
}
long long mirage_arena_offset(void) {
  return (long long)kernel::DeviceMemoryManager::get_instance()->offset;
}
long long mirage_arena_total(void) {
  return (long long)kernel::DeviceMemoryManager::get_instance()->total_size;
}

}  // extern "C"
