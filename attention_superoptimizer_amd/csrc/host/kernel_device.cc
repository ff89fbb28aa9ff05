// Device half of every kernel-level operator: fingerprint(), profile(), run() and
// DTensor::has_same_fingerprint.  In the reference these live in
// src/kernel/cuda/*.cu and call CUDA / cuBLAS directly; here they bind the C ABI of
// mi355_abi.h and nothing else touches HIP.  fingerprint() enqueues on the backend
// stream without a device-wide sync (the reference syncs after every operator);
// has_same_fingerprint and profile synchronise.
#include "mi355_abi.h"
#include "mirage/kernel/device_memory_manager.h"
#include "mirage/kernel/graph.h"
#include "mirage/layout.h"
#include "mirage/utils/hip_types.h"

#include <cstring>
#include <fstream>
#include <map>
#include <sstream>
#include <string>
#include <vector>

namespace mirage {
namespace kernel {

using namespace mirage::type;

#define MI355_CALL(expr) MIRAGE_CHECK((expr) == MI355_OK, mi355_last_error())

// ---- compare (reference src/kernel/cuda/device_tensor_kernel.cu:22-53) ---------------
bool DTensor::has_same_fingerprint(DTensor const &ref) const {
  if (data_type != ref.data_type || layout != ref.layout || num_dims != ref.num_dims) {
    return false;
  }
  for (int i = 0; i < num_dims; i++) {
    if (dim[i] != ref.dim[i]) {
      return false;
    }
  }
  require_device("has_same_fingerprint");
  int equal = 0;
  MI355_CALL(mi355_fp_equal(fp_ptr, ref.fp_ptr, num_elements(), &equal));
  return equal != 0;
}

// ---- input (reference src/kernel/cuda/input_kernel.cu:40-72) ----------------------------
bool KNInputOp::profile(ProfileResult &profile) {
  require_device("KNInputOp::profile");
  DTensor const &t = output_tensors[0];
  MIRAGE_CHECK(t.data_type == DT_FLOAT16, "only fp16 inputs are supported");
  MI355_CALL(mi355_f16_fill_iota(t.data_ptr, t.num_elements(), t.dim[t.num_dims - 1]));
  MI355_CALL(mi355_sync());
  profile.run_time = 0.0f;
  return true;
}

bool KNInputOp::fingerprint(void) {
  require_device("KNInputOp::fingerprint");
  DTensor const &t = output_tensors[0];
  MI355_CALL(mi355_fp_fill_iota(t.fp_ptr, t.num_elements()));
  return true;
}

// ---- matmul (reference src/kernel/cuda/matmul_kernel.cu:28-203) --------------------------
static void matmul_extents(DTensor const &A, DTensor const &B, int &batch, int &m, int &n,
                           int &k) {
  int const nd = A.num_dims;
  m = A.dim[nd - 2];
  k = A.dim[nd - 1];
  n = B.dim[nd - 1];
  batch = 1;
  for (int i = 0; i < nd - 2; i++) {
    batch *= A.dim[i];
  }
}

// The fp16 data of a DmemColumnMajor tensor holds each matrix column by column.  The GEMM reads
// either order (as the reference's does, matmul_kernel.cu:61-76); the element-wise operators
// and reductions index their inputs flat, so a column-major input is first copied row-major
// into a temporary at the top of the arena (freed again before the call returns: LIFO).
static bool column_major(DTensor const &t) {
  return t.layout == mirage::layout::DmemColumnMajor && t.num_dims >= 2;
}

namespace {
struct RowMajorCopy {
  void *ptr = nullptr;  // what the operator reads
  DTensor temp;
  bool held = false;
  explicit RowMajorCopy(DTensor const &t) : ptr(t.data_ptr) {
    if (!column_major(t)) {
      return;
    }
    temp = t;
    temp.layout = mirage::layout::DmemRowMajor;
    DeviceMemoryManager::get_instance()->allocate(temp, false);
    held = true;
    int batch = 1;
    for (int i = 0; i < t.num_dims - 2; i++) {
      batch *= t.dim[i];
    }
    // the buffer is `batch` matrices of [cols][rows]
    MI355_CALL(mi355_f16_transpose(t.data_ptr, temp.data_ptr, batch, t.dim[t.num_dims - 1],
                                   t.dim[t.num_dims - 2]));
    ptr = temp.data_ptr;
  }
  RowMajorCopy(RowMajorCopy const &) = delete;
  RowMajorCopy &operator=(RowMajorCopy const &) = delete;
  ~RowMajorCopy() {
    if (held) {
      mi355_sync();
      DeviceMemoryManager::get_instance()->free(temp);
    }
  }
};
// The result side of the same: an element-wise operator or reduction hands its output tensor
// the layout of its first input (src/kernel/element_unary.cc:57, element_binary.cc:97,
// reduction.cc:63), so the output of an operator on a column-major tensor is column-major too.
// The kernel writes a row-major temporary; finish() stores it column by column.
struct RowMajorResult {
  void *ptr = nullptr;  // what the operator writes
  DTensor const &out;
  DTensor temp;
  bool held = false;
  explicit RowMajorResult(DTensor const &t) : ptr(t.data_ptr), out(t) {
    if (!column_major(t)) {
      return;
    }
    temp = t;
    temp.layout = mirage::layout::DmemRowMajor;
    DeviceMemoryManager::get_instance()->allocate(temp, false);
    held = true;
    ptr = temp.data_ptr;
  }
  RowMajorResult(RowMajorResult const &) = delete;
  RowMajorResult &operator=(RowMajorResult const &) = delete;
  void finish() {
    if (held) {
      int batch = 1;
      for (int i = 0; i < out.num_dims - 2; i++) {
        batch *= out.dim[i];
      }
      MI355_CALL(mi355_f16_transpose(temp.data_ptr, out.data_ptr, batch, out.dim[out.num_dims - 2],
                                     out.dim[out.num_dims - 1]));
    }
  }
  ~RowMajorResult() {
    if (held) {
      mi355_sync();
      DeviceMemoryManager::get_instance()->free(temp);
    }
  }
};
}  // namespace

// One run of an element-wise operator or reduction on row-major views of its tensors.
template <typename Launch>
static void on_row_major(std::vector<DTensor> const &inputs, DTensor const &output, Launch launch) {
  // (temporaries are freed in reverse order of their allocation: the arena is a stack)
  RowMajorCopy const a(inputs[0]);
  if (inputs.size() > 1) {
    RowMajorCopy const b(inputs[1]);
    RowMajorResult o(output);
    launch(a.ptr, b.ptr, o.ptr);
    o.finish();
  } else {
    RowMajorResult o(output);
    launch(a.ptr, nullptr, o.ptr);
    o.finish();
  }
}

bool KNMatmulOp::profile(ProfileResult &result) {
  require_device("KNMatmulOp::profile");
  int batch, m, n, k;
  matmul_extents(input_tensors[0], input_tensors[1], batch, m, n, k);
  int const iters = 16;
  int const a_cm = column_major(input_tensors[0]) ? 1 : 0, b_cm = column_major(input_tensors[1]) ? 1 : 0;
  MI355_CALL(mi355_f16_matmul_layout(input_tensors[0].data_ptr, input_tensors[1].data_ptr,
                                     output_tensors[0].data_ptr, batch, m, n, k, a_cm, b_cm));
  MI355_CALL(mi355_timer_start());
  for (int i = 0; i < iters; i++) {
    MI355_CALL(mi355_f16_matmul_layout(input_tensors[0].data_ptr, input_tensors[1].data_ptr,
                                       output_tensors[0].data_ptr, batch, m, n, k, a_cm, b_cm));
  }
  float ms = 0.0f;
  MI355_CALL(mi355_timer_stop(&ms));
  result.run_time = ms / iters;
  return true;
}

bool KNMatmulOp::fingerprint(void) {
  require_device("KNMatmulOp::fingerprint");
  int batch, m, n, k;
  matmul_extents(input_tensors[0], input_tensors[1], batch, m, n, k);
  MI355_CALL(mi355_fp_matmul(input_tensors[0].fp_ptr, input_tensors[1].fp_ptr,
                             output_tensors[0].fp_ptr, batch, m, n, k));
  return true;
}

// ---- element-wise unary (reference src/kernel/cuda/element_unary_kernel.cu:44-112) -------
// Element-wise, so flat in either storage order while input and output share a layout (what the
// operator's constructor sets up); a layout search may declare them differently, and then the
// result is stored in the order its tensor declares.
static void run_unary(mirage::type::KNOperatorType type, std::vector<DTensor> const &inputs,
                      DTensor const &output, size_t n) {
  if (column_major(inputs[0]) == column_major(output)) {
    MI355_CALL(mi355_f16_unary(type, inputs[0].data_ptr, output.data_ptr, n));
    return;
  }
  on_row_major(inputs, output,
               [&](void *pa, void *, void *po) { MI355_CALL(mi355_f16_unary(type, pa, po, n)); });
}

bool KNElementUnaryOp::profile(ProfileResult &result) {
  require_device("KNElementUnaryOp::profile");
  size_t const n = input_tensors[0].num_elements();
  int const iters = ProfileResult::NUM_ITERATIONS;
  auto once = [&]() { run_unary(op_type, input_tensors, output_tensors[0], n); };
  once();
  MI355_CALL(mi355_timer_start());
  for (int i = 0; i < iters; i++) {
    once();
  }
  float ms = 0.0f;
  MI355_CALL(mi355_timer_stop(&ms));
  result.run_time = ms / iters;
  return true;
}

bool KNElementUnaryOp::fingerprint(void) {
  require_device("KNElementUnaryOp::fingerprint");
  MI355_CALL(mi355_fp_unary(op_type, input_tensors[0].fp_ptr, output_tensors[0].fp_ptr,
                            input_tensors[0].num_elements()));
  return true;
}

// ---- element-wise binary (reference src/kernel/cuda/element_binary_kernel.cu:53-199) -----
bool KNElementBinaryOp::profile(ProfileResult &result) {
  require_device("KNElementBinaryOp::profile");
  DTensor const &a = input_tensors[0], &b = input_tensors[1], &o = output_tensors[0];
  int const iters = 16;
  float ms = 0.0f;
  on_row_major(input_tensors, o, [&](void *pa, void *pb, void *po) {
    MI355_CALL(mi355_f16_binary(op_type, pa, a.dim, pb, b.dim, po, o.dim, o.num_dims));
    MI355_CALL(mi355_timer_start());
    for (int i = 0; i < iters; i++) {
      MI355_CALL(mi355_f16_binary(op_type, pa, a.dim, pb, b.dim, po, o.dim, o.num_dims));
    }
    MI355_CALL(mi355_timer_stop(&ms));
  });
  result.run_time = ms / iters;
  return true;
}

bool KNElementBinaryOp::fingerprint(void) {
  require_device("KNElementBinaryOp::fingerprint");
  DTensor const &a = input_tensors[0], &b = input_tensors[1], &o = output_tensors[0];
  MI355_CALL(
      mi355_fp_binary(op_type, a.fp_ptr, a.dim, b.fp_ptr, b.dim, o.fp_ptr, o.dim, o.num_dims));
  return true;
}

// ---- reduction (reference src/kernel/cuda/reduction_kernel.cu:45-133) --------------------
static void reduction_strides(DTensor const &in, DTensor const &out, int dim, int &factor,
                              int &in_stride, int &out_stride) {
  out_stride = 1;
  in_stride = 1;
  for (int i = dim; i < out.num_dims; i++) {
    out_stride *= out.dim[i];
    in_stride *= in.dim[i];
  }
  factor = in.dim[dim] / out.dim[dim];
  MIRAGE_CHECK(out_stride * factor == in_stride, "reduction strides disagree");
}

bool KNReductionOp::profile(ProfileResult &result) {
  require_device("KNReductionOp::profile");
  int factor, is, os;
  reduction_strides(input_tensors[0], output_tensors[0], reduction_dim_idx, factor, is, os);
  size_t const n = output_tensors[0].num_elements();
  int const iters = ProfileResult::NUM_ITERATIONS;
  float ms = 0.0f;
  on_row_major(input_tensors, output_tensors[0], [&](void *pi, void *, void *po) {
    MI355_CALL(mi355_f16_reduce(pi, po, n, factor, is, os));
    MI355_CALL(mi355_timer_start());
    for (int i = 0; i < iters; i++) {
      MI355_CALL(mi355_f16_reduce(pi, po, n, factor, is, os));
    }
    MI355_CALL(mi355_timer_stop(&ms));
  });
  result.run_time = ms / iters;
  return true;
}

bool KNReductionOp::fingerprint(void) {
  require_device("KNReductionOp::fingerprint");
  int factor, is, os;
  reduction_strides(input_tensors[0], output_tensors[0], reduction_dim_idx, factor, is, os);
  MI355_CALL(mi355_fp_reduce(input_tensors[0].fp_ptr, output_tensors[0].fp_ptr,
                             output_tensors[0].num_elements(), factor, is, os));
  return true;
}

// ---- customized (reference src/kernel/cuda/customized_kernel.cu:605-678) -----------------
struct LoweredOp {
  mi355_plan plan;
  void const *inputs[MI355_MAX_DMEM_INPUTS];
  void *outputs[MI355_MAX_DMEM_OUTPUTS];
};

static LoweredOp lower(KNCustomizedOp const &op, bool fingerprint) {
  mirage::threadblock::NewKernelParams p = op.bgraph.get_new_kernel_params(fingerprint);
  LoweredOp l;
  std::memset(&l, 0, sizeof(l));
  l.plan.grid_dim[0] = op.bgraph.grid_dim.x;
  l.plan.grid_dim[1] = op.bgraph.grid_dim.y;
  l.plan.grid_dim[2] = op.bgraph.grid_dim.z;
  l.plan.block_dim[0] = op.bgraph.block_dim.x;
  l.plan.block_dim[1] = op.bgraph.block_dim.y;
  l.plan.block_dim[2] = op.bgraph.block_dim.z;
  l.plan.forloop_range = op.bgraph.forloop_range;
  l.plan.reduction_dimx = op.bgraph.reduction_dimx;
  l.plan.smem_bytes = (int)op.bgraph.smem_offset;
  l.plan.num_operators = p.num_operators;
  l.plan.num_parameters = p.num_parameters;
  l.plan.num_dmem_inputs = p.num_dmem_inputs;
  l.plan.num_dmem_outputs = p.num_dmem_outputs;
  for (int i = 0; i < p.num_operators; i++) {
    l.plan.operator_types[i] = p.operator_types[i];
  }
  std::memcpy(l.plan.parameters, p.parameters, sizeof(int) * p.num_parameters);
  for (int i = 0; i < p.num_dmem_inputs; i++) {
    l.inputs[i] = p.dmem_input_ptrs[i];
  }
  for (int i = 0; i < p.num_dmem_outputs; i++) {
    l.outputs[i] = p.dmem_output_ptrs[i];
  }
  // every tile the program touches must lie inside its device tensor
  long long in_ext[MI355_MAX_DMEM_INPUTS], out_ext[MI355_MAX_DMEM_OUTPUTS];
  MI355_CALL(mi355_plan_extents(&l.plan, in_ext, out_ext, nullptr, nullptr));
  int ii = 0, oo = 0;
  for (mirage::threadblock::TBOperator *t : op.bgraph.operators) {
    if (t->op_type == TB_INPUT_OP) {
      auto *in = static_cast<mirage::threadblock::TBInputOp *>(t);
      MIRAGE_CHECK(in_ext[ii] <= (long long)in->dtensor.num_elements(),
                   "input loader would read past its tensor");
      ii++;
    } else if (t->op_type == TB_OUTPUT_OP) {
      auto *out = static_cast<mirage::threadblock::TBOutputOp *>(t);
      MIRAGE_CHECK(out_ext[oo] <= (long long)out->dtensor.num_elements(),
                   "output saver would write past its tensor");
      oo++;
    }
  }
  return l;
}

// for batched submission (verify.cc): the lowered program and its bound pointers
void lower_customized(KNCustomizedOp const &op, bool fingerprint, mi355_plan *plan,
                      void const **inputs, void **outputs) {
  LoweredOp l = lower(op, fingerprint);
  *plan = l.plan;
  std::memcpy(inputs, l.inputs, sizeof(l.inputs));
  std::memcpy(outputs, l.outputs, sizeof(l.outputs));
}

void KNCustomizedOp::run() {
  require_device("KNCustomizedOp::run");
  LoweredOp l = lower(*this, false);
  MI355_CALL(mi355_customized_run(&l.plan, l.inputs, l.outputs));
}

bool KNCustomizedOp::profile(ProfileResult &result) {
  require_device("KNCustomizedOp::profile");
  LoweredOp l = lower(*this, false);
  float ms = 0.0f;
  int const rc = mi355_customized_profile(&l.plan, l.inputs, l.outputs, 0, ProfileResult::NUM_WARPUP_ITERATIONS,
                                          ProfileResult::NUM_ITERATIONS, &ms);
  if (rc == MI355_ERR_UNSUPPORTED) {
    // no kernel of this backend runs the program as declared (say, tiles that only a fused
    // kernel keeps out of LDS, under layouts the fused kernels do not take): not a candidate
    result = ProfileResult::infinity();
    return false;
  }
  MIRAGE_CHECK(rc == MI355_OK, mi355_last_error());
  result.run_time = ms;
  return true;
}

bool KNCustomizedOp::fingerprint(void) {
  require_device("KNCustomizedOp::fingerprint");
  LoweredOp l = lower(*this, true);
  MI355_CALL(mi355_customized_fp(&l.plan, l.inputs, l.outputs));
  return true;
}

}  // namespace kernel
}  // namespace mirage

// ---- source emission (reference src/kernel/triton_code_gen.cc:354-450) ---------------------
namespace mirage {
namespace kernel {

void Graph::generate_hip_program(char const *file_path) {
  std::ofstream file(file_path);
  MIRAGE_CHECK(file.good(), "generate_hip_program: cannot open the output file");
  file << mi355_emit_hip_preamble();
  // device tensors are numbered in creation order: every operator's outputs
  std::map<int, int> index_of;  // guid -> number
  std::vector<long long> elements;
  std::vector<bool> is_input;
  for (KNOperator *op : operators) {
    for (DTensor const &t : op->output_tensors) {
      index_of[t.guid] = (int)elements.size();
      elements.push_back((long long)t.num_elements());
      is_input.push_back(op->op_type == mirage::type::KN_INPUT_OP);
    }
  }
  std::stringstream launcher;
  launcher << "// Launches every customized operator of the graph in order.  dtensors[i] is device\n"
              "// tensor i in creation order (see graphdef_tensor_elements).\n"
              "GRAPHDEF_API int graphdef_launch(void *const *dtensors, hipStream_t stream) {\n";
  int kernels = 0;
  for (KNOperator *op : operators) {
    if (op->op_type != mirage::type::KN_CUSTOMIZED_OP) {
      continue;  // as the reference: only customized operators are emitted
    }
    LoweredOp l = lower(*static_cast<KNCustomizedOp *>(op), false);
    std::string const name = "graphdef_kernel_" + std::to_string(kernels++);
    long long const n = mi355_emit_hip_kernel(&l.plan, name.c_str(), 0, nullptr, 0);
    MIRAGE_CHECK(n >= 0, mi355_last_error());
    std::vector<char> text((size_t)n + 1);
    MIRAGE_CHECK(mi355_emit_hip_kernel(&l.plan, name.c_str(), 0, text.data(), n + 1) == n,
                 "generate_hip_program: emission changed size");
    file << text.data();
    launcher << "  {\n    void const *in[] = {";
    for (size_t i = 0; i < op->input_tensors.size(); i++) {
      launcher << (i ? ", " : "") << "dtensors[" << index_of.at(op->input_tensors[i].guid) << "]";
    }
    launcher << "};\n    void *out[] = {";
    for (size_t i = 0; i < op->output_tensors.size(); i++) {
      launcher << (i ? ", " : "") << "dtensors[" << index_of.at(op->output_tensors[i].guid) << "]";
    }
    launcher << "};\n    if (int rc = " << name << "_launch(in, out, stream)) {\n      return rc;\n    }\n  }\n";
  }
  launcher << "  return 0;\n}\n\n";
  file << "static long long const kTensorElements[] = {";
  for (size_t i = 0; i < elements.size(); i++) {
    file << (i ? ", " : "") << elements[i];
  }
  file << "};\nstatic int const kTensorIsInput[] = {";
  for (size_t i = 0; i < elements.size(); i++) {
    file << (i ? ", " : "") << (is_input[i] ? 1 : 0);
  }
  file << "};\n"
          "GRAPHDEF_API int graphdef_num_tensors(void) { return " << elements.size() << "; }\n"
          "GRAPHDEF_API long long graphdef_tensor_elements(int i) { return kTensorElements[i]; }\n"
          "GRAPHDEF_API int graphdef_sync(void) { return (int)hipDeviceSynchronize(); }\n\n";
  file << launcher.str();
  // the profiling main: random fp16 tensors, 1000 warm-up launches, 1000 timed
  file << R"HIP(#ifndef GRAPHDEF_NO_MAIN
static uint64_t mix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

int main() {
  int const n = graphdef_num_tensors();
  std::vector<void *> dtensors(n);
  for (int t = 0; t < n; t++) {
    long long const e = kTensorElements[t];
    GRAPHDEF_HIP(hipMalloc(&dtensors[t], (size_t)e * 2));
    std::vector<_Float16> host((size_t)e);
    for (long long i = 0; i < e; i++) {
      // N(0, 1) / 8 by Box-Muller on two 24-bit uniforms
      uint64_t const r = mix64(((uint64_t)t << 40) ^ (uint64_t)i);
      float const u1 = ((r >> 40) + 1) * (1.0f / 16777216.0f), u2 = ((r >> 16) & 0xffffff) * (1.0f / 16777216.0f);
      host[(size_t)i] = (_Float16)(0.125f * __builtin_sqrtf(-2.0f * __builtin_logf(u1)) * __builtin_cosf(6.2831853f * u2));
    }
    GRAPHDEF_HIP(hipMemcpy(dtensors[t], host.data(), (size_t)e * 2, hipMemcpyHostToDevice));
  }
  hipStream_t stream;
  GRAPHDEF_HIP(hipStreamCreate(&stream));
  hipEvent_t e0, e1;
  GRAPHDEF_HIP(hipEventCreate(&e0));
  GRAPHDEF_HIP(hipEventCreate(&e1));
  for (int i = 0; i < 1000; i++) {
    if (graphdef_launch(dtensors.data(), stream)) {
      return 1;
    }
  }
  GRAPHDEF_HIP(hipEventRecord(e0, stream));
  for (int i = 0; i < 1000; i++) {
    if (graphdef_launch(dtensors.data(), stream)) {
      return 1;
    }
  }
  GRAPHDEF_HIP(hipEventRecord(e1, stream));
  GRAPHDEF_HIP(hipEventSynchronize(e1));
  float ms = 0.0f;
  GRAPHDEF_HIP(hipEventElapsedTime(&ms, e0, e1));
  printf("%.6f ms per launch of the whole graph (mean of 1000)\n", ms / 1000.0f);
  for (void *p : dtensors) {
    GRAPHDEF_HIP(hipFree(p));
  }
  return 0;
}
#endif
)HIP";
  file.close();
}

}  // namespace kernel
}  // namespace mirage

// ---- one fp16 execution of any operator (extension: the reference only offers
// profile(), which runs an operator hundreds of times) -----------------------------------
namespace mirage {
namespace kernel {

void execute_once(KNOperator *op) {
  require_device("execute_once");
  using namespace mirage::type;
  switch (op->op_type) {
    case KN_INPUT_OP:
      break;  // inputs hold whatever the caller wrote
    case KN_MATMUL_OP: {
      int batch, m, n, k;
      matmul_extents(op->input_tensors[0], op->input_tensors[1], batch, m, n, k);
      MI355_CALL(mi355_f16_matmul_layout(op->input_tensors[0].data_ptr, op->input_tensors[1].data_ptr,
                                         op->output_tensors[0].data_ptr, batch, m, n, k,
                                         column_major(op->input_tensors[0]) ? 1 : 0,
                                         column_major(op->input_tensors[1]) ? 1 : 0));
      break;
    }
    case KN_EXP_OP:
    case KN_SILU_OP:
      run_unary(op->op_type, op->input_tensors, op->output_tensors[0], op->input_tensors[0].num_elements());
      break;
    case KN_ADD_OP:
    case KN_MUL_OP:
    case KN_DIV_OP: {
      DTensor const &a = op->input_tensors[0], &b = op->input_tensors[1],
                    &o = op->output_tensors[0];
      on_row_major(op->input_tensors, o, [&](void *pa, void *pb, void *po) {
        MI355_CALL(mi355_f16_binary(op->op_type, pa, a.dim, pb, b.dim, po, o.dim, o.num_dims));
      });
      break;
    }
    case KN_REDUCTION_0_OP:
    case KN_REDUCTION_1_OP:
    case KN_REDUCTION_2_OP: {
      auto *r = static_cast<KNReductionOp *>(op);
      int factor, is, os;
      reduction_strides(op->input_tensors[0], op->output_tensors[0], r->reduction_dim_idx,
                        factor, is, os);
      on_row_major(op->input_tensors, op->output_tensors[0], [&](void *pi, void *, void *po) {
        MI355_CALL(mi355_f16_reduce(pi, po, op->output_tensors[0].num_elements(), factor, is, os));
      });
      break;
    }
    case KN_CUSTOMIZED_OP:
      static_cast<KNCustomizedOp *>(op)->run();
      break;
    default:
      MIRAGE_CHECK(false, "operator cannot be executed");
  }
}

}  // namespace kernel
}  // namespace mirage
