// Small value types of the host runtime: dtype sizes, enum names, DTensor / STensor
// construction, equality and hashing.
#include "mirage/kernel/device_tensor.h"
#include "mirage/layout.h"
#include "mirage/profile_result.h"
#include "mirage/threadblock/smem_tensor.h"
#include "mirage/type.h"
#include "mirage/utils/hip_types.h"

#include <limits>

namespace mirage {

// reference src/profile_result.cc:7-9: "infinity" is a finite sentinel (1000 ms), so a
// checkpoint whose best profile was never set still serialises as a number
ProfileResult ProfileResult::infinity() {
  ProfileResult r;
  r.run_time = 1000.0f;
  return r;
}

namespace type {

// reference src/base/data_type.cc:21-36
size_t get_datatype_size(DataType type) {
  switch (type) {
    case DT_INT8:
      return 1;
    case DT_UINT16:
    case DT_BFLOAT16:
    case DT_FLOAT16:
      return 2;
    case DT_FLOAT32:
      return 4;
    case DT_DOUBLE:
      return 8;
    default:
      MIRAGE_CHECK(false, "unknown data type");
  }
  return 0;
}

char const *to_string(KNOperatorType t) {
  switch (t) {
    case KN_INPUT_OP: return "kn_input_op";
    case KN_MATMUL_OP: return "kn_matmul_op";
    case KN_REDUCTION_0_OP: return "kn_reduction_0_op";
    case KN_REDUCTION_1_OP: return "kn_reduction_1_op";
    case KN_REDUCTION_2_OP: return "kn_reduction_2_op";
    case KN_EXP_OP: return "kn_exp_op";
    case KN_ADD_OP: return "kn_add_op";
    case KN_MUL_OP: return "kn_mul_op";
    case KN_DIV_OP: return "kn_div_op";
    case KN_SILU_OP: return "kn_silu_op";
    case KN_CUSTOMIZED_OP: return "kn_customized_op";
    default: return "kn_unkown";
  }
}

char const *to_string(TBOperatorType t) {
  switch (t) {
    case TB_INPUT_OP: return "tb_input_op";
    case TB_OUTPUT_OP: return "tb_output_op";
    case TB_MATMUL_OP: return "tb_matmul_op";
    case TB_EXP_OP: return "tb_exp_op";
    case TB_ADD_OP: return "tb_add_op";
    case TB_MUL_OP: return "tb_mul_op";
    case TB_DIV_OP: return "tb_div_op";
    case TB_SILU_OP: return "tb_silu_op";
    case TB_REDUCTION_0_OP: return "tb_reduction_0_op";
    case TB_REDUCTION_1_OP: return "tb_reduction_1_op";
    case TB_REDUCTION_2_OP: return "tb_reduction_2_op";
    case TB_REDUCTION_0_TO_DIMX_OP: return "tb_reduction_0_to_dimx_op";
    case TB_REDUCTION_1_TO_DIMX_OP: return "tb_reduction_1_to_dimx_op";
    case TB_REDUCTION_2_TO_DIMX_OP: return "tb_reduction_2_to_dimx_op";
    case TB_CONCAT_0_OP: return "tb_concat_0_op";
    case TB_CONCAT_1_OP: return "tb_concat_1_op";
    case TB_CONCAT_2_OP: return "tb_concat_2_op";
    case TB_CUSTOMIZED_OP: return "tb_customized_op";
    default: return "tb_unkown";
  }
}

}  // namespace type

namespace layout {

char const *to_string(DmemLayout l) {
  switch (l) {
    case DmemRowMajor: return "DmemRowMajor";
    case DmemColumnMajor: return "DmemColumnMajor";
    default: return "DmemUnknownLayout";
  }
}

char const *to_string(SmemLayout l) {
  switch (l) {
    case SmemRowMajor: return "SmemRowMajor";
    case SmemColumnMajor: return "SmemColumnMajor";
    case SmemRowMajorTensorOpMultiplicand_Crosswise16: return "SmemRowMajorTensorOpMultiplicand_Crosswise16";
    case SmemRowMajorTensorOpMultiplicand_Crosswise32: return "SmemRowMajorTensorOpMultiplicand_Crosswise32";
    case SmemRowMajorTensorOpMultiplicand_Crosswise64: return "SmemRowMajorTensorOpMultiplicand_Crosswise64";
    case SmemColumnMajorTensorOpMultiplicand_Crosswise16: return "SmemColumnMajorTensorOpMultiplicand_Crosswise16";
    case SmemColumnMajorTensorOpMultiplicand_Crosswise32: return "SmemColumnMajorTensorOpMultiplicand_Crosswise32";
    case SmemColumnMajorTensorOpMultiplicand_Crosswise64: return "SmemColumnMajorTensorOpMultiplicand_Crosswise64";
    default: return "SmemUnknownLayout";
  }
}

}  // namespace layout

namespace kernel {

int DTensor::next_guid = 20000;  // reference src/kernel/device_tensor.cc:49

DTensor::DTensor()
    : data_type(mirage::type::DT_UNKNOWN), layout(mirage::layout::DmemUnknownLayout), num_dims(0),
      guid(0), owner_op(nullptr), owner_ts_idx(-1000), data_ptr(nullptr), fp_ptr(nullptr) {
  for (int i = 0; i < MAX_TENSOR_DIMS; i++) {
    dim[i] = 0;
  }
}

bool DTensor::operator==(DTensor const &b) const {
  if (data_type != b.data_type || layout != b.layout || num_dims != b.num_dims) {
    return false;
  }
  for (int i = 0; i < num_dims; i++) {
    if (dim[i] != b.dim[i]) {
      return false;
    }
  }
  return owner_op == b.owner_op && owner_ts_idx == b.owner_ts_idx;
}

}  // namespace kernel

namespace threadblock {

int STensor::next_guid = 10000;  // reference src/threadblock/smem_tensor.cc:22

STensor::STensor()
    : data_type(mirage::type::DT_UNKNOWN), layout(mirage::layout::SmemUnknownLayout), num_dims(0),
      guid(0), owner_op(nullptr), owner_ts_idx(-1000), smem_offset(128) {
  for (int i = 0; i < MAX_TENSOR_DIMS; i++) {
    dim[i] = 0;
  }
}

bool STensor::operator==(STensor const &b) const {
  if (data_type != b.data_type || layout != b.layout || num_dims != b.num_dims) {
    return false;
  }
  for (int i = 0; i < num_dims; i++) {
    if (dim[i] != b.dim[i]) {
      return false;
    }
  }
  return owner_op == b.owner_op && owner_ts_idx == b.owner_ts_idx && smem_offset == b.smem_offset;
}

size_t STensor::num_elements() const {
  size_t n = 1;
  for (int i = 0; i < num_dims; i++) {
    n *= dim[i];
  }
  return n;
}

size_t STensor::size() const {
  MIRAGE_CHECK(data_type != mirage::type::DT_UNKNOWN, "tile without a data type");
  return num_elements() * mirage::type::get_datatype_size(data_type);
}

}  // namespace threadblock
}  // namespace mirage

namespace {
inline void mix(size_t &seed, size_t v) { seed ^= v + 0x9e3779b9 + (seed << 6) + (seed >> 2); }
}  // namespace

namespace std {

size_t hash<mirage::kernel::DTensor>::operator()(mirage::kernel::DTensor const &t) const {
  size_t h = std::hash<int>()(t.data_type);
  mix(h, t.layout);
  mix(h, t.num_dims);
  for (int i = 0; i < t.num_dims; i++) {
    mix(h, t.dim[i]);
  }
  mix(h, reinterpret_cast<size_t>(t.owner_op));
  mix(h, t.owner_ts_idx);
  mix(h, reinterpret_cast<size_t>(t.data_ptr));
  return h;
}

size_t hash<mirage::threadblock::STensor>::operator()(mirage::threadblock::STensor const &t) const {
  size_t h = std::hash<int>()(t.data_type);
  mix(h, t.layout);
  mix(h, t.num_dims);
  for (int i = 0; i < t.num_dims; i++) {
    mix(h, t.dim[i]);
  }
  mix(h, reinterpret_cast<size_t>(t.owner_op));
  mix(h, t.owner_ts_idx);
  mix(h, t.smem_offset);
  return h;
}

}  // namespace std
