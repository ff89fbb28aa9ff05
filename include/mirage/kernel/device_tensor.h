// DTensor: a value-type handle of a tensor in device memory — shape, declared
// layout, producer, and the two arena buffers every tensor owns (fp16 data and
// uint16 fingerprint).  Field-for-field the reference's struct
// (include/mirage/kernel/device_tensor.h:31-124) so plans and callers carry over.
#pragma once

#include "mirage/layout.h"
#include "mirage/type.h"
#include <cstddef>
#include <functional>

namespace mirage {
namespace kernel {

#define MAX_TENSOR_DIMS 4

class KNOperator;

struct alignas(16) DTensor {
  DTensor(void);
  // Same tensor: equal metadata and the same producer slot.
  bool operator==(DTensor const &b) const;
  bool operator!=(DTensor const &b) const { return !(*this == b); }

  size_t num_elements() const {
    size_t n = 1;
    for (int i = 0; i < num_dims; i++) {
      n *= dim[i];
    }
    return n;
  }
  size_t data_size() const { return num_elements() * mirage::type::get_datatype_size(data_type); }
  size_t fingerprint_size() const { return num_elements() * sizeof(mirage::type::FPType); }

  // Element-wise equality of the two fingerprint buffers, decided on the device
  // (the reference copies both tensors to the host,
  // src/kernel/cuda/device_tensor_kernel.cu:22-53).  Requires equal dtype,
  // layout and dims, as there.
  bool has_same_fingerprint(DTensor const &ref) const;

  mirage::type::DataType data_type;
  mirage::layout::DmemLayout layout;
  int num_dims;
  int dim[MAX_TENSOR_DIMS];
  size_t guid;
  KNOperator *owner_op;
  int owner_ts_idx;
  void *data_ptr;                // fp16 payload
  mirage::type::FPType *fp_ptr;  // uint16 fingerprint

  static int next_guid;
};

}  // namespace kernel
}  // namespace mirage

namespace std {
template <>
struct hash<mirage::kernel::DTensor> {
  size_t operator()(mirage::kernel::DTensor const &) const;
};
}  // namespace std
