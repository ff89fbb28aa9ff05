// STensor: a tile of a thread-block graph.  `smem_offset` is the tile's address
// in the graph's STensor address space (a bump allocation, 16-byte granules,
// 2 bytes per element); it identifies the tile in the lowered program.  The
// backend decides where — LDS or registers — the tile really lives.
// Fields as in the reference's include/mirage/threadblock/smem_tensor.h:32-167.
#pragma once

#include "mirage/layout.h"
#include "mirage/type.h"
#include <cstddef>
#include <functional>

namespace mirage {
namespace threadblock {

#ifndef MAX_TENSOR_DIMS
#define MAX_TENSOR_DIMS 4
#endif

class TBOperator;

struct alignas(16) STensor {
  STensor(void);
  bool operator==(STensor const &b) const;
  bool operator!=(STensor const &b) const { return !(*this == b); }
  size_t size() const;  // bytes
  size_t num_elements() const;

  mirage::type::DataType data_type;
  mirage::layout::SmemLayout layout;
  int num_dims;
  int dim[MAX_TENSOR_DIMS];
  int guid;
  TBOperator *owner_op;
  int owner_ts_idx;
  int smem_offset;

  static int next_guid;
};

}  // namespace threadblock
}  // namespace mirage

namespace std {
template <>
struct hash<mirage::threadblock::STensor> {
  size_t operator()(mirage::threadblock::STensor const &) const;
};
}  // namespace std
