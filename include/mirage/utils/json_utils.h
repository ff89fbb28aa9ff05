// A small JSON value type and the wire format of mugraphs.
//
// The reference serialises graphs with nlohmann::json (include/mirage/utils/json_utils.h,
// NLOHMANN_DEFINE_TYPE_NON_INTRUSIVE on DTensor / STensor / ExecutionPlan, `operator
// json()` on every operator, to_json / from_json on kernel::Graph,
// src/kernel/graph.cc:33-159).  That library is a dependency this backend does not
// have; `json` below covers what the wire format needs — parse, dump (object keys in
// sorted order, as nlohmann's default std::map object gives), building and reading
// objects, arrays, integers, strings, booleans and null — and the functions keep the
// reference's names and schema, so checkpoints written by the reference load here and
// what is written here loads there.
#pragma once

#include "mirage/kernel/graph.h"
#include "mirage/utils/json_value.h"

// ---- the wire format (reference schema) ----------------------------------------------
// int3 / dim3 as {"x","y","z"} (src/utils/json_utils.cc:3-25)
void to_json(json &j, int3 const &v);
void from_json(json const &j, int3 &v);
void to_json(json &j, dim3 const &v);
void from_json(json const &j, dim3 &v);

namespace mirage {
namespace kernel {
// {data_type, layout, num_dims, dim[4], guid} (device_tensor.h:126-127)
void to_json(json &j, DTensor const &t);
void from_json(json const &j, DTensor &t);
// the operator's entry of a graph: op_type (by name, type.h:64-78), input_tensors,
// output_tensors, and for a customized op bgraph + plan (src/kernel/customized.cc:315-321)
void to_json(json &j, KNOperator const &op);
// a graph is the array of its operators (src/kernel/graph.cc:33-37); from_json rebuilds
// it through the graph API, matching tensors by guid (:39-159), and throws
// std::runtime_error on a document that does not follow the schema (the reference asserts)
void to_json(json &j, Graph const &g);
void from_json(json const &j, Graph &g);
}  // namespace kernel

namespace threadblock {
// {data_type, layout, num_dims, dim[4], smem_offset, guid} (smem_tensor.h:169-170)
void to_json(json &j, STensor const &t);
void from_json(json const &j, STensor &t);
// all ExecutionPlan fields (graph.h:44-53); reduction_dimx defaults to 64 when a
// checkpoint predates the field
void to_json(json &j, ExecutionPlan const &p);
void from_json(json const &j, ExecutionPlan &p);
void to_json(json &j, TBOperator const &op);
// {graph_level, grid_dim, block_dim, forloop_range, reduction_dimx, operators,
// smem_offset} (src/threadblock/graph.cc:476-489)
void to_json(json &j, Graph const &g);
}  // namespace threadblock
}  // namespace mirage
