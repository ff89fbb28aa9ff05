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
#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace mirage {
namespace utils {

class Json {
public:
  enum Kind { Null, Bool, Int, Float, String, Array, Object };

  Json() : kind_(Null) {}
  Json(std::nullptr_t) : kind_(Null) {}
  Json(bool b) : kind_(Bool), int_(b ? 1 : 0) {}
  Json(int v) : kind_(Int), int_(v) {}
  Json(unsigned v) : kind_(Int), int_(v) {}
  Json(long v) : kind_(Int), int_(v) {}
  Json(long long v) : kind_(Int), int_(v) {}
  Json(unsigned long v) : kind_(Int), int_((long long)v) {}
  Json(unsigned long long v) : kind_(Int), int_((long long)v) {}
  Json(double v) : kind_(Float), float_(v) {}
  Json(char const *s) : kind_(String), str_(s) {}
  Json(std::string const &s) : kind_(String), str_(s) {}

  static Json array() {
    Json j;
    j.kind_ = Array;
    return j;
  }
  static Json object() {
    Json j;
    j.kind_ = Object;
    return j;
  }
  // Throws std::runtime_error with the byte offset on malformed input.
  static Json parse(std::string const &text);
  // indent < 0: one line; otherwise pretty-printed with that many spaces per level.
  std::string dump(int indent = -1) const;

  Kind kind() const { return kind_; }
  bool is_null() const { return kind_ == Null; }
  bool is_array() const { return kind_ == Array; }
  bool is_object() const { return kind_ == Object; }
  bool contains(std::string const &key) const { return kind_ == Object && obj_.count(key) != 0; }
  size_t size() const { return kind_ == Array ? arr_.size() : kind_ == Object ? obj_.size() : 0; }

  // Object access: operator[] creates (turning a null value into an object), at() throws.
  Json &operator[](std::string const &key);
  Json const &at(std::string const &key) const;
  // Array access.
  Json &operator[](size_t i) { return arr_.at(i); }
  Json const &operator[](size_t i) const { return arr_.at(i); }
  Json const &at(size_t i) const { return arr_.at(i); }
  void push_back(Json const &v);  // turns a null value into an array
  std::vector<Json> const &items() const { return arr_; }
  std::map<std::string, Json> const &members() const { return obj_; }

  long long as_int() const;
  double as_double() const;
  bool as_bool() const;
  std::string const &as_string() const;
  void get_to(int &v) const { v = (int)as_int(); }
  void get_to(size_t &v) const { v = (size_t)as_int(); }
  void get_to(long long &v) const { v = as_int(); }
  void get_to(std::string &v) const { v = as_string(); }
  void get_to(bool &v) const { v = as_bool(); }

  bool operator==(Json const &o) const;
  bool operator!=(Json const &o) const { return !(*this == o); }

private:
  Kind kind_;
  long long int_ = 0;
  double float_ = 0.0;
  std::string str_;
  std::vector<Json> arr_;
  std::map<std::string, Json> obj_;
};

}  // namespace utils
}  // namespace mirage

using json = mirage::utils::Json;

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
