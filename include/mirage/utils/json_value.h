// A small JSON value type (the reference uses nlohmann::json, a dependency this backend
// does not have): parse, dump (object keys in sorted order, as nlohmann's default std::map
// object gives), building and reading objects, arrays, integers, strings, booleans and null.
// `json` names it, as in the reference's sources, so `operator json()` of the operator
// classes and `json(*op)` at their call sites read the same.
#pragma once

#include <cstddef>
#include <cstdint>
#include <iosfwd>
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

// `ifs >> j` reads the rest of the stream as one document; `os << j` writes it on one line
// (the two uses the reference's cpp_examples/profile.cc makes of nlohmann's operators).
std::istream &operator>>(std::istream &in, mirage::utils::Json &j);
std::ostream &operator<<(std::ostream &out, mirage::utils::Json const &j);

