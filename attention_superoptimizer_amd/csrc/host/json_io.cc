// JSON value type and the mugraph wire format (reference include/mirage/utils/json_utils.h,
// src/utils/json_utils.cc, src/kernel/graph.cc:33-159, the `operator json()` of every
// operator and the NLOHMANN_DEFINE_TYPE_NON_INTRUSIVE lists of DTensor / STensor /
// ExecutionPlan).  Host only.
#include "mirage/utils/json_utils.h"
#include <istream>
#include <iterator>
#include <ostream>

#include "mirage/utils/hip_types.h"

#include <cmath>
#include <cstdio>
#include <memory>
#include <cstring>
#include <cstdlib>
#include <stdexcept>
#include <unordered_map>

namespace mirage {
namespace utils {

// ---- value ---------------------------------------------------------------------------
Json &Json::operator[](std::string const &key) {
  if (kind_ == Null) {
    kind_ = Object;
  }
  if (kind_ != Object) {
    throw std::runtime_error("json: not an object");
  }
  return obj_[key];
}

Json const &Json::at(std::string const &key) const {
  if (kind_ != Object) {
    throw std::runtime_error("json: not an object (looking up \"" + key + "\")");
  }
  auto it = obj_.find(key);
  if (it == obj_.end()) {
    throw std::runtime_error("json: key \"" + key + "\" not found");
  }
  return it->second;
}

void Json::push_back(Json const &v) {
  if (kind_ == Null) {
    kind_ = Array;
  }
  if (kind_ != Array) {
    throw std::runtime_error("json: not an array");
  }
  arr_.push_back(v);
}

long long Json::as_int() const {
  if (kind_ == Int || kind_ == Bool) {
    return int_;
  }
  if (kind_ == Float && std::floor(float_) == float_) {
    return (long long)float_;
  }
  throw std::runtime_error("json: not an integer");
}

double Json::as_double() const {
  if (kind_ == Float) {
    return float_;
  }
  if (kind_ == Int) {
    return (double)int_;
  }
  throw std::runtime_error("json: not a number");
}

bool Json::as_bool() const {
  if (kind_ != Bool) {
    throw std::runtime_error("json: not a boolean");
  }
  return int_ != 0;
}

std::string const &Json::as_string() const {
  if (kind_ != String) {
    throw std::runtime_error("json: not a string");
  }
  return str_;
}

bool Json::operator==(Json const &o) const {
  if (kind_ != o.kind_) {
    return false;
  }
  switch (kind_) {
    case Null: return true;
    case Bool:
    case Int: return int_ == o.int_;
    case Float: return float_ == o.float_;
    case String: return str_ == o.str_;
    case Array: return arr_ == o.arr_;
    case Object: return obj_ == o.obj_;
  }
  return false;
}

// ---- writer --------------------------------------------------------------------------
static void dump_string(std::string const &s, std::string &out) {
  out.push_back('"');
  for (unsigned char ch : s) {
    switch (ch) {
      case '"': out += "\\\""; break;
      case '\\': out += "\\\\"; break;
      case '\n': out += "\\n"; break;
      case '\r': out += "\\r"; break;
      case '\t': out += "\\t"; break;
      case '\b': out += "\\b"; break;
      case '\f': out += "\\f"; break;
      default:
        if (ch < 0x20) {
          char buf[8];
          std::snprintf(buf, sizeof(buf), "\\u%04x", ch);
          out += buf;
        } else {
          out.push_back((char)ch);
        }
    }
  }
  out.push_back('"');
}

static void dump_value(Json const &j, int indent, int level, std::string &out) {
  auto newline = [&](int lv) {
    if (indent >= 0) {
      out.push_back('\n');
      out.append((size_t)(indent * lv), ' ');
    }
  };
  switch (j.kind()) {
    case Json::Null: out += "null"; break;
    case Json::Bool: out += j.as_bool() ? "true" : "false"; break;
    case Json::Int: out += std::to_string(j.as_int()); break;
    case Json::Float: {
      // JSON has no spelling for infinities and NaNs: null, as nlohmann-json writes them
      if (!std::isfinite(j.as_double())) {
        out += "null";
        break;
      }
      char buf[40];
      std::snprintf(buf, sizeof(buf), "%.17g", j.as_double());
      out += buf;
      break;
    }
    case Json::String: dump_string(j.as_string(), out); break;
    case Json::Array: {
      if (j.size() == 0) {
        out += "[]";
        break;
      }
      out.push_back('[');
      bool first = true;
      for (Json const &v : j.items()) {
        if (!first) {
          out.push_back(',');
        }
        first = false;
        newline(level + 1);
        dump_value(v, indent, level + 1, out);
      }
      newline(level);
      out.push_back(']');
      break;
    }
    case Json::Object: {
      if (j.size() == 0) {
        out += "{}";
        break;
      }
      out.push_back('{');
      bool first = true;
      for (auto const &kv : j.members()) {
        if (!first) {
          out.push_back(',');
        }
        first = false;
        newline(level + 1);
        dump_string(kv.first, out);
        out += indent >= 0 ? ": " : ":";
        dump_value(kv.second, indent, level + 1, out);
      }
      newline(level);
      out.push_back('}');
      break;
    }
  }
}

std::string Json::dump(int indent) const {
  std::string out;
  dump_value(*this, indent, 0, out);
  return out;
}

// ---- parser --------------------------------------------------------------------------
namespace {

struct Parser {
  std::string const &s;
  size_t p = 0;
  explicit Parser(std::string const &text) : s(text) {}

  [[noreturn]] void fail(char const *what) const {
    throw std::runtime_error("json: " + std::string(what) + " at byte " + std::to_string(p));
  }
  void skip() {
    while (p < s.size() && (s[p] == ' ' || s[p] == '\n' || s[p] == '\t' || s[p] == '\r')) {
      p++;
    }
  }
  bool eat(char c) {
    skip();
    if (p < s.size() && s[p] == c) {
      p++;
      return true;
    }
    return false;
  }
  void expect_word(char const *w) {
    for (; *w; w++, p++) {
      if (p >= s.size() || s[p] != *w) {
        fail("bad literal");
      }
    }
  }
  static void append_utf8(unsigned cp, std::string &out) {
    if (cp < 0x80) {
      out.push_back((char)cp);
    } else if (cp < 0x800) {
      out.push_back((char)(0xC0 | (cp >> 6)));
      out.push_back((char)(0x80 | (cp & 0x3F)));
    } else if (cp < 0x10000) {
      out.push_back((char)(0xE0 | (cp >> 12)));
      out.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
      out.push_back((char)(0x80 | (cp & 0x3F)));
    } else {
      out.push_back((char)(0xF0 | (cp >> 18)));
      out.push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
      out.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
      out.push_back((char)(0x80 | (cp & 0x3F)));
    }
  }
  unsigned hex4() {
    unsigned v = 0;
    for (int i = 0; i < 4; i++, p++) {
      if (p >= s.size()) {
        fail("truncated \\u escape");
      }
      char c = s[p];
      v <<= 4;
      if (c >= '0' && c <= '9') {
        v |= (unsigned)(c - '0');
      } else if (c >= 'a' && c <= 'f') {
        v |= (unsigned)(c - 'a' + 10);
      } else if (c >= 'A' && c <= 'F') {
        v |= (unsigned)(c - 'A' + 10);
      } else {
        fail("bad \\u escape");
      }
    }
    return v;
  }
  std::string string() {
    std::string out;
    if (!eat('"')) {
      fail("expected a string");
    }
    while (true) {
      if (p >= s.size()) {
        fail("unterminated string");
      }
      char c = s[p++];
      if (c == '"') {
        return out;
      }
      if (c != '\\') {
        out.push_back(c);
        continue;
      }
      if (p >= s.size()) {
        fail("unterminated escape");
      }
      char e = s[p++];
      switch (e) {
        case '"': out.push_back('"'); break;
        case '\\': out.push_back('\\'); break;
        case '/': out.push_back('/'); break;
        case 'n': out.push_back('\n'); break;
        case 'r': out.push_back('\r'); break;
        case 't': out.push_back('\t'); break;
        case 'b': out.push_back('\b'); break;
        case 'f': out.push_back('\f'); break;
        case 'u': {
          unsigned cp = hex4();
          if (cp >= 0xD800 && cp < 0xDC00 && p + 1 < s.size() && s[p] == '\\' && s[p + 1] == 'u') {
            p += 2;
            unsigned lo = hex4();
            cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
          }
          append_utf8(cp, out);
          break;
        }
        default: fail("bad escape");
      }
    }
  }
  Json number() {
    size_t const start = p;
    if (p < s.size() && s[p] == '-') {
      p++;
    }
    bool is_float = false;
    while (p < s.size() && ((s[p] >= '0' && s[p] <= '9') || s[p] == '.' || s[p] == 'e' ||
                            s[p] == 'E' || s[p] == '+' || s[p] == '-')) {
      if (s[p] == '.' || s[p] == 'e' || s[p] == 'E') {
        is_float = true;
      }
      p++;
    }
    std::string tok = s.substr(start, p - start);
    if (tok.empty() || tok == "-") {
      fail("expected a number");
    }
    if (is_float) {
      return Json(std::strtod(tok.c_str(), nullptr));
    }
    return Json(std::strtoll(tok.c_str(), nullptr, 10));
  }
  Json value(int depth) {
    if (depth > 256) {
      fail("nesting too deep");
    }
    skip();
    if (p >= s.size()) {
      fail("unexpected end");
    }
    char c = s[p];
    if (c == '{') {
      p++;
      Json o = Json::object();
      if (eat('}')) {
        return o;
      }
      do {
        skip();
        std::string key = string();
        if (!eat(':')) {
          fail("expected ':'");
        }
        o[key] = value(depth + 1);
      } while (eat(','));
      if (!eat('}')) {
        fail("expected '}'");
      }
      return o;
    }
    if (c == '[') {
      p++;
      Json a = Json::array();
      if (eat(']')) {
        return a;
      }
      do {
        a.push_back(value(depth + 1));
      } while (eat(','));
      if (!eat(']')) {
        fail("expected ']'");
      }
      return a;
    }
    if (c == '"') {
      return Json(string());
    }
    if (c == 't') {
      expect_word("true");
      return Json(true);
    }
    if (c == 'f') {
      expect_word("false");
      return Json(false);
    }
    if (c == 'n') {
      expect_word("null");
      return Json(nullptr);
    }
    return number();
  }
};

}  // namespace

Json Json::parse(std::string const &text) {
  Parser ps(text);
  Json v = ps.value(0);
  ps.skip();
  if (ps.p != text.size()) {
    ps.fail("trailing characters");
  }
  return v;
}

}  // namespace utils
}  // namespace mirage

// ======================================================================================
// wire format
// ======================================================================================
using namespace mirage::type;
using namespace mirage::layout;

namespace {

// malformed documents are reported by exception (the C facade turns it into NULL)
inline void json_require(bool ok, char const *what) {
  if (!ok) {
    throw std::runtime_error(what);
  }
}

struct EnumName {
  int value;
  char const *name;
};

// reference include/mirage/type.h:64-78
EnumName const kKnOps[] = {
    {KN_UNKOWN, "kn_unkown"},
    {KN_INPUT_OP, "kn_input_op"},
    {KN_MATMUL_OP, "kn_matmul_op"},
    {KN_REDUCTION_0_OP, "kn_reduction_0_op"},
    {KN_REDUCTION_1_OP, "kn_reduction_1_op"},
    {KN_REDUCTION_2_OP, "kn_reduction_2_op"},
    {KN_EXP_OP, "kn_exp_op"},
    {KN_ADD_OP, "kn_add_op"},
    {KN_MUL_OP, "kn_mul_op"},
    {KN_DIV_OP, "kn_div_op"},
    {KN_SILU_OP, "kn_silu_op"},  // extension
    {KN_CUSTOMIZED_OP, "kn_customized_op"},
};
// reference include/mirage/type.h:105-129
EnumName const kTbOps[] = {
    {TB_UNKOWN, "tb_unkown"},
    {TB_INPUT_OP, "tb_input_op"},
    {TB_OUTPUT_OP, "tb_output_op"},
    {TB_MATMUL_OP, "tb_matmul_op"},
    {TB_REDUCTION_0_OP, "tb_reduction_0_op"},
    {TB_REDUCTION_1_OP, "tb_reduction_1_op"},
    {TB_REDUCTION_2_OP, "tb_reduction_2_op"},
    {TB_EXP_OP, "tb_exp_op"},
    {TB_ADD_OP, "tb_add_op"},
    {TB_MUL_OP, "tb_mul_op"},
    {TB_DIV_OP, "tb_div_op"},
    {TB_SILU_OP, "tb_silu_op"},  // extension
    {TB_REDUCTION_0_TO_DIMX_OP, "tb_reduction_0_to_dimx_op"},
    {TB_REDUCTION_1_TO_DIMX_OP, "tb_reduction_1_to_dimx_op"},
    {TB_REDUCTION_2_TO_DIMX_OP, "tb_reduction_2_to_dimx_op"},
    {TB_CONCAT_0_OP, "tb_concat_0_op"},
    {TB_CONCAT_1_OP, "tb_concat_1_op"},
    {TB_CONCAT_2_OP, "tb_concat_2_op"},
    {TB_CUSTOMIZED_OP, "tb_customized_op"},
};
// reference include/mirage/layout.h:28-58
EnumName const kDmem[] = {
    {DmemRowMajor, "DmemRowMajor"},
    {DmemColumnMajor, "DmemColumnMajor"},
    {DmemUnknownLayout, "DmemUnknownLayout"},
};
EnumName const kSmem[] = {
    {SmemRowMajor, "SmemRowMajor"},
    {SmemColumnMajor, "SmemColumnMajor"},
    {SmemRowMajorTensorOpMultiplicand_Crosswise16, "SmemRowMajorTensorOpMultiplicand_Crosswise16"},
    {SmemRowMajorTensorOpMultiplicand_Crosswise32, "SmemRowMajorTensorOpMultiplicand_Crosswise32"},
    {SmemRowMajorTensorOpMultiplicand_Crosswise64, "SmemRowMajorTensorOpMultiplicand_Crosswise64"},
    {SmemColumnMajorTensorOpMultiplicand_Crosswise16,
     "SmemColumnMajorTensorOpMultiplicand_Crosswise16"},
    {SmemColumnMajorTensorOpMultiplicand_Crosswise32,
     "SmemColumnMajorTensorOpMultiplicand_Crosswise32"},
    {SmemColumnMajorTensorOpMultiplicand_Crosswise64,
     "SmemColumnMajorTensorOpMultiplicand_Crosswise64"},
    {SmemUnknownLayout, "SmemUnknownLayout"},
};

template <size_t N>
json enum_to_json(EnumName const (&table)[N], int v) {
  for (EnumName const &e : table) {
    if (e.value == v) {
      return json(e.name);
    }
  }
  return json(table[0].name);  // nlohmann falls back to the first pair
}

template <size_t N>
int enum_from_json(EnumName const (&table)[N], json const &j) {
  if (j.kind() == json::Int) {
    return (int)j.as_int();
  }
  for (EnumName const &e : table) {
    if (j.as_string() == e.name) {
      return e.value;
    }
  }
  return table[0].value;
}

template <class T>
json array_of(std::vector<T> const &v) {
  json a = json::array();
  for (T const &x : v) {
    json e;
    to_json(e, x);
    a.push_back(e);
  }
  return a;
}

}  // namespace

void to_json(json &j, int3 const &v) {
  j = json::object();
  j["x"] = v.x;
  j["y"] = v.y;
  j["z"] = v.z;
}
void from_json(json const &j, int3 &v) {
  j.at("x").get_to(v.x);
  j.at("y").get_to(v.y);
  j.at("z").get_to(v.z);
}
void to_json(json &j, dim3 const &v) {
  j = json::object();
  j["x"] = v.x;
  j["y"] = v.y;
  j["z"] = v.z;
}
void from_json(json const &j, dim3 &v) {
  v.x = (unsigned)j.at("x").as_int();
  v.y = (unsigned)j.at("y").as_int();
  v.z = (unsigned)j.at("z").as_int();
}

namespace mirage {
namespace kernel {

void to_json(json &j, DTensor const &t) {
  j = json::object();
  j["data_type"] = (int)t.data_type;
  j["layout"] = enum_to_json(kDmem, t.layout);
  j["num_dims"] = t.num_dims;
  json d = json::array();
  for (int i = 0; i < MAX_TENSOR_DIMS; i++) {
    d.push_back(i < t.num_dims ? t.dim[i] : 0);
  }
  j["dim"] = d;
  j["guid"] = t.guid;
}

void from_json(json const &j, DTensor &t) {
  t.data_type = (DataType)j.at("data_type").as_int();
  t.layout = (DmemLayout)enum_from_json(kDmem, j.at("layout"));
  j.at("num_dims").get_to(t.num_dims);
  json_require(t.num_dims >= 0 && t.num_dims <= MAX_TENSOR_DIMS, "json: bad num_dims");
  for (int i = 0; i < MAX_TENSOR_DIMS; i++) {
    t.dim[i] = i < (int)j.at("dim").size() ? (int)j.at("dim").at((size_t)i).as_int() : 0;
  }
  j.at("guid").get_to(t.guid);
}

void to_json(json &j, KNOperator const &op) {
  j = json::object();
  j["op_type"] = enum_to_json(kKnOps, op.op_type);
  j["input_tensors"] = array_of(op.input_tensors);
  j["output_tensors"] = array_of(op.output_tensors);
  if (op.op_type == KN_CUSTOMIZED_OP) {
    auto const &c = static_cast<KNCustomizedOp const &>(op);
    json b, p;
    mirage::threadblock::to_json(b, c.bgraph);
    mirage::threadblock::to_json(p, c.plan);
    j["bgraph"] = b;
    j["plan"] = p;
  }
}

void to_json(json &j, Graph const &g) {
  j = json::array();
  for (KNOperator const *op : g.operators) {
    json e;
    to_json(e, *op);
    j.push_back(e);
  }
}

void from_json(json const &j, Graph &g) {
  // guid in the file -> tensor of the graph being rebuilt
  std::unordered_map<size_t, DTensor> by_file_guid;
  auto tensor_of = [&](json const &jt) -> DTensor const & {
    size_t guid = 0;
    jt.at("guid").get_to(guid);
    auto it = by_file_guid.find(guid);
    json_require(it != by_file_guid.end(), "json: operator consumes a tensor nobody produced");
    return it->second;
  };
  auto bind = [&](json const &jop, size_t i, DTensor const &t) {
    size_t guid = 0;
    jop.at("output_tensors").at(i).at("guid").get_to(guid);
    by_file_guid[guid] = t;
  };
  for (json const &jop : j.items()) {
    int const op_type = enum_from_json(kKnOps, jop.at("op_type"));
    switch (op_type) {
      case KN_INPUT_OP: {
        DTensor meta;
        from_json(jop.at("output_tensors").at(0), meta);
        std::vector<int> dims(meta.dim, meta.dim + meta.num_dims);
        bind(jop, 0, g.new_input(dims, meta.data_type, meta.layout));
        break;
      }
      case KN_MATMUL_OP:
        bind(jop, 0, g.matmul(tensor_of(jop.at("input_tensors").at(0)),
                              tensor_of(jop.at("input_tensors").at(1))));
        break;
      case KN_EXP_OP:
        bind(jop, 0, g.exp(tensor_of(jop.at("input_tensors").at(0))));
        break;
      case KN_SILU_OP:
        bind(jop, 0, g.silu(tensor_of(jop.at("input_tensors").at(0))));
        break;
      case KN_ADD_OP:
        bind(jop, 0, g.add(tensor_of(jop.at("input_tensors").at(0)),
                           tensor_of(jop.at("input_tensors").at(1))));
        break;
      case KN_MUL_OP:
        bind(jop, 0, g.mul(tensor_of(jop.at("input_tensors").at(0)),
                           tensor_of(jop.at("input_tensors").at(1))));
        break;
      case KN_DIV_OP:
        bind(jop, 0, g.div(tensor_of(jop.at("input_tensors").at(0)),
                           tensor_of(jop.at("input_tensors").at(1))));
        break;
      case KN_REDUCTION_0_OP:
      case KN_REDUCTION_1_OP:
      case KN_REDUCTION_2_OP: {
        // the reference rebuilds with size 1 (graph.cc:110-120); the recorded output
        // shape also covers reductions to a size other than 1
        int const dim = op_type - KN_REDUCTION_0_OP;
        DTensor out;
        from_json(jop.at("output_tensors").at(0), out);
        bind(jop, 0, g.reduction(tensor_of(jop.at("input_tensors").at(0)), dim, out.dim[dim]));
        break;
      }
      case KN_CUSTOMIZED_OP: {
        std::vector<DTensor> inputs;
        for (json const &jt : jop.at("input_tensors").items()) {
          inputs.push_back(tensor_of(jt));
        }
        mirage::threadblock::ExecutionPlan plan;
        mirage::threadblock::from_json(jop.at("plan"), plan);
        if (!jop.at("plan").contains("reduction_dimx") && jop.contains("bgraph") &&
            jop.at("bgraph").contains("reduction_dimx")) {
          jop.at("bgraph").at("reduction_dimx").get_to(plan.reduction_dimx);
        }
        std::vector<DTensor> outputs = g.customized(inputs, plan);
        json_require(outputs.size() == jop.at("output_tensors").size(), "json: customized op has a different number of outputs than recorded");
        for (size_t i = 0; i < outputs.size(); i++) {
          bind(jop, i, outputs[i]);
        }
        // carry the recorded tile layouts over (graph.cc:139-152)
        if (jop.contains("bgraph")) {
          auto *op = static_cast<KNCustomizedOp *>(g.operators.back());
          json const &jops = jop.at("bgraph").at("operators");
          json_require(op->bgraph.operators.size() == jops.size(), "json: thread-block graph has a different number of operators than recorded");
          for (size_t i = 0; i < jops.size(); i++) {
            mirage::threadblock::TBOperator *bop = op->bgraph.operators[i];
            json const &jb = jops.at(i);
            for (size_t k = 0; k < bop->input_tensors.size() && k < jb.at("input_tensors").size(); k++) {
              bop->input_tensors[k].layout =
                  (SmemLayout)enum_from_json(kSmem, jb.at("input_tensors").at(k).at("layout"));
            }
            for (size_t k = 0; k < bop->output_tensors.size() && k < jb.at("output_tensors").size(); k++) {
              bop->output_tensors[k].layout =
                  (SmemLayout)enum_from_json(kSmem, jb.at("output_tensors").at(k).at("layout"));
            }
          }
        }
        break;
      }
      default:
        json_require(false, "json: cannot deserialize this operator");
    }
  }
}

}  // namespace kernel

namespace threadblock {

void to_json(json &j, STensor const &t) {
  j = json::object();
  j["data_type"] = (int)t.data_type;
  j["layout"] = enum_to_json(kSmem, t.layout);
  j["num_dims"] = t.num_dims;
  json d = json::array();
  for (int i = 0; i < MAX_TENSOR_DIMS; i++) {
    d.push_back(i < t.num_dims ? t.dim[i] : 0);
  }
  j["dim"] = d;
  j["smem_offset"] = t.smem_offset;
  j["guid"] = t.guid;
}

void from_json(json const &j, STensor &t) {
  t.data_type = (DataType)j.at("data_type").as_int();
  t.layout = (SmemLayout)enum_from_json(kSmem, j.at("layout"));
  j.at("num_dims").get_to(t.num_dims);
  json_require(t.num_dims >= 0 && t.num_dims <= MAX_TENSOR_DIMS, "json: bad num_dims");
  for (int i = 0; i < MAX_TENSOR_DIMS; i++) {
    t.dim[i] = i < (int)j.at("dim").size() ? (int)j.at("dim").at((size_t)i).as_int() : 0;
  }
  j.at("smem_offset").get_to(t.smem_offset);
  j.at("guid").get_to(t.guid);
}

void to_json(json &j, ExecutionPlan const &p) {
  j = json::object();
  json ops = json::array();
  for (auto const &op : p.ops) {
    json pair = json::array();
    pair.push_back(enum_to_json(kTbOps, op.first));
    json operands = json::array();
    for (auto const &idx : op.second) {
      json two = json::array();
      two.push_back(idx.first);
      two.push_back(idx.second);
      operands.push_back(two);
    }
    pair.push_back(operands);
    ops.push_back(pair);
  }
  j["ops"] = ops;
  j["input_map"] = array_of(p.input_map);
  json fd = json::array();
  for (int v : p.forloop_dim) {
    fd.push_back(v);
  }
  j["forloop_dim"] = fd;
  json lay = json::array();
  for (SmemLayout l : p.input_smem_layouts) {
    lay.push_back(enum_to_json(kSmem, l));
  }
  j["input_smem_layouts"] = lay;
  json om, gd, bd;
  ::to_json(om, p.output_map);
  ::to_json(gd, p.grid_dim);
  ::to_json(bd, p.block_dim);
  j["output_map"] = om;
  j["forloop_range"] = p.forloop_range;
  j["reduction_dimx"] = p.reduction_dimx;
  j["grid_dim"] = gd;
  j["block_dim"] = bd;
}

void from_json(json const &j, ExecutionPlan &p) {
  p = ExecutionPlan();
  for (json const &jop : j.at("ops").items()) {
    std::vector<std::pair<int, int>> operands;
    for (json const &two : jop.at(1).items()) {
      operands.emplace_back((int)two.at(0).as_int(), (int)two.at(1).as_int());
    }
    p.ops.emplace_back((TBOperatorType)enum_from_json(kTbOps, jop.at(0)), operands);
  }
  for (json const &m : j.at("input_map").items()) {
    int3 v;
    ::from_json(m, v);
    p.input_map.push_back(v);
  }
  for (json const &v : j.at("forloop_dim").items()) {
    p.forloop_dim.push_back((int)v.as_int());
  }
  for (json const &l : j.at("input_smem_layouts").items()) {
    p.input_smem_layouts.push_back((SmemLayout)enum_from_json(kSmem, l));
  }
  ::from_json(j.at("output_map"), p.output_map);
  j.at("forloop_range").get_to(p.forloop_range);
  if (j.contains("reduction_dimx")) {  // absent from checkpoints that predate the field
    j.at("reduction_dimx").get_to(p.reduction_dimx);
  }
  ::from_json(j.at("grid_dim"), p.grid_dim);
  ::from_json(j.at("block_dim"), p.block_dim);
}

void to_json(json &j, TBOperator const &op) {
  j = json::object();
  j["op_type"] = enum_to_json(kTbOps, op.op_type);
  j["input_tensors"] = array_of(op.input_tensors);
  j["output_tensors"] = array_of(op.output_tensors);
  if (op.op_type == TB_INPUT_OP) {
    auto const &in = static_cast<TBInputOp const &>(op);
    json dt, im;
    mirage::kernel::to_json(dt, in.dtensor);
    ::to_json(im, in.input_map);
    j["dtensor"] = dt;
    j["input_map"] = im;
    j["forloop_dim"] = in.forloop_dim;
  } else if (op.op_type == TB_OUTPUT_OP) {
    auto const &out = static_cast<TBOutputOp const &>(op);
    json dt, om;
    mirage::kernel::to_json(dt, out.dtensor);
    ::to_json(om, out.output_map);
    j["dtensor"] = dt;
    j["output_map"] = om;
  } else if (op.op_type >= TB_REDUCTION_0_OP && op.op_type <= TB_REDUCTION_2_TO_DIMX_OP) {
    auto const &r = static_cast<TBReductionOp const &>(op);
    j["reduce_dim"] = r.reduce_dim;
    j["reduce_size"] = r.reduce_size;
  } else if (op.op_type >= TB_CONCAT_0_OP && op.op_type <= TB_CONCAT_2_OP) {
    j["concat_dim"] = static_cast<TBConcatOp const &>(op).concat_dim;
  }
}

void to_json(json &j, Graph const &g) {
  j = json::object();
  j["graph_level"] = "thread_block_graph";
  json gd, bd;
  ::to_json(gd, g.grid_dim);
  ::to_json(bd, g.block_dim);
  j["grid_dim"] = gd;
  j["block_dim"] = bd;
  j["forloop_range"] = g.forloop_range;
  j["reduction_dimx"] = g.reduction_dimx;
  json ops = json::array();
  for (TBOperator const *op : g.operators) {
    json e;
    to_json(e, *op);
    ops.push_back(e);
  }
  j["operators"] = ops;
  j["smem_offset"] = g.smem_offset;
}

}  // namespace threadblock
}  // namespace mirage

std::istream &operator>>(std::istream &in, mirage::utils::Json &j) {
  std::string text((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
  j = mirage::utils::Json::parse(text);
  return in;
}

std::ostream &operator<<(std::ostream &out, mirage::utils::Json const &j) { return out << j.dump(); }

// ---- operator json() of the operator classes ---------------------------------------------
// One definition per class, as in the reference (src/kernel/{operator,matmul,element_unary,
// element_binary,reduction,customized}.cc, src/threadblock/{input_loader,output,matmul,
// element_unary,element_binary,reduction,concat,graph}.cc): each gives the entry that
// to_json writes for it, so `json(*op)` and `to_json(j, *op)` agree by construction.
namespace mirage {
namespace kernel {
#define MIRAGE_KN_JSON(CLASS)                          \
  CLASS::operator json() const {                       \
    json j;                                            \
    to_json(j, static_cast<KNOperator const &>(*this)); \
    return j;                                          \
  }
MIRAGE_KN_JSON(KNInputOp)
MIRAGE_KN_JSON(KNMatmulOp)
MIRAGE_KN_JSON(KNElementUnaryOp)
MIRAGE_KN_JSON(KNElementBinaryOp)
MIRAGE_KN_JSON(KNReductionOp)
MIRAGE_KN_JSON(KNCustomizedOp)
#undef MIRAGE_KN_JSON

Graph::operator json() const {
  json j;
  to_json(j, *this);
  return j;
}
}  // namespace kernel

namespace threadblock {
#define MIRAGE_TB_JSON(CLASS)                          \
  CLASS::operator json() const {                       \
    json j;                                            \
    to_json(j, static_cast<TBOperator const &>(*this)); \
    return j;                                          \
  }
MIRAGE_TB_JSON(TBInputOp)
MIRAGE_TB_JSON(TBOutputOp)
MIRAGE_TB_JSON(TBMatmulOp)
MIRAGE_TB_JSON(TBElementUnaryOp)
MIRAGE_TB_JSON(TBElementBinaryOp)
MIRAGE_TB_JSON(TBReductionOp)
MIRAGE_TB_JSON(TBConcatOp)
#undef MIRAGE_TB_JSON

Graph::operator json() const {
  json j;
  to_json(j, *this);
  return j;
}
}  // namespace threadblock
}  // namespace mirage

// ---- C facade ------------------------------------------------------------------------
extern "C" {

// Parses a kernel graph in the reference's JSON schema and rebuilds it through the graph
// API.  Returns a graph handle (mirage_graph_destroy frees it) or NULL on malformed text.
void *mirage_graph_from_json(char const *text) {
  try {
    json j = json::parse(text);
    std::unique_ptr<mirage::kernel::Graph> g(new mirage::kernel::Graph());
    mirage::kernel::from_json(j, *g);
    return g.release();
  } catch (std::exception const &e) {
    std::fprintf(stderr, "mirage_graph_from_json: %s\n", e.what());
    return nullptr;
  }
}

// Writes the graph's JSON (one line) into buf if it fits; returns the length needed,
// terminator excluded.
long long mirage_graph_to_json(void *graph, char *buf, long long capacity) {
  json j;
  mirage::kernel::to_json(j, *static_cast<mirage::kernel::Graph *>(graph));
  std::string s = j.dump();
  if (buf != nullptr && (long long)s.size() < capacity) {
    std::memcpy(buf, s.c_str(), s.size() + 1);
  }
  return (long long)s.size();
}

}  // extern "C"
