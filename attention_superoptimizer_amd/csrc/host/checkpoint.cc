// Checkpoint objects and the profile.cc measurement (see mirage/search/checkpoint.h).
#include "mirage/search/checkpoint.h"

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <sstream>
#include <stdexcept>

namespace mirage {
namespace search {

void from_json(json const &j, Checkpoint &c) {
  if (!j.is_object() || !j.contains("computation_graph") || !j.contains("generated_graphs") ||
      !j.at("generated_graphs").is_array()) {
    throw std::runtime_error("json: not a checkpoint object");
  }
  c = Checkpoint{};
  c.computation_graph = j.at("computation_graph");
  c.best_graph = j.contains("best_graph") ? j.at("best_graph") : json();
  c.best_profile_result = ProfileResult::infinity();
  // (a null run_time is how a writer spells a non-finite float: it stays "infinity")
  if (j.contains("best_profile_result") && j.at("best_profile_result").is_object() &&
      j.at("best_profile_result").contains("run_time") &&
      !j.at("best_profile_result").at("run_time").is_null()) {
    c.best_profile_result.run_time = (float)j.at("best_profile_result").at("run_time").as_double();
  }
  c.config = j.contains("config") ? j.at("config") : json::object();
  c.callstack = j.contains("callstack") ? j.at("callstack") : json::array();
  for (json const &g : j.at("generated_graphs").items()) {
    c.generated_graphs.push_back(g);
  }
  auto counter = [&](char const *key) {
    return j.contains(key) ? j.at(key).as_int() : 0LL;
  };
  c.num_total_kernel_graphs = counter("num_total_kernel_graphs");
  c.num_total_random_tests = counter("num_total_random_tests");
  c.num_valid_kernel_graphs = counter("num_valid_kernel_graphs");
}

void to_json(json &j, Checkpoint const &c) {
  j = json::object();
  j["computation_graph"] = c.computation_graph;
  j["best_graph"] = c.best_graph;
  json r = json::object();
  r["run_time"] = (double)c.best_profile_result.run_time;
  j["best_profile_result"] = r;
  j["config"] = c.config;
  j["callstack"] = c.callstack;
  json gs = json::array();
  for (json const &g : c.generated_graphs) {
    gs.push_back(g);
  }
  j["generated_graphs"] = gs;
  j["num_total_kernel_graphs"] = c.num_total_kernel_graphs;
  j["num_total_random_tests"] = c.num_total_random_tests;
  j["num_valid_kernel_graphs"] = c.num_valid_kernel_graphs;
}

Checkpoint load_checkpoint_file(std::string const &path) {
  std::ifstream in(path);
  if (!in) {
    throw std::runtime_error("cannot open " + path);
  }
  std::stringstream text;
  text << in.rdbuf();
  json const j = json::parse(text.str());
  Checkpoint c;
  if (j.is_array()) {  // one kernel graph
    c.computation_graph = j;
    c.best_profile_result = ProfileResult::infinity();
    c.config = json::object();
    c.callstack = json::array();
    c.generated_graphs.push_back(j);
    c.num_valid_kernel_graphs = 1;
    return c;
  }
  from_json(j, c);
  return c;
}

GraphProfile profile_graph(mirage::kernel::Graph &g) {
  GraphProfile out;
  for (auto *op : g.operators) {
    op->fingerprint();
  }
  for (auto *op : g.operators) {
    ProfileResult r;
    r.run_time = 0.0f;
    op->profile(r);
    out.op_ms.push_back(r.run_time);
    out.run_time += r.run_time;
  }
  return out;
}

}  // namespace search
}  // namespace mirage

// ---- C facade -------------------------------------------------------------------------------
extern "C" {

// A checkpoint (or single-graph) file; nullptr with a message on stderr if it cannot be read.
void *mirage_checkpoint_load(char const *path) {
  try {
    return new mirage::search::Checkpoint(mirage::search::load_checkpoint_file(path));
  } catch (std::exception const &e) {
    std::fprintf(stderr, "mirage_checkpoint_load: %s\n", e.what());
    return nullptr;
  }
}

void mirage_checkpoint_destroy(void *c) { delete static_cast<mirage::search::Checkpoint *>(c); }

// (every accessor below returns an error value for a null handle)
int mirage_checkpoint_num_graphs(void *c) {
  if (c == nullptr) {
    return -1;
  }
  return (int)static_cast<mirage::search::Checkpoint *>(c)->generated_graphs.size();
}

// counters[0..2] = num_total_kernel_graphs, num_total_random_tests, num_valid_kernel_graphs;
// returns best_profile_result.run_time
float mirage_checkpoint_summary(void *c, long long *counters) {
  if (c == nullptr) {
    return -1.0f;
  }
  auto *cp = static_cast<mirage::search::Checkpoint *>(c);
  if (counters != nullptr) {
    counters[0] = cp->num_total_kernel_graphs;
    counters[1] = cp->num_total_random_tests;
    counters[2] = cp->num_valid_kernel_graphs;
  }
  return cp->best_profile_result.run_time;
}

// The whole checkpoint (index -2), its computation graph (index -1) or generated graph
// `index` as JSON text; returns the length, copies at most capacity - 1 bytes.
long long mirage_checkpoint_json(void *c, int index, char *buf, long long capacity) {
  if (c == nullptr) {
    return -1;
  }
  auto *cp = static_cast<mirage::search::Checkpoint *>(c);
  std::string text;
  if (index == -2) {
    json j;
    mirage::search::to_json(j, *cp);
    text = j.dump();
  } else if (index == -1) {
    text = cp->computation_graph.dump();
  } else if (index >= 0 && index < (int)cp->generated_graphs.size()) {
    text = cp->generated_graphs[(size_t)index].dump();
  } else {
    return -1;
  }
  if (buf != nullptr && capacity > 0) {
    long long n = std::min<long long>((long long)text.size(), capacity - 1);
    std::memcpy(buf, text.data(), (size_t)n);
    buf[n] = '\0';
  }
  return (long long)text.size();
}

// profile.cc's measurement on an open graph: per-operator mean milliseconds into op_ms (up to
// capacity entries); returns the sum.
float mirage_graph_profile(void *graph, float *op_ms, int capacity) {
  if (graph == nullptr) {
    return -1.0f;
  }
  mirage::search::GraphProfile p =
      mirage::search::profile_graph(*static_cast<mirage::kernel::Graph *>(graph));
  for (int i = 0; op_ms != nullptr && i < capacity && i < (int)p.op_ms.size(); i++) {
    op_ms[i] = p.op_ms[(size_t)i];
  }
  return p.run_time;
}

}  // extern "C"
