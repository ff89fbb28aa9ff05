// The search checkpoint as a data carrier, and the measurement the reference's
// cpp_examples/profile.cc makes on a graph file.
//
// A checkpoint (reference include/mirage/search/search.h:46-68) is what the reference's
// search writes: the computation graph, the graphs it found fingerprint-equal to it
// (`generated_graphs`, each in the wire format of mirage/utils/json_utils.h), the best of
// them with its measured time, the generator's configuration and call stack, and three
// counters.  The search itself is not part of this backend; its two fields that only the
// search interprets (`config`, `callstack`) are kept as JSON values and written back as
// they were read, so a checkpoint passes through unchanged.
#pragma once

#include "mirage/kernel/graph.h"
#include "mirage/profile_result.h"
#include "mirage/utils/json_utils.h"
#include <string>
#include <vector>

namespace mirage {
namespace search {

struct Checkpoint {
  json computation_graph;  // a kernel graph in wire format: from_json(computation_graph, g)
  json best_graph;         // null until a layout search has run
  ProfileResult best_profile_result;
  json config;             // GeneratorConfig (search/config.h:45-56), uninterpreted
  json callstack;          // std::vector<LayerCheckpoint>, uninterpreted
  std::vector<json> generated_graphs;
  long long num_total_kernel_graphs = 0;
  long long num_total_random_tests = 0;
  long long num_valid_kernel_graphs = 0;
};

// throws std::runtime_error on a document that is not a checkpoint object
void from_json(json const &j, Checkpoint &c);
void to_json(json &j, Checkpoint const &c);

// Reads a file that holds either a checkpoint object or a single kernel graph (an array of
// operators, what profile.cc takes); a single graph comes back as a checkpoint whose
// generated_graphs holds just that graph.
Checkpoint load_checkpoint_file(std::string const &path);

struct GraphProfile {
  float run_time = 0.0f;      // sum of the operators' mean milliseconds per launch
  std::vector<float> op_ms;   // per operator, in graph order (input operators: 0)
};

// cpp_examples/profile.cc:25-34: fingerprint() of every operator, then profile() of every
// operator (ProfileResult's 1024 + 1024 launches each), run times summed.
GraphProfile profile_graph(mirage::kernel::Graph &g);

}  // namespace search
}  // namespace mirage
