// mirage_profile: the reference's cpp_examples/profile.cc for this backend.
//
//   mirage_profile <graph.json | checkpoint.json> [first [count]]
//
// A graph file (an array of operators) is loaded, printed back as JSON, fingerprinted
// and every operator profiled; the sum of the operators' mean times is printed, as
// profile.cc:17-36 does.  A checkpoint file (search.h:46-68) gets the same treatment for
// each of its generated graphs (optionally a range of them), one line per graph, then the
// minimum / median / maximum.
#include "mirage/kernel/graph.h"
#include "mirage/search/checkpoint.h"
#include "mirage/threadblock/graph.h"

#include <algorithm>
#include <cstdlib>
#include <fstream>
#include <iostream>

using namespace mirage;
using namespace mirage::search;

int main(int argc, char **argv) {
  if (argc < 2) {
    std::cerr << "Miss graph file name" << std::endl;
    return 1;
  }
  Checkpoint cp;
  try {
    cp = load_checkpoint_file(argv[1]);
  } catch (std::exception const &e) {
    std::cerr << e.what() << std::endl;
    return 1;
  }
  bool const single = cp.generated_graphs.size() == 1 && cp.computation_graph == cp.generated_graphs[0];
  size_t first = argc > 2 ? (size_t)std::atoll(argv[2]) : 0;
  size_t count = argc > 3 ? (size_t)std::atoll(argv[3]) : cp.generated_graphs.size();
  std::vector<float> times;
  for (size_t i = first; i < cp.generated_graphs.size() && i < first + count; i++) {
    kernel::Graph g;
    GraphProfile p;
    try {
      from_json(cp.generated_graphs[i], g);
      if (single) {
        std::cout << json(g) << std::endl;
      }
      p = profile_graph(g);
    } catch (std::exception const &e) {
      std::cerr << "graph " << i << ": " << e.what() << std::endl;
      return 1;
    }
    times.push_back(p.run_time);
    if (single) {
      std::cout << "Profiled running time: " << p.run_time << std::endl;
    } else {
      std::cout << "graph " << i << ": " << g.operators.size() << " operators, profiled running time: "
                << p.run_time << " ms" << std::endl;
    }
  }
  if (!single && !times.empty()) {
    std::sort(times.begin(), times.end());
    std::cout << times.size() << " graphs: min " << times.front() << " ms, median "
              << times[times.size() / 2] << " ms, max " << times.back() << " ms" << std::endl;
  }
  return 0;
}
