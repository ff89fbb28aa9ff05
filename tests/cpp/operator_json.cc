// Call sites of the reference that this translation unit must compile and run unchanged:
//   src/kernel/graph.cc:35        j.push_back(json(*op))          op: KNOperator*
//   src/threadblock/graph.cc:485  j["operators"].push_back(json(*op))   op: TBOperator*
//   src/kernel/customized.cc:318  j["bgraph"] = json(bgraph)
//   cpp_examples/profile.cc:19-22 ifs >> j; from_json(j, g); std::cout << json(g)
// Builds the C1-style tiled matmul mugraph through the host API (host-only runtime), writes
// it through `operator json()`, reads it back and prints both forms.
#include "mirage/kernel/graph.h"
#include "mirage/threadblock/graph.h"
#include "mirage/utils/json_utils.h"

#include <iostream>
#include <sstream>

using namespace mirage;

int main() {
  kernel::Graph g;
  kernel::DTensor A = g.new_input({64, 256}, type::DT_FLOAT16, layout::DmemRowMajor);
  kernel::DTensor B = g.new_input({256, 128}, type::DT_FLOAT16, layout::DmemColumnMajor);
  {
    threadblock::ExecutionPlan plan;
    plan.ops.push_back({type::TB_MATMUL_OP, {{0, 0}, {1, 0}}});
    plan.ops.push_back({type::TB_EXP_OP, {{2, 0}}});
    plan.ops.push_back({type::TB_REDUCTION_1_OP, {{3, 0}}});
    plan.input_map = {{-1, -1, -1}, {1, -1, -1}};
    plan.forloop_dim = {1, 0};
    plan.input_smem_layouts = {layout::SmemRowMajor, layout::SmemColumnMajor};
    plan.output_map = {1, -1, -1};
    plan.forloop_range = 4;
    plan.grid_dim = {2, 1, 1};
    plan.block_dim = {128, 1, 1};
    std::vector<kernel::DTensor> outs = g.customized({A, B}, plan);
    g.exp(outs[0]);
  }
  // graph.cc:33-37
  json by_operator = json::array();
  for (kernel::KNOperator *const op : g.operators) {
    by_operator.push_back(json(*op));
  }
  json whole;
  to_json(whole, g);
  if (by_operator != whole || json(g) != whole) {
    std::cerr << "json(*op) and to_json(j, graph) disagree" << std::endl;
    return 1;
  }
  // threadblock/graph.cc:476-489 and customized.cc:315-321
  auto *c = static_cast<kernel::KNCustomizedOp *>(g.operators[2]);
  json ops = json::array();
  for (threadblock::TBOperator *const op : c->bgraph.operators) {
    ops.push_back(json(*op));
  }
  json const b = json(c->bgraph);
  if (b.at("operators") != ops || whole.at(2).at("bgraph") != b ||
      b.at("operators").size() != 6 || ops.at(4).at("reduce_dim").as_int() != 1) {
    std::cerr << "thread-block operator json mismatch" << std::endl;
    return 2;
  }
  // profile.cc:17-22
  std::stringstream file;
  file << whole;
  kernel::Graph g2;
  json j;
  file >> j;
  from_json(j, g2);
  std::cout << json(g2) << std::endl;
  return json(g2).size() == whole.size() ? 0 : 3;
}
