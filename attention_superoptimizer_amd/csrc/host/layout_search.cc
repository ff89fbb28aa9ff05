// Layout selection (reference src/search/search.cc:625-777); see
// include/mirage/search/layout.h for what a layout means on this backend.
#include "mirage/search/layout.h"

#include "mi355_abi.h"
#include "mirage/utils/json_utils.h"

#include <map>
#include <utility>

namespace mirage {
namespace search {

using mirage::kernel::DTensor;
using mirage::kernel::KNCustomizedOp;
using mirage::kernel::KNOperator;
using mirage::threadblock::STensor;
using mirage::threadblock::TBOperator;
using namespace mirage::layout;
using namespace mirage::type;

// search.cc:625-697.  The candidate list is the one the reference explores (the
// Crosswise16 members are commented out there, :629-637).
std::vector<SmemLayout> get_valid_output_layout(TBOperator const *op, int idx) {
  (void)idx;
  static std::vector<SmemLayout> const explore = {
      SmemRowMajor,
      SmemColumnMajor,
      SmemRowMajorTensorOpMultiplicand_Crosswise32,
      SmemRowMajorTensorOpMultiplicand_Crosswise64,
      SmemColumnMajorTensorOpMultiplicand_Crosswise32,
      SmemColumnMajorTensorOpMultiplicand_Crosswise64,
  };
  switch (op->op_type) {
    case TB_INPUT_OP:
      return explore;
    case TB_MATMUL_OP: {
      SmemLayout const a = op->input_tensors[0].layout, b = op->input_tensors[1].layout;
      bool const pair =
          (a == SmemRowMajor && b == SmemColumnMajor) ||
          (a == SmemRowMajorTensorOpMultiplicand_Crosswise32 &&
           b == SmemColumnMajorTensorOpMultiplicand_Crosswise32) ||
          (a == SmemRowMajorTensorOpMultiplicand_Crosswise64 &&
           b == SmemColumnMajorTensorOpMultiplicand_Crosswise64);
      return pair ? explore : std::vector<SmemLayout>{};
    }
    case TB_OUTPUT_OP: {
      SmemLayout const in = op->input_tensors[0].layout;
      if (in == SmemRowMajor || in == SmemRowMajorTensorOpMultiplicand_Crosswise16 ||
          in == SmemRowMajorTensorOpMultiplicand_Crosswise32 ||
          in == SmemRowMajorTensorOpMultiplicand_Crosswise64) {
        return {in};
      }
      return {};
    }
    case TB_EXP_OP:
    case TB_SILU_OP:  // extension operator, same rule as exp
    case TB_DIV_OP:
    case TB_ADD_OP:
    case TB_MUL_OP:  // extension operator, same rule as add
    case TB_CONCAT_0_OP:
    case TB_CONCAT_1_OP:
    case TB_CONCAT_2_OP:
      return {op->input_tensors[0].layout};
    case TB_REDUCTION_0_OP:
    case TB_REDUCTION_1_OP:
    case TB_REDUCTION_2_OP:
    case TB_REDUCTION_0_TO_DIMX_OP:
    case TB_REDUCTION_1_TO_DIMX_OP:
    case TB_REDUCTION_2_TO_DIMX_OP: {
      SmemLayout const in = op->input_tensors[0].layout;
      if (in == SmemRowMajor || in == SmemColumnMajor) {
        return {in};
      }
      return {};
    }
    default:
      return {};
  }
}

// What the cost of `op` may depend on: the layouts of the device tensors it reads, of those it
// writes (an input operator only publishes its tensor: none) and, for a customized operator,
// of its loaders' tiles.
std::vector<int> cost_layouts(KNOperator const *op) {
  std::vector<int> key;
  if (op->op_type == KN_INPUT_OP) {
    return key;
  }
  for (DTensor const &t : op->input_tensors) {
    key.push_back((int)t.layout);
  }
  for (DTensor const &t : op->output_tensors) {
    key.push_back((int)t.layout);
  }
  if (op->op_type == KN_CUSTOMIZED_OP) {
    auto const *c = static_cast<KNCustomizedOp const *>(op);
    for (TBOperator *bop : c->bgraph.operators) {
      if (bop->op_type == TB_INPUT_OP) {
        key.push_back((int)bop->output_tensors[0].layout);
      }
    }
  }
  return key;
}

namespace {

// cost of an operator whose profile() reports that nothing runs it
constexpr float kUnrunnable = -1.0f;

struct Searcher {
  mirage::kernel::Graph &g;
  LayoutSearchConfig const &cfg;
  LayoutSearchResult res;
  // (operator, layouts its time depends on) -> ms.  The layouts: those of the device tensors
  // it reads and writes, then those of its loaders' tiles.
  std::map<std::pair<int, std::vector<int>>, float> known;
  // Customized operators that took a fused kernel under given device-tensor layouts: the
  // kernel stages operands its own way, so the tiles' layouts cannot change that time.
  std::map<std::pair<int, std::vector<int>>, float> fused_cost;
  std::vector<int> best;                                    // snapshot of every layout
  bool have_best = false;

  Searcher(mirage::kernel::Graph &graph, LayoutSearchConfig const &c) : g(graph), cfg(c) {}

  // every layout slot of the graph, in the order the search assigns them
  template <typename F>
  void for_each_slot(F f) {
    for (KNOperator *op : g.operators) {
      for (DTensor &t : op->output_tensors) {
        f(reinterpret_cast<int &>(t.layout));
      }
      if (op->op_type == KN_CUSTOMIZED_OP) {
        auto *c = static_cast<KNCustomizedOp *>(op);
        for (TBOperator *bop : c->bgraph.operators) {
          for (STensor &t : bop->output_tensors) {
            f(reinterpret_cast<int &>(t.layout));
          }
        }
      }
    }
  }

  void set_dtensor_layout(int op_idx, int ts_idx, DmemLayout l) {
    DTensor &t = g.operators[op_idx]->output_tensors[ts_idx];
    t.layout = l;
    for (KNOperator *op : g.operators) {
      for (DTensor &in : op->input_tensors) {
        if (in.guid == t.guid) {
          in.layout = l;
        }
      }
      // the loaders and savers of a customized operator keep their own copies of the device
      // tensors; the lowered program takes the layouts from those
      if (op->op_type == KN_CUSTOMIZED_OP) {
        for (TBOperator *bop : static_cast<KNCustomizedOp *>(op)->bgraph.operators) {
          if (bop->op_type == TB_INPUT_OP) {
            auto *in = static_cast<mirage::threadblock::TBInputOp *>(bop);
            if (in->dtensor.guid == t.guid) {
              in->dtensor.layout = l;
            }
          } else if (bop->op_type == TB_OUTPUT_OP) {
            auto *out = static_cast<mirage::threadblock::TBOutputOp *>(bop);
            if (out->dtensor.guid == t.guid) {
              out->dtensor.layout = l;
            }
          }
        }
      }
    }
  }

  static void set_stensor_layout(KNCustomizedOp *c, int bop_idx, int bts_idx, SmemLayout l) {
    STensor &t = c->bgraph.operators[bop_idx]->output_tensors[bts_idx];
    t.layout = l;
    for (TBOperator *bop : c->bgraph.operators) {
      for (STensor &in : bop->input_tensors) {
        if (in.guid == t.guid) {
          in.layout = l;
        }
      }
    }
  }

  float op_cost(int op_idx) {
    KNOperator *op = g.operators[op_idx];
    std::vector<int> key = cost_layouts(op);
    auto it = known.find({op_idx, key});
    if (it != known.end()) {
      return it->second;
    }
    std::vector<int> device_key;
    for (int l : key) {
      if (l < (int)SmemRowMajor) {
        device_key.push_back(l);
      }
    }
    auto fl = fused_cost.find({op_idx, device_key});
    if (fl != fused_cost.end()) {
      return fl->second;
    }
    float ms;
    if (cfg.cost) {
      ms = cfg.cost(op);
    } else {
      ProfileResult r;
      bool const ran = op->profile(r);
      ms = ran ? r.run_time : kUnrunnable;
      mi355_launch_info li{};
      if (ran && op->op_type == KN_CUSTOMIZED_OP && mi355_last_launch(&li) == MI355_OK &&
          li.kernel_id != MI355_KERNEL_F16_INTERP) {
        fused_cost[{op_idx, device_key}] = ms;
      }
    }
    res.measurements++;
    known[{op_idx, key}] = ms;
    return ms;
  }

  // update_best_graph, search.cc:765-777
  void evaluate() {
    if (res.assignments >= cfg.max_assignments) {
      res.truncated = true;
      return;
    }
    float total = 0.0f;
    bool runnable = true;
    for (int i = 0; i < (int)g.operators.size(); i++) {
      float const ms = op_cost(i);
      runnable = runnable && ms != kUnrunnable;
      total += ms;
    }
    res.assignments++;
    if (!runnable) {
      // an operator no kernel of the backend runs under these layouts: not a candidate
      res.unrunnable++;
      return;
    }
    if (!have_best) {
      res.first_run_time = res.worst_run_time = total;
    }
    res.worst_run_time = total > res.worst_run_time ? total : res.worst_run_time;
    if (!have_best || total < res.best_run_time) {
      have_best = true;
      res.best_run_time = total;
      best.clear();
      for_each_slot([&](int &l) { best.push_back(l); });
    }
  }

  // optimize_layout(g, op_idx, ts_idx, bop_idx, bts_idx), search.cc:703-763
  void walk(int op_idx, int ts_idx, int bop_idx, int bts_idx) {
    if (res.truncated) {
      return;
    }
    if (bop_idx != -1) {
      auto *c = static_cast<KNCustomizedOp *>(g.operators[op_idx]);
      if (bop_idx >= (int)c->bgraph.operators.size()) {
        walk(op_idx + 1, 0, -1, -1);
        return;
      }
      TBOperator *bop = c->bgraph.operators[bop_idx];
      if (bts_idx >= (int)bop->output_tensors.size()) {
        walk(op_idx, ts_idx, bop_idx + 1, 0);
        return;
      }
      SmemLayout const before = bop->output_tensors[bts_idx].layout;
      for (SmemLayout l : get_valid_output_layout(bop, bts_idx)) {
        set_stensor_layout(c, bop_idx, bts_idx, l);
        walk(op_idx, ts_idx, bop_idx, bts_idx + 1);
      }
      set_stensor_layout(c, bop_idx, bts_idx, before);
      return;
    }
    if (op_idx >= (int)g.operators.size()) {
      evaluate();
      return;
    }
    KNOperator *op = g.operators[op_idx];
    if (ts_idx >= (int)op->output_tensors.size()) {
      if (op->op_type == KN_CUSTOMIZED_OP) {
        walk(op_idx, ts_idx, 0, 0);
      } else {
        walk(op_idx + 1, 0, -1, -1);
      }
      return;
    }
    DmemLayout const before = op->output_tensors[ts_idx].layout;
    for (DmemLayout l : {DmemRowMajor, DmemColumnMajor}) {
      if (op->op_type == KN_MATMUL_OP && l != DmemRowMajor) {
        continue;
      }
      set_dtensor_layout(op_idx, ts_idx, l);
      walk(op_idx, ts_idx + 1, -1, -1);
    }
    set_dtensor_layout(op_idx, ts_idx, before);
  }

  void apply_best() {
    size_t n = 0;
    int op_idx = 0;
    for (KNOperator *op : g.operators) {
      for (int ts = 0; ts < (int)op->output_tensors.size(); ts++) {
        set_dtensor_layout(op_idx, ts, (DmemLayout)best[n++]);
      }
      if (op->op_type == KN_CUSTOMIZED_OP) {
        auto *c = static_cast<KNCustomizedOp *>(op);
        for (int b = 0; b < (int)c->bgraph.operators.size(); b++) {
          for (int ts = 0; ts < (int)c->bgraph.operators[b]->output_tensors.size(); ts++) {
            set_stensor_layout(c, b, ts, (SmemLayout)best[n++]);
          }
        }
      }
      op_idx++;
    }
  }
};

}  // namespace

void optimize_layout(mirage::kernel::Graph &g, LayoutSearchResult *result,
                     LayoutSearchConfig const *config) {
  LayoutSearchConfig const defaults;
  LayoutSearchConfig const &cfg = config != nullptr ? *config : defaults;
  Searcher s(g, cfg);
  bool const measure = !cfg.cost;
  if (measure) {
    MIRAGE_CHECK(mi355_set_option(MI355_OPT_PLAN_SMEM_LAYOUT, 1) == MI355_OK,
                 "optimize_layout: the backend refused to honour declared layouts");
  }
  s.walk(0, 0, -1, -1);
  if (measure) {
    mi355_set_option(MI355_OPT_PLAN_SMEM_LAYOUT, 0);
  }
  if (s.have_best) {
    s.apply_best();
    json j;
    mirage::kernel::to_json(j, g);
    s.res.best_graph = j.dump();
  }
  if (result != nullptr) {
    *result = s.res;
  }
}

}  // namespace search
}  // namespace mirage

// ---- C facade -------------------------------------------------------------------
extern "C" {

struct mirage_layout_stats {
  long long assignments;
  long long measurements;
  long long unrunnable;
  int truncated;
  float first_ms, best_ms, worst_ms;
};

// cost(user, operator index, the layouts the operator's cost may depend on, their count) in
// ms; NULL measures with KNOperator::profile.  The layouts: those of the device tensors the
// operator reads, then of those it writes (DmemLayout values), then of its loaders' tiles
// (SmemLayout values); none for an input operator.
typedef float (*mirage_layout_cost_fn)(void *user, int op_index, int const *layouts, int n);

int mirage_optimize_layout(void *graph, long long max_assignments, mirage_layout_cost_fn cost,
                           void *user, mirage_layout_stats *out) {
  auto &G = *static_cast<mirage::kernel::Graph *>(graph);
  mirage::search::LayoutSearchConfig cfg;
  if (max_assignments > 0) {
    cfg.max_assignments = max_assignments;
  }
  if (cost != nullptr) {
    cfg.cost = [&G, cost, user](mirage::kernel::KNOperator *op) {
      int index = 0;
      while (G.operators[index] != op) {
        index++;
      }
      std::vector<int> const layouts = mirage::search::cost_layouts(op);
      return cost(user, index, layouts.data(), (int)layouts.size());
    };
  }
  mirage::search::LayoutSearchResult r;
  mirage::search::optimize_layout(G, &r, &cfg);
  if (out != nullptr) {
    out->assignments = r.assignments;
    out->measurements = r.measurements;
    out->unrunnable = r.unrunnable;
    out->truncated = r.truncated ? 1 : 0;
    out->first_ms = r.first_run_time;
    out->best_ms = r.best_run_time;
    out->worst_ms = r.worst_run_time;
  }
  return 0;
}

}  // extern "C"
