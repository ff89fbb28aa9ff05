// Layout selection for a verified kernel graph: the reference's
// KernelGraphGenerator::{get_valid_output_layout, optimize_layout, update_best_graph}
// (src/search/search.cc:625-777) as free functions.
//
// The search walks every kernel-level output tensor (row- or column-major; a matmul
// result stays row-major) and, inside every customized operator, every tile a
// thread-block operator defines (the layouts its operator admits), profiles each
// complete assignment with KNOperator::profile and keeps the fastest.
//
// What a layout means on this backend.  A device tensor's layout is the storage order of
// its fp16 data (DmemColumnMajor: each matrix column by column): loaders, savers and the
// kernel-level operators honour it, and it decides which kernel a customized operator gets --
// the fused kernels read key / value and weight tiles in either order at different speeds and
// store rows only, so a column-major result runs on the interpreter.  A tile's layout is its
// LDS layout while the fp16 interpreter runs with MI355_OPT_PLAN_SMEM_LAYOUT = 1 (row- or
// column-major, unpadded or padded against bank conflicts); a fused kernel stages operands
// its own way.  The cost of an operator is therefore measured once per distinct set of the
// layouts it depends on (cost_layouts), and once per set of device-tensor layouts when that
// measurement ran on a fused kernel.
#pragma once

#include "mirage/kernel/graph.h"
#include <functional>
#include <string>
#include <vector>

namespace mirage {
namespace search {

// Layouts the `idx`-th output tile of a thread-block operator may take, given the
// layouts of its inputs (search.cc:625-697).  Empty: the inputs' layouts rule the
// operator out.
std::vector<mirage::layout::SmemLayout>
    get_valid_output_layout(mirage::threadblock::TBOperator const *op, int idx);

// The layouts the cost of `op` may depend on: those of the device tensors it reads, then of
// those it writes, then (customized operator) of its loaders' tiles; none for an input operator.
std::vector<int> cost_layouts(mirage::kernel::KNOperator const *op);

struct LayoutSearchConfig {
  // Assignments evaluated at most; the search stops there and reports `truncated`.
  long long max_assignments = 1 << 22;
  // Cost of one operator under the graph's current layouts, in milliseconds.  Must
  // depend on nothing but the operator and cost_layouts(operator).  Empty:
  // KNOperator::profile with the backend honouring declared loader layouts.
  std::function<float(mirage::kernel::KNOperator *)> cost;
};

struct LayoutSearchResult {
  long long assignments = 0;   // complete layout assignments evaluated
  long long measurements = 0;  // operator costs actually measured (the rest were known: same
                               // layouts seen before, or a fused kernel under the same
                               // device-tensor layouts)
  long long unrunnable = 0;    // assignments under which some operator has no kernel to run on
                               // (KNOperator::profile returned false): counted, never chosen
  bool truncated = false;
  float first_run_time = 0.0f;  // total of the first runnable assignment evaluated
  float best_run_time = 0.0f;
  float worst_run_time = 0.0f;
  std::string best_graph;  // JSON of the graph under the best assignment
};

// Leaves `g` under the best assignment found (every tensor's and tile's `layout`,
// and the copies its consumers hold).  A graph with no valid assignment is left as
// it was and reports assignments == 0.
void optimize_layout(mirage::kernel::Graph &g, LayoutSearchResult *result = nullptr,
                     LayoutSearchConfig const *config = nullptr);

}  // namespace search
}  // namespace mirage
