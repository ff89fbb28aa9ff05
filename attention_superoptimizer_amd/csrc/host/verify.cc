// Batched verification of candidate kernel graphs (reference
// KernelGraphGenerator::verify / have_same_fingerprint, src/search/search.cc:569-623).
// One synchronisation per batch: fingerprint kernels and compares are enqueued back to
// back on the backend stream and only the compare bits come back.
#include "mirage/search/verify.h"

#include "mi355_abi.h"
#include "mirage/kernel/device_memory_manager.h"
#include "mirage/utils/hip_types.h"

#include <algorithm>
#include <numeric>
#include <unordered_set>

namespace mirage {
namespace search {

using kernel::DTensor;
using kernel::KNOperator;
using namespace mirage::type;

#define MI355_CALL(expr) MIRAGE_CHECK((expr) == MI355_OK, mi355_last_error())

std::vector<DTensor> graph_outputs(kernel::Graph const &g) {
  std::unordered_set<size_t> consumed;
  for (KNOperator const *op : g.operators) {
    for (DTensor const &t : op->input_tensors) {
      consumed.insert(t.guid);
    }
  }
  std::vector<DTensor> outs;
  for (KNOperator const *op : g.operators) {
    for (DTensor const &t : op->output_tensors) {
      if (consumed.count(t.guid) == 0) {
        outs.push_back(t);
      }
    }
  }
  return outs;
}

static void account(KNOperator const *op, VerifyStats *stats) {
  if (stats == nullptr) {
    return;
  }
  stats->kernel_ops++;
  for (DTensor const &t : op->input_tensors) {
    stats->fp_bytes += (long long)t.fingerprint_size();
  }
  for (DTensor const &t : op->output_tensors) {
    stats->fp_bytes += (long long)t.fingerprint_size();
  }
  if (op->op_type == KN_MATMUL_OP) {
    DTensor const &A = op->input_tensors[0];
    stats->matmul_macs +=
        (long long)op->output_tensors[0].num_elements() * A.dim[A.num_dims - 1];
  } else if (op->op_type == KN_CUSTOMIZED_OP) {
    stats->customized_ops++;
    auto const *c = static_cast<kernel::KNCustomizedOp const *>(op);
    long long const launches = (long long)c->bgraph.grid_dim.x * c->bgraph.grid_dim.y *
                               c->bgraph.grid_dim.z * c->bgraph.forloop_range;
    for (threadblock::TBOperator const *t : c->bgraph.operators) {
      if (t->op_type == TB_MATMUL_OP) {
        threadblock::STensor const &A = t->input_tensors[0];
        stats->matmul_macs += launches * (long long)t->output_tensors[0].num_elements() *
                              A.dim[A.num_dims - 1];
      }
    }
  }
}

void fingerprint_graph(kernel::Graph const &g, uint64_t input_seed, VerifyStats *stats) {
  kernel::require_device("fingerprint_graph");
  uint64_t ordinal = 0;
  for (KNOperator *op : g.operators) {
    account(op, stats);
    if (op->op_type == KN_INPUT_OP && input_seed != 0) {
      DTensor const &t = op->output_tensors[0];
      MI355_CALL(mi355_fp_fill_uniform(t.fp_ptr, t.num_elements(),
                                       input_seed ^ (ordinal << 40)));
    } else {
      op->fingerprint();
    }
    if (op->op_type == KN_INPUT_OP) {
      ordinal++;
    }
  }
}

static bool comparable(DTensor const &a, DTensor const &b) {
  if (a.data_type != b.data_type || a.layout != b.layout || a.num_dims != b.num_dims) {
    return false;
  }
  for (int i = 0; i < a.num_dims; i++) {
    if (a.dim[i] != b.dim[i]) {
      return false;
    }
  }
  return true;
}

void verify_batch(std::vector<kernel::Graph *> const &candidates,
                  std::vector<DTensor> const &reference_outputs, uint64_t input_seed,
                  std::vector<uint8_t> &equal, VerifyStats *stats) {
  kernel::require_device("verify_batch");
  size_t const n = candidates.size(), no = reference_outputs.size();
  equal.assign(n, 0);
  struct Pending {
    std::vector<DTensor> outputs;
    int first_slot = -1;  // no*no slots, row = reference output, column = candidate output
  };
  std::vector<Pending> pend(n);
  int slots = 0;
  for (size_t i = 0; i < n; i++) {
    pend[i].outputs = graph_outputs(*candidates[i]);
    if (pend[i].outputs.size() == no) {
      pend[i].first_slot = slots;
      slots += (int)(no * no);
    }
  }
  MIRAGE_CHECK(slots <= MI355_COMPARE_SLOTS, "too many compares for one verify_batch call");
  MI355_CALL(mi355_fp_equal_reset(0, slots));
  // which (reference, candidate) output pairs can be equal at all
  std::vector<uint8_t> possible((size_t)slots, 0);
  for (size_t i = 0; i < n; i++) {
    fingerprint_graph(*candidates[i], input_seed, stats);
    if (pend[i].first_slot < 0) {
      continue;
    }
    for (size_t r = 0; r < no; r++) {
      for (size_t c = 0; c < no; c++) {
        if (!comparable(reference_outputs[r], pend[i].outputs[c])) {
          continue;
        }
        int const slot = pend[i].first_slot + (int)(r * no + c);
        possible[slot] = 1;
        MI355_CALL(mi355_fp_equal_enqueue(reference_outputs[r].fp_ptr,
                                          pend[i].outputs[c].fp_ptr,
                                          reference_outputs[r].num_elements(), slot));
        if (stats != nullptr) {
          stats->compares++;
          stats->fp_bytes += 2 * (long long)reference_outputs[r].fingerprint_size();
        }
      }
    }
  }
  std::vector<uint8_t> same((size_t)slots, 0);
  MI355_CALL(mi355_fp_equal_collect(0, slots, same.data()));
  std::vector<int> perm(no);
  for (size_t i = 0; i < n; i++) {
    if (pend[i].first_slot < 0) {
      continue;
    }
    std::iota(perm.begin(), perm.end(), 0);
    do {  // search.cc:605-609: any output permutation may match
      bool ok = true;
      for (size_t r = 0; r < no && ok; r++) {
        int const slot = pend[i].first_slot + (int)(r * no + perm[r]);
        ok = possible[slot] && same[slot];
      }
      if (ok) {
        equal[i] = 1;
        break;
      }
    } while (std::next_permutation(perm.begin(), perm.end()));
  }
}

}  // namespace search
}  // namespace mirage

// ---- C facade -----------------------------------------------------------------------
extern "C" {

typedef struct mirage_verify_stats {
  int kernel_ops, customized_ops, compares;
  long long fp_bytes, matmul_macs;
} mirage_verify_stats;

static void export_stats(mirage::search::VerifyStats const &s, mirage_verify_stats *out) {
  if (out != nullptr) {
    out->kernel_ops = s.kernel_ops;
    out->customized_ops = s.customized_ops;
    out->compares = s.compares;
    out->fp_bytes = s.fp_bytes;
    out->matmul_macs = s.matmul_macs;
  }
}

int mirage_graph_fingerprint(void *graph, unsigned long long input_seed,
                             mirage_verify_stats *stats) {
  mirage::search::VerifyStats s;
  mirage::search::fingerprint_graph(*static_cast<mirage::kernel::Graph *>(graph), input_seed, &s);
  export_stats(s, stats);
  return 0;
}

// Candidates are compared with the outputs of `reference` (which must already be
// fingerprinted, e.g. by mirage_graph_fingerprint with the same seed).
int mirage_verify_batch(void *const *candidates, int n, void *reference,
                        unsigned long long input_seed, unsigned char *equal,
                        mirage_verify_stats *stats) {
  std::vector<mirage::kernel::Graph *> c(n);
  for (int i = 0; i < n; i++) {
    c[i] = static_cast<mirage::kernel::Graph *>(candidates[i]);
  }
  std::vector<mirage::kernel::DTensor> ref =
      mirage::search::graph_outputs(*static_cast<mirage::kernel::Graph *>(reference));
  std::vector<uint8_t> eq;
  mirage::search::VerifyStats s;
  mirage::search::verify_batch(c, ref, input_seed, eq, &s);
  for (int i = 0; i < n; i++) {
    equal[i] = eq[i];
  }
  export_stats(s, stats);
  return 0;
}

}  // extern "C"
