// Batched probabilistic verification of candidate kernel graphs: the device half
// of the reference's KernelGraphGenerator::verify / have_same_fingerprint
// (src/search/search.cc:569-623), restated for many candidates at once.
//
// The reference verifies one candidate at a time: fingerprint() of every operator
// (a device-wide sync after each), then one blocking has_same_fingerprint per
// output and permutation.  Here every candidate's fingerprint kernels and one
// on-device compare per (reference output, candidate output) pair are enqueued
// back to back; the host synchronises once per batch and resolves the output
// permutations from the compare matrix.
#pragma once

#include "mirage/kernel/graph.h"
#include <cstdint>
#include <vector>

namespace mirage {
namespace search {

// Tensors of `g` that no operator of `g` consumes, in creation order
// (search.cc:580-593: `num_consumers[i] == 0`).
std::vector<mirage::kernel::DTensor> graph_outputs(mirage::kernel::Graph const &g);

struct VerifyStats {
  int kernel_ops = 0;         // operators fingerprinted (inputs included)
  int customized_ops = 0;     // of which customized
  int compares = 0;           // on-device compares enqueued
  long long fp_bytes = 0;     // 2 B x (input + output elements) over all operators
  long long matmul_macs = 0;  // m*n*k over kernel-level and thread-block matmuls
  double enqueue_seconds = 0; // host time spent lowering and enqueueing (verify_batch)
  double wait_seconds = 0;    // host time spent in the final synchronisation
};

// equal[i] = 1 iff candidate i has as many outputs as `reference_outputs` and some
// permutation of them is fingerprint-equal to the reference outputs (same dtype,
// layout and dims, search.cc:611-619).  Every operator of every candidate is
// fingerprinted first.  input_seed == 0 fills inputs as the reference does
// (`idx % 25651`, src/kernel/cuda/input_kernel.cu:56-61); otherwise input number j of
// each graph holds uniform values generated from (input_seed, j), so graphs built
// over the same inputs see the same data (the batched operators read inputs number j of
// equal element count through the first such graph's tensor, so every candidate's tensors
// must stay allocated until the verdicts are in).  The reference outputs must already hold
// their fingerprints.  At most MI355_COMPARE_SLOTS compares per call.
void verify_batch(std::vector<mirage::kernel::Graph *> const &candidates,
                  std::vector<mirage::kernel::DTensor> const &reference_outputs,
                  uint64_t input_seed, std::vector<uint8_t> &equal,
                  VerifyStats *stats = nullptr);

// The same in two calls, so that several batches can be in flight: while the device works
// on one, the caller builds and submits the next.  verify_batch_begin lowers and enqueues
// everything from worker threads (one per backend queue) and returns at once;
// verify_batch_end waits for exactly this batch's compares and fills `equal`.
// `reference_to_fingerprint` != nullptr: that graph (whose outputs `reference_outputs` are)
// is fingerprinted as part of the batch; nullptr: the caller has already enqueued its
// fingerprints on its own queue.  Between the two calls the caller must not enqueue device
// work on the worker queues itself, and the candidates, the reference and their tensors
// must stay alive.  At most 32 batches, MI355_COMPARE_SLOTS compares in all, may be in flight
// (begun and not yet ended): a batch owns its compare slots and its pair of marks until
// verify_batch_end has read them, and a verify_batch_begin that finds no free pair or no free
// stretch of slots aborts with a message rather than reuse what a live batch still owns.
// How many backend queues (and worker threads) a batch is dealt over, MI355_NUM_QUEUES by
// default.  Successive batches take successive groups of queues, so with two batches in
// flight and 2 queues per batch each batch has half of the queues to itself: twice as many
// candidates share every launch and the batches' chains of dependent launches run side by
// side instead of one after the other.
void set_verify_queues_per_batch(int queues);
struct VerifyTicket;
VerifyTicket *verify_batch_begin(std::vector<mirage::kernel::Graph *> const &candidates,
                                 std::vector<mirage::kernel::DTensor> const &reference_outputs,
                                 uint64_t input_seed,
                                 mirage::kernel::Graph *reference_to_fingerprint = nullptr);
void verify_batch_end(VerifyTicket *ticket, std::vector<uint8_t> &equal, VerifyStats *stats = nullptr);

// fingerprint() of every operator of one graph with the same input convention.
void fingerprint_graph(mirage::kernel::Graph const &g, uint64_t input_seed,
                       VerifyStats *stats = nullptr);

}  // namespace search
}  // namespace mirage
