// Batched verification of candidate kernel graphs (reference
// KernelGraphGenerator::verify / have_same_fingerprint, src/search/search.cc:569-623).
// One synchronisation per batch: fingerprint kernels and compares are enqueued back to
// back on the backend stream and only the compare bits come back.
#include "mirage/search/verify.h"

#include "mi355_abi.h"
#include "mirage/kernel/device_memory_manager.h"
#include "mirage/utils/hip_types.h"

#include <algorithm>
#include <chrono>
#include <condition_variable>
#include <deque>
#include <map>
#include <functional>
#include <memory>
#include <mutex>
#include <numeric>
#include <thread>
#include <unordered_map>
#include <unordered_set>

namespace mirage {
namespace kernel {
// kernel_device.cc: the lowered program of a customized operator and its bound pointers
void lower_customized(KNCustomizedOp const &op, bool fingerprint, mi355_plan *plan,
                      void const **inputs, void **outputs);
}  // namespace kernel

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

// Inputs depend on nothing: the inputs of all the graphs given are filled by as few
// launches as the backend's tensor list allows.  Input number j of every graph draws from
// (input_seed, j).
static void fill_inputs(std::vector<kernel::Graph const *> const &graphs, uint64_t input_seed) {
  kernel::require_device("fingerprint_graph");
  uint16_t *ptrs[MI355_MAX_FILL_TENSORS];
  size_t counts[MI355_MAX_FILL_TENSORS];
  uint64_t seeds[MI355_MAX_FILL_TENSORS];
  int pending = 0;
  auto flush = [&]() {
    if (pending > 0) {
      MI355_CALL(mi355_fp_fill_many(ptrs, counts, seeds, pending, input_seed == 0 ? 1 : 0));
      pending = 0;
    }
  };
  for (kernel::Graph const *g : graphs) {
    uint64_t ordinal = 0;
    for (KNOperator *op : g->operators) {
      if (op->op_type != KN_INPUT_OP) {
        continue;
      }
      DTensor const &t = op->output_tensors[0];
      ptrs[pending] = t.fp_ptr;
      counts[pending] = t.num_elements();
      seeds[pending] = input_seed ^ (ordinal << 40);
      ordinal++;
      if (++pending == MI355_MAX_FILL_TENSORS) {
        flush();
      }
    }
  }
  flush();
}

void fingerprint_graph(kernel::Graph const &g, uint64_t input_seed, VerifyStats *stats) {
  fill_inputs({&g}, input_seed);
  for (KNOperator *op : g.operators) {
    account(op, stats);
    if (op->op_type != KN_INPUT_OP) {
      op->fingerprint();
    }
  }
}

// Fingerprints several independent graphs on the calling thread's queue, round by round.
// In a round every graph advances through its unary operators and reductions (enqueued
// one by one) up to its next matmul, element-wise binary or customized operator; those
// are collected and submitted together (mi355_fp_matmul_many, mi355_fp_binary_many,
// mi355_customized_fp_batch: a handful of launches for all of them).  The queue is in
// order, so an operator's producers are always ahead of it.
static void fingerprint_graphs(std::vector<kernel::Graph *> const &graphs, uint64_t input_seed,
                               VerifyStats *stats) {
  size_t const n = graphs.size();
  std::vector<size_t> cursor(n, 0);
  fill_inputs(std::vector<kernel::Graph const *>(graphs.begin(), graphs.end()), input_seed);
  // Input number j of every graph is filled from (input_seed, j), so inputs j of two graphs
  // with the same element count hold the same values (candidates of one problem: all of them).
  // The batched operators below read such an input through the first graph's tensor: the
  // backend then sees one operand where there were many copies, splits it into residue planes
  // once per launch, and the launch's programs share its cache lines.
  std::unordered_map<void const *, uint16_t *> first_equal;
  {
    std::map<std::pair<uint64_t, size_t>, uint16_t *> by_content;
    for (kernel::Graph *g : graphs) {
      uint64_t ordinal = 0;
      for (KNOperator *op : g->operators) {
        if (op->op_type != KN_INPUT_OP) {
          continue;
        }
        DTensor const &t = op->output_tensors[0];
        auto it = by_content.emplace(std::make_pair(ordinal, (size_t)t.num_elements()), t.fp_ptr).first;
        first_equal[t.fp_ptr] = it->second;
        ordinal++;
      }
    }
  }
  auto shared_input = [&](uint16_t *p) -> uint16_t * {
    auto it = first_equal.find(p);
    return it == first_equal.end() ? p : it->second;
  };
  for (kernel::Graph *g : graphs) {
    for (KNOperator *op : g->operators) {
      account(op, stats);
    }
  }
  std::vector<mi355_plan> plans;
  std::vector<void const *> ins;
  std::vector<void *> outs;
  int b_op[MI355_MAX_BINARY_OPS], b_nd[MI355_MAX_BINARY_OPS];
  uint16_t const *b_in1[MI355_MAX_BINARY_OPS], *b_in2[MI355_MAX_BINARY_OPS];
  uint16_t *b_out[MI355_MAX_BINARY_OPS];
  int b_d1[4 * MI355_MAX_BINARY_OPS], b_d2[4 * MI355_MAX_BINARY_OPS], b_od[4 * MI355_MAX_BINARY_OPS];
  uint16_t const *m_a[MI355_MAX_MATMULS], *m_b[MI355_MAX_MATMULS];
  uint16_t *m_c[MI355_MAX_MATMULS];
  int m_batch[MI355_MAX_MATMULS], m_m[MI355_MAX_MATMULS], m_n[MI355_MAX_MATMULS], m_k[MI355_MAX_MATMULS];
  int matmuls = 0;
  auto flush_matmuls = [&]() {
    if (matmuls > 0) {
      MI355_CALL(mi355_fp_matmul_many(m_a, m_b, m_c, m_batch, m_m, m_n, m_k, matmuls));
      matmuls = 0;
    }
  };
  int binaries = 0;
  auto flush_binaries = [&]() {
    if (binaries > 0) {
      MI355_CALL(mi355_fp_binary_many(b_op, b_in1, b_d1, b_in2, b_d2, b_out, b_od, b_nd, binaries));
      binaries = 0;
    }
  };
  for (;;) {
    plans.clear();
    ins.clear();
    outs.clear();
    bool any = false;
    for (size_t k = 0; k < n; k++) {
      std::vector<KNOperator *> const &ops = graphs[k]->operators;
      while (cursor[k] < ops.size()) {
        KNOperator *op = ops[cursor[k]++];
        if (op->op_type == KN_INPUT_OP) {
          continue;
        }
        any = true;
        if (op->op_type == KN_MATMUL_OP) {
          DTensor const &a = op->input_tensors[0], &b = op->input_tensors[1];
          int const nd = a.num_dims;
          int batch = 1;
          for (int d = 0; d < nd - 2; d++) {
            batch *= a.dim[d];
          }
          m_a[matmuls] = shared_input(a.fp_ptr);
          m_b[matmuls] = shared_input(b.fp_ptr);
          m_c[matmuls] = op->output_tensors[0].fp_ptr;
          m_batch[matmuls] = batch;
          m_m[matmuls] = a.dim[nd - 2];
          m_k[matmuls] = a.dim[nd - 1];
          m_n[matmuls] = b.dim[nd - 1];
          if (++matmuls == MI355_MAX_MATMULS) {
            flush_matmuls();
          }
          break;
        }
        if (op->op_type == KN_ADD_OP || op->op_type == KN_MUL_OP || op->op_type == KN_DIV_OP) {
          DTensor const &a = op->input_tensors[0], &b = op->input_tensors[1],
                        &o = op->output_tensors[0];
          bool small = true;
          for (int d = 0; d < o.num_dims; d++) {
            small = small && o.dim[d] <= 65535;
          }
          if (!small || o.num_elements() > 0xffffffffull) {
            op->fingerprint();  // beyond the batched form's index range
            continue;
          }
          b_op[binaries] = op->op_type;
          b_nd[binaries] = o.num_dims;
          b_in1[binaries] = shared_input(a.fp_ptr);
          b_in2[binaries] = shared_input(b.fp_ptr);
          b_out[binaries] = o.fp_ptr;
          for (int d = 0; d < 4; d++) {
            b_d1[4 * binaries + d] = d < o.num_dims ? a.dim[d] : 1;
            b_d2[4 * binaries + d] = d < o.num_dims ? b.dim[d] : 1;
            b_od[4 * binaries + d] = d < o.num_dims ? o.dim[d] : 1;
          }
          if (++binaries == MI355_MAX_BINARY_OPS) {
            flush_binaries();
          }
          break;
        }
        if (op->op_type != KN_CUSTOMIZED_OP) {
          op->fingerprint();
          continue;
        }
        plans.emplace_back();
        ins.resize(ins.size() + MI355_MAX_DMEM_INPUTS, nullptr);
        outs.resize(outs.size() + MI355_MAX_DMEM_OUTPUTS, nullptr);
        kernel::lower_customized(*static_cast<kernel::KNCustomizedOp *>(op), true, &plans.back(),
                                 &ins[ins.size() - MI355_MAX_DMEM_INPUTS],
                                 &outs[outs.size() - MI355_MAX_DMEM_OUTPUTS]);
        for (size_t i = ins.size() - MI355_MAX_DMEM_INPUTS; i < ins.size(); i++) {
          if (ins[i] != nullptr) {
            ins[i] = shared_input(static_cast<uint16_t *>(const_cast<void *>(ins[i])));
          }
        }
        break;
      }
    }
    flush_matmuls();
    flush_binaries();
    if (!plans.empty()) {
      MI355_CALL(mi355_customized_fp_batch(plans.data(), (int)plans.size(), ins.data(), outs.data()));
    }
    if (!any) {
      break;
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

// ---- worker threads ----------------------------------------------------------------
// One host thread per backend queue, started on first use and kept: candidate i of a batch
// is lowered and enqueued by thread i % queues.  A queue is only ever driven by its own
// thread (and by the caller's thread for queue 0 while no batch is being enqueued), which is
// what the backend's per-queue staging memory needs.
namespace {

class WorkerPool {
public:
  static WorkerPool &get() {
    static WorkerPool pool;
    return pool;
  }
  void post(int worker, std::function<void()> job) {
    Worker &w = *workers_[(size_t)worker];
    {
      std::lock_guard<std::mutex> lock(w.m);
      w.jobs.push_back(std::move(job));
    }
    w.cv.notify_one();
  }
  int size() const { return (int)workers_.size(); }

private:
  struct Worker {
    std::thread th;
    std::mutex m;
    std::condition_variable cv;
    std::deque<std::function<void()>> jobs;
    bool stop = false;
  };
  std::vector<std::unique_ptr<Worker>> workers_;

  WorkerPool() {
    for (int i = 0; i < MI355_NUM_QUEUES; i++) {
      workers_.emplace_back(new Worker);
      Worker *w = workers_.back().get();
      w->th = std::thread([w, i]() {
        MI355_CALL(mi355_queue_select(i));
        for (;;) {
          std::function<void()> job;
          {
            std::unique_lock<std::mutex> lock(w->m);
            w->cv.wait(lock, [w]() { return w->stop || !w->jobs.empty(); });
            if (w->jobs.empty()) {
              return;
            }
            job = std::move(w->jobs.front());
            w->jobs.pop_front();
          }
          job();
        }
      });
    }
  }
  ~WorkerPool() {
    for (auto &w : workers_) {
      {
        std::lock_guard<std::mutex> lock(w->m);
        w->stop = true;
      }
      w->cv.notify_one();
      w->th.join();
    }
  }
};

struct Pending {
  std::vector<DTensor> outputs;
  int first_slot = -1;  // no*no slots, row = reference output, column = candidate output
};

}  // namespace

struct VerifyTicket {
  std::vector<kernel::Graph *> candidates;
  std::vector<DTensor> reference_outputs;
  kernel::Graph *reference = nullptr;  // fingerprinted by worker 0 when set
  uint64_t input_seed = 0;
  std::vector<Pending> pend;
  std::vector<uint8_t> possible;  // which (reference, candidate) output pairs can be equal at all
  int first_slot = 0, slots = 0;
  int mark_reference = 0, mark_done = 0;
  int ticket = -1;  // owns mark pair (2 ticket, 2 ticket + 1) and the slot range until the end call
  int reference_queue = 0;
  int workers = 0, first_worker = 0;  // worker w of the batch is pool thread (first_worker + w) % queues
  std::vector<VerifyStats> local;
  std::mutex m;
  std::condition_variable cv;
  bool reference_recorded = false;
  int enqueueing = 0;
  std::chrono::steady_clock::time_point t_begin, t_enqueued;
};

// Compare-slot ranges and mark pairs of the batches in flight.  A range or a mark pair is
// handed out only while no unfinished batch owns it: resetting the slots of a live batch
// would clear mismatch flags the device has already written (its candidates would then read
// back as EQUAL), and sharing a mark with a live batch could drop that batch's wait.
// verify_batch_begin takes both, verify_batch_end gives them back.
namespace {
struct InFlight {
  struct Range {
    int first, count, ticket;
  };
  std::vector<Range> live;
  int next_slot = 0;
  int next_ticket = 0;
  static constexpr int kTickets = MI355_NUM_MARKS / 2;

  bool overlaps(int first, int count, int *end_of_blocker) const {
    for (Range const &r : live) {
      if (r.count > 0 && first < r.first + r.count && r.first < first + count) {
        *end_of_blocker = r.first + r.count;
        return true;
      }
    }
    return false;
  }

  // false: every mark pair is owned, or no free stretch of `count` slots exists
  bool acquire(int count, int *first_slot, int *ticket) {
    if (count < 0 || count > MI355_COMPARE_SLOTS || (int)live.size() >= kTickets) {
      return false;
    }
    int id = -1;
    for (int i = 0; i < kTickets && id < 0; i++) {
      int const cand = (next_ticket + i) % kTickets;
      bool used = false;
      for (Range const &r : live) {
        used = used || r.ticket == cand;
      }
      if (!used) {
        id = cand;
      }
    }
    if (id < 0) {
      return false;
    }
    // first fit from the ring position, wrapping once
    int pos = next_slot;
    bool wrapped = false, found = false;
    for (int guard = 0; guard < 4 * kTickets + 4 && !found; guard++) {
      if (pos + count > MI355_COMPARE_SLOTS) {
        if (wrapped) {
          break;
        }
        wrapped = true;
        pos = 0;
      }
      int blocker_end = 0;
      if (count > 0 && overlaps(pos, count, &blocker_end)) {
        pos = blocker_end;
      } else {
        found = true;
      }
      if (wrapped && pos >= next_slot && !found) {
        break;
      }
    }
    if (!found) {
      return false;
    }
    live.push_back(Range{pos, count, id});
    next_slot = pos + count;
    next_ticket = (id + 1) % kTickets;
    *first_slot = pos;
    *ticket = id;
    return true;
  }

  void release(int ticket) {
    for (size_t i = 0; i < live.size(); i++) {
      if (live[i].ticket == ticket) {
        live.erase(live.begin() + (long)i);
        return;
      }
    }
  }
};
}  // namespace

static std::mutex g_ring_mutex;
static InFlight g_in_flight;
static int g_queues_per_batch = MI355_NUM_QUEUES;
static int g_next_queue = 0;

void set_verify_queues_per_batch(int queues) {
  std::lock_guard<std::mutex> lock(g_ring_mutex);
  g_queues_per_batch = std::max(1, std::min(queues, (int)MI355_NUM_QUEUES));
}

VerifyTicket *verify_batch_begin(std::vector<kernel::Graph *> const &candidates,
                                 std::vector<DTensor> const &reference_outputs,
                                 uint64_t input_seed, kernel::Graph *reference_to_fingerprint) {
  kernel::require_device("verify_batch");
  std::unique_ptr<VerifyTicket> t(new VerifyTicket);
  t->t_begin = std::chrono::steady_clock::now();
  t->candidates = candidates;
  t->reference_outputs = reference_outputs;
  t->reference = reference_to_fingerprint;
  t->input_seed = input_seed;
  size_t const n = candidates.size(), no = reference_outputs.size();
  t->pend.resize(n);
  for (size_t i = 0; i < n; i++) {
    t->pend[i].outputs = graph_outputs(*candidates[i]);
    if (t->pend[i].outputs.size() == no) {
      t->pend[i].first_slot = t->slots;
      t->slots += (int)(no * no);
    }
  }
  MIRAGE_CHECK(t->slots <= MI355_COMPARE_SLOTS, "too many compares for one verify_batch call");
  {
    std::lock_guard<std::mutex> lock(g_ring_mutex);
    int ticket = -1;
    bool const ok = g_in_flight.acquire(t->slots, &t->first_slot, &ticket);
    MIRAGE_CHECK(ok, "too many verification batches in flight: every verify_batch_begin needs a "
                     "free mark pair (32 in all) and a free stretch of compare slots; call "
                     "verify_batch_end on an earlier ticket first");
    t->ticket = ticket;
    t->mark_reference = 2 * ticket;
    t->mark_done = 2 * ticket + 1;
    t->workers = g_queues_per_batch;
    t->first_worker = g_next_queue;
    g_next_queue = (g_next_queue + g_queues_per_batch) % MI355_NUM_QUEUES;
  }
  for (Pending &p : t->pend) {
    if (p.first_slot >= 0) {
      p.first_slot += t->first_slot;
    }
  }
  t->possible.assign((size_t)t->slots, 0);
  MI355_CALL(mi355_fp_equal_reset(t->first_slot, t->slots));
  WorkerPool &pool = WorkerPool::get();
  t->workers = (int)std::min<size_t>((size_t)t->workers, std::max<size_t>(n, 1));
  t->local.resize((size_t)t->workers);
  t->enqueueing = t->workers;
  if (t->reference == nullptr) {
    // the caller has enqueued the reference graph's fingerprints on its own queue: the
    // compares of the other queues start after them
    t->reference_queue = mi355_queue_current();
    MI355_CALL(mi355_mark_record(t->mark_reference));
    t->reference_recorded = true;
  }
  VerifyTicket *const T = t.get();
  for (int w = 0; w < T->workers; w++) {
    pool.post((T->first_worker + w) % pool.size(), [T, w]() {
      size_t const n = T->candidates.size(), no = T->reference_outputs.size();
      if (w == 0 && T->reference != nullptr) {
        T->reference_queue = mi355_queue_current();
        fingerprint_graphs({T->reference}, T->input_seed, &T->local[0]);
        MI355_CALL(mi355_mark_record(T->mark_reference));
        {
          std::lock_guard<std::mutex> lock(T->m);
          T->reference_recorded = true;
        }
        T->cv.notify_all();
      }
      std::vector<kernel::Graph *> mine;
      for (size_t i = (size_t)w; i < n; i += (size_t)T->workers) {
        mine.push_back(T->candidates[i]);
      }
      fingerprint_graphs(mine, T->input_seed, &T->local[(size_t)w]);
      {
        std::unique_lock<std::mutex> lock(T->m);
        T->cv.wait(lock, [T]() { return T->reference_recorded; });
      }
      MI355_CALL(mi355_mark_wait_queue(T->mark_reference, T->reference_queue));
      // this worker's compares, MI355_MAX_COMPARE_PAIRS per launch
      uint16_t const *ca[MI355_MAX_COMPARE_PAIRS], *cb[MI355_MAX_COMPARE_PAIRS];
      size_t cn[MI355_MAX_COMPARE_PAIRS];
      int cs[MI355_MAX_COMPARE_PAIRS];
      int pairs = 0;
      auto flush = [&]() {
        if (pairs > 0) {
          MI355_CALL(mi355_fp_equal_enqueue_many(ca, cb, cn, cs, pairs));
          pairs = 0;
        }
      };
      for (size_t i = (size_t)w; i < n; i += (size_t)T->workers) {
        if (T->pend[i].first_slot < 0) {
          continue;
        }
        for (size_t r = 0; r < no; r++) {
          for (size_t c = 0; c < no; c++) {
            if (!comparable(T->reference_outputs[r], T->pend[i].outputs[c])) {
              continue;
            }
            int const slot = T->pend[i].first_slot + (int)(r * no + c);
            T->possible[(size_t)(slot - T->first_slot)] = 1;
            ca[pairs] = T->reference_outputs[r].fp_ptr;
            cb[pairs] = T->pend[i].outputs[c].fp_ptr;
            cn[pairs] = T->reference_outputs[r].num_elements();
            cs[pairs] = slot;
            if (++pairs == MI355_MAX_COMPARE_PAIRS) {
              flush();
            }
            T->local[(size_t)w].compares++;
            T->local[(size_t)w].fp_bytes += 2 * (long long)T->reference_outputs[r].fingerprint_size();
          }
        }
      }
      flush();
      MI355_CALL(mi355_mark_record(T->mark_done));
      {
        std::lock_guard<std::mutex> lock(T->m);
        if (--T->enqueueing == 0) {
          T->t_enqueued = std::chrono::steady_clock::now();
        }
      }
      T->cv.notify_all();
    });
  }
  return t.release();
}

void verify_batch_end(VerifyTicket *ticket, std::vector<uint8_t> &equal, VerifyStats *stats) {
  std::unique_ptr<VerifyTicket> t(ticket);
  size_t const n = t->candidates.size(), no = t->reference_outputs.size();
  equal.assign(n, 0);
  auto const t_wait = std::chrono::steady_clock::now();
  {
    std::unique_lock<std::mutex> lock(t->m);
    t->cv.wait(lock, [&]() { return t->enqueueing == 0; });
  }
  MI355_CALL(mi355_mark_wait_host(t->mark_done));
  std::vector<uint8_t> same((size_t)t->slots, 0);
  MI355_CALL(mi355_fp_equal_read(t->first_slot, t->slots, same.data()));
  {
    std::lock_guard<std::mutex> lock(g_ring_mutex);
    g_in_flight.release(t->ticket);  // slots read, marks waited for: both may be handed out again
  }
  if (stats != nullptr) {
    auto const t_done = std::chrono::steady_clock::now();
    for (VerifyStats const &l : t->local) {
      stats->kernel_ops += l.kernel_ops;
      stats->customized_ops += l.customized_ops;
      stats->compares += l.compares;
      stats->fp_bytes += l.fp_bytes;
      stats->matmul_macs += l.matmul_macs;
    }
    stats->enqueue_seconds += std::chrono::duration<double>(t->t_enqueued - t->t_begin).count();
    stats->wait_seconds += std::chrono::duration<double>(t_done - std::max(t_wait, t->t_enqueued)).count();
  }
  std::vector<int> perm(no);
  for (size_t i = 0; i < n; i++) {
    if (t->pend[i].first_slot < 0) {
      continue;
    }
    std::iota(perm.begin(), perm.end(), 0);
    do {  // search.cc:605-609: any output permutation may match
      bool ok = true;
      for (size_t r = 0; r < no && ok; r++) {
        int const slot = t->pend[i].first_slot + (int)(r * no + perm[r]);
        ok = t->possible[(size_t)(slot - t->first_slot)] && same[(size_t)(slot - t->first_slot)];
      }
      if (ok) {
        equal[i] = 1;
        break;
      }
    } while (std::next_permutation(perm.begin(), perm.end()));
  }
}

void verify_batch(std::vector<kernel::Graph *> const &candidates,
                  std::vector<DTensor> const &reference_outputs, uint64_t input_seed,
                  std::vector<uint8_t> &equal, VerifyStats *stats) {
  verify_batch_end(verify_batch_begin(candidates, reference_outputs, input_seed, nullptr), equal, stats);
}

}  // namespace search
}  // namespace mirage

// ---- C facade -----------------------------------------------------------------------
extern "C" {

typedef struct mirage_verify_stats {
  int kernel_ops, customized_ops, compares;
  long long fp_bytes, matmul_macs;
  double enqueue_seconds, wait_seconds;
} mirage_verify_stats;

static void export_stats(mirage::search::VerifyStats const &s, mirage_verify_stats *out) {
  if (out != nullptr) {
    out->kernel_ops = s.kernel_ops;
    out->customized_ops = s.customized_ops;
    out->compares = s.compares;
    out->fp_bytes = s.fp_bytes;
    out->matmul_macs = s.matmul_macs;
    out->enqueue_seconds = s.enqueue_seconds;
    out->wait_seconds = s.wait_seconds;
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
// Two-call form: several batches may be in flight.  `fingerprint_reference` != 0: the
// reference graph is fingerprinted as part of the batch (on a worker's queue); otherwise it
// must already have been, on the calling thread's queue.  The candidates, the reference and
// their tensors stay alive until the matching mirage_verify_batch_end returns.
void *mirage_verify_batch_begin(void *const *candidates, int n, void *reference,
                                unsigned long long input_seed, int fingerprint_reference) {
  std::vector<mirage::kernel::Graph *> c(n);
  for (int i = 0; i < n; i++) {
    c[i] = static_cast<mirage::kernel::Graph *>(candidates[i]);
  }
  mirage::kernel::Graph *ref = static_cast<mirage::kernel::Graph *>(reference);
  return mirage::search::verify_batch_begin(c, mirage::search::graph_outputs(*ref), input_seed,
                                            fingerprint_reference ? ref : nullptr);
}

// The bookkeeping of slot ranges and mark pairs by itself (no device): a scratch instance for
// host-side tests.  acquire returns 0 and fills first_slot / ticket, or -1 when nothing is free.
using mirage::search::InFlight;
void *mirage_verify_ring_create(void) { return new InFlight(); }
void mirage_verify_ring_destroy(void *ring) { delete static_cast<InFlight *>(ring); }
int mirage_verify_ring_acquire(void *ring, int slots, int *first_slot, int *ticket) {
  return static_cast<InFlight *>(ring)->acquire(slots, first_slot, ticket) ? 0 : -1;
}
void mirage_verify_ring_release(void *ring, int ticket) { static_cast<InFlight *>(ring)->release(ticket); }

void mirage_verify_set_queues_per_batch(int queues) {
  mirage::search::set_verify_queues_per_batch(queues);
}

int mirage_verify_batch_end(void *ticket, int n, unsigned char *equal, mirage_verify_stats *stats) {
  std::vector<uint8_t> eq;
  mirage::search::VerifyStats s;
  mirage::search::verify_batch_end(static_cast<mirage::search::VerifyTicket *>(ticket), eq, &s);
  for (int i = 0; i < n && i < (int)eq.size(); i++) {
    equal[i] = eq[i];
  }
  export_stats(s, stats);
  return 0;
}

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
