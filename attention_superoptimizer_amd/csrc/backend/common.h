// Shared state and helpers of the gfx950 backend (internal; not part of the ABI).
#pragma once

#include "mi355_abi.h"
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

namespace mi355 {

// Fingerprint ring constants (reference include/mirage/type.h:26-34).
constexpr uint32_t FP_P = 227;
constexpr uint32_t FP_Q = 113;
constexpr uint32_t FP_EXP_BASE = 3;
constexpr uint32_t FP_PQ = 25651;
constexpr uint32_t FP_P_MUL_Q_MOD_1 = 227;
constexpr uint32_t FP_Q_MUL_P_MOD_1 = 25425;

// Operator type codes (reference include/mirage/type.h:50-62, 79-103).
enum : int {
  KN_EXP_OP = 1007,
  KN_ADD_OP = 1008,
  KN_MUL_OP = 1009,
  KN_DIV_OP = 1010,
  KN_SILU_OP = 1011,  // extension
  TB_INPUT_OP = 2001,
  TB_OUTPUT_OP = 2002,
  TB_MATMUL_OP = 2003,
  TB_EXP_OP = 2007,
  TB_ADD_OP = 2008,
  TB_MUL_OP = 2009,
  TB_DIV_OP = 2010,
  TB_SILU_OP = 2012,  // extension
  TB_REDUCTION_0_OP = 2101,
  TB_REDUCTION_2_TO_DIMX_OP = 2106,
  TB_CONCAT_0_OP = 2200,
  TB_CONCAT_2_OP = 2202,
};

extern thread_local int tls_queue;  // the calling thread's queue, see mi355_queue_select

struct State {
  bool ready = false;
  int device = 0;
  // Work is enqueued on the calling host thread's selected queue (queue 0 unless the
  // thread chose another); the others exist so independent candidates can overlap their
  // small kernels and host threads can enqueue side by side.
  hipStream_t queues[MI355_NUM_QUEUES] = {};
  hipStream_t stream() const { return queues[tls_queue]; }
  char *arena = nullptr;
  size_t arena_bytes = 0;
  // device copies of the lookup tables, reference layout
  uint16_t *exp_tbl = nullptr, *div_p = nullptr, *div_q = nullptr;
  int *flag = nullptr;        // device scratch of mi355_fp_equal: one int per queue, 64 bytes apart
  int *flag_host = nullptr;   // pinned mirror, same layout
  int *queue_flag() const { return flag + 16 * tls_queue; }
  int *queue_flag_host() const { return flag_host + 16 * tls_queue; }
  int *cmp_host = nullptr;    // MI355_COMPARE_SLOTS mismatch flags of deferred compares, in
                              // pinned host memory
  int *cmp_slots = nullptr;   // the same memory as the device addresses it
  hipEvent_t marks[MI355_NUM_MARKS][MI355_NUM_QUEUES] = {};
  hipEvent_t ev0[MI355_NUM_QUEUES] = {}, ev1[MI355_NUM_QUEUES] = {};  // timer pair per queue
  hipEvent_t pace[MI355_NUM_QUEUES][2] = {};  // markers that bound how far a timed loop runs ahead
  int max_lds = 65536;
  // staging of batched launches (mi355_customized_fp_batch): per queue a small ring of
  // pinned host / device buffer pairs that carry the program records of one call
  static constexpr int kBatchSlots = 16;
  static constexpr size_t kBatchSlotBytes = (size_t)256 << 10;
  struct BatchSlot {
    char *host = nullptr;
    char *dev = nullptr;
    hipEvent_t copied = nullptr;  // the host buffer may be rewritten once this has passed
  };
  BatchSlot batch[MI355_NUM_QUEUES][kBatchSlots];
  int batch_next[MI355_NUM_QUEUES] = {};
  // what the last customized-op call of each queue launched (a queue is driven by one host
  // thread at a time, so per-queue records never mix)
  mi355_launch_info launches[MI355_NUM_QUEUES] = {};
  mi355_launch_info &last() { return launches[tls_queue]; }
  int force_interpreter = 0;
  int attention_mode = 0;  // 0 auto, 1 latency kernel only, 2 throughput kernel when it fits
  int fp_vector_dot_only = 0;  // 1: fingerprint matmuls never take the matrix-core kernels
  int fp_big_tiles = 1;        // 0: large kernel-level matmuls keep 64 x 64 tiles
  int fp_big_tiles_ok = 1;     // 0: the self-check of the 128-row tile kernels failed on this
                               // device / build: they stay off whatever fp_big_tiles says
  int plan_smem_layout = 0;  // 1: loader tiles take the LDS layout their plan declares
  int direct_lanes = 0;      // MI355_OPT_DIRECT_LANES
  int gemm_mode = 0;         // MI355_OPT_GEMM_MODE
  int f16_matmul_route = 0;  // MI355_OPT_F16_MATMUL_ROUTE
  // phase timestamps of the direct-staging attention kernel (MI355_OPT_PHASE_TRACE): while
  // set, launches of that kernel record six wall-clock stamps per wavefront here
  unsigned long long *phase_trace = nullptr;        // null while tracing is off
  unsigned long long *phase_trace_store = nullptr;  // the allocation (first use of the option)
  size_t phase_trace_bytes = 0;
  // fused-kernel workspace: fp16 range sums of split for-loops
  // (each queue has its own slice of scratch_base, so concurrent queues never share)
  size_t scratch_bytes = 0;  // per queue
  char *scratch_base = nullptr;
  void *scratch() const {
    return scratch_base == nullptr ? nullptr : scratch_base + (size_t)tls_queue * scratch_bytes;
  }
  // residue planes of the matrix-core fingerprint matmul (per queue, like scratch)
  size_t planes_bytes = 0;
  char *planes_base = nullptr;
  char *planes() const {
    return planes_base == nullptr ? nullptr : planes_base + (size_t)tls_queue * planes_bytes;
  }
};

State &state();

// Matrix-core fingerprint matmul (fp_mfma.hip): whether a single matmul is large enough to
// repay the extra launch that splits its operands into residue planes, and its launch.
bool mfma_matmul_pays(int batch, int m, int n, int k);
int launch_mfma_matmul(uint16_t const *A, uint16_t const *B, uint16_t *C, int batch, int m, int n,
                       int k);
int sync_all_queues();
// Drops what mi355_customized_profile keeps of its last call per queue (tb_interp.hip).
void drop_profile_replays();
// The vendor library's GEMM on the calling thread's queue (vendor_gemm.cc): row-major C =
// A . B for `batch` matrices, each operand in either storage order; MI355_ERR_UNSUPPORTED
// when the library cannot be loaded.  vendor_gemm_release drops its per-queue handles.
int vendor_gemm(void const *A, void const *B, void *C, int batch, int m, int n, int k, int a_column_major,
                int b_column_major);
int vendor_gemm_release();
// Looks up the device address of the file-scope scratch array behind
// mi355_customized_fp_static (tb_interp.hip); called by mi355_init with `device` current.
int static_scratch_setup(int device);
int fail(int code, char const *fmt, ...);

#define MI355_HIP(expr)                                                             \
  do {                                                                              \
    hipError_t e_ = (expr);                                                         \
    if (e_ != hipSuccess) {                                                         \
      return ::mi355::fail(MI355_ERR_HIP, "%s failed: %s (%s:%d)", #expr,           \
                           hipGetErrorString(e_), __FILE__, __LINE__);              \
    }                                                                               \
  } while (0)

#define MI355_REQUIRE_INIT()                                                        \
  do {                                                                              \
    if (!::mi355::state().ready) {                                                  \
      return ::mi355::fail(MI355_ERR_NOT_INITIALISED, "mi355_init has not run");    \
    }                                                                               \
  } while (0)

// x mod 25651 / 227 / 113 for 32-bit x.  The compiler lowers `%` by a constant to
// a multiply-high; kept as functions so every kernel spells it the same way.
__device__ __forceinline__ uint32_t mod_pq(uint32_t x) { return x % FP_PQ; }
__device__ __forceinline__ uint32_t mod_p(uint32_t x) { return x % FP_P; }
__device__ __forceinline__ uint32_t mod_q(uint32_t x) { return x % FP_Q; }

// Fingerprint value of a matmul output from its two residue sums (matrix-core kernels).
// u * 25425 + v * 227 has residue u modulo 227 and v modulo 113 whatever the integers u and v
// are (25425 = 113 * 225 = 1 mod 227, 227 = 1 mod 113), so the sums need not be reduced modulo
// their own primes first: each is brought below 25651 and one more reduction finishes.
// sum_p may be negative (operands recentred to [-113, 113]), |sum_p| < 2^31 - 2^17; adding
// 83715 * 25651 makes it non-negative without changing a residue.  sum_q >= 0.
__device__ __forceinline__ uint32_t fp_from_residue_sums(int sum_p, int sum_q) {
  uint32_t const a = (static_cast<uint32_t>(sum_p) + 2147373465u) % FP_PQ;  // unsigned: wraps by definition
  uint32_t const b = static_cast<uint32_t>(sum_q) % FP_PQ;
  return (a * FP_Q_MUL_P_MOD_1 + b * FP_P_MUL_Q_MOD_1) % FP_PQ;
}

// The fingerprint lookup tables in device memory and the ring operations built on them
// (kernel-level operators, and the operand prologue of the matrix-core matmul).
struct FpTables {
  uint16_t const *exp_tbl, *div_p, *div_q;
};

__device__ __forceinline__ uint32_t fp_exp_value(FpTables t, uint32_t x) {
  // reference element_unary_kernel.cu:85-89
  return (t.exp_tbl[x % FP_Q] * FP_Q_MUL_P_MOD_1) % FP_PQ;
}

__device__ __forceinline__ uint32_t fp_div_value(FpTables t, uint32_t x, uint32_t y) {
  // reference element_binary_kernel.cu:155-160
  uint32_t z = (x % FP_P) * t.div_p[y % FP_P] * FP_Q_MUL_P_MOD_1 +
               (x % FP_Q) * t.div_q[y % FP_Q] * FP_P_MUL_Q_MOD_1;
  return z % FP_PQ;
}

__device__ __forceinline__ uint32_t fp_silu_value(FpTables t, uint32_t x) {
  // extension: x / (1 + exp(-x)) from the ring primitives above
  uint32_t neg = (FP_PQ - x) % FP_PQ;
  uint32_t den = (1u + fp_exp_value(t, neg)) % FP_PQ;
  return fp_div_value(t, x, den);
}

inline FpTables tables() {
  State &s = state();
  return FpTables{s.exp_tbl, s.div_p, s.div_q};
}

}  // namespace mi355
