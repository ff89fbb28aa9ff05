// Lifetime, memory and timing entry points of the gfx950 backend.
//
// Stands in for the device half of the reference's DeviceMemoryManager
// (src/kernel/device_memory_manager.cu:26-96): one arena allocation, the three
// fingerprint lookup tables, and the event pairs every profile() uses.
#include "common.h"
#include <atomic>
#include <cstring>
#include <vector>

namespace mi355 {

static State g_state;
// which queues have recorded under each mark since its last host wait
static std::atomic<unsigned> g_mark_bits[MI355_NUM_MARKS];
thread_local char g_error[512] = "";  // per host thread: several may enqueue side by side

State &state() { return g_state; }

int fail(int code, char const *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

thread_local int tls_queue = 0;

int sync_all_queues() {
  State &s = state();
  for (int i = 0; i < MI355_NUM_QUEUES; i++) {
    if (s.queues[i] != nullptr) {
      MI355_HIP(hipStreamSynchronize(s.queues[i]));
    }
  }
  return MI355_OK;
}

}  // namespace mi355

using namespace mi355;

extern "C" char const *mi355_last_error(void) { return g_error; }

extern "C" int mi355_is_initialised(void) { return state().ready ? 1 : 0; }

extern "C" int mi355_init(size_t arena_bytes, void **arena_base) {
  State &s = state();
  if (s.ready) {
    if (arena_base != nullptr) {
      *arena_base = s.arena;
    }
    if (arena_bytes > s.arena_bytes) {
      return fail(MI355_ERR_INVALID, "backend already initialised with a smaller arena");
    }
    return MI355_OK;
  }
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0) {
    return fail(MI355_ERR_NO_DEVICE, "no HIP device visible (%s)",
                e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
  }
  MI355_HIP(hipSetDevice(0));
  hipDeviceProp_t prop;
  MI355_HIP(hipGetDeviceProperties(&prop, 0));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    return fail(MI355_ERR_NO_DEVICE, "device 0 is %s; this backend is built for gfx950 only",
                prop.gcnArchName);
  }
  int optin = 0;
  if (hipDeviceGetAttribute(&optin, hipDeviceAttributeMaxSharedMemoryPerBlock, 0) == hipSuccess &&
      optin > 0) {
    s.max_lds = optin;
  }
  if (int rc = static_scratch_setup(s.device)) {
    return rc;
  }
  for (int i = 0; i < MI355_NUM_QUEUES; i++) {
    MI355_HIP(hipStreamCreate(&s.queues[i]));  // default priority, all of them
  }
  tls_queue = 0;
  MI355_HIP(hipMalloc(reinterpret_cast<void **>(&s.arena), arena_bytes));
  s.arena_bytes = arena_bytes;
  // Tables: exp[i] = 3^i mod 227 (i < 113); div_p / div_q = modular inverses with
  // entries 0 and 1 both mapped to 1 (device_memory_manager.cu:41-90).
  uint16_t exp_h[FP_Q], divp_h[FP_P], divq_h[FP_Q];
  exp_h[0] = 1;
  for (uint32_t i = 1; i < FP_Q; i++) {
    exp_h[i] = static_cast<uint16_t>((exp_h[i - 1] * FP_EXP_BASE) % FP_P);
  }
  if ((exp_h[FP_Q - 1] * FP_EXP_BASE) % FP_P != 1) {
    return fail(MI355_ERR_INVALID, "exp base does not have order Q modulo P");
  }
  auto inverse_table = [](uint16_t *t, uint32_t mod) {
    for (uint32_t i = 0; i < mod; i++) {
      t[i] = 1;
      for (uint32_t j = 1; j < mod; j++) {
        if ((i * j) % mod == 1) {
          t[i] = static_cast<uint16_t>(j);
        }
      }
    }
  };
  inverse_table(divp_h, FP_P);
  inverse_table(divq_h, FP_Q);
  uint16_t *tbl = nullptr;
  MI355_HIP(hipMalloc(reinterpret_cast<void **>(&tbl), 1024));
  s.exp_tbl = tbl;         // 113 entries, 226 B -> next at 240 B
  s.div_p = tbl + 120;     // 227 entries, 454 B -> next at 704 B
  s.div_q = tbl + 352;     // 113 entries
  MI355_HIP(hipMemcpy(s.exp_tbl, exp_h, sizeof(exp_h), hipMemcpyHostToDevice));
  MI355_HIP(hipMemcpy(s.div_p, divp_h, sizeof(divp_h), hipMemcpyHostToDevice));
  MI355_HIP(hipMemcpy(s.div_q, divq_h, sizeof(divq_h), hipMemcpyHostToDevice));
  MI355_HIP(hipMalloc(reinterpret_cast<void **>(&s.flag), 256));
  MI355_HIP(hipHostMalloc(reinterpret_cast<void **>(&s.flag_host), 256, hipHostMallocDefault));
  MI355_HIP(hipHostMalloc(reinterpret_cast<void **>(&s.cmp_host), sizeof(int) * MI355_COMPARE_SLOTS,
                          hipHostMallocDefault));
  memset(s.cmp_host, 0, sizeof(int) * MI355_COMPARE_SLOTS);
  MI355_HIP(hipHostGetDevicePointer(reinterpret_cast<void **>(&s.cmp_slots), s.cmp_host, 0));
  for (int m = 0; m < MI355_NUM_MARKS; m++) {
    for (int q = 0; q < MI355_NUM_QUEUES; q++) {
      MI355_HIP(hipEventCreateWithFlags(&s.marks[m][q], hipEventDisableTiming));
    }
    g_mark_bits[m].store(0);
  }
  for (int q = 0; q < MI355_NUM_QUEUES; q++) {
    MI355_HIP(hipEventCreate(&s.ev0[q]));
    MI355_HIP(hipEventCreate(&s.ev1[q]));
    MI355_HIP(hipEventCreateWithFlags(&s.pace[q][0], hipEventDisableTiming));
    MI355_HIP(hipEventCreateWithFlags(&s.pace[q][1], hipEventDisableTiming));
  }
  for (int q = 0; q < MI355_NUM_QUEUES; q++) {
    for (int b = 0; b < State::kBatchSlots; b++) {
      State::BatchSlot &slot = s.batch[q][b];
      MI355_HIP(hipHostMalloc(reinterpret_cast<void **>(&slot.host), State::kBatchSlotBytes,
                              hipHostMallocDefault));
      MI355_HIP(hipMalloc(reinterpret_cast<void **>(&slot.dev), State::kBatchSlotBytes));
      MI355_HIP(hipEventCreateWithFlags(&slot.copied, hipEventDisableTiming));
    }
    s.batch_next[q] = 0;
  }
  s.scratch_bytes = (size_t)64 << 20;  // per queue
  MI355_HIP(hipMalloc(reinterpret_cast<void **>(&s.scratch_base),
                      s.scratch_bytes * MI355_NUM_QUEUES));
  s.planes_bytes = (size_t)128 << 20;  // per queue
  MI355_HIP(hipMalloc(reinterpret_cast<void **>(&s.planes_base),
                      s.planes_bytes * MI355_NUM_QUEUES));
  s.ready = true;
  if (arena_base != nullptr) {
    *arena_base = s.arena;
  }
  // the kernels whose loads the compiler cannot see are checked once on the device they run on
  return mi355_fp_big_tiles_check(nullptr);
}

extern "C" int mi355_shutdown(void) {
  State &s = state();
  if (!s.ready) {
    return MI355_OK;
  }
  if (int rc = sync_all_queues()) {
    return rc;
  }
  vendor_gemm_release();  // its handles are bound to the queues destroyed below
  drop_profile_replays();
  for (int q = 0; q < MI355_NUM_QUEUES; q++) {
    MI355_HIP(hipEventDestroy(s.ev0[q]));
    MI355_HIP(hipEventDestroy(s.ev1[q]));
    MI355_HIP(hipEventDestroy(s.pace[q][0]));
    MI355_HIP(hipEventDestroy(s.pace[q][1]));
  }
  MI355_HIP(hipFree(s.arena));
  MI355_HIP(hipFree(s.exp_tbl));
  MI355_HIP(hipFree(s.flag));
  MI355_HIP(hipHostFree(s.flag_host));
  MI355_HIP(hipHostFree(s.cmp_host));
  for (int m = 0; m < MI355_NUM_MARKS; m++) {
    for (int q = 0; q < MI355_NUM_QUEUES; q++) {
      MI355_HIP(hipEventDestroy(s.marks[m][q]));
    }
  }
  MI355_HIP(hipFree(s.scratch_base));
  MI355_HIP(hipFree(s.planes_base));
  s.planes_base = nullptr;
  if (s.phase_trace_store != nullptr) {
    MI355_HIP(hipFree(s.phase_trace_store));
  }
  for (int q = 0; q < MI355_NUM_QUEUES; q++) {
    for (int b = 0; b < State::kBatchSlots; b++) {
      MI355_HIP(hipHostFree(s.batch[q][b].host));
      MI355_HIP(hipFree(s.batch[q][b].dev));
      MI355_HIP(hipEventDestroy(s.batch[q][b].copied));
    }
  }
  for (int i = 0; i < MI355_NUM_QUEUES; i++) {
    MI355_HIP(hipStreamDestroy(s.queues[i]));
  }
  s = State{};
  return MI355_OK;
}

extern "C" int mi355_get_device_info(mi355_device_info *info) {
  MI355_REQUIRE_INIT();
  if (info == nullptr) {
    return fail(MI355_ERR_INVALID, "null info");
  }
  hipDeviceProp_t prop;
  MI355_HIP(hipGetDeviceProperties(&prop, state().device));
  memset(info, 0, sizeof(*info));
  // some driver stacks report an empty marketing name: fall back to the architecture string
  strncpy(info->name, prop.name[0] != '\0' ? prop.name : prop.gcnArchName, sizeof(info->name) - 1);
  strncpy(info->arch, prop.gcnArchName, sizeof(info->arch) - 1);
  info->compute_units = prop.multiProcessorCount;
  info->clock_mhz = prop.clockRate / 1000;
  info->memory_clock_mhz = prop.memoryClockRate / 1000;
  info->lds_bytes_per_block = state().max_lds;
  info->total_memory = prop.totalGlobalMem;
  return MI355_OK;
}

extern "C" int mi355_mark_record(int mark) {
  MI355_REQUIRE_INIT();
  if (mark < 0 || mark >= MI355_NUM_MARKS) {
    return fail(MI355_ERR_INVALID, "mark %d out of range", mark);
  }
  MI355_HIP(hipEventRecord(state().marks[mark][tls_queue], state().stream()));
  g_mark_bits[mark].fetch_or(1u << tls_queue);
  return MI355_OK;
}

extern "C" int mi355_mark_wait_queue(int mark, int queue) {
  MI355_REQUIRE_INIT();
  if (mark < 0 || mark >= MI355_NUM_MARKS || queue < 0 || queue >= MI355_NUM_QUEUES) {
    return fail(MI355_ERR_INVALID, "mark %d / queue %d out of range", mark, queue);
  }
  if (queue != tls_queue && (g_mark_bits[mark].load() & (1u << queue)) != 0) {
    MI355_HIP(hipStreamWaitEvent(state().stream(), state().marks[mark][queue], 0));
  }
  return MI355_OK;
}

extern "C" int mi355_mark_wait_host(int mark) {
  MI355_REQUIRE_INIT();
  if (mark < 0 || mark >= MI355_NUM_MARKS) {
    return fail(MI355_ERR_INVALID, "mark %d out of range", mark);
  }
  unsigned const bits = g_mark_bits[mark].exchange(0);
  for (int q = 0; q < MI355_NUM_QUEUES; q++) {
    if (bits & (1u << q)) {
      MI355_HIP(hipEventSynchronize(state().marks[mark][q]));
    }
  }
  return MI355_OK;
}

extern "C" int mi355_set_option(int option, int value) {
  drop_profile_replays();
  if (option == MI355_OPT_FORCE_INTERPRETER) {
    state().force_interpreter = value;
    return MI355_OK;
  }
  if (option == MI355_OPT_ATTENTION_MODE && value >= 0 && value <= 3) {
    state().attention_mode = value;
    return MI355_OK;
  }
  if (option == MI355_OPT_PLAN_SMEM_LAYOUT && (value == 0 || value == 1)) {
    state().plan_smem_layout = value;
    return MI355_OK;
  }
  if (option == MI355_OPT_FP_MATMUL_ROUTE && value >= 0 && value <= 2) {
    state().fp_vector_dot_only = value == 1;
    state().fp_big_tiles = value != 2;
    return MI355_OK;
  }
  if (option == MI355_OPT_DIRECT_LANES && (value == 0 || value == 1 || value == 4)) {
    state().direct_lanes = value;
    return MI355_OK;
  }
  if (option == MI355_OPT_GEMM_MODE && value >= 0 && value <= 2) {
    state().gemm_mode = value;
    return MI355_OK;
  }
  if (option == MI355_OPT_F16_MATMUL_ROUTE && (value == 0 || value == 1)) {
    state().f16_matmul_route = value;
    return MI355_OK;
  }
  if (option == MI355_OPT_PHASE_TRACE && (value == 0 || value == 1)) {
    MI355_REQUIRE_INIT();
    State &s = state();
    if (value == 1 && s.phase_trace_store == nullptr) {
      s.phase_trace_bytes = (size_t)8 << 20;
      MI355_HIP(hipMalloc(reinterpret_cast<void **>(&s.phase_trace_store), s.phase_trace_bytes));
    }
    s.phase_trace = value == 1 ? s.phase_trace_store : nullptr;
    return MI355_OK;
  }
  return fail(MI355_ERR_INVALID, "unknown option %d", option);
}

namespace mi355 {
__global__ void empty_kernel() {}

// plain device-to-device copy, 16 bytes per lane per step
__global__ void copy_kernel(uint4 const *__restrict__ src, uint4 *__restrict__ dst, size_t n16,
                            unsigned char const *__restrict__ src_tail,
                            unsigned char *__restrict__ dst_tail, int tail) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n16; i += stride) {
    dst[i] = src[i];
  }
  if (blockIdx.x == 0 && (int)threadIdx.x < tail) {
    dst_tail[threadIdx.x] = src_tail[threadIdx.x];
  }
}
}  // namespace mi355

extern "C" int mi355_copy(void *dst, void const *src, size_t bytes) {
  MI355_REQUIRE_INIT();
  if (((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15) != 0) {
    return fail(MI355_ERR_INVALID, "mi355_copy needs 16-byte aligned pointers");
  }
  if (bytes == 0) {
    return MI355_OK;
  }
  size_t n16 = bytes / 16;
  int tail = (int)(bytes % 16);
  size_t blocks = (n16 + 255) / 256;
  blocks = blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks);
  copy_kernel<<<(unsigned)blocks, 256, 0, state().stream()>>>(
      static_cast<uint4 const *>(src), static_cast<uint4 *>(dst), n16,
      static_cast<unsigned char const *>(src) + n16 * 16, static_cast<unsigned char *>(dst) + n16 * 16,
      tail);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_launch_floor(int iters, float *us) {
  MI355_REQUIRE_INIT();
  if (iters < 1 || us == nullptr) {
    return fail(MI355_ERR_INVALID, "bad arguments");
  }
  State &s = state();
  // The same way mi355_customized_profile repeats a call: chains of 256 kernel nodes, one graph
  // launch each, so that the figure is the device's launch-to-launch time and not the host's
  // time per launch call.
  constexpr int kChain = 256;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  MI355_HIP(hipStreamBeginCapture(s.stream(), hipStreamCaptureModeThreadLocal));
  for (int i = 0; i < kChain; i++) {
    empty_kernel<<<1, 64, 0, s.stream()>>>();
  }
  MI355_HIP(hipStreamEndCapture(s.stream(), &graph));
  hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  if (e == hipSuccess) {
    e = hipGraphLaunch(exec, s.stream());  // warm-up
  }
  int const chains = (iters + kChain - 1) / kChain;
  if (e == hipSuccess) {
    e = hipEventRecord(s.ev0[tls_queue], s.stream());
  }
  for (int i = 0; i < chains && e == hipSuccess; i++) {
    e = hipGraphLaunch(exec, s.stream());
  }
  if (e == hipSuccess) {
    e = hipEventRecord(s.ev1[tls_queue], s.stream());
  }
  if (e == hipSuccess) {
    e = hipEventSynchronize(s.ev1[tls_queue]);
  }
  float ms = 0.0f;
  if (e == hipSuccess) {
    e = hipEventElapsedTime(&ms, s.ev0[tls_queue], s.ev1[tls_queue]);
  }
  if (exec != nullptr) {
    (void)hipGraphExecDestroy(exec);
  }
  (void)hipGraphDestroy(graph);
  MI355_HIP(e);
  *us = ms * 1000.0f / ((float)chains * kChain);
  return MI355_OK;
}

extern "C" int mi355_get_tables(void const **exp_tbl, void const **div_p, void const **div_q) {
  MI355_REQUIRE_INIT();
  *exp_tbl = state().exp_tbl;
  *div_p = state().div_p;
  *div_q = state().div_q;
  return MI355_OK;
}

extern "C" int mi355_memcpy_h2d(void *dst, void const *src, size_t bytes) {
  MI355_REQUIRE_INIT();
  if (int rc = sync_all_queues()) {  // work on any queue may still read dst
    return rc;
  }
  MI355_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, state().stream()));
  MI355_HIP(hipStreamSynchronize(state().stream()));
  return MI355_OK;
}

extern "C" int mi355_memcpy_d2h(void *dst, void const *src, size_t bytes) {
  MI355_REQUIRE_INIT();
  if (int rc = sync_all_queues()) {  // src may be produced on any queue
    return rc;
  }
  MI355_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, state().stream()));
  MI355_HIP(hipStreamSynchronize(state().stream()));
  return MI355_OK;
}

extern "C" int mi355_queue_select(int queue) {
  MI355_REQUIRE_INIT();
  State &s = state();
  if (queue < 0 || queue >= MI355_NUM_QUEUES) {
    return fail(MI355_ERR_INVALID, "queue %d out of range [0, %d)", queue, MI355_NUM_QUEUES);
  }
  tls_queue = queue;
  return MI355_OK;
}

extern "C" int mi355_queue_current(void) { return tls_queue; }

extern "C" int mi355_memset(void *dst, int value, size_t bytes) {
  MI355_REQUIRE_INIT();
  MI355_HIP(hipMemsetAsync(dst, value, bytes, state().stream()));
  return MI355_OK;
}

extern "C" int mi355_sync(void) {
  MI355_REQUIRE_INIT();
  return sync_all_queues();
}

extern "C" int mi355_timer_start(void) {
  MI355_REQUIRE_INIT();
  MI355_HIP(hipEventRecord(state().ev0[tls_queue], state().stream()));
  return MI355_OK;
}

extern "C" int mi355_timer_stop(float *ms) {
  MI355_REQUIRE_INIT();
  MI355_HIP(hipEventRecord(state().ev1[tls_queue], state().stream()));
  MI355_HIP(hipEventSynchronize(state().ev1[tls_queue]));
  MI355_HIP(hipEventElapsedTime(ms, state().ev0[tls_queue], state().ev1[tls_queue]));
  return MI355_OK;
}

extern "C" int mi355_phase_trace_read(unsigned long long *stamps, size_t count) {
  MI355_REQUIRE_INIT();
  State &s = state();
  if (stamps == nullptr || s.phase_trace_store == nullptr || count * 8 > s.phase_trace_bytes) {
    return fail(MI355_ERR_INVALID, "no trace buffer, or more stamps asked for than it holds");
  }
  if (int rc = sync_all_queues()) {
    return rc;
  }
  MI355_HIP(hipMemcpy(stamps, s.phase_trace_store, count * 8, hipMemcpyDeviceToHost));
  return MI355_OK;
}

extern "C" int mi355_last_launch(mi355_launch_info *info) {
  if (info == nullptr) {
    return fail(MI355_ERR_INVALID, "null info");
  }
  *info = state().last();
  return MI355_OK;
}
