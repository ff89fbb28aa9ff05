/*
 * mi355_abi.h — C ABI of the MI355X (gfx950) mugraph execution / fingerprint
 * backend.
 *
 * The reference (Mirage) has no C ABI for this path: its host classes call
 * CUDA directly from .cu member functions.  This header is the boundary those
 * member functions bind to instead; each entry point names the reference code
 * it stands in for (paths relative to the reference root).  Plain pointers and
 * sizes only; every function returns 0 on success and a negative code on
 * failure, with mi355_last_error() giving the text.  All device pointers must
 * come from the arena returned by mi355_init() (or any hipMalloc'ed memory).
 * Work is enqueued on one of MI355_NUM_QUEUES backend-owned in-order queues (HIP streams):
 * the queue the calling host thread selected with mi355_queue_select, queue 0 by default.
 * Calls are asynchronous unless stated otherwise.  Several host threads may call at once
 * provided each drives a queue of its own (a queue is driven by one thread at a time);
 * timers, the blocking compare and the launch record are kept per queue.  The reference
 * itself has one stream and a single caller thread; a caller that never selects a queue
 * gets exactly that.
 */
#ifndef MI355_ABI_H
#define MI355_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_OK 0
#define MI355_ERR_NO_DEVICE (-1)
#define MI355_ERR_HIP (-2)
#define MI355_ERR_INVALID (-3)
#define MI355_ERR_UNSUPPORTED (-4)
#define MI355_ERR_NOT_INITIALISED (-5)

/* Limits of the reference's flat-int program
 * (include/mirage/threadblock/serializer/kernel_params.h:25-35). */
#define MI355_MAX_OPERATORS 16
#define MI355_MAX_PARAMETERS 120
#define MI355_MAX_DMEM_INPUTS 4
#define MI355_MAX_DMEM_OUTPUTS 4

/* POD mirror of NewKernelParams plus the launch shape that the reference keeps
 * on threadblock::Graph (include/mirage/threadblock/graph.h:110-116).
 * `parameters` is the reference's serialised per-operator bytecode verbatim
 * (serializer/{input_loader,output_saver,matmul,element_unary,element_binary,
 * reduction,concat}_serializer.h); `smem_bytes` is bgraph.smem_offset, the size
 * of the thread-block graph's STensor address space. */
typedef struct mi355_plan {
  int grid_dim[3];
  int block_dim[3]; /* the plan's logical block shape; a hint on this backend */
  int forloop_range;
  int reduction_dimx;
  int smem_bytes;
  int num_operators;
  int num_parameters;
  int num_dmem_inputs;
  int num_dmem_outputs;
  int operator_types[MI355_MAX_OPERATORS];
  int parameters[MI355_MAX_PARAMETERS];
} mi355_plan;

typedef struct mi355_device_info {
  char name[128];
  char arch[64];
  int compute_units;
  int clock_mhz;
  int memory_clock_mhz;
  int lds_bytes_per_block;
  size_t total_memory;
} mi355_device_info;

/* How a customized op was executed (for reporting / tests). */
typedef struct mi355_launch_info {
  int kernel_id;        /* MI355_KERNEL_* */
  int workgroups;       /* physical workgroups launched */
  int threads;          /* threads per workgroup */
  int lds_bytes;        /* LDS actually requested */
  int row_split;        /* workgroups cooperating on one logical thread block */
} mi355_launch_info;

#define MI355_KERNEL_FP_INTERP 1
#define MI355_KERNEL_F16_INTERP 2
#define MI355_KERNEL_F16_ATTENTION 3 /* fused register-resident attention family */
#define MI355_KERNEL_F16_GEMM 4      /* fused skinny-GEMM family (split for-loop, ordered fix-up) */
#define MI355_KERNEL_F16_COMBINE 5   /* fused fold-partials-and-divide family */
#define MI355_KERNEL_FP_GEMM 6       /* fused fingerprint tiled-matmul family (uint16) */

/* Backend options (mi355_set_option).  FORCE_INTERPRETER = 1 sends every customized op,
 * fp16 or fingerprint, through the generic LDS interpreter instead of a fused kernel
 * (both must agree with the oracle; tests run the two against each other). */
#define MI355_OPT_FORCE_INTERPRETER 1
/* ATTENTION_MODE: 0 = choose by problem size (default), 1 = always a latency
 * variant of the fused attention kernel, 2 = the throughput variant whenever the
 * tile shape allows it, 3 = the latency variant with register-transposed staging
 * only (not the one that streams tiles straight into LDS). */
#define MI355_OPT_ATTENTION_MODE 2
/* PLAN_SMEM_LAYOUT: 0 = the lowering gives every fp16 tile the LDS layout its
 * consumers want (default); 1 = a loader's tile takes the layout its plan declares
 * (the stensor layout word of the input-loader bytecode, values of the reference's
 * include/mirage/layout.h:37-47): the RowMajor family is stored row-major, the
 * ColumnMajor family column-major; the plain layouts are unpadded, the
 * TensorOpMultiplicand_Crosswise{16,32,64} ones pad every row / column by 8, 16 and
 * 32 bytes to spread matrix-core operand fetches over the LDS banks.
 * SmemUnknownLayout leaves the choice to the lowering.  Results do not depend on
 * the layout; this is the knob the layout search (reference
 * src/search/search.cc:625-763) turns with profile() as its cost.  Fused kernels
 * keep their own staging layouts. */
#define MI355_OPT_PLAN_SMEM_LAYOUT 3
/* FP_MATMUL_ROUTE: 0 = fingerprint matmuls (kernel-level and the fused tiled-matmul plans)
 * take the int8 matrix-core kernels whenever their shapes allow (default); 1 = always the
 * packed 4 x 8-bit vector-dot kernels; 2 = as 0, but large kernel-level matmuls keep the
 * 64 x 64 tiles of the smaller ones instead of 128 x 128 tiles staged through LDS.  Results
 * are bit-identical; tests run all three. */
#define MI355_OPT_FP_MATMUL_ROUTE 4
/* PHASE_TRACE: 1 = launches of the direct-staging attention kernel record six wall-clock
 * stamps (100 MHz) per wavefront -- start, loads issued, first tiles landed, arithmetic done,
 * joined, stores issued -- read back with mi355_phase_trace_read; 0 = off (default).  A
 * measurement aid: the traced kernel is a separate instantiation, the normal one carries no
 * trace code. */
#define MI355_OPT_PHASE_TRACE 5
/* DIRECT_LANES: shape of the direct-staging attention kernel.  0 = chosen by the backend
 * (default: wavefronts of two row groups where that still fills the chip; eight
 * single-buffered iteration lanes for a lone row group with a long for-loop); 1 = one row
 * group per wavefront always; 4 = four double-buffered lanes for a lone row group.  Results
 * are identical; a measurement knob that the tests use to cover every instantiation. */
#define MI355_OPT_DIRECT_LANES 6
/* GEMM_MODE: which fused kernel runs a skinny-GEMM plan.  0 = chosen by the backend (one
 * launch with the output tile cut into 16 x 16 pieces for plans that would otherwise leave
 * most of the chip idle; the for-loop cut into ranges, plus a launch that adds them, for
 * plans whose traffic, not the launch, sets the time); 1 = always the range-splitting kernel; 2 = the one-launch
 * kernel wherever it applies.  Both keep the accumulation order of the sequential loop;
 * results agree to the last bit.  A measurement knob that the tests use to cover both. */
#define MI355_OPT_GEMM_MODE 7
/* F16_MATMUL_ROUTE: what runs a kernel-level fp16 matmul (mi355_f16_matmul,
 * mi355_f16_matmul_layout).  0 = this library's kernels (default); 1 = the vendor's BLAS
 * (rocblas_gemm_strided_batched_ex, fp16 in and out, fp32 accumulation, atomics off), which
 * is what the reference calls on its side (cublasGemmStridedBatchedEx,
 * src/kernel/cuda/matmul_kernel.cu:86-131).  rocBLAS is opened at run time on the first
 * such call; when it cannot be, the call fails with MI355_ERR_UNSUPPORTED and nothing else
 * runs in its place.  Both routes accumulate in fp32 and round once; their sums differ in
 * order, so results agree to fp16 rounding, not to the bit. */
#define MI355_OPT_F16_MATMUL_ROUTE 8

/* ---- lifetime ------------------------------------------------------------
 * Replaces DeviceMemoryManager's constructor / destructor
 * (src/kernel/device_memory_manager.cu:26-96): one device allocation of
 * `arena_bytes`, the exp / div lookup tables built and uploaded.  The caller
 * keeps the bump/LIFO bookkeeping (the reference's `offset`) itself. */
int mi355_init(size_t arena_bytes, void **arena_base);
int mi355_shutdown(void);
int mi355_is_initialised(void);
/* message of the calling host thread's most recent failed call */
char const *mi355_last_error(void);
int mi355_get_device_info(mi355_device_info *info);
int mi355_set_option(int option, int value);
/* Mean microseconds per launch of an empty kernel, `iters` launches (rounded up to whole
 * chains of 256 kernel nodes, one graph launch each, as mi355_customized_profile repeats a
 * call) back to back on the backend stream: the floor under any per-launch figure
 * (blocking). */
int mi355_launch_floor(int iters, float *us);
/* Device addresses of the three uint16 tables (113, 227, 113 entries), in the
 * reference's layout: exp[i] = 3^i mod 227; div_p[i], div_q[i] = inverse of i
 * with [0] = [1] = 1 (device_memory_manager.cu:41-90). */
int mi355_get_tables(void const **exp_tbl, void const **div_p, void const **div_q);

/* Blocking copies and sync (the reference uses cudaMemcpy / cudaDeviceSynchronize). */
int mi355_memcpy_h2d(void *dst, void const *src, size_t bytes);
int mi355_memcpy_d2h(void *dst, void const *src, size_t bytes);
int mi355_memset(void *dst, int value, size_t bytes);
/* Asynchronous device-to-device copy by a plain kernel (16-byte aligned pointers).
 * Also the known-size reference that hardware byte counters are scaled against. */
int mi355_copy(void *dst, void const *src, size_t bytes);
int mi355_sync(void);
/* The backend owns MI355_NUM_QUEUES in-order queues (HIP streams, all at the default
 * priority).  Every call enqueues on the queue its host thread selected (queue 0 until the
 * thread selects another), so host threads can enqueue side by side; work on different
 * queues may overlap on the device, which is how a batch of independent candidate graphs
 * fills the chip with its many small kernels (the reference has one stream and a
 * cudaDeviceSynchronize after every fingerprint launch, customized_kernel.cu:676).
 * mi355_sync, the memcpy calls and mi355_fp_equal_collect wait for all queues.  The
 * caller orders dependent work itself: same queue, a mi355_sync in between, or a mark.
 * A queue is driven by one host thread at a time (several entry points enqueue more than
 * one launch and keep per-queue staging memory between them). */
#define MI355_NUM_QUEUES 4
int mi355_queue_select(int queue);
int mi355_queue_current(void); /* the calling thread's queue */
/* Marks order work across queues and let the host wait for part of the work only (the
 * reference has one stream and device-wide syncs, so no counterpart).  mi355_mark_record:
 * everything enqueued so far on the calling thread's queue is "before" (mark, that queue).
 * mi355_mark_wait_queue: work enqueued from now on the calling thread's queue starts after
 * what `queue` recorded under `mark` (a device-side wait; the host does not block; a no-op
 * if nothing was recorded).  mi355_mark_wait_host: blocks until everything recorded under
 * `mark`, on any queue, since the last host wait on it has completed.  A mark is reusable
 * after its host wait. */
#define MI355_NUM_MARKS 64
int mi355_mark_record(int mark);
int mi355_mark_wait_queue(int mark, int queue);
int mi355_mark_wait_host(int mark);

/* ---- fingerprint path (uint16 over Z_25651, integer only) ------------------ */
/* init_input_fingerprint, src/kernel/cuda/input_kernel.cu:56-72: fp[i] = i % 25651 */
int mi355_fp_fill_iota(uint16_t *fp, size_t n);
/* seeded inputs: fp[i] = splitmix64(seed + i) % 25651 (no reference counterpart;
 * the reference's FIXME at input_kernel.cu:59 asks for random inputs) */
int mi355_fp_fill_uniform(uint16_t *fp, size_t n, uint64_t seed);
/* Up to MI355_MAX_FILL_TENSORS input tensors (of one graph or of several) in a single
 * launch (init_input_fingerprint once per tensor in the reference, input_kernel.cu:56-72):
 * tensor i gets `idx % 25651` when iota != 0, else the uniform values of
 * mi355_fp_fill_uniform with seeds[i]. */
#define MI355_MAX_FILL_TENSORS 64
int mi355_fp_fill_many(uint16_t *const *fp, size_t const *n, uint64_t const *seeds, int count,
                       int iota);
/* compute_matmul_fingerprint, src/kernel/cuda/matmul_kernel.cu:145-203 */
int mi355_fp_matmul(uint16_t const *A, uint16_t const *B, uint16_t *C, int batch, int m,
                    int n, int k);
/* Several independent matmuls in one submission (compute_matmul_fingerprint once per
 * operator in the reference, matmul_kernel.cu:175-203): C[i] = A[i] . B[i] with extents
 * batch[i], m[i], n[i], k[i], bit-identical to mi355_fp_matmul of each.  Operands are split
 * once into signed-byte residue planes (mod 227 recentred, mod 113) in backend memory and
 * multiplied with int8 matrix instructions; up to MI355_MAX_MATMULS go out as two launches
 * (one more per tile shape when the list holds matmuls large enough for the kernels that
 * stage operands through LDS), longer lists in groups.  Outputs must not alias inputs of the
 * same call. */
#define MI355_MAX_MATMULS 32
int mi355_fp_matmul_many(uint16_t const *const *A, uint16_t const *const *B, uint16_t *const *C,
                         int const *batch, int const *m, int const *n, int const *k, int count);
/* compute_elementunary_fingerprint, src/kernel/cuda/element_unary_kernel.cu:77-112;
 * op = KN_EXP_OP (1007) or the silu extension (1011) */
int mi355_fp_unary(int op, uint16_t const *in, uint16_t *out, size_t n);
/* compute_elementbinary_fingerprint, src/kernel/cuda/element_binary_kernel.cu:97-199;
 * op = KN_ADD_OP / KN_MUL_OP / KN_DIV_OP (1008 / 1009 / 1010) */
int mi355_fp_binary(int op, uint16_t const *in1, int const *dims1, uint16_t const *in2,
                    int const *dims2, uint16_t *out, int const *dims_out, int num_dims);
/* Self-check of the two fingerprint-matmul kernels that work on 128-row tiles.  They prefetch
 * one operand with loads issued from inline assembly, whose completion the compiler does not
 * track; the build verifies that they use no scratch memory and keep their occupancy, this call
 * verifies the results where they run: a [2048, 512] x [512, 2048] and a [2048, 512] x [512, 1024]
 * product on those kernels against the 64 x 64-tile kernel (ordinary loads), which must agree
 * bit for bit.  mi355_init runs it once; on a difference the 128-row kernels stay off for the
 * process (MI355_OPT_FP_MATMUL_ROUTE cannot switch them back on) and a line goes to stderr.
 * *passed (may be NULL): 1 = equal.  Allocates and frees 30 MB of device memory; blocking.
 * No counterpart in the reference, whose matmul fingerprint is one scalar kernel
 * (src/kernel/cuda/matmul_kernel.cu:133-203). */
int mi355_fp_big_tiles_check(int *passed);
/* `count` <= MI355_MAX_BINARY_OPS independent operators of the kind above in one launch (a
 * verification batch holds one per candidate): operator e uses ops[e], in1[e], in2[e], out[e],
 * num_dims[e] and the dims at dims1 / dims2 / dims_out + 4 * e.  Every dim <= 65535. */
#define MI355_MAX_BINARY_OPS 32
int mi355_fp_binary_many(int const *ops, uint16_t const *const *in1, int const *dims1,
                         uint16_t const *const *in2, int const *dims2, uint16_t *const *out,
                         int const *dims_out, int const *num_dims, int count);
/* compute_reduction_fingerprint, src/kernel/cuda/reduction_kernel.cu:80-133 */
int mi355_fp_reduce(uint16_t const *in, uint16_t *out, size_t n_out, int factor,
                    int in_stride, int out_stride);
/* DTensor::has_same_fingerprint's element loop, src/kernel/cuda/device_tensor_kernel.cu:36-52,
 * done on the device; writes 1/0 to *equal (blocking: 4 bytes come back, not 2 tensors) */
int mi355_fp_equal(uint16_t const *a, uint16_t const *b, size_t n, int *equal);
/* The same compare without the round trip, for verifying many candidates
 * (the verify loop of src/search/search.cc:569-623 calls has_same_fingerprint once per
 * candidate output and blocks each time).  The backend keeps MI355_COMPARE_SLOTS result
 * slots: reset a range, enqueue one compare per slot behind the
 * fingerprint kernels on the backend stream, then collect the range with a single
 * synchronisation; equal[i] = 1/0 for slot first_slot + i.  A slot that several
 * compares target reports their conjunction. */
#define MI355_COMPARE_SLOTS 65536
int mi355_fp_equal_reset(int first_slot, int count);
int mi355_fp_equal_enqueue(uint16_t const *a, uint16_t const *b, size_t n, int slot);
/* `count` <= MI355_MAX_COMPARE_PAIRS compares in one launch: pair i is (a[i], b[i]) of n[i]
 * elements and reports into slots[i]. */
#define MI355_MAX_COMPARE_PAIRS 64
int mi355_fp_equal_enqueue_many(uint16_t const *const *a, uint16_t const *const *b,
                                size_t const *n, int const *slots, int count);
int mi355_fp_equal_collect(int first_slot, int count, uint8_t *equal);
/* The slots live in host memory that the device writes directly: mi355_fp_equal_reset
 * clears a range at once, on the host (the range must not be the target of compares still
 * in flight), and mi355_fp_equal_read reports a range WITHOUT waiting for anything: for
 * callers that have waited for exactly the compares they care about (mi355_mark_wait_host)
 * while other batches are still running. */
int mi355_fp_equal_read(int first_slot, int count, uint8_t *equal);
/* KNCustomizedOp::fingerprint + compute_customizedop_fingerprint,
 * src/kernel/cuda/customized_kernel.cu:307-603,655-678 */
int mi355_customized_fp(mi355_plan const *plan, void const *const *inputs,
                        void *const *outputs);

/* The same fingerprint, for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * It calls no hipMalloc / hipFree and uses none of the memory mi355_init allocated beyond
 * the lookup tables: the partial sums of a split for-loop go to a file-scope device array
 * of MI355_STATIC_SCRATCH_BYTES instead of the backend's scratch slab, and the plan always
 * runs on the generic interpreter (the matrix-core route needs residue planes in allocated
 * memory).  Bit-identical to mi355_customized_fp.  The for-loop is cut into the ranges
 * mi355_customized_fp would take, or into fewer while their partial sums (ranges x output
 * elements x 2 bytes) do not fit the array -- any split gives the same sum in the ring.  A
 * plan of which not even two ranges fit (more than 2 Mi output elements, on a grid small
 * enough to be split) is refused with MI355_ERR_UNSUPPORTED.  Every call on a GPU shares that GPU's array:
 * calls that overlap on one GPU (different queues or host threads) race; calls on one
 * queue are ordered.  Nothing in the array needs clearing between calls. */
#define MI355_STATIC_SCRATCH_BYTES (8 << 20)
int mi355_customized_fp_static(mi355_plan const *plan, void const *const *inputs,
                               void *const *outputs);

/* n independent customized-op fingerprints in one call (the batched form of the entry above
 * for a verification loop that holds many candidates, src/search/search.cc:601-603):
 * operator i reads inputs[4*i .. 4*i+3] and writes outputs[4*i .. 4*i+3].  The operators must
 * not depend on each other: they run as a handful of launches on the caller's queue, each
 * covering many operators (grouped by LDS need; workgroup -> operator by a prefix table in
 * device memory), plus one launch that folds the partial sums of every split for-loop. */
int mi355_customized_fp_batch(mi355_plan const *plans, int n, void const *const *inputs,
                              void *const *outputs);

/* Host-only check of a plan (no device needed): 1 + the largest element index the
 * plan reads from each input / writes to each output, and the LDS the two
 * interpreters would request.  Callers compare the extents with their tensors'
 * element counts before launching; the reference relies on device asserts
 * (include/mirage/threadblock/cuda/input_loader.h:463) instead.  Any pointer may
 * be NULL. */
int mi355_plan_extents(mi355_plan const *plan, long long *in_elems, long long *out_elems,
                       int *lds_bytes_fp, int *lds_bytes_f16);

/* ---- fp16 execution path --------------------------------------------------- */
/* KNCustomizedOp::run + customized_kernel_function,
 * src/kernel/cuda/customized_kernel.cu:39-305,605-613 */
int mi355_customized_run(mi355_plan const *plan, void const *const *inputs,
                         void *const *outputs);
/* KNCustomizedOp::profile, customized_kernel.cu:615-653: `warmup` untimed then
 * `iters` timed launches between two events on the backend stream; *ms = mean.
 * What one call launches is captured once (a stream capture that is not executed) and
 * repeated from there: kernel by kernel, or, for 512 launches and more, 256 calls at a time
 * as one chain of kernel nodes (one graph launch); a call that enqueues anything other than
 * kernels is repeated by calling it.  So the loop times the device: plan matching and
 * parameter set-up cost the host 2.8 - 3.9 us a launch here, more than a 3.5 us kernel takes.
 * The host never runs more than two batches of 1024 launches ahead of the device (a marker
 * per batch, waited for one batch later): with several thousand launches queued every
 * launch takes longer. */
int mi355_customized_profile(mi355_plan const *plan, void const *const *inputs,
                             void *const *outputs, int fingerprint, int warmup, int iters,
                             float *ms);
/* What the last mi355_customized_{fp,run,profile} call launched. */
int mi355_last_launch(mi355_launch_info *info);
/* Copies the first `count` 64-bit stamps the last traced launch wrote (blocking):
 * wavefront w of workgroup g (linear block index) is at [(g * wavefronts + w) * 6 .. + 5]. */
int mi355_phase_trace_read(unsigned long long *stamps, size_t count);

/* init_input<half>, src/kernel/cuda/input_kernel.cu:29-54: x[i] = (half)(i % last_dim) */
int mi355_f16_fill_iota(void *x, size_t n, int last_dim);
/* seeded N(0, std) inputs rounded to fp16 (counter-based: splitmix64 + Box-Muller) */
int mi355_f16_fill_normal(void *x, size_t n, float std, uint64_t seed);
/* KNMatmulOp::profile's GEMM, src/kernel/cuda/matmul_kernel.cu:28-143 (row-major) */
int mi355_f16_matmul(void const *A, void const *B, void *C, int batch, int m, int n, int k);
/* The same with the operands' storage order stated, as matmul_kernel.cu:61-76 turns
 * DmemColumnMajor operands into transposed GEMM arguments: a column-major [rows, cols]
 * matrix holds element (r, c) at c * rows + r.  C is row-major (matmul_kernel.cu:74-75). */
int mi355_f16_matmul_layout(void const *A, void const *B, void *C, int batch, int m, int n, int k,
                            int a_column_major, int b_column_major);
/* out[b][c][r] = in[b][r][c] for `batch` [rows, cols] matrices: the row-major copy of a
 * DmemColumnMajor tensor (call it with rows = the tensor's columns and cols = its rows) for
 * the element-wise operators and reductions, which index their inputs flat as
 * element_unary_kernel.cu:30-42 and element_binary_kernel.cu:30-51 do. */
int mi355_f16_transpose(void const *in, void *out, int batch, int rows, int cols);
/* execute_elementunary, src/kernel/cuda/element_unary_kernel.cu:30-42 */
int mi355_f16_unary(int op, void const *in, void *out, size_t n);
/* execute_elementbinary, src/kernel/cuda/element_binary_kernel.cu:30-51, with the
 * fingerprint kernel's per-dim broadcast rule so both paths agree on shapes */
int mi355_f16_binary(int op, void const *in1, int const *dims1, void const *in2,
                     int const *dims2, void *out, int const *dims_out, int num_dims);
/* execute_reduction, src/kernel/cuda/reduction_kernel.cu:30-42 is a stand-in in the
 * reference; this one computes the strided sum the fingerprint kernel defines */
int mi355_f16_reduce(void const *in, void *out, size_t n_out, int factor, int in_stride,
                     int out_stride);

/* ---- timing -----------------------------------------------------------------
 * cudaEvent pairs of every profile() in the reference (e.g. matmul_kernel.cu:63-70). */
int mi355_timer_start(void);
int mi355_timer_stop(float *ms); /* blocking */

/* ---- source emission -------------------------------------------------------
 * Replaces generate_kernel_code (src/kernel/triton_code_gen.cc:84-352): the fp16
 * lowering of one customized op printed as a specialised gfx950 kernel named `name`
 * plus `extern "C" int <name>_launch(void const *const *in, void *const *out,
 * hipStream_t)`.  Host code only, no device needed.  Returns the length of the text
 * (without the terminator) and copies at most capacity - 1 bytes of it into `buf`;
 * -1 on error (mi355_last_error).  max_lds_bytes <= 0 means gfx950's 160 KB.
 * mi355_emit_hip_preamble: the includes, typedefs and tile helpers the kernels use,
 * once per file. */
char const *mi355_emit_hip_preamble(void);
long long mi355_emit_hip_kernel(mi355_plan const *plan, char const *name, int max_lds_bytes,
                                char *buf, long long capacity);

#ifdef __cplusplus
}
#endif
#endif /* MI355_ABI_H */
