/*
 * CPU oracle for the mugraph execute / fingerprint path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a scalar restatement, in plain C,
 * of the arithmetic the reference performs on the GPU.  Nothing in the shipped
 * package may call, link or load it; only tests, the smoke check and the
 * bench's cpu_baseline leg do, and only as the checker / reported baseline.
 *
 * Every function cites the reference lines it follows (paths relative to the
 * reference root).  Storage is uint16, temporaries uint32, the modulus is
 * applied after every multiply-accumulate exactly as the reference writes it.
 * All tensors are indexed row-major whatever their declared layout
 * (include/mirage/threadblock/cuda/input_loader.h:457-467,
 *  include/mirage/threadblock/cuda/matmul.h:762-763).
 *
 * Parity status of each function (what pins it besides transcription):
 *   tables                 closed forms (Fermat inverses, order of 3 mod 227)
 *   matmul/add/mul/reduce  ring homomorphism vs exact big-integer arithmetic
 *   exp/div                algebraic identities + the 69 reference-verified
 *                          graphs of demo/checkpoint_group_query_attn_spec_decode.json
 *   customized interpreter the 69 graphs, the reference's 13 hand-written
 *                          example equivalences, degenerate-grid reduction to
 *                          the kernel-level ops, an independent numpy statement
 *   silu                   EXTENSION the reference never defines, so there is no
 *                          reference value to be equal to; the definition
 *                          x / (1 + exp(-x)) over the reference's ring primitives is
 *                          pinned by a residue-by-residue closed form in Python
 *                          integers over all 25651 inputs, by silu(x) * (1 + exp(-x))
 *                          == x (the denominator is always invertible) and by the
 *                          composition through the public add / exp / div entry points
 *   tb add/mul             EXTENSIONS at thread-block level (the reference's lowering
 *                          asserts on them); the kernel-level formulas
 *                          (element_binary_kernel.cu:117-119,136-138) under the
 *                          thread-block broadcast indexer, pinned by exact Python
 *                          big-integer arithmetic over every broadcast a 3-D tile admits
 *   f16 golden             semantics of src/kernel/triton_code_gen.cc; the
 *                          reference holds no numeric fp16 outputs: pinned only
 *                          by textbook special cases (GEMM, softmax attention)
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* include/mirage/type.h:26-34 */
#define FP_P 227u
#define FP_Q 113u
#define FP_EXP_BASE 3u
#define FP_PQ 25651u
#define FP_P_MUL_Q_MOD_1 227u
#define FP_Q_MUL_P_MOD_1 25425u

/* include/mirage/type.h:50-62, 79-103 (numeric values verbatim) */
enum {
  KN_ADD_OP = 1008,
  KN_MUL_OP = 1009,
  KN_DIV_OP = 1010,
  TB_INPUT_OP = 2001,
  TB_OUTPUT_OP = 2002,
  TB_MATMUL_OP = 2003,
  TB_EXP_OP = 2007,
  TB_ADD_OP = 2008,
  TB_MUL_OP = 2009,
  TB_DIV_OP = 2010,
  TB_SILU_OP = 2012, /* extension, absent from the reference */
  TB_REDUCTION_0_OP = 2101,
  TB_REDUCTION_2_TO_DIMX_OP = 2106,
  TB_CONCAT_0_OP = 2200,
  TB_CONCAT_2_OP = 2202,
};

typedef uint16_t fp_t;

static fp_t g_exp[FP_Q], g_divp[FP_P], g_divq[FP_Q];
static int g_tables_ready = 0;

/* src/kernel/device_memory_manager.cu:41-90 */
void orc_build_tables(fp_t *exp_tbl, fp_t *divp, fp_t *divq) {
  exp_tbl[0] = 1;
  for (unsigned i = 1; i < FP_Q; i++) {
    exp_tbl[i] = (fp_t)((exp_tbl[i - 1] * FP_EXP_BASE) % FP_P);
  }
  for (unsigned i = 0; i < FP_P; i++) {
    divp[i] = 1;
    for (unsigned j = 1; j < FP_P; j++) {
      if ((i * j) % FP_P == 1) {
        divp[i] = (fp_t)j;
      }
    }
  }
  for (unsigned i = 0; i < FP_Q; i++) {
    divq[i] = 1;
    for (unsigned j = 1; j < FP_Q; j++) {
      if ((i * j) % FP_Q == 1) {
        divq[i] = (fp_t)j;
      }
    }
  }
}

static void ensure_tables(void) {
  if (!g_tables_ready) {
    orc_build_tables(g_exp, g_divp, g_divq);
    g_tables_ready = 1;
  }
}

/* src/kernel/cuda/input_kernel.cu:56-61 */
void orc_fp_input(fp_t *fp, size_t n) {
  for (size_t i = 0; i < n; i++) {
    fp[i] = (fp_t)(i % FP_PQ);
  }
}

/* src/kernel/cuda/matmul_kernel.cu:145-173 */
void orc_fp_matmul(fp_t const *A, fp_t const *B, fp_t *C, int batch, int m,
                   int n, int k) {
  size_t mk = (size_t)m * k, mn = (size_t)m * n, nk = (size_t)n * k;
  for (int b = 0; b < batch; b++) {
    for (int row = 0; row < m; row++) {
      for (int col = 0; col < n; col++) {
        uint32_t r = 0;
        for (int i = 0; i < k; i++) {
          uint32_t a = A[b * mk + (size_t)row * k + i];
          uint32_t bv = B[b * nk + (size_t)i * n + col];
          r = (r + a * bv) % FP_PQ;
        }
        C[b * mn + (size_t)row * n + col] = (fp_t)r;
      }
    }
  }
}

static inline fp_t fp_exp1(fp_t x) {
  /* src/kernel/cuda/element_unary_kernel.cu:85-89,
     include/mirage/threadblock/cuda/element_unary.h:61-66 */
  uint32_t r = g_exp[x % FP_Q];
  return (fp_t)((r * FP_Q_MUL_P_MOD_1) % FP_PQ);
}

static inline fp_t fp_div1(uint32_t x, uint32_t y) {
  /* src/kernel/cuda/element_binary_kernel.cu:155-160,
     include/mirage/threadblock/cuda/element_binary.h:100-105 */
  uint32_t z = (x % FP_P) * g_divp[y % FP_P] * FP_Q_MUL_P_MOD_1 +
               (x % FP_Q) * g_divq[y % FP_Q] * FP_P_MUL_Q_MOD_1;
  return (fp_t)(z % FP_PQ);
}

/* EXTENSION (not in the reference): silu(x) = x / (1 + exp(-x)) written with
   the reference's own ring primitives. */
static inline fp_t fp_silu1(fp_t x) {
  fp_t neg = (fp_t)((FP_PQ - x) % FP_PQ);
  uint32_t den = (1u + fp_exp1(neg)) % FP_PQ;
  return fp_div1(x, den);
}

void orc_fp_exp(fp_t const *in, fp_t *out, size_t n) {
  ensure_tables();
  for (size_t i = 0; i < n; i++) {
    out[i] = fp_exp1(in[i]);
  }
}

void orc_fp_silu(fp_t const *in, fp_t *out, size_t n) {
  ensure_tables();
  for (size_t i = 0; i < n; i++) {
    out[i] = fp_silu1(in[i]);
  }
}

/* src/kernel/cuda/element_binary_kernel.cu:97-168 */
void orc_fp_binary(int op, fp_t const *in1, int const *dims1, fp_t const *in2,
                   int const *dims2, fp_t *out, int const *dims_out, int nd) {
  ensure_tables();
  size_t n = 1;
  for (int d = 0; d < nd; d++) {
    n *= (size_t)dims_out[d];
  }
  for (size_t t = 0; t < n; t++) {
    size_t i = t;
    size_t s1 = 1, i1 = 0, s2 = 1, i2 = 0;
    for (int d = nd - 1; d >= 0; d--) {
      i1 += (i % dims1[d]) * s1;
      i2 += (i % dims2[d]) * s2;
      s1 *= dims1[d];
      s2 *= dims2[d];
      i /= dims_out[d];
    }
    uint32_t x = in1[i1], y = in2[i2];
    if (op == KN_ADD_OP) {
      out[t] = (fp_t)((x + y) % FP_PQ);
    } else if (op == KN_MUL_OP) {
      out[t] = (fp_t)((x * y) % FP_PQ);
    } else {
      out[t] = fp_div1(x, y);
    }
  }
}

/* src/kernel/cuda/reduction_kernel.cu:80-108 */
void orc_fp_reduce(fp_t const *in, fp_t *out, size_t n_out, int factor,
                   int in_stride, int out_stride) {
  for (size_t i = 0; i < n_out; i++) {
    uint32_t r = 0;
    size_t n = i / out_stride, m = i % out_stride;
    for (int k = 0; k < factor; k++) {
      r = (r + in[n * in_stride + m + (size_t)k * out_stride]) % FP_PQ;
    }
    out[i] = (fp_t)r;
  }
}

/* src/kernel/cuda/device_tensor_kernel.cu:42-49 (element loop only) */
int orc_fp_equal(fp_t const *a, fp_t const *b, size_t n) {
  for (size_t i = 0; i < n; i++) {
    if (a[i] != b[i]) {
      return 0;
    }
  }
  return 1;
}

/* ---- fp16 helpers (software, round-to-nearest-even) --------------------- */
static inline float h2f(uint16_t h) {
  uint32_t s = (uint32_t)(h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ff, u;
  if (e == 0) {
    if (m == 0) {
      u = s;
    } else {
      int sh = 0;
      while (!(m & 0x400)) {
        m <<= 1;
        sh++;
      }
      m &= 0x3ff;
      u = s | ((uint32_t)(127 - 15 - sh + 1) << 23) | (m << 13);
    }
  } else if (e == 31) {
    u = s | 0x7f800000u | (m << 13);
  } else {
    u = s | ((e + 112) << 23) | (m << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f2h(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t s = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(s | 0x7c00u | ((a > 0x7f800000u) ? 0x200u : 0));
  }
  if (a >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(s | 0x7c00u);
  }
  if (a < 0x38800000u) { /* subnormal half or zero */
    if (a < 0x33000000u) {
      return (uint16_t)s; /* < 2^-25 -> 0 */
    }
    uint32_t e = a >> 23;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;
    uint32_t shift = 126 - e; /* 14..24 */
    uint32_t r = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (r & 1))) {
      r++;
    }
    return (uint16_t)(s | r);
  }
  uint32_t e = (a >> 23) - 112, m = (a >> 13) & 0x3ff;
  uint32_t r = (e << 10) | m, rem = a & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) {
    r++;
  }
  return (uint16_t)(s | r);
}

void orc_f16_to_f32(uint16_t const *in, float *out, size_t n) {
  for (size_t i = 0; i < n; i++) {
    out[i] = h2f(in[i]);
  }
}
void orc_f32_to_f16(float const *in, uint16_t *out, size_t n) {
  for (size_t i = 0; i < n; i++) {
    out[i] = f2h(in[i]);
  }
}

/* ---- the customized-op interpreter --------------------------------------
 * Program format = the reference's NewKernelParams flat ints
 * (include/mirage/threadblock/serializer/kernel_params.h:25-35 and the
 * per-op serializers beside it).  The walk below restates
 * src/kernel/cuda/customized_kernel.cu:307-603 with one host loop standing in
 * for the thread-strided loops of the TB*Fingerprinter classes.
 *
 * `f16 != 0` selects the fp16 golden: same program, real arithmetic in fp32,
 * every STensor rounded to fp16 when written, accumulators fp16 starting at 0
 * and `accum = accum + x` each iteration, stored once after the loop
 * (src/kernel/triton_code_gen.cc:223-232,246-268,292-333).
 */
typedef struct {
  int num_operators, num_parameters;
  int const *op_types;
  int const *params;
  int grid[3];
  int forloop_range;
  int smem_bytes;
  void *const *in_ptrs;
  void *const *out_ptrs;
  int num_inputs, num_outputs;
  int f16;
  /* work split: positions [block_begin, block_end) of block_list (or, when
     block_list is NULL, the linear block indices themselves) */
  int block_begin, block_end;
  int const *block_list;
} interp_job;

static void run_block(interp_job const *J, int bx, int by, int bz,
                      uint16_t *smem) {
  int const *P = J->params;
  int const f16 = J->f16;
  int const out_start = J->num_operators - J->num_outputs;
  for (int it = 0; it < J->forloop_range; it++) {
    int pi = 0;
    for (int op = 0; op < J->num_operators; op++) {
      int t = J->op_types[op];
      if (t == TB_INPUT_OP) {
        /* customized_kernel.cu:327-385 + input_loader.h:457-467 */
        int const *q = P + pi;
        pi += 19;
        int row0 = bx * q[0] + by * q[1] + bz * q[2] + it * q[6];
        int col0 = bx * q[3] + by * q[4] + bz * q[5] + it * q[7];
        long goff = (long)bx * q[8] + (long)by * q[9] + (long)bz * q[10] +
                    (long)it * q[11];
        int dcols = q[13], srows = q[14], scols = q[15];
        uint16_t const *d = (uint16_t const *)J->in_ptrs[op] + goff;
        uint16_t *s = smem + q[18] / 2;
        for (int idx = 0; idx < srows * scols; idx++) {
          int r = row0 + idx / scols, c = col0 + idx % scols;
          s[idx] = d[(long)r * dcols + c];
        }
      } else if (t == TB_OUTPUT_OP) {
        /* customized_kernel.cu:387-458 + output_saver.h:373-401,418-447 */
        int const *q = P + pi;
        pi += 17;
        int srows = q[11], scols = q[12], dcols = q[10];
        uint16_t const *in = smem + q[15] / 2;
        uint16_t *acc = smem + q[16] / 2;
        int n = srows * scols;
        if (f16) {
          /* triton_code_gen.cc:223-230: zeros then accum = accum + x */
          for (int idx = 0; idx < n; idx++) {
            float a = (it == 0) ? 0.0f : h2f(acc[idx]);
            acc[idx] = f2h(a + h2f(in[idx]));
          }
        } else if (it == 0) {
          for (int idx = 0; idx < n; idx++) {
            acc[idx] = in[idx];
          }
        } else {
          for (int idx = 0; idx < n; idx++) {
            uint32_t v = in[idx];
            acc[idx] = (uint16_t)((v + acc[idx]) % FP_PQ);
          }
        }
        if (it == J->forloop_range - 1) {
          int row0 = bx * q[0] + by * q[1] + bz * q[2];
          int col0 = bx * q[3] + by * q[4] + bz * q[5];
          long goff = (long)bx * q[6] + (long)by * q[7] + (long)bz * q[8];
          uint16_t *d = (uint16_t *)J->out_ptrs[op - out_start] + goff;
          for (int idx = 0; idx < n; idx++) {
            int r = row0 + idx / scols, c = col0 + idx % scols;
            d[(long)r * dcols + c] = acc[idx];
          }
        }
      } else if (t == TB_MATMUL_OP) {
        /* matmul.h:773-804 */
        int m = P[pi], n = P[pi + 1], k = P[pi + 2];
        uint16_t const *A = smem + P[pi + 3] / 2;
        uint16_t const *B = smem + P[pi + 4] / 2;
        uint16_t *C = smem + P[pi + 5] / 2;
        pi += 6;
        for (int i = 0; i < m * n; i++) {
          int mm = i / n, nn = i % n;
          if (f16) {
            float r = 0.0f;
            for (int kk = 0; kk < k; kk++) {
              r += h2f(A[mm * k + kk]) * h2f(B[kk * n + nn]);
            }
            C[i] = f2h(r);
          } else {
            uint32_t r = 0;
            for (int kk = 0; kk < k; kk++) {
              uint32_t a = A[mm * k + kk], b = B[kk * n + nn];
              r = (r + a * b) % FP_PQ;
            }
            C[i] = (uint16_t)r;
          }
        }
      } else if (t == TB_EXP_OP || t == TB_SILU_OP) {
        /* element_unary.h:59-67 (exp); silu is an extension */
        uint16_t *p = smem + P[pi] / 2;
        int n = P[pi + 1];
        pi += 2;
        for (int i = 0; i < n; i++) {
          if (f16) {
            float x = h2f(p[i]);
            p[i] = f2h(t == TB_EXP_OP ? expf(x) : x / (1.0f + expf(-x)));
          } else {
            p[i] = (t == TB_EXP_OP) ? fp_exp1(p[i]) : fp_silu1(p[i]);
          }
        }
      } else if (t == TB_DIV_OP || t == TB_ADD_OP || t == TB_MUL_OP) {
        /* element_binary.h:74-105; add/mul take the kernel-level formulas
           (element_binary_kernel.cu:117-119,136-138) and are extensions at
           thread-block level: the reference asserts false there */
        int d1[3] = {P[pi], P[pi + 1], P[pi + 2]};
        int d2[3] = {P[pi + 3], P[pi + 4], P[pi + 5]};
        uint16_t const *i1 = smem + P[pi + 6] / 2;
        uint16_t const *i2 = smem + P[pi + 7] / 2;
        uint16_t *o = smem + P[pi + 8] / 2;
        pi += 9;
        int od[3];
        for (int d = 0; d < 3; d++) {
          od[d] = d1[d] > d2[d] ? d1[d] : d2[d];
        }
        int n = od[0] * od[1] * od[2];
        for (int i = 0; i < n; i++) {
          int idx = i, s1 = 1, x1 = 0, s2 = 1, x2 = 0;
          for (int d = 2; d >= 0; d--) {
            x1 += (idx % d1[d]) * s1;
            x2 += (idx % d2[d]) * s2;
            s1 *= d1[d];
            s2 *= d2[d];
            idx /= od[d];
          }
          if (f16) {
            float x = h2f(i1[x1]), y = h2f(i2[x2]);
            o[i] = f2h(t == TB_DIV_OP ? x / y : (t == TB_ADD_OP ? x + y : x * y));
          } else {
            uint32_t x = i1[x1], y = i2[x2];
            o[i] = t == TB_DIV_OP   ? fp_div1(x, y)
                   : t == TB_ADD_OP ? (uint16_t)((x + y) % FP_PQ)
                                    : (uint16_t)((x * y) % FP_PQ);
          }
        }
      } else if (t >= TB_REDUCTION_0_OP && t <= TB_REDUCTION_2_TO_DIMX_OP) {
        /* reduction.h:147-156 */
        int n_out = P[pi], deg = P[pi + 1], inner = P[pi + 2];
        uint16_t const *in = smem + P[pi + 3] / 2;
        uint16_t *o = smem + P[pi + 4] / 2;
        pi += 5;
        for (int i = 0; i < n_out; i++) {
          int pos = (i / inner) * (inner * deg) + i % inner;
          if (f16) {
            float r = 0.0f;
            for (int k = 0; k < deg; k++, pos += inner) {
              r += h2f(in[pos]);
            }
            o[i] = f2h(r);
          } else {
            uint32_t r = 0;
            for (int k = 0; k < deg; k++, pos += inner) {
              r = (r + in[pos]) % FP_PQ;
            }
            o[i] = (uint16_t)r;
          }
        }
      } else if (t >= TB_CONCAT_0_OP && t <= TB_CONCAT_2_OP) {
        /* concat.h:90-101 */
        int n_out = P[pi], a = P[pi + 1], b = P[pi + 2], inner = P[pi + 3];
        uint16_t const *A = smem + P[pi + 4] / 2;
        uint16_t const *B = smem + P[pi + 5] / 2;
        uint16_t *o = smem + P[pi + 6] / 2;
        pi += 7;
        for (int i = 0; i < n_out; i++) {
          int in_i = i % inner;
          int cd = (i / inner) % (a + b);
          int outer = (i / inner) / (a + b);
          o[i] = cd < a ? A[in_i + cd * inner + outer * inner * a]
                        : B[in_i + (cd - a) * inner + outer * inner * b];
        }
      }
    }
  }
}

static void *interp_worker(void *arg) {
  interp_job const *J = (interp_job const *)arg;
  uint16_t *smem = (uint16_t *)malloc((size_t)J->smem_bytes + 64);
  for (int i = J->block_begin; i < J->block_end; i++) {
    int b = J->block_list ? J->block_list[i] : i;
    int bx = b % J->grid[0];
    int by = (b / J->grid[0]) % J->grid[1];
    int bz = b / (J->grid[0] * J->grid[1]);
    run_block(J, bx, by, bz, smem);
  }
  free(smem);
  return NULL;
}

/* Returns 0 on success.  `threads` > 1 splits the thread blocks of the op
   over that many host threads (blocks write disjoint output tiles).
   `block_list` (may be NULL = every block) names the linear block indices
   bx + grid.x * (by + grid.y * bz) to run: thread blocks are independent
   (customized_kernel.cu:307-603 shares nothing between them), so a subset
   reproduces exactly those blocks' output tiles and leaves the rest of the
   outputs untouched -- how a full-size op is checked on a slice. */
int orc_customized_blocks(int num_operators, int num_parameters,
                          int const *op_types, int const *params,
                          int const *grid, int forloop_range, int smem_bytes,
                          void *const *in_ptrs, int num_inputs,
                          void *const *out_ptrs, int num_outputs, int f16,
                          int threads, int const *block_list, int num_listed) {
  ensure_tables();
  int nblocks = grid[0] * grid[1] * grid[2];
  if (block_list) {
    for (int i = 0; i < num_listed; i++) {
      if (block_list[i] < 0 || block_list[i] >= nblocks) {
        return -2;
      }
    }
    nblocks = num_listed;
  }
  if (nblocks < 1) {
    return 0;
  }
  if (threads < 1) {
    threads = 1;
  }
  if (threads > nblocks) {
    threads = nblocks;
  }
  if (threads > 256) {
    threads = 256;
  }
  interp_job jobs[256];
  pthread_t tids[256];
  for (int t = 0; t < threads; t++) {
    interp_job *J = &jobs[t];
    J->num_operators = num_operators;
    J->num_parameters = num_parameters;
    J->op_types = op_types;
    J->params = params;
    memcpy(J->grid, grid, sizeof(int) * 3);
    J->forloop_range = forloop_range;
    J->smem_bytes = smem_bytes;
    J->in_ptrs = in_ptrs;
    J->out_ptrs = out_ptrs;
    J->num_inputs = num_inputs;
    J->num_outputs = num_outputs;
    J->f16 = f16;
    J->block_begin = (int)((long)nblocks * t / threads);
    J->block_end = (int)((long)nblocks * (t + 1) / threads);
    J->block_list = block_list;
  }
  if (threads == 1) {
    interp_worker(&jobs[0]);
    return 0;
  }
  for (int t = 0; t < threads; t++) {
    if (pthread_create(&tids[t], NULL, interp_worker, &jobs[t]) != 0) {
      return -1;
    }
  }
  for (int t = 0; t < threads; t++) {
    pthread_join(tids[t], NULL);
  }
  return 0;
}

int orc_customized(int num_operators, int num_parameters, int const *op_types,
                   int const *params, int const *grid, int forloop_range,
                   int smem_bytes, void *const *in_ptrs, int num_inputs,
                   void *const *out_ptrs, int num_outputs, int f16,
                   int threads) {
  return orc_customized_blocks(num_operators, num_parameters, op_types, params,
                               grid, forloop_range, smem_bytes, in_ptrs,
                               num_inputs, out_ptrs, num_outputs, f16, threads,
                               NULL, 0);
}

/* ---- kernel-level fp16 golden ops (same rounding rule: fp32 math, one fp16
 * rounding per stored element) -------------------------------------------- */
void orc_f16_matmul(uint16_t const *A, uint16_t const *B, uint16_t *C,
                    int batch, int m, int n, int k) {
  size_t mk = (size_t)m * k, mn = (size_t)m * n, nk = (size_t)n * k;
  float *row = (float *)malloc(sizeof(float) * (size_t)n);
  for (int b = 0; b < batch; b++) {
    for (int r = 0; r < m; r++) {
      for (int c = 0; c < n; c++) {
        row[c] = 0.0f;
      }
      for (int i = 0; i < k; i++) {
        float a = h2f(A[b * mk + (size_t)r * k + i]);
        uint16_t const *bp = B + b * nk + (size_t)i * n;
        for (int c = 0; c < n; c++) {
          row[c] += a * h2f(bp[c]);
        }
      }
      for (int c = 0; c < n; c++) {
        C[b * mn + (size_t)r * n + c] = f2h(row[c]);
      }
    }
  }
  free(row);
}
