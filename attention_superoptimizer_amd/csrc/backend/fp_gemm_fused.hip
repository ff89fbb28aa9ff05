// Fused fingerprint kernel for the plainest customized op: load A tile, load B tile,
// matmul, accumulate over the for-loop, store (the shape of the reference's
// tests/threadblock/matmul.cu:163-189 and of most matmul rewrites a search proposes).
//
// The interpreter runs such a plan as four operators per iteration with a barrier after
// each: raw tiles into LDS, a packing pass, the dot products, a CRT recombination, the
// accumulating saver.  In the ring Z_25651 the saver's sum over iterations is exact, so
// the whole for-loop is ONE sum of products: this kernel keeps both residue sums of its
// outputs in registers across all iterations and recombines once at the end, and the raw
// tiles of step s + 1 are in flight in registers while step s is multiplied (one barrier
// per step).  Tiles are read through the plan's own strides, iteration by iteration, so a
// wrong input map or for-loop dim still gives the wrong answer.  Bit-identical to the
// interpreter (and to the reference's `(r + a*b) % 25651` chains,
// include/mirage/threadblock/cuda/matmul.h:773-804 and output_saver.h:373-401).
// Integer only: residues mod 227 / 113 packed four to a dword, v_dot4_u32_u8.
#include "common.h"
#include "tb_program.h"
#include <atomic>

namespace mi355 {

namespace {

constexpr int kThreads = 256;
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void residues4(uint32_t v0, uint32_t v1, uint32_t v2, uint32_t v3,
                                          uint32_t &pp, uint32_t &qq) {
  pp = (v0 % FP_P) | ((v1 % FP_P) << 8) | ((v2 % FP_P) << 16) | ((v3 % FP_P) << 24);
  qq = (v0 % FP_Q) | ((v1 % FP_Q) << 8) | ((v2 % FP_Q) << 16) | ((v3 % FP_Q) << 24);
}

__device__ __forceinline__ long long origin(DevOp const &op, int it, int bx, int by, int bz) {
  int const row0 = bx * op.row_bs[0] + by * op.row_bs[1] + bz * op.row_bs[2] + it * op.row_fs;
  int const col0 = bx * op.col_bs[0] + by * op.col_bs[1] + bz * op.col_bs[2] + it * op.col_fs;
  long long const base = (long long)bx * op.g_bs[0] + (long long)by * op.g_bs[1] +
                         (long long)bz * op.g_bs[2] + (long long)it * op.g_fs;
  return base + (long long)row0 * op.d_cols + col0;
}

// One workgroup: logical block (bx, by, bz), part `split` of the for-loop.
// LDS: two buffers of Ap[2][kc/4][m + 4] and Bp[2][kc/4][n] dwords.
// Thread roles while staging: up to 4 A items (one row, 8 consecutive k) and one B item
// (4 consecutive k x 8 columns).  Output: TPT register tiles of 4 x 4 per thread.
template <int TPT>
__device__ __forceinline__ void fp_gemm_block(DevProgram const &P, uint32_t *lds, int bx, int by,
                                              int bz, int split) {
  DevOp const &la = P.ops[P.fg[0]], &lb = P.ops[P.fg[1]], &so = P.ops[3];
  int const m = P.t[la.dst].rows, kt = P.t[la.dst].cols, n = P.t[lb.dst].cols;
  int const kc = P.fg[2], kq = kc / 4, lda = m + 4;
  int const buf_dwords = 2 * kq * (lda + n);
  int const tid = threadIdx.x;
  int const F = P.forloop_range;
  // (32-bit: a for-loop is cut into at most 64 parts, and 64 F is far below 2^32)
  unsigned const parts = (unsigned)P.splits;
  int const it_begin = parts == 1 ? 0 : (int)((unsigned)F * (unsigned)split / parts);
  int const it_end = parts == 1 ? F : (int)((unsigned)F * (unsigned)(split + 1) / parts);
  int const chunks = kt / kc, steps = (it_end - it_begin) * chunks;
  uint16_t const *inA = static_cast<uint16_t const *>(P.in[la.io]);
  uint16_t const *inB = static_cast<uint16_t const *>(P.in[lb.io]);

  // staging roles (the same every step)
  int const a_per_row = kc / 8, a_items = m * a_per_row;
  int a_row[4], a_k8[4];
#pragma unroll
  for (int u = 0; u < 4; u++) {
    int const e = tid + u * kThreads;
    a_row[u] = e / a_per_row;
    a_k8[u] = (e % a_per_row) * 8;
  }
  int const b_per_q = n / 8;
  bool const b_active = tid < kq * b_per_q;
  int const b_q = tid / b_per_q, b_c8 = (tid % b_per_q) * 8;

  uint4v ra[4], rb[4];
  auto fetch = [&](int step) {
    int const it = it_begin + step / chunks, k0 = (step % chunks) * kc;
    uint16_t const *ga = inA + origin(la, it, bx, by, bz) + k0;
    uint16_t const *gb = inB + origin(lb, it, bx, by, bz) + (long long)k0 * lb.d_cols;
#pragma unroll
    for (int u = 0; u < 4; u++) {
      if (tid + u * kThreads < a_items) {
        ra[u] = *reinterpret_cast<uint4v const *>(ga + (long long)a_row[u] * la.d_cols + a_k8[u]);
      }
    }
    if (b_active) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        rb[j] = *reinterpret_cast<uint4v const *>(gb + (long long)(4 * b_q + j) * lb.d_cols + b_c8);
      }
    }
  };
  auto stage = [&](int buf) {
    uint32_t *Ap = lds + buf * buf_dwords, *Bp = Ap + 2 * kq * lda;
#pragma unroll
    for (int u = 0; u < 4; u++) {
      if (tid + u * kThreads < a_items) {
        int const q = a_k8[u] / 4, row = a_row[u];
        uint32_t pp, qq;
        residues4(ra[u][0] & 0xffffu, ra[u][0] >> 16, ra[u][1] & 0xffffu, ra[u][1] >> 16, pp, qq);
        Ap[q * lda + row] = pp;
        Ap[(kq + q) * lda + row] = qq;
        residues4(ra[u][2] & 0xffffu, ra[u][2] >> 16, ra[u][3] & 0xffffu, ra[u][3] >> 16, pp, qq);
        Ap[(q + 1) * lda + row] = pp;
        Ap[(kq + q + 1) * lda + row] = qq;
      }
    }
    if (b_active) {
      uint32_t bp[8], bq[8];
#pragma unroll
      for (int w = 0; w < 4; w++) {  // dword w of each row holds columns 2w and 2w + 1
        residues4(rb[0][w] & 0xffffu, rb[1][w] & 0xffffu, rb[2][w] & 0xffffu, rb[3][w] & 0xffffu,
                  bp[2 * w], bq[2 * w]);
        residues4(rb[0][w] >> 16, rb[1][w] >> 16, rb[2][w] >> 16, rb[3][w] >> 16, bp[2 * w + 1],
                  bq[2 * w + 1]);
      }
      uint32_t *dp = Bp + b_q * n + b_c8, *dq = Bp + (kq + b_q) * n + b_c8;
      *reinterpret_cast<uint4v *>(dp) = uint4v{bp[0], bp[1], bp[2], bp[3]};
      *reinterpret_cast<uint4v *>(dp + 4) = uint4v{bp[4], bp[5], bp[6], bp[7]};
      *reinterpret_cast<uint4v *>(dq) = uint4v{bq[0], bq[1], bq[2], bq[3]};
      *reinterpret_cast<uint4v *>(dq + 4) = uint4v{bq[4], bq[5], bq[6], bq[7]};
    }
  };

  int const tiles_n = n / 4, tiles = (m / 4) * tiles_n;
  // A small output tile leaves most threads without a register tile; they form further
  // groups of `tiles` threads that each take every kgroups-th k quad of a step, and the
  // groups' sums are added at the end (exact in the ring).  kgroups == 1 when TPT > 1.
  int const kgroups = TPT == 1 ? P.fg[4] : 1;
  int const kgroup = TPT == 1 ? tid / tiles : 0;
  int r0[TPT], c0[TPT];
  uint32_t accp[TPT][4][4], accq[TPT][4][4];
#pragma unroll
  for (int u = 0; u < TPT; u++) {
    int const t = TPT == 1 ? tid % tiles : tid + u * kThreads;
    int const tt = t < tiles ? t : 0;  // idle threads shadow tile 0 and store nothing
    r0[u] = (tt / tiles_n) * 4;
    c0[u] = (tt % tiles_n) * 4;
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        accp[u][i][j] = 0;
        accq[u][i][j] = 0;
      }
    }
  }

  if (steps > 0) {
    fetch(0);
    stage(0);
  }
  __syncthreads();
  for (int s = 0; s < steps; s++) {
    if (s + 1 < steps) {
      fetch(s + 1);
    }
    uint32_t const *Ap = lds + (s & 1) * buf_dwords, *Bp = Ap + 2 * kq * lda;
    for (int q = kgroup < kgroups ? kgroup : kq; q < kq; q += kgroups) {
#pragma unroll
      for (int u = 0; u < TPT; u++) {
        uint4v const a_p = *reinterpret_cast<uint4v const *>(Ap + q * lda + r0[u]);
        uint4v const a_q = *reinterpret_cast<uint4v const *>(Ap + (kq + q) * lda + r0[u]);
        uint4v const b_p = *reinterpret_cast<uint4v const *>(Bp + q * n + c0[u]);
        uint4v const b_q4 = *reinterpret_cast<uint4v const *>(Bp + (kq + q) * n + c0[u]);
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
          for (int j = 0; j < 4; j++) {
            accp[u][i][j] = __builtin_amdgcn_udot4(a_p[i], b_p[j], accp[u][i][j], false);
            accq[u][i][j] = __builtin_amdgcn_udot4(a_q[i], b_q4[j], accq[u][i][j], false);
          }
        }
      }
    }
    // a step adds at most kc * 226^2 < 2^22 to a sum: fold long before 2^32
    if ((s & 511) == 511) {
#pragma unroll
      for (int u = 0; u < TPT; u++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
          for (int j = 0; j < 4; j++) {
            accp[u][i][j] %= FP_P;
            accq[u][i][j] %= FP_Q;
          }
        }
      }
    }
    if (s + 1 < steps) {
      stage((s + 1) & 1);  // that buffer was last read in step s - 1
    }
    __syncthreads();
  }

  if (TPT == 1 && kgroups > 1) {
    // the step loop ended with a barrier: the staging buffers are free to carry the sums
    uint32_t *red = lds;
    if (kgroup > 0 && kgroup < kgroups) {
      uint32_t *mine = red + ((kgroup - 1) * tiles + tid % tiles) * 32;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        *reinterpret_cast<uint4v *>(mine + 4 * i) = uint4v{accp[0][i][0] % FP_P, accp[0][i][1] % FP_P,
                                                           accp[0][i][2] % FP_P, accp[0][i][3] % FP_P};
        *reinterpret_cast<uint4v *>(mine + 16 + 4 * i) =
            uint4v{accq[0][i][0] % FP_Q, accq[0][i][1] % FP_Q, accq[0][i][2] % FP_Q, accq[0][i][3] % FP_Q};
      }
    }
    __syncthreads();
    if (kgroup == 0) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          accp[0][i][j] %= FP_P;
          accq[0][i][j] %= FP_Q;
        }
      }
      for (int gk = 1; gk < kgroups; gk++) {
        uint32_t const *other = red + ((gk - 1) * tiles + tid) * 32;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          uint4v const vp = *reinterpret_cast<uint4v const *>(other + 4 * i);
          uint4v const vq = *reinterpret_cast<uint4v const *>(other + 16 + 4 * i);
#pragma unroll
          for (int j = 0; j < 4; j++) {
            accp[0][i][j] += vp[j];
            accq[0][i][j] += vq[j];
          }
        }
      }
    }
  }
  uint16_t *g = (P.splits > 1 ? P.part[so.io] + (long long)split * P.part_stride[so.io]
                              : static_cast<uint16_t *>(P.out[so.io])) +
                origin(so, 0, bx, by, bz);
#pragma unroll
  for (int u = 0; u < TPT; u++) {
    if (tid + u * kThreads < tiles) {  // with k groups: the threads of group 0
#pragma unroll
      for (int i = 0; i < 4; i++) {
        uint32_t z[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          z[j] = ((accp[u][i][j] % FP_P) * FP_Q_MUL_P_MOD_1 + (accq[u][i][j] % FP_Q) * FP_P_MUL_Q_MOD_1) %
                 FP_PQ;
        }
        uint2 out;
        out.x = z[0] | (z[1] << 16);
        out.y = z[2] | (z[3] << 16);
        *reinterpret_cast<uint2 *>(g + (long long)(r0[u] + i) * so.d_cols + c0[u]) = out;
      }
    }
  }
}

template <int TPT>
__global__ __launch_bounds__(kThreads) void fp_gemm_kernel(DevProgram const P) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  fp_gemm_block<TPT>(P, reinterpret_cast<uint32_t *>(lds), blockIdx.x % P.grid[0], blockIdx.y,
                     blockIdx.z, blockIdx.x / P.grid[0]);
}

// Many programs in one launch, as fp_interp_multi_kernel: workgroup -> program by a prefix
// table, the program record copied to LDS above the staging buffers.
template <int TPT>
__global__ __launch_bounds__(kThreads) void fp_gemm_multi_kernel(
    DevProgram const *__restrict__ progs, int const *__restrict__ first_block, int n,
    int program_lds_offset) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  int lo = 0, hi = n;
  int const w = blockIdx.x;
  while (hi - lo > 1) {
    int const mid = (lo + hi) / 2;
    if (first_block[mid] <= w) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  uint4v const *src = reinterpret_cast<uint4v const *>(progs + lo);
  uint4v *dst = reinterpret_cast<uint4v *>(lds + program_lds_offset);
  for (int i = threadIdx.x; i < (int)(sizeof(DevProgram) / 16); i += kThreads) {
    dst[i] = src[i];
  }
  __syncthreads();
  DevProgram const &P = *reinterpret_cast<DevProgram const *>(lds + program_lds_offset);
  int v = w - first_block[lo];
  int const gx = P.grid[0] * P.splits;
  int const x = v % gx;
  v /= gx;
  fp_gemm_block<TPT>(P, reinterpret_cast<uint32_t *>(lds), x % P.grid[0], v % P.grid[1], v / P.grid[1],
                     x / P.grid[0]);
}

template <int TPT>
int raise_lds(int lds_total) {
  static std::atomic<int> granted_single{0}, granted_multi{0};
  State &s = state();
  if (lds_total > 65536 && (granted_single < s.max_lds || granted_multi < s.max_lds)) {
    MI355_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(fp_gemm_kernel<TPT>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, s.max_lds));
    MI355_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(fp_gemm_multi_kernel<TPT>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, s.max_lds));
    granted_single = granted_multi = s.max_lds;
  }
  return MI355_OK;
}

}  // namespace

// Recognises the family in a lowered uint16 program; on success marks it (fused = 4),
// records which loader feeds which operand, the k chunk and the register tiles per thread,
// and replaces the LDS need by the staging buffers'.
bool fp_gemm_applicable(DevProgram &P) {
  // load, load, [exp / silu of a loaded tile, in place]*, matmul, [exp / silu of the product,
  // in place], save
  int const last = P.num_ops - 1;
  int mm = -1;
  for (int o = 2; o < last; o++) {
    if (P.ops[o].kind == DOP_MATMUL) {
      mm = mm < 0 ? o : P.num_ops;  // exactly one
    }
  }
  if (P.num_ops < 4 || P.num_ops > 7 || mm < 0 || mm >= last || mm < last - 2 ||
      P.ops[0].kind != DOP_LOAD || P.ops[1].kind != DOP_LOAD || P.ops[last].kind != DOP_OUTPUT ||
      P.ops[last].src0 != P.ops[mm].dst) {
    return false;
  }
  int a = -1, b = -1;
  for (int i = 0; i < 2; i++) {
    if (P.ops[i].dst == P.ops[mm].src0) {
      a = i;
    }
    if (P.ops[i].dst == P.ops[mm].src1) {
      b = i;
    }
  }
  if (a < 0 || b < 0 || a == b) {
    return false;
  }
  P.fp_unary[0] = P.fp_unary[1] = P.fp_unary[2] = 0;
  for (int o = 2; o < mm; o++) {
    DevOp const &u = P.ops[o];
    int const which = u.dst == P.ops[a].dst ? 0 : (u.dst == P.ops[b].dst ? 1 : -1);
    if (u.kind != DOP_UNARY || which < 0 || u.src0 != u.dst || P.fp_unary[which] != 0) {
      return false;
    }
    P.fp_unary[which] = u.sub;
  }
  if (mm == last - 2) {
    DevOp const &u = P.ops[last - 1];
    if (u.kind != DOP_UNARY || u.dst != P.ops[mm].dst || u.src0 != u.dst) {
      return false;
    }
    P.fp_unary[2] = u.sub;
  }
  DevOp const &la = P.ops[a], &lb = P.ops[b], &so = P.ops[last];
  int const m = P.t[la.dst].rows, kt = P.t[la.dst].cols, n = P.t[lb.dst].cols;
  if (fp_needs_matrix_cores(P)) {
    // only the matrix-core route applies these operators; whether it fits (shapes, plane
    // memory) is for the caller to ask fp_mfma_gemm_fits before it relies on this mark
    P.fused = 4;
    P.fg[0] = a;
    P.fg[1] = b;
    P.fg[2] = P.fg[3] = P.fg[4] = P.fg[5] = 0;
    return true;
  }
  if (!la.vec8 || !lb.vec8 || !so.vec8 || m % 4 != 0 || n % 8 != 0 || kt % 8 != 0 ||
      (reinterpret_cast<uintptr_t>(P.out[so.io]) & 15) != 0 ||
      (reinterpret_cast<uintptr_t>(P.in[la.io]) & 15) != 0 ||
      (reinterpret_cast<uintptr_t>(P.in[lb.io]) & 15) != 0) {
    return false;
  }
  int kc = 0;
  for (int cand : {64, 32, 16, 8}) {
    if (kt % cand == 0 && (cand / 4) * (n / 8) <= kThreads && m * (cand / 8) <= 4 * kThreads) {
      kc = cand;
      break;
    }
  }
  int const tiles = (m / 4) * (n / 4);
  if (kc == 0 || tiles > 4 * kThreads) {
    return false;
  }
  int const tpt = tiles <= kThreads ? 1 : (tiles <= 2 * kThreads ? 2 : 4);
  P.fused = 4;
  P.fg[0] = a;
  P.fg[1] = b;
  P.fg[2] = kc;
  P.fg[3] = tpt;
  int kgroups = 1;
  if (tpt == 1) {
    kgroups = kThreads / tiles;
    kgroups = kgroups > kc / 4 ? kc / 4 : kgroups;
    kgroups = kgroups > 8 ? 8 : kgroups;
  }
  P.fg[4] = kgroups;
  P.fg[5] = 0;
  int const staging = 2 * (2 * (kc / 4) * (m + 4 + n)) * 4;
  int const reduce = (kgroups - 1) * tiles * 32 * 4;
  P.lds_bytes = staging > reduce ? staging : reduce;
  return true;
}

int launch_fp_gemm(DevProgram const &P, hipStream_t stream) {
  dim3 grid(P.grid[0] * P.splits, P.grid[1], P.grid[2]);
  switch (P.fg[3]) {
    case 1:
      if (int rc = raise_lds<1>(P.lds_bytes)) return rc;
      fp_gemm_kernel<1><<<grid, kThreads, P.lds_bytes, stream>>>(P);
      break;
    case 2:
      if (int rc = raise_lds<2>(P.lds_bytes)) return rc;
      fp_gemm_kernel<2><<<grid, kThreads, P.lds_bytes, stream>>>(P);
      break;
    default:
      if (int rc = raise_lds<4>(P.lds_bytes)) return rc;
      fp_gemm_kernel<4><<<grid, kThreads, P.lds_bytes, stream>>>(P);
      break;
  }
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

int launch_fp_gemm_multi(DevProgram const *progs, int const *first_block, int n, int blocks, int tpt,
                         int staging_bytes, hipStream_t stream) {
  int const program_off = (staging_bytes + 15) / 16 * 16;
  int const lds_total = program_off + (int)sizeof(DevProgram);
  switch (tpt) {
    case 1:
      if (int rc = raise_lds<1>(lds_total)) return rc;
      fp_gemm_multi_kernel<1><<<blocks, kThreads, lds_total, stream>>>(progs, first_block, n, program_off);
      break;
    case 2:
      if (int rc = raise_lds<2>(lds_total)) return rc;
      fp_gemm_multi_kernel<2><<<blocks, kThreads, lds_total, stream>>>(progs, first_block, n, program_off);
      break;
    default:
      if (int rc = raise_lds<4>(lds_total)) return rc;
      fp_gemm_multi_kernel<4><<<blocks, kThreads, lds_total, stream>>>(progs, first_block, n, program_off);
      break;
  }
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

}  // namespace mi355
