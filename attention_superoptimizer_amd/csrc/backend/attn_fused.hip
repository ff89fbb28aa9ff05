// Fused, register-resident kernel for the attention family of thread-block graphs:
//
//   form A   S = Q.K ; E = exp(S) ; r = rowsum(E) ; P = E / r ; O = P.V        -> accumulate O
//   form B   S = Q.K ; E = exp(S) ; O = E.V ; r = rowsum(E)                     -> accumulate O and r
//
// (the single-op GQA decode plan and the reference's two-output split-KV plans,
// e.g. cpp_examples/group_query_attn_inc_decode.cc:47-74).  Same arithmetic and the
// same fp16 rounding points as the generic interpreter, but no intermediate tile
// ever touches LDS:
//
//  * one wavefront owns 16 query rows; a logical thread block's rows are split over
//    as many workgroups as it takes to fill the chip (the plan's grid is a lower
//    bound on parallelism, not the launch shape);
//  * S is produced TRANSPOSED (S^T = K^T.Q^T) with 16x16x32 fp16 MFMA, so that each
//    lane ends up holding four consecutive keys of one query row — exactly the
//    A-operand layout of the next MFMA.  exp, the row sum (two cross-lane adds) and
//    the division happen on those accumulator registers; P.V consumes them directly;
//  * K tiles arrive [head_dim][keys] and V tiles [keys][dv], both with the MFMA's
//    reduction index strided in memory, so they are transposed once while being
//    staged into LDS (four 16-byte global reads -> eight 8-byte LDS writes per 4x8
//    patch) and every operand fetch is one contiguous LDS read;
//  * as many for-loop iterations as fit are staged per barrier, so their loads are
//    in flight together;
//  * the for-loop accumulators live in VGPRs (fp16-rounded each iteration, as the
//    reference's generated programs do) and are written once, through LDS, as full
//    16-byte row segments.
#include "common.h"
#include "tb_program.h"

namespace mi355 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

struct TileAddr {
  void const *ptr;
  int row_bs[3], col_bs[3], row_fs, col_fs;
  int g_bs[3], g_fs;
  int d_cols;
};

struct AttnParams {
  TileAddr q, k, v, o, r;  // r: row-sum output (form B only)
  int forloop_range;
  int split;   // workgroups per logical thread block
  int stages;  // for-loop iterations staged per barrier
  int lds_stage_bytes;
};

__device__ __forceinline__ long long tile_offset(TileAddr const &t, int bx, int by, int bz,
                                                 int it) {
  int row0 = bx * t.row_bs[0] + by * t.row_bs[1] + bz * t.row_bs[2] + it * t.row_fs;
  int col0 = bx * t.col_bs[0] + by * t.col_bs[1] + bz * t.col_bs[2] + it * t.col_fs;
  long long base = (long long)bx * t.g_bs[0] + (long long)by * t.g_bs[1] +
                   (long long)bz * t.g_bs[2] + (long long)it * t.g_fs;
  return base + (long long)row0 * t.d_cols + col0;
}

// src: R x C tile, columns contiguous, row stride ld.  dst[c][r] with row stride LD.
__device__ __forceinline__ void stage_transposed(_Float16 const *__restrict__ src, int ld, int R,
                                                 int C, _Float16 *__restrict__ dst, int LD,
                                                 int tid, int nthreads) {
  int const cblocks = C / 8, patches = (R / 4) * cblocks;
  for (int p = tid; p < patches; p += nthreads) {
    int const cb = p % cblocks, rb = p / cblocks;
    _Float16 const *s = src + (long long)(4 * rb) * ld + 8 * cb;
    uint4v x0 = *reinterpret_cast<uint4v const *>(s);
    uint4v x1 = *reinterpret_cast<uint4v const *>(s + ld);
    uint4v x2 = *reinterpret_cast<uint4v const *>(s + 2 * (long long)ld);
    uint4v x3 = *reinterpret_cast<uint4v const *>(s + 3 * (long long)ld);
    _Float16 *d = dst + (8 * cb) * LD + 4 * rb;
#pragma unroll
    for (int w = 0; w < 4; w++) {
      uint2v even, odd;  // columns 2w and 2w+1, rows 0..3
      even.x = (x0[w] & 0xffffu) | (x1[w] << 16);
      even.y = (x2[w] & 0xffffu) | (x3[w] << 16);
      odd.x = (x0[w] >> 16) | (x1[w] & 0xffff0000u);
      odd.y = (x2[w] >> 16) | (x3[w] & 0xffff0000u);
      *reinterpret_cast<uint2v *>(d + (2 * w) * LD) = even;
      *reinterpret_cast<uint2v *>(d + (2 * w + 1) * LD) = odd;
    }
  }
}

template <int D, int NK, int DV, bool HAS_DIV>
__global__ __launch_bounds__(256) void attn_fused_kernel(AttnParams const P) {
  constexpr int LDK = D + 8;    // K^T rows: [key][head_dim]
  constexpr int LDV = NK + 8;   // V^T rows: [dv][key]
  constexpr int LDO = DV + 8;
  constexpr int KB = NK / 16, DB = DV / 16, DK = D / 32;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

  int const tid = threadIdx.x, nthreads = blockDim.x;
  int const lane = tid % 64, wave = tid / 64, nwaves = nthreads / 64;
  int const g = lane / 16, c = lane % 16;
  int const bx = blockIdx.x / P.split, slice = blockIdx.x % P.split;
  int const by = blockIdx.y, bz = blockIdx.z;
  int const row_base = (slice * nwaves + wave) * 16;  // first query row of this wavefront
  int const F = P.forloop_range;

  // Q fragments (B operand of S^T): Q[row c][32kk + 8g .. +7], loop invariant
  half8 qf[DK];
  {
    _Float16 const *q = static_cast<_Float16 const *>(P.q.ptr) + tile_offset(P.q, bx, by, bz, 0) +
                        (long long)(row_base + c) * P.q.d_cols + 8 * g;
#pragma unroll
    for (int kk = 0; kk < DK; kk++) {
      qf[kk] = *reinterpret_cast<half8 const *>(q + 32 * kk);
    }
  }

  _Float16 oacc[DB][4];  // O[row 4g + r][16t + c], fp16 like the reference's accumulators
  _Float16 racc = (_Float16)0.0f;
#pragma unroll
  for (int t = 0; t < DB; t++) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      oacc[t][r] = (_Float16)0.0f;
    }
  }

  _Float16 *o_stage = reinterpret_cast<_Float16 *>(lds + P.stages * P.lds_stage_bytes);

  for (int it0 = 0; it0 < F; it0 += P.stages) {
    int const n_st = (F - it0) < P.stages ? (F - it0) : P.stages;
    if (it0 > 0) {
      __syncthreads();  // previous chunk fully consumed
    }
    for (int s = 0; s < n_st; s++) {
      _Float16 *kt = reinterpret_cast<_Float16 *>(lds + s * P.lds_stage_bytes);
      _Float16 *vt = kt + NK * LDK;
      _Float16 const *kg =
          static_cast<_Float16 const *>(P.k.ptr) + tile_offset(P.k, bx, by, bz, it0 + s);
      _Float16 const *vg =
          static_cast<_Float16 const *>(P.v.ptr) + tile_offset(P.v, bx, by, bz, it0 + s);
      stage_transposed(kg, P.k.d_cols, D, NK, kt, LDK, tid, nthreads);   // [D][NK] -> [NK][D]
      stage_transposed(vg, P.v.d_cols, NK, DV, vt, LDV, tid, nthreads);  // [NK][DV] -> [DV][NK]
    }
    __syncthreads();
    for (int s = 0; s < n_st; s++) {
      int const it = it0 + s;
      _Float16 const *kt = reinterpret_cast<_Float16 const *>(lds + s * P.lds_stage_bytes);
      _Float16 const *vt = kt + NK * LDK;
      // ---- S^T = K^T . Q^T, exp, row sum ------------------------------------------
      half4 e[KB];  // e[j][r] = E[row c][key 16j + 4g + r]
      float rs = 0.0f;
#pragma unroll
      for (int j = 0; j < KB; j++) {
        float4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int kk = 0; kk < DK; kk++) {
          half8 a = *reinterpret_cast<half8 const *>(kt + (16 * j + c) * LDK + 32 * kk + 8 * g);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qf[kk], acc, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
          _Float16 s16 = static_cast<_Float16>(acc[r]);                       // S tile (fp16)
          _Float16 e16 = static_cast<_Float16>(__expf(static_cast<float>(s16)));  // E tile
          e[j][r] = e16;
          rs += static_cast<float>(e16);
        }
      }
      rs += __shfl_xor(rs, 16, 64);
      rs += __shfl_xor(rs, 32, 64);
      _Float16 const r16 = static_cast<_Float16>(rs);  // row-sum tile (fp16)
      if (HAS_DIV) {
        float const den = static_cast<float>(r16);
#pragma unroll
        for (int j = 0; j < KB; j++) {
#pragma unroll
          for (int r = 0; r < 4; r++) {
            e[j][r] = static_cast<_Float16>(static_cast<float>(e[j][r]) / den);
          }
        }
      } else {
        racc = (it == 0) ? r16
                         : static_cast<_Float16>(static_cast<float>(racc) + static_cast<float>(r16));
      }
      // ---- O = P . V: the accumulators of S^T are the A operand as they stand -----
#pragma unroll
      for (int t = 0; t < DB; t++) {
        float4v o = {0.0f, 0.0f, 0.0f, 0.0f};
        _Float16 const *vrow = vt + (16 * t + c) * LDV + 4 * g;
#pragma unroll
        for (int jj = 0; jj < KB / 2; jj++) {
          half4 b0 = *reinterpret_cast<half4 const *>(vrow + 32 * jj);
          half4 b1 = *reinterpret_cast<half4 const *>(vrow + 32 * jj + 16);
          half8 a = __builtin_shufflevector(e[2 * jj], e[2 * jj + 1], 0, 1, 2, 3, 4, 5, 6, 7);
          half8 b = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
          o = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, o, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
          _Float16 o16 = static_cast<_Float16>(o[r]);  // O tile (fp16)
          oacc[t][r] = (it == 0) ? o16
                                 : static_cast<_Float16>(static_cast<float>(oacc[t][r]) +
                                                         static_cast<float>(o16));
        }
      }
    }
  }

  // ---- store: through LDS so every lane writes a 16-byte row segment ----------------
  _Float16 *ow = o_stage + wave * 16 * LDO;
#pragma unroll
  for (int t = 0; t < DB; t++) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      ow[(4 * g + r) * LDO + 16 * t + c] = oacc[t][r];
    }
  }
  __syncthreads();
  {
    _Float16 *og = static_cast<_Float16 *>(const_cast<void *>(P.o.ptr)) +
                   tile_offset(P.o, bx, by, bz, 0) + (long long)row_base * P.o.d_cols;
    constexpr int CH = DV / 8;  // 16-byte chunks per row
    for (int e = lane; e < 16 * CH; e += 64) {
      int rr = e / CH, cc = (e % CH) * 8;
      *reinterpret_cast<uint4v *>(og + (long long)rr * P.o.d_cols + cc) =
          *reinterpret_cast<uint4v const *>(ow + rr * LDO + cc);
    }
  }
  if (!HAS_DIV && g == 0) {
    _Float16 *rg = static_cast<_Float16 *>(const_cast<void *>(P.r.ptr)) +
                   tile_offset(P.r, bx, by, bz, 0);
    rg[(long long)(row_base + c) * P.r.d_cols] = racc;
  }
}

// ---------------------------------------------------------------------------------------
// host: recognise the family in a lowered program and launch
// ---------------------------------------------------------------------------------------
namespace {

TileAddr tile_addr(DevOp const &op, void const *ptr) {
  TileAddr t;
  t.ptr = ptr;
  for (int i = 0; i < 3; i++) {
    t.row_bs[i] = op.row_bs[i];
    t.col_bs[i] = op.col_bs[i];
    t.g_bs[i] = op.g_bs[i];
  }
  t.row_fs = op.row_fs;
  t.col_fs = op.col_fs;
  t.g_fs = op.g_fs;
  t.d_cols = op.d_cols;
  return t;
}

struct Match {
  int q, k, v;        // load op indices
  int out_o, out_r;   // output op indices (out_r < 0 in form A)
  bool has_div;
  int m, D, NK, DV;
};

bool match(DevProgram const &P, Match &M) {
  if (P.num_ops < 9 || P.ops[0].kind != DOP_LOAD || P.ops[1].kind != DOP_LOAD ||
      P.ops[2].kind != DOP_LOAD || P.ops[3].kind != DOP_MATMUL) {
    return false;
  }
  auto loader_of = [&](int tensor) {
    for (int i = 0; i < 3; i++) {
      if (P.ops[i].dst == tensor) {
        return i;
      }
    }
    return -1;
  };
  DevOp const &mm1 = P.ops[3];
  DevOp const &ex = P.ops[4];
  M.q = loader_of(mm1.src0);
  M.k = loader_of(mm1.src1);
  if (M.q < 0 || M.k < 0 || M.q == M.k || ex.kind != DOP_UNARY || ex.sub != TB_EXP_OP ||
      ex.dst != mm1.dst) {
    return false;
  }
  int const E = mm1.dst;
  auto is_rowsum = [&](DevOp const &op) {
    return op.kind == DOP_REDUCE && op.src0 == E && P.t[op.dst].cols == 1 &&
           P.t[op.dst].rows == P.t[E].rows && op.red_inner == 1 && op.red_deg == P.t[E].cols;
  };
  int mm2 = -1, red = -1;
  if (P.num_ops == 9 && is_rowsum(P.ops[5]) && P.ops[6].kind == DOP_BINARY &&
      P.ops[6].sub == TB_DIV_OP && P.ops[6].src0 == E && P.ops[6].src1 == P.ops[5].dst &&
      P.ops[7].kind == DOP_MATMUL && P.ops[7].src0 == P.ops[6].dst &&
      P.ops[8].kind == DOP_OUTPUT && P.ops[8].src0 == P.ops[7].dst) {
    M.has_div = true;
    mm2 = 7;
    M.out_o = 8;
    M.out_r = -1;
  } else if (P.num_ops == 9 && P.ops[7].kind == DOP_OUTPUT && P.ops[8].kind == DOP_OUTPUT) {
    if (P.ops[5].kind == DOP_MATMUL && is_rowsum(P.ops[6])) {
      mm2 = 5;
      red = 6;
    } else if (is_rowsum(P.ops[5]) && P.ops[6].kind == DOP_MATMUL) {
      mm2 = 6;
      red = 5;
    } else {
      return false;
    }
    if (P.ops[mm2].src0 != E) {
      return false;
    }
    M.has_div = false;
    M.out_o = M.out_r = -1;
    for (int o = 7; o <= 8; o++) {
      if (P.ops[o].src0 == P.ops[mm2].dst) {
        M.out_o = o;
      } else if (P.ops[o].src0 == P.ops[red].dst) {
        M.out_r = o;
      }
    }
    if (M.out_o < 0 || M.out_r < 0) {
      return false;
    }
  } else {
    return false;
  }
  M.v = loader_of(P.ops[mm2].src1);
  if (M.v < 0 || M.v == M.q || M.v == M.k) {
    return false;
  }
  DevTensor const &tq = P.t[P.ops[M.q].dst], &tk = P.t[P.ops[M.k].dst], &tv = P.t[P.ops[M.v].dst];
  M.m = tq.rows;
  M.D = tq.cols;
  M.NK = tk.cols;
  M.DV = tv.cols;
  if (tk.rows != M.D || tv.rows != M.NK || M.m % 16 != 0) {
    return false;
  }
  // Q must be loop invariant; all tiles reachable with 16-byte accesses
  DevOp const &lq = P.ops[M.q];
  if (lq.row_fs != 0 || lq.col_fs != 0 || lq.g_fs != 0) {
    return false;
  }
  if (!lq.galign || !P.ops[M.k].galign || !P.ops[M.v].galign || !P.ops[M.out_o].galign) {
    return false;
  }
  for (void const *p : {P.in[lq.io], P.in[P.ops[M.k].io], P.in[P.ops[M.v].io],
                        (void const *)P.out[P.ops[M.out_o].io]}) {
    if ((reinterpret_cast<uintptr_t>(p) & 15) != 0) {
      return false;
    }
  }
  return true;
}

template <int D, int NK, int DV>
int launch_shape(AttnParams const &A, bool has_div, dim3 grid, int threads, int lds) {
  State &s = state();
  auto set_lds = [&](void const *fn) -> int {
    if (lds > 65536) {
      MI355_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    }
    return MI355_OK;
  };
  if (has_div) {
    int rc = set_lds(reinterpret_cast<void const *>(attn_fused_kernel<D, NK, DV, true>));
    if (rc != MI355_OK) {
      return rc;
    }
    attn_fused_kernel<D, NK, DV, true><<<grid, threads, lds, s.stream>>>(A);
  } else {
    int rc = set_lds(reinterpret_cast<void const *>(attn_fused_kernel<D, NK, DV, false>));
    if (rc != MI355_OK) {
      return rc;
    }
    attn_fused_kernel<D, NK, DV, false><<<grid, threads, lds, s.stream>>>(A);
  }
  MI355_HIP(hipGetLastError());
  return 1;
}

}  // namespace

static bool shape_supported(Match const &M) {
  return (M.D == 64 && M.DV == 64 && (M.NK == 64 || M.NK == 128 || M.NK == 256)) ||
         (M.D == 128 && M.DV == 128 && M.NK == 64);
}

bool attention_applicable(DevProgram const &P) {
  Match M;
  return match(P, M) && shape_supported(M);
}

int try_launch_attention(DevProgram const &P) {
  Match M;
  if (!match(P, M) || !shape_supported(M)) {
    return 0;
  }
  State &s = state();
  AttnParams A;
  A.q = tile_addr(P.ops[M.q], P.in[P.ops[M.q].io]);
  A.k = tile_addr(P.ops[M.k], P.in[P.ops[M.k].io]);
  A.v = tile_addr(P.ops[M.v], P.in[P.ops[M.v].io]);
  A.o = tile_addr(P.ops[M.out_o], P.out[P.ops[M.out_o].io]);
  A.r = M.out_r >= 0 ? tile_addr(P.ops[M.out_r], P.out[P.ops[M.out_r].io]) : A.o;
  A.forloop_range = P.forloop_range;
  // wavefronts per workgroup: as many as the tile has 16-row groups, at most 4, fewer
  // when that is what it takes to put a workgroup on every compute unit
  int const groups = M.m / 16;
  int nw = groups >= 4 && groups % 4 == 0 ? 4 : (groups % 2 == 0 ? 2 : 1);
  long long const blocks = (long long)P.grid[0] * P.grid[1] * P.grid[2];
  while (nw > 1 && blocks * (groups / nw) < 256) {
    nw /= 2;
  }
  A.split = groups / nw;
  if ((long long)P.grid[0] * A.split > 2147483647LL) {
    return 0;
  }
  int const stage_bytes = (M.NK * (M.D + 8) + M.DV * (M.NK + 8)) * 2;
  int const out_bytes = nw * 16 * (M.DV + 8) * 2;
  int stages = (96 * 1024 - out_bytes) / stage_bytes;
  stages = stages < 1 ? 1 : (stages > P.forloop_range ? P.forloop_range : stages);
  A.stages = stages;
  A.lds_stage_bytes = stage_bytes;
  int const lds = stages * stage_bytes + out_bytes;
  if (lds > s.max_lds) {
    return 0;
  }
  dim3 grid(P.grid[0] * A.split, P.grid[1], P.grid[2]);
  int rc;
  if (M.D == 64 && M.NK == 64) {
    rc = launch_shape<64, 64, 64>(A, M.has_div, grid, nw * 64, lds);
  } else if (M.D == 64 && M.NK == 128) {
    rc = launch_shape<64, 128, 64>(A, M.has_div, grid, nw * 64, lds);
  } else if (M.D == 64 && M.NK == 256) {
    rc = launch_shape<64, 256, 64>(A, M.has_div, grid, nw * 64, lds);
  } else {
    rc = launch_shape<128, 64, 128>(A, M.has_div, grid, nw * 64, lds);
  }
  if (rc == 1) {
    s.last_launch.kernel_id = MI355_KERNEL_F16_ATTENTION;
    s.last_launch.workgroups = grid.x * grid.y * grid.z;
    s.last_launch.threads = nw * 64;
    s.last_launch.lds_bytes = lds;
    s.last_launch.row_split = A.split;
  }
  return rc;
}

}  // namespace mi355
