// Fused kernel for the skinny-GEMM family of thread-block graphs: a handful of rows
// of activations against streamed weight tiles, accumulated over the for-loop.
//
//   plain      O  = sum_i pro(A_i) . B_i                         pro in {id, exp, silu}
//   two-weight O1 = sum_i A_i . B1_i ;  O2 = sum_i A_i . B2_i    (gated MLP, first half)
//   gate       O  = sum_i (silu(G_i) * U_i) . B_i                (gated MLP, second half)
//   lora       O  = sum_i [X_i | X_i.A_i] . [W_i ; B]            (concat-then-matmul,
//                                                                 cpp_examples/lora.cc:45-67)
//
// These are HBM-bound: what matters is how many bytes of weights are in flight, not
// the MFMAs.  Design:
//  * the plan's grid is a lower bound on parallelism.  Each logical block's for-loop
//    is cut into `ksplit` contiguous ranges handled by different workgroups, sized so
//    that a few workgroups sit on every compute unit; a workgroup issues every load
//    of an iteration before it waits for any, so one compute unit keeps several
//    whole tiles in flight;
//  * the reference's generated programs round each iteration's product to fp16 and
//    add it to an fp16 accumulator in iteration order (src/kernel/triton_code_gen.cc:
//    223-232).  A workgroup that owns a whole for-loop does exactly that in registers.
//    When the for-loop is cut into ranges, summing each range by itself would regroup
//    the fp16 additions ((t0+t1)+(t2+t3) instead of ((t0+t1)+t2)+t3), which is a
//    different rounding sequence; so a range's workgroup stores every iteration's fp16
//    product tile to a scratch slab instead (a few percent of the weight bytes) and a
//    second, small launch adds the tiles of each block in ITERATION order, rounding to
//    fp16 after each add: the same sequence of roundings as the unsplit loop;
//  * products are formed transposed (weights as the first MFMA operand), which leaves a
//    lane with four consecutive output columns of one row: 8-byte stores;
//  * weight tiles arrive [k][n] with n contiguous while the MFMA wants k contiguous
//    per lane, so they are transposed once while being staged into LDS (4 x 16 B
//    global reads -> 8 x 8 B LDS writes per 4x8 patch), into unpadded rows with a
//    16-byte-chunk XOR swizzle; activation tiles are staged as they are, with the
//    element-wise prologue applied on the way;
//  * the LoRA inner product is produced transposed ((X.A)^T = A^T.X^T), which leaves
//    each lane holding the A-operand fragment of the following [X.A].B MFMA, so it
//    never leaves registers and the two concats cost nothing.
#include "common.h"
#include "tb_program.h"

namespace mi355 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

enum { PRO_NONE = 0, PRO_EXP = 1, PRO_SILU = 2, PRO_SILU_MUL = 3 };

struct GTile {
  void const *ptr;
  int row_bs[3], col_bs[3], row_fs, col_fs;
  int g_bs[3], g_fs;
  int d_cols;
};

struct GemmParams {
  GTile a0, a1;      // activation-side tiles [M][KT] (a1: second operand of the gate form)
  GTile b0, b1;      // weight tiles [KT][64]
  GTile la, lb;      // lora: A tile [KT][16], B tile [16][64] (loop invariant)
  GTile o0, o1;      // outputs
  int M, KT;         // rows of the activation tile, k extent of one iteration
  int forloop_range;
  int ksplit;        // workgroups per logical block
  _Float16 *scratch; // [blocks][forloop_range][NB][M][64] fp16 product tiles (ksplit > 1)
};

__device__ __forceinline__ long long gtile_offset(GTile const &t, int bx, int by, int bz, int it) {
  int row0 = bx * t.row_bs[0] + by * t.row_bs[1] + bz * t.row_bs[2] + it * t.row_fs;
  int col0 = bx * t.col_bs[0] + by * t.col_bs[1] + bz * t.col_bs[2] + it * t.col_fs;
  long long base = (long long)bx * t.g_bs[0] + (long long)by * t.g_bs[1] +
                   (long long)bz * t.g_bs[2] + (long long)it * t.g_fs;
  return base + (long long)row0 * t.d_cols + col0;
}

// 16-byte chunk `chunk` of row `row` in a swizzled LDS tile with LD halfs per row.
// `mask` = (chunks per row - 1) & 7 keeps the XOR inside the row for narrow tiles.
__device__ __forceinline__ int sw_chunk(int row, int chunk, int LD, int mask) {
  return row * LD + ((chunk ^ ((row ^ (row >> 3)) & mask)) << 3);
}

__device__ __forceinline__ float prologue(int pro, float x) {
  if (pro == PRO_EXP) {
    return __expf(x);
  }
  return x / (1.0f + __expf(-x));
}

// Transposing stage of a [R][C] tile (C contiguous, row stride ld) into dst[C][R]
// (swizzled, R halfs per row).  All loads first, then the register transposes and
// the LDS writes.  PPT = patches per thread (compile-time bound).
template <int PPT>
__device__ __forceinline__ void stage_weight(_Float16 const *__restrict__ src, int ld, int R, int C,
                                             _Float16 *__restrict__ dst, int tid, int nthreads) {
  int const cblocks = C / 8, patches = (R / 4) * cblocks;
  int const mask = ((R / 8) - 1) & 7;
  uint4v x[PPT][4];
#pragma unroll
  for (int i = 0; i < PPT; i++) {
    int p = tid + i * nthreads;
    if (p < patches) {
      int cb = p % cblocks, rb = p / cblocks;
      _Float16 const *s = src + (long long)(4 * rb) * ld + 8 * cb;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        x[i][j] = *reinterpret_cast<uint4v const *>(s + (long long)j * ld);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < PPT; i++) {
    int p = tid + i * nthreads;
    if (p < patches) {
      int cb = p % cblocks, rb = p / cblocks;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        uint2v even, odd;
        even.x = (x[i][0][w] & 0xffffu) | (x[i][1][w] << 16);
        even.y = (x[i][2][w] & 0xffffu) | (x[i][3][w] << 16);
        odd.x = (x[i][0][w] >> 16) | (x[i][1][w] & 0xffff0000u);
        odd.y = (x[i][2][w] >> 16) | (x[i][3][w] & 0xffff0000u);
        int row = 8 * cb + 2 * w;
        *reinterpret_cast<uint2v *>(dst + sw_chunk(row, rb >> 1, R, mask) + (rb & 1) * 4) = even;
        *reinterpret_cast<uint2v *>(dst + sw_chunk(row + 1, rb >> 1, R, mask) + (rb & 1) * 4) = odd;
      }
    }
  }
}

// The two halves of stage_weight for tiles that are prefetched: the global loads of the
// next iteration's tile are issued before the current one is multiplied and the
// register transposes / LDS writes happen an iteration later.
template <int PPT>
__device__ __forceinline__ void load_weight(_Float16 const *__restrict__ src, int ld, int R, int C,
                                            uint4v (&x)[PPT][4], int tid, int nthreads) {
  int const cblocks = C / 8, patches = (R / 4) * cblocks;
#pragma unroll
  for (int i = 0; i < PPT; i++) {
    int p = tid + i * nthreads;
    if (p < patches) {
      int cb = p % cblocks, rb = p / cblocks;
      _Float16 const *s = src + (long long)(4 * rb) * ld + 8 * cb;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        x[i][j] = *reinterpret_cast<uint4v const *>(s + (long long)j * ld);
      }
    }
  }
}

template <int PPT>
__device__ __forceinline__ void store_weight(uint4v const (&x)[PPT][4], int R, int C,
                                             _Float16 *__restrict__ dst, int tid, int nthreads) {
  int const cblocks = C / 8, patches = (R / 4) * cblocks;
  int const mask = ((R / 8) - 1) & 7;
#pragma unroll
  for (int i = 0; i < PPT; i++) {
    int p = tid + i * nthreads;
    if (p < patches) {
      int cb = p % cblocks, rb = p / cblocks;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        uint2v even, odd;  // byte permute: selector bytes 0-3 from the second operand
        even.x = __builtin_amdgcn_perm(x[i][1][w], x[i][0][w], 0x05040100u);
        even.y = __builtin_amdgcn_perm(x[i][3][w], x[i][2][w], 0x05040100u);
        odd.x = __builtin_amdgcn_perm(x[i][1][w], x[i][0][w], 0x07060302u);
        odd.y = __builtin_amdgcn_perm(x[i][3][w], x[i][2][w], 0x07060302u);
        int row = 8 * cb + 2 * w;
        *reinterpret_cast<uint2v *>(dst + sw_chunk(row, rb >> 1, R, mask) + (rb & 1) * 4) = even;
        *reinterpret_cast<uint2v *>(dst + sw_chunk(row + 1, rb >> 1, R, mask) + (rb & 1) * 4) = odd;
      }
    }
  }
}

// MT m-tiles of 16 rows, NB weight matrices, 4 wavefronts = the 4 column tiles of a
// 64-column weight tile.  KTMAX bounds the staging register arrays.
template <int MT, int NB, int PRO, bool LORA, int KTMAX>
__global__ __launch_bounds__(256) void gemm_fused_kernel(GemmParams const P) {
  constexpr int NT = 256;
  constexpr int WPPT = ((KTMAX / 4) * 8 + NT - 1) / NT;  // weight patches per thread
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  int const tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  int const g = lane / 16, c = lane % 16;
  int const M = P.M, KT = P.KT, F = P.forloop_range;
  int const kmask = ((KT / 8) - 1) & 7;

  // logical block and k range of this workgroup; consecutive ids share a block so the
  // block's partial products are written and read from one XCD's L2 where possible
  int const ks = blockIdx.x % P.ksplit;
  int const bx = blockIdx.x / P.ksplit, by = blockIdx.y, bz = blockIdx.z;
  int const per = (F + P.ksplit - 1) / P.ksplit;
  int const it_begin = ks * per, it_end = (it_begin + per) < F ? (it_begin + per) : F;
  int const block_linear = bx + (gridDim.x / P.ksplit) * (by + gridDim.y * bz);

  // LDS: activation tile [16*MT][KT] | weight tiles NB x [64][KT] | lora A^T [16][KT] |
  // lora B^T [64][16]
  _Float16 *a_lds = reinterpret_cast<_Float16 *>(lds);
  _Float16 *b_lds = a_lds + 16 * MT * KT;
  _Float16 *la_lds = b_lds + NB * 64 * KT;
  _Float16 *lb_lds = la_lds + (LORA ? 16 * KT : 0);

  if (LORA) {
    // B [16][64] -> B^T [64][16], loop invariant: 32 patches
    _Float16 const *src = static_cast<_Float16 const *>(P.lb.ptr) + gtile_offset(P.lb, bx, by, bz, 0);
    stage_weight<1>(src, P.lb.d_cols, 16, 64, lb_lds, tid, NT);
  }

  _Float16 acc16[NB][MT][4];  // O[16mt + c][16*wave + 4g + r], used when ksplit == 1
#pragma unroll
  for (int b = 0; b < NB; b++) {
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        acc16[b][mt][r] = (_Float16)0.0f;
      }
    }
  }

  // Prefetch registers: the raw tiles of the next iteration.
  constexpr int APT = (16 * MT * (KTMAX / 8) + NT - 1) / NT;  // activation chunks per thread
  constexpr int LPPT = (KTMAX / 4) * 2 / NT + 1;             // lora A patches per thread
  uint4v wreg[NB][WPPT][4];
  uint4v lreg[LORA ? LPPT : 1][4];
  half8 areg[APT], ureg[PRO == PRO_SILU_MUL ? APT : 1];
  int const chunks_a = KT / 8;
  auto fetch = [&](int it) {
    _Float16 const *a0 = static_cast<_Float16 const *>(P.a0.ptr) + gtile_offset(P.a0, bx, by, bz, it);
    _Float16 const *a1 = PRO == PRO_SILU_MUL
                             ? static_cast<_Float16 const *>(P.a1.ptr) + gtile_offset(P.a1, bx, by, bz, it)
                             : a0;
#pragma unroll
    for (int i = 0; i < APT; i++) {
      int const e = tid + i * NT;
      int const row = e / chunks_a, ch = e % chunks_a;
      if (e < 16 * MT * chunks_a && row < M) {
        areg[i] = *reinterpret_cast<half8 const *>(a0 + (long long)row * P.a0.d_cols + 8 * ch);
        if (PRO == PRO_SILU_MUL) {
          ureg[i] = *reinterpret_cast<half8 const *>(a1 + (long long)row * P.a1.d_cols + 8 * ch);
        }
      }
    }
#pragma unroll
    for (int b = 0; b < NB; b++) {
      GTile const &bt = b == 0 ? P.b0 : P.b1;
      _Float16 const *src = static_cast<_Float16 const *>(bt.ptr) + gtile_offset(bt, bx, by, bz, it);
      load_weight<WPPT>(src, bt.d_cols, KT, 64, wreg[b], tid, NT);
    }
    if (LORA) {
      _Float16 const *src = static_cast<_Float16 const *>(P.la.ptr) + gtile_offset(P.la, bx, by, bz, it);
      load_weight<LORA ? LPPT : 1>(src, P.la.d_cols, KT, 16, lreg, tid, NT);
    }
  };
  // registers -> LDS: activation tile as it is (prologue applied), weights transposed
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < APT; i++) {
      int const e = tid + i * NT;
      int const row = e / chunks_a, ch = e % chunks_a;
      if (e < 16 * MT * chunks_a) {
        half8 v;
        if (row < M) {
          v = areg[i];
          if (PRO == PRO_EXP || PRO == PRO_SILU) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
              v[j] = static_cast<_Float16>(prologue(PRO, static_cast<float>(v[j])));
            }
          } else if (PRO == PRO_SILU_MUL) {
            half8 u = ureg[i];
#pragma unroll
            for (int j = 0; j < 8; j++) {
              _Float16 sg = static_cast<_Float16>(prologue(PRO_SILU, static_cast<float>(v[j])));
              v[j] = static_cast<_Float16>(static_cast<float>(sg) * static_cast<float>(u[j]));
            }
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; j++) {
            v[j] = (_Float16)0.0f;  // rows past M (M == 8) contribute nothing
          }
        }
        *reinterpret_cast<half8 *>(a_lds + sw_chunk(row, ch, KT, kmask)) = v;
      }
    }
#pragma unroll
    for (int b = 0; b < NB; b++) {
      store_weight<WPPT>(wreg[b], KT, 64, b_lds + b * 64 * KT, tid, NT);
    }
    if (LORA) {
      store_weight<LORA ? LPPT : 1>(lreg, KT, 16, la_lds, tid, NT);
    }
  };
  bool const split = P.ksplit > 1;
  auto compute = [&](int it) {
    // ---- lora inner product, transposed: D^T = A^T . X^T (rows past M are zero) -----
    half4 dfrag = {(_Float16)0.0f, (_Float16)0.0f, (_Float16)0.0f, (_Float16)0.0f};
    if (LORA) {
      float4v d = {0.0f, 0.0f, 0.0f, 0.0f};
      for (int k0 = 0; k0 < KT; k0 += 32) {
        int ch = (k0 >> 3) + g;
        half8 a = *reinterpret_cast<half8 const *>(la_lds + sw_chunk(c, ch, KT, kmask));  // A^T[n=c]
        half8 x = *reinterpret_cast<half8 const *>(a_lds + sw_chunk(c, ch, KT, kmask));   // X[m=c]
        d = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, x, d, 0, 0, 0);
      }
      // d[r] = D[m = c][n = 4g + r]: the A fragment of a 16x16x16 MFMA over k = n
#pragma unroll
      for (int r = 0; r < 4; r++) {
        dfrag[r] = static_cast<_Float16>(d[r]);  // the [X.A] tile, fp16
      }
    }
    // ---- main products: wavefront `wave` owns output columns 16*wave .. +15 ---------
#pragma unroll
    for (int b = 0; b < NB; b++) {
      float4v o[MT];
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        o[mt] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
      }
      _Float16 const *bt = b_lds + b * 64 * KT;
      for (int k0 = 0; k0 < KT; k0 += 32) {
        int ch = (k0 >> 3) + g;
        half8 w = *reinterpret_cast<half8 const *>(bt + sw_chunk(16 * wave + c, ch, KT, kmask));
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
          half8 a = *reinterpret_cast<half8 const *>(a_lds + sw_chunk(16 * mt + c, ch, KT, kmask));
          // weights first: o[mt][r] = O[m = 16mt + c][n = 16 wave + 4g + r]
          o[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, a, o[mt], 0, 0, 0);
        }
      }
      if (LORA) {
        // + [X.A] . B over the 16 concatenated k; B^T rows hold 16 halfs (2 chunks)
        half4 w = *reinterpret_cast<half4 const *>(lb_lds + sw_chunk(16 * wave + c, g >> 1, 16, 1) +
                                                   (g & 1) * 4);
        o[0] = __builtin_amdgcn_mfma_f32_16x16x16f16(w, dfrag, o[0], 0, 0, 0);
      }
      if (split) {
        // this iteration's fp16 product tile goes to its slot of the scratch slab
        _Float16 *tile = P.scratch + (((long long)block_linear * F + it) * NB + b) * (long long)M * 64;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
          half4 p16;
#pragma unroll
          for (int r = 0; r < 4; r++) {
            p16[r] = static_cast<_Float16>(o[mt][r]);
          }
          if (16 * mt + c < M) {
            *reinterpret_cast<half4 *>(tile + (16 * mt + c) * 64 + 16 * wave + 4 * g) = p16;
          }
        }
      } else {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
#pragma unroll
          for (int r = 0; r < 4; r++) {
            _Float16 p16 = static_cast<_Float16>(o[mt][r]);  // this iteration's product tile
            acc16[b][mt][r] = static_cast<_Float16>(static_cast<float>(acc16[b][mt][r]) +
                                                    static_cast<float>(p16));
          }
        }
      }
    }
  };

  // Steady state is branch-free: the next iteration's loads are issued as soon as this
  // iteration's tiles are in LDS and stay in flight while it is multiplied; the last
  // iteration is peeled.
  fetch(it_begin);
  for (int it = it_begin; it + 1 < it_end; it++) {
    __syncthreads();  // previous iteration's tiles fully consumed
    stash();
    __syncthreads();
    fetch(it + 1);
    __builtin_amdgcn_sched_barrier(0);  // keep the loads ahead of the products
    compute(it);
  }
  __syncthreads();
  stash();
  __syncthreads();
  compute(it_end - 1);

  // ---- finish ---------------------------------------------------------------------------
  // A split for-loop has left every iteration's tile in the scratch slab.  Otherwise the
  // workgroup's fp16 sums go through LDS so that they leave as 16-byte row segments.
  if (split) {
    return;
  }
  constexpr int LDT = 64 + 8;
  _Float16 *t_lds = reinterpret_cast<_Float16 *>(lds);  // the tiles are dead by now
  __syncthreads();
#pragma unroll
  for (int b = 0; b < NB; b++) {
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      half4 v;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        v[r] = acc16[b][mt][r];
      }
      *reinterpret_cast<half4 *>(t_lds + (b * 16 * MT + 16 * mt + c) * LDT + 16 * wave + 4 * g) = v;
    }
  }
  __syncthreads();
  int const chunks = M * 8;  // 16-byte chunks of one [M][64] tile
#pragma unroll
  for (int b = 0; b < NB; b++) {
    GTile const &ot = b == 0 ? P.o0 : P.o1;
    _Float16 *og = static_cast<_Float16 *>(const_cast<void *>(ot.ptr)) + gtile_offset(ot, bx, by, bz, 0);
    for (int e = tid; e < chunks; e += NT) {
      int row = e / 8, col = (e % 8) * 8;
      *reinterpret_cast<uint4v *>(og + (long long)row * ot.d_cols + col) =
          *reinterpret_cast<uint4v const *>(t_lds + (b * 16 * MT + row) * LDT + col);
    }
  }
}

// Second pass of a split for-loop: adds the fp16 product tiles of every logical block in
// iteration order (fp16 rounding after each add: the rounding sequence of the sequential
// loop) and stores the block's output tile.  A separate launch rather than a last-arriver
// fix-up: the kernel boundary makes the slabs visible without device-scope fences,
// which on this part write back and invalidate a whole L2 each time.
template <int NB>
__global__ __launch_bounds__(256) void gemm_combine_kernel(GemmParams const P) {
  int const tid = threadIdx.x, M = P.M, F = P.forloop_range;
  int const bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  int const block_linear = bx + gridDim.x * (by + gridDim.y * bz);
  long long const slab = (long long)NB * M * 64;  // one iteration's tiles
  _Float16 const *all = P.scratch + (long long)block_linear * F * slab;
  // 4-byte pieces (two neighbouring columns), so that even an 8-row tile keeps every thread
  // busy, and sixteen iterations' loads in flight per piece: the adds are a dependent chain,
  // the loads are not.
  typedef _Float16 half2v __attribute__((ext_vector_type(2)));
  int const pieces = M * 32;
#pragma unroll
  for (int b = 0; b < NB; b++) {
    GTile const &ot = b == 0 ? P.o0 : P.o1;
    _Float16 *og = static_cast<_Float16 *>(const_cast<void *>(ot.ptr)) + gtile_offset(ot, bx, by, bz, 0);
    for (int e = tid; e < pieces; e += 256) {
      int row = e / 32, col = (e % 32) * 2;
      _Float16 const *sp = all + (long long)b * M * 64 + row * 64 + col;
      float a0 = 0.0f, a1 = 0.0f;  // hold fp16 values between the adds
      int q = 0;
      for (; q + 16 <= F; q += 16) {
        half2v v[16];
#pragma unroll
        for (int u = 0; u < 16; u++) {
          v[u] = *reinterpret_cast<half2v const *>(sp + (long long)(q + u) * slab);
        }
#pragma unroll
        for (int u = 0; u < 16; u++) {
          a0 = static_cast<float>(static_cast<_Float16>(a0 + static_cast<float>(v[u][0])));
          a1 = static_cast<float>(static_cast<_Float16>(a1 + static_cast<float>(v[u][1])));
        }
      }
      for (; q < F; q++) {
        half2v v = *reinterpret_cast<half2v const *>(sp + (long long)q * slab);
        a0 = static_cast<float>(static_cast<_Float16>(a0 + static_cast<float>(v[0])));
        a1 = static_cast<float>(static_cast<_Float16>(a1 + static_cast<float>(v[1])));
      }
      half2v r;
      r[0] = static_cast<_Float16>(a0);
      r[1] = static_cast<_Float16>(a1);
      *reinterpret_cast<half2v *>(og + (long long)row * ot.d_cols + col) = r;
    }
  }
}

// ---------------------------------------------------------------------------------------
// host: recognise the family and launch
// ---------------------------------------------------------------------------------------
namespace {

GTile gtile(DevOp const &op, void const *ptr) {
  GTile t;
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

struct GMatch {
  int pro, nb;
  bool lora;
  int a0, a1, b0, b1, la, lb;  // load op indices (-1 when absent)
  int o0, o1;                  // output op indices
  int M, KT;
};

int loader_of(DevProgram const &P, int nloads, int tensor) {
  for (int i = 0; i < nloads; i++) {
    if (P.ops[i].dst == tensor) {
      return i;
    }
  }
  return -1;
}

bool gmatch(DevProgram const &P, GMatch &G) {
  int nl = 0;
  while (nl < P.num_ops && P.ops[nl].kind == DOP_LOAD) {
    nl++;
  }
  G.a1 = G.b1 = G.la = G.lb = G.o1 = -1;
  G.pro = PRO_NONE;
  G.nb = 1;
  G.lora = false;
  DevOp const *o = P.ops + nl;
  int const n = P.num_ops - nl;
  auto L = [&](int tensor) { return loader_of(P, nl, tensor); };
  if (nl == 2 && n == 2 && o[0].kind == DOP_MATMUL && o[1].kind == DOP_OUTPUT &&
      o[1].src0 == o[0].dst) {
    G.a0 = L(o[0].src0);
    G.b0 = L(o[0].src1);
    G.o0 = nl + 1;
  } else if (nl == 2 && n == 3 && o[0].kind == DOP_UNARY && o[1].kind == DOP_MATMUL &&
             o[1].src0 == o[0].dst && o[2].kind == DOP_OUTPUT && o[2].src0 == o[1].dst) {
    G.pro = o[0].sub == TB_EXP_OP ? PRO_EXP : PRO_SILU;
    G.a0 = L(o[0].src0);
    G.b0 = L(o[1].src1);
    G.o0 = nl + 2;
  } else if (nl == 3 && n == 4 && o[0].kind == DOP_MATMUL && o[1].kind == DOP_MATMUL &&
             o[0].src0 == o[1].src0 && o[2].kind == DOP_OUTPUT && o[3].kind == DOP_OUTPUT &&
             o[2].src0 == o[0].dst && o[3].src0 == o[1].dst) {
    G.nb = 2;
    G.a0 = L(o[0].src0);
    G.b0 = L(o[0].src1);
    G.b1 = L(o[1].src1);
    G.o0 = nl + 2;
    G.o1 = nl + 3;
  } else if (nl == 3 && n == 4 && o[0].kind == DOP_UNARY && o[0].sub == TB_SILU_OP &&
             o[1].kind == DOP_BINARY && o[1].sub == TB_MUL_OP && o[1].src0 == o[0].dst &&
             o[2].kind == DOP_MATMUL && o[2].src0 == o[1].dst && o[3].kind == DOP_OUTPUT &&
             o[3].src0 == o[2].dst) {
    G.pro = PRO_SILU_MUL;
    G.a0 = L(o[0].src0);
    G.a1 = L(o[1].src1);
    G.b0 = L(o[2].src1);
    G.o0 = nl + 3;
    if (G.a1 < 0 || P.t[P.ops[G.a1].dst].rows != P.t[o[0].dst].rows ||
        P.t[P.ops[G.a1].dst].cols != P.t[o[0].dst].cols) {
      return false;
    }
  } else if (nl == 4 && n == 5 && o[0].kind == DOP_MATMUL && o[1].kind == DOP_CONCAT &&
             o[2].kind == DOP_CONCAT && o[3].kind == DOP_MATMUL && o[4].kind == DOP_OUTPUT &&
             o[1].src0 == o[0].src0 && o[1].src1 == o[0].dst &&   // [X | X.A]
             o[3].src0 == o[1].dst && o[3].src1 == o[2].dst && o[4].src0 == o[3].dst &&
             P.t[o[1].dst].rows == P.t[o[0].src0].rows &&          // concat along columns
             P.t[o[2].dst].cols == P.t[o[2].src0].cols) {          // concat along rows
    G.lora = true;
    G.a0 = L(o[0].src0);
    G.la = L(o[0].src1);
    G.b0 = L(o[2].src0);
    G.lb = L(o[2].src1);
    G.o0 = nl + 4;
    if (G.la < 0 || G.lb < 0) {
      return false;
    }
    DevTensor const &ta = P.t[P.ops[G.la].dst], &tb = P.t[P.ops[G.lb].dst];
    DevOp const &lb = P.ops[G.lb];
    if (ta.cols != 16 || tb.rows != 16 || tb.cols != 64 || lb.row_fs != 0 || lb.col_fs != 0 ||
        lb.g_fs != 0 || !P.ops[G.la].galign || !lb.galign) {
      return false;
    }
  } else {
    return false;
  }
  if (G.a0 < 0 || G.b0 < 0 || (G.nb == 2 && G.b1 < 0)) {
    return false;
  }
  DevTensor const &ta = P.t[P.ops[G.a0].dst], &tb = P.t[P.ops[G.b0].dst];
  G.M = ta.rows;
  G.KT = ta.cols;
  if (tb.rows != G.KT || tb.cols != 64 || G.KT % 32 != 0 || G.KT < 64 || G.KT > 512 ||
      !(G.M == 8 || (G.M % 16 == 0 && G.M <= 64))) {
    return false;
  }
  if (G.lora && (G.M != 16 || ta.rows != 16)) {
    return false;
  }
  if (G.nb == 2 && (P.t[P.ops[G.b1].dst].rows != G.KT || P.t[P.ops[G.b1].dst].cols != 64)) {
    return false;
  }
  for (int i : {G.a0, G.a1, G.b0, G.b1, G.la, G.lb}) {
    if (i >= 0 && (!P.ops[i].galign || (reinterpret_cast<uintptr_t>(P.in[P.ops[i].io]) & 15) != 0)) {
      return false;
    }
  }
  if (G.lora && (ta.cols != P.t[P.ops[G.la].dst].rows)) {
    return false;
  }
  for (int i : {G.o0, G.o1}) {
    if (i >= 0 && (!P.ops[i].galign || (reinterpret_cast<uintptr_t>(P.out[P.ops[i].io]) & 15) != 0)) {
      return false;
    }
  }
  return true;
}

template <int MT, int NB, int PRO, bool LORA>
int launch_kt(GemmParams const &A, dim3 grid, int lds) {
  State &s = state();
  auto go = [&](auto *fn) -> int {
    if (lds > 65536) {
      MI355_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(fn),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    }
    fn<<<grid, 256, lds, s.stream()>>>(A);
    MI355_HIP(hipGetLastError());
    return 1;
  };
  if (A.KT <= 64) {
    return go(gemm_fused_kernel<MT, NB, PRO, LORA, 64>);
  }
  if (A.KT <= 256) {
    return go(gemm_fused_kernel<MT, NB, PRO, LORA, 256>);
  }
  return go(gemm_fused_kernel<MT, NB, PRO, LORA, 512>);
}

}  // namespace

bool gemm_applicable(DevProgram const &P) {
  GMatch G;
  return gmatch(P, G);
}

int try_launch_gemm(DevProgram const &P) {
  GMatch G;
  if (!gmatch(P, G)) {
    return 0;
  }
  State &s = state();
  GemmParams A{};
  auto in_tile = [&](int i) { return gtile(P.ops[i], P.in[P.ops[i].io]); };
  A.a0 = in_tile(G.a0);
  A.a1 = G.a1 >= 0 ? in_tile(G.a1) : A.a0;
  A.b0 = in_tile(G.b0);
  A.b1 = G.b1 >= 0 ? in_tile(G.b1) : A.b0;
  A.la = G.la >= 0 ? in_tile(G.la) : A.a0;
  A.lb = G.lb >= 0 ? in_tile(G.lb) : A.a0;
  A.o0 = gtile(P.ops[G.o0], P.out[P.ops[G.o0].io]);
  A.o1 = G.o1 >= 0 ? gtile(P.ops[G.o1], P.out[P.ops[G.o1].io]) : A.o0;
  A.M = G.M;
  A.KT = G.KT;
  A.forloop_range = P.forloop_range;
  int const mt = (G.M + 15) / 16;
  long long const blocks = (long long)P.grid[0] * P.grid[1] * P.grid[2];
  // Ranges per block: the split that minimises (rounds of resident workgroups) x
  // (iterations per workgroup + a fixed cost per workgroup + the combine's cost per range),
  // with two workgroups resident per compute unit.  Never more ranges than iterations.
  int ksplit = 1;
  {
    double best = 1e30;
    for (int cand = 1; cand <= P.forloop_range; cand++) {
      int const per = (P.forloop_range + cand - 1) / cand;
      if ((P.forloop_range + per - 1) / per != cand) {
        continue;  // would leave empty ranges
      }
      long long const rounds = (blocks * cand + 511) / 512;
      double const cost = (double)rounds * (per + 1.5 + 0.15 * cand);
      if (cost < best - 1e-9) {
        best = cost;
        ksplit = cand;
      }
    }
  }
  long long const scratch_elems = blocks * P.forloop_range * G.nb * G.M * 64;
  if (ksplit > 1 && (scratch_elems * 2 > (long long)s.scratch_bytes)) {
    ksplit = 1;
  }
  A.ksplit = ksplit;
  A.scratch = static_cast<_Float16 *>(s.scratch());
  int const tile_lds = (16 * mt * G.KT + G.nb * 64 * G.KT + (G.lora ? 16 * G.KT + 64 * 16 : 0)) * 2;
  int const out_lds = G.nb * 16 * mt * (64 + 8) * 2;
  int const lds = tile_lds > out_lds ? tile_lds : out_lds;
  if (lds > s.max_lds || (long long)P.grid[0] * ksplit > 2147483647LL) {
    return 0;
  }
  dim3 grid(P.grid[0] * ksplit, P.grid[1], P.grid[2]);
  int rc = 0;
#define MI355_GEMM_CASE(MTV, NBV, PROV, LORAV)                                        \
  if (mt == MTV && G.nb == NBV && G.pro == PROV && G.lora == LORAV) {                 \
    rc = launch_kt<MTV, NBV, PROV, LORAV>(A, grid, lds);                              \
  }
  MI355_GEMM_CASE(1, 1, PRO_NONE, false)
  MI355_GEMM_CASE(2, 1, PRO_NONE, false)
  MI355_GEMM_CASE(4, 1, PRO_NONE, false)
  MI355_GEMM_CASE(1, 1, PRO_EXP, false)
  MI355_GEMM_CASE(1, 1, PRO_SILU, false)
  MI355_GEMM_CASE(1, 2, PRO_NONE, false)
  MI355_GEMM_CASE(1, 1, PRO_SILU_MUL, false)
  MI355_GEMM_CASE(1, 1, PRO_NONE, true)
#undef MI355_GEMM_CASE
  if (rc == 1 && ksplit > 1) {
    dim3 cgrid(P.grid[0], P.grid[1], P.grid[2]);
    if (G.nb == 1) {
      gemm_combine_kernel<1><<<cgrid, 256, 0, s.stream()>>>(A);
    } else {
      gemm_combine_kernel<2><<<cgrid, 256, 0, s.stream()>>>(A);
    }
    MI355_HIP(hipGetLastError());
  }
  if (rc == 1) {
    s.last().kernel_id = MI355_KERNEL_F16_GEMM;
    s.last().workgroups = grid.x * grid.y * grid.z;
    s.last().threads = 256;
    s.last().lds_bytes = lds;
    s.last().row_split = ksplit;
  }
  return rc;
}

}  // namespace mi355
