// Device code of the fused skinny-GEMM kernels (gemm_fused_kernel and its fold gemm_combine_kernel,
// gemm_lanes_kernel) and the parameter blocks they take.  Header-only and free of host state:
// the backend library (gemm_fused.hip recognises the family, chooses kernel and launch shape) and
// the programs Graph::generate_hip_program writes both instantiate these templates.  They are
// what an emitted program of this backend runs where the reference emits Triton source
// (src/kernel/triton_code_gen.cc:84-352).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernarg.h"

namespace mi355 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

enum { PRO_NONE = 0, PRO_EXP = 1, PRO_SILU = 2, PRO_SILU_MUL = 3 };

// Where a tile of a device tensor starts: the element offset is linear in the block
// coordinates and the for-loop iteration, so the host folds the plan's row / column / batch
// strides into one stride per coordinate (a few scalar multiplies per tile address).
struct GTile {
  void const *ptr;
  int lin[4];  // elements per step of bx, by, bz and of the iteration (the host takes a plan on
               // these kernels only when every tile origin fits 31 bits: the parameter block
               // of the one-launch kernel then fits the scalar registers, and a tile address is
               // four 32-bit multiplies)
  int d_cols;  // row stride of the tensor
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
  return (long long)(bx * t.lin[0] + by * t.lin[1] + bz * t.lin[2] + it * t.lin[3]);
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

// Column-major weights (a [R][C] tile stored column by column: C rows of R contiguous halfs,
// `ld` halfs apart) already have k contiguous: the same two halves without the transpose.
// The tile is dst[C][R], R / 8 chunks of 16 bytes per row; slot (i, j) of thread `tid` is chunk
// (4 i + j) * nthreads + tid, so that the lanes of one load or store instruction walk
// consecutive chunks of a row (whole cache lines per instruction).
template <int PPT>
__device__ __forceinline__ void load_weight_cm(_Float16 const *__restrict__ src, int ld, int R, int C,
                                               uint4v (&x)[PPT][4], int tid, int nthreads) {
  int const cpr = R / 8, chunks = C * cpr;
#pragma unroll
  for (int i = 0; i < PPT; i++) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      int const q = (4 * i + j) * nthreads + tid;
      if (q < chunks) {
        x[i][j] = *reinterpret_cast<uint4v const *>(src + (long long)(q / cpr) * ld + 8 * (q % cpr));
      }
    }
  }
}

template <int PPT>
__device__ __forceinline__ void store_weight_cm(uint4v const (&x)[PPT][4], int R, int C,
                                                _Float16 *__restrict__ dst, int tid, int nthreads) {
  int const cpr = R / 8, chunks = C * cpr;
  int const mask = (cpr - 1) & 7;
#pragma unroll
  for (int i = 0; i < PPT; i++) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      int const q = (4 * i + j) * nthreads + tid;
      if (q < chunks) {
        *reinterpret_cast<uint4v *>(dst + sw_chunk(q / cpr, q % cpr, R, mask)) = x[i][j];
      }
    }
  }
}

// MT m-tiles of 16 rows, NB weight matrices, 4 wavefronts = the 4 column tiles of a
// 64-column weight tile.  KTMAX bounds the staging register arrays.  WCM: every weight-side
// operand (weights, lora A and B) is a column-major tensor.
template <int MT, int NB, int PRO, bool LORA, int KTMAX, bool WCM>
__global__ __launch_bounds__(256) void gemm_fused_kernel(GemmParams const P) {
  fetch_kernel_arguments<sizeof(GemmParams), 2>();  // every line of the block, one trip (gridDim.x, .y are read)
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
    if (WCM) {  // already B^T [64][16]: 128 chunks, copied as they are
      uint4v x[1][4];
      load_weight_cm<1>(src, P.lb.d_cols, 16, 64, x, tid, NT);
      store_weight_cm<1>(x, 16, 64, lb_lds, tid, NT);
    } else {
      stage_weight<1>(src, P.lb.d_cols, 16, 64, lb_lds, tid, NT);
    }
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
      if (WCM) {
        load_weight_cm<WPPT>(src, bt.d_cols, KT, 64, wreg[b], tid, NT);
      } else {
        load_weight<WPPT>(src, bt.d_cols, KT, 64, wreg[b], tid, NT);
      }
    }
    if (LORA) {
      _Float16 const *src = static_cast<_Float16 const *>(P.la.ptr) + gtile_offset(P.la, bx, by, bz, it);
      if (WCM) {
        load_weight_cm<LORA ? LPPT : 1>(src, P.la.d_cols, KT, 16, lreg, tid, NT);
      } else {
        load_weight<LORA ? LPPT : 1>(src, P.la.d_cols, KT, 16, lreg, tid, NT);
      }
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
      if (WCM) {
        store_weight_cm<WPPT>(wreg[b], KT, 64, b_lds + b * 64 * KT, tid, NT);
      } else {
        store_weight<WPPT>(wreg[b], KT, 64, b_lds + b * 64 * KT, tid, NT);
      }
    }
    if (LORA) {
      if (WCM) {
        store_weight_cm<LORA ? LPPT : 1>(lreg, KT, 16, la_lds, tid, NT);
      } else {
        store_weight<LORA ? LPPT : 1>(lreg, KT, 16, la_lds, tid, NT);
      }
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
  // A split for-loop leaves every iteration's tile in its own slot of the slab, so a workgroup
  // may walk its range in any order: each starts at a different iteration (rotating through the
  // range), so that at any moment the workgroups of the chip read at many different offsets
  // along k.  Started in step they would all sit at the same one or two offsets within the
  // operand's power-of-two row or column stride, i.e. on a fraction of the memory channels.
  int const n_it = it_end - it_begin;
  int const rot = split ? (int)((blockIdx.x / P.ksplit * 5u + blockIdx.y * 3u + blockIdx.z) % (unsigned)n_it) : 0;
  auto nth = [&](int i) {
    int const j = i + rot;
    return it_begin + (j >= n_it ? j - n_it : j);
  };
  fetch(nth(0));
  for (int i = 0; i + 1 < n_it; i++) {
    __syncthreads();  // previous iteration's tiles fully consumed
    stash();
    __syncthreads();
    fetch(nth(i + 1));
    __builtin_amdgcn_sched_barrier(0);  // keep the loads ahead of the products
    compute(nth(i));
  }
  __syncthreads();
  stash();
  __syncthreads();
  compute(nth(n_it - 1));

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
// which on this part write back and invalidate a whole L2 each time (with a fence per
// workgroup the LoRA plan took 77 us instead of 13).
template <int NB>
__global__ __launch_bounds__(256) void gemm_combine_kernel(GemmParams const P) {
  fetch_kernel_arguments<sizeof(GemmParams), 2>();  // (gridDim.x, .y are read)
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
      if (q < F) {
        // the tail's loads go out together as well (past the end: the last tile again, left out
        // of the sums), not one latency after the other
        half2v v[16];
#pragma unroll
        for (int u = 0; u < 16; u++) {
          int const it = q + u < F ? q + u : F - 1;
          v[u] = *reinterpret_cast<half2v const *>(sp + (long long)it * slab);
        }
#pragma unroll
        for (int u = 0; u < 16; u++) {
          if (q + u < F) {
            a0 = static_cast<float>(static_cast<_Float16>(a0 + static_cast<float>(v[u][0])));
            a1 = static_cast<float>(static_cast<_Float16>(a1 + static_cast<float>(v[u][1])));
          }
        }
      }
      half2v r;
      r[0] = static_cast<_Float16>(a0);
      r[1] = static_cast<_Float16>(a1);
      *reinterpret_cast<half2v *>(og + (long long)row * ot.d_cols + col) = r;
    }
  }
}


// ---------------------------------------------------------------------------------------
// One launch, no scratch: the output tile of a logical block is cut into 16-row x 16-column
// pieces and every piece is a workgroup of its own (four pieces across the 64 columns, one
// row of pieces per 16 activation rows), so a plan with a handful of blocks still covers the
// chip.  Inside a workgroup the wavefronts are ITERATION LANES: lane ip takes iterations ip,
// ip + IP, ... of the for-loop and needs nobody else for them --
//   * its activation rows arrive as MFMA operands straight from global memory (a lane's eight
//     consecutive k of one row are 16 contiguous bytes), the element-wise prologue is applied
//     in registers;
//   * its 16-column strip of each weight tile ([KT][16], 32 contiguous bytes per k) is copied
//     by direct-to-LDS loads into a buffer of its own and read back with transposing LDS
//     reads, which hand a lane the eight consecutive k of one column;
//   * one wait for all of its loads, then KT / 32 MFMAs per weight matrix (weights as the
//     first operand: a lane ends up with four consecutive columns of one row);
// so the workgroup is IP independent streams with no barrier in the loop.  Every iteration's
// product piece is rounded to fp16 into an LDS slot of its own; after ONE barrier the
// pieces are added in ITERATION order, rounding to fp16 after each add -- the arithmetic of
// the sequential loop (src/kernel/triton_code_gen.cc:223-232) -- and stored.
// Workgroup ids put the four column pieces of a block on ids that are equal modulo 8, i.e. on
// one XCD: the 128-byte lines of a weight row that the pieces share are fetched into one L2.
struct LaneParams {
  GemmParams g;
  int gx, gy;        // the plan's grid (x, y): the logical block index is decoded from a flat id
  int blocks;        // logical blocks
  int mtiles;        // 16-row pieces per block
  int slot_base;     // byte offset of the product slots in LDS (after the lanes' buffers)
  // multiply-high division magics (fast_div_magic) of 8 * 4 * mtiles, 4 * mtiles, gx and gy:
  // the decode of the flat id is on the path to the first load
  uint32_t m_group, m_pieces, m_gx, m_gy;
};

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void lane_dma16(_Float16 const *gbase, uint32_t lane_byte_offset,
                                           uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_wave_base)), "v"(lane_byte_offset),
                 "s"(gbase)
               : "m0", "memory");
}
#pragma clang diagnostic pop
__device__ __forceinline__ uint32_t lane_lds_address(void const *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void const *)p;
}
// within 16 lanes, lane 4a + b names four halfs T[row0 + a][col0 + 4b ..]; lane i receives
// T[row0 + 0..3][col0 + i]
__device__ __forceinline__ half4 lane_tr16(_Float16 const *p) {
  typedef short short4v __attribute__((ext_vector_type(4)));
  short4v const v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (short4v __attribute__((address_space(3))) *)(__attribute__((address_space(3))) void *)(p));
  return __builtin_bit_cast(half4, v);
}

// Column-major weights (WCM): column n of a weight tile is KT contiguous halfs, so a lane's
// operand -- eight consecutive k of one column -- is 16 contiguous bytes of global memory, like
// its activation rows: every operand goes straight into registers, the strips and the
// transposing reads disappear, LDS holds the product slots only, and a piece's sixteen columns
// are sixteen streams of whole cache lines that no other workgroup touches.
template <int KT, int NB, int PRO, bool LORA, bool WCM>
__global__ __launch_bounds__(1024) void gemm_lanes_kernel(LaneParams const L) {
  fetch_kernel_arguments<sizeof(LaneParams), 4>();  // every line of the block, one trip (blockDim.x is read)
  GemmParams const &P = L.g;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  constexpr int KS = KT / 32;                                // MFMA steps (and 1 KB loads) per strip
  constexpr int STRIPS = NB + (LORA ? 1 : 0);
  // (row-major weights: the strips, + the [16][16] piece of lora B)
  constexpr int WAVE_BYTES = WCM ? 0 : STRIPS * KT * 32 + (LORA ? 512 : 0);
  int const tid = threadIdx.x, lane = tid % 64, IP = blockDim.x / 64;
  int const ip = __builtin_amdgcn_readfirstlane(tid / 64);  // (wave-uniform: addresses stay scalar)
  int const g = lane / 16, c = lane % 16;
  int const F = P.forloop_range, M = P.M;

  // flat id -> (logical block, row piece, column piece): ids that differ by 8 x piece index
  // share a block
  auto div = [](unsigned v, uint32_t magic) { return magic == 0 ? v : __umulhi(v, magic); };
  unsigned const S = 4 * L.mtiles;
  unsigned const id = blockIdx.x;
  unsigned const eighth = id >> 3;
  int const blk = (int)(div(id, L.m_group) * 8 + (id & 7));
  int const sub = (int)(eighth - div(eighth, L.m_pieces) * S);
  if (blk >= L.blocks) {
    return;
  }
  int const piece = sub % 4, mt = sub / 4;
  unsigned const q1 = div((unsigned)blk, L.m_gx);  // blk / gx
  unsigned const q2 = div(q1, L.m_gy);             // blk / (gx * gy)
  int const bx = (int)((unsigned)blk - q1 * (unsigned)L.gx), by = (int)(q1 - q2 * (unsigned)L.gy), bz = (int)q2;
  int const n0 = 16 * piece;

  unsigned char *mine = lds + ip * WAVE_BYTES;
  _Float16 const *strip[STRIPS];
#pragma unroll
  for (int b = 0; b < STRIPS; b++) {
    strip[b] = reinterpret_cast<_Float16 const *>(mine + b * KT * 32);
  }
  _Float16 const *lb_piece = reinterpret_cast<_Float16 const *>(mine + STRIPS * KT * 32);
  _Float16 *slots = reinterpret_cast<_Float16 *>(lds + L.slot_base);  // [F][NB][16][16]

  // this lane's place in a strip load (64 lanes x 16 bytes = 32 rows of 32 bytes) and in the
  // transposing reads
  int const ld_row = lane / 2, ld_half = lane % 2;
  int const tr_off = (c / 4) * 16 + 4 * (c % 4);
  int const row = 16 * mt + c;                 // activation row of this lane's fragments
  bool const row_ok = row < M;
  int const row_ld = row_ok ? row : M - 1;

  half4 lb_frag = {(_Float16)0.0f, (_Float16)0.0f, (_Float16)0.0f, (_Float16)0.0f};
  if (LORA) {
    _Float16 const *src = static_cast<_Float16 const *>(P.lb.ptr) + gtile_offset(P.lb, bx, by, bz, 0);
    if (WCM) {
      // lora B^T[n0 + c][k = 4g .. + 3]: 8 bytes, loop invariant
      lb_frag = *reinterpret_cast<half4 const *>(src + (long long)(n0 + c) * P.lb.d_cols + 4 * g);
    } else if (lane < 32) {
      // lora B [16][64], loop invariant: this piece's 16 columns, rows of 32 bytes
      lane_dma16(src + n0, (uint32_t)((ld_row * P.lb.d_cols + 8 * ld_half) * 2), lane_lds_address(lb_piece));
    }
  }

  for (int it = ip; it < F; it += IP) {
    // (the previous iteration's operand reads must be out of LDS before the transfers that
    // overwrite the strips are issued; the compiler would otherwise move them up among that
    // iteration's last matrix instructions, past the waits for those reads)
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // ---- issue everything this iteration needs -------------------------------------------
    uint4v wr[WCM ? STRIPS : 1][KS];  // column-major weights: the operands themselves
#pragma unroll
    for (int b = 0; b < STRIPS; b++) {
      GTile const &bt = b == NB ? P.la : (b == 0 ? P.b0 : P.b1);
      int const col0 = b == NB ? 0 : n0;  // the lora A tile is [KT][16]: whole
      if (WCM) {
        // W^T[col0 + c][32j + 8g + 0..7]
        _Float16 const *src = static_cast<_Float16 const *>(bt.ptr) + gtile_offset(bt, bx, by, bz, it) +
                              (long long)(col0 + c) * bt.d_cols + 8 * g;
#pragma unroll
        for (int j = 0; j < KS; j++) {
          wr[b][j] = *reinterpret_cast<uint4v const *>(src + 32 * j);
        }
      } else {
        _Float16 const *src = static_cast<_Float16 const *>(bt.ptr) + gtile_offset(bt, bx, by, bz, it) + col0;
        uint32_t const off = (uint32_t)((ld_row * bt.d_cols + 8 * ld_half) * 2);
#pragma unroll
        for (int j = 0; j < KS; j++) {
          lane_dma16(src + (long long)(32 * j) * bt.d_cols, off, lane_lds_address(strip[b]) + j * 1024);
        }
      }
    }
    _Float16 const *a0 = static_cast<_Float16 const *>(P.a0.ptr) + gtile_offset(P.a0, bx, by, bz, it) +
                         (long long)row_ld * P.a0.d_cols + 8 * g;
    uint4v xr[KS], ur[PRO == PRO_SILU_MUL ? KS : 1];
#pragma unroll
    for (int j = 0; j < KS; j++) {
      xr[j] = *reinterpret_cast<uint4v const *>(a0 + 32 * j);
    }
    if (PRO == PRO_SILU_MUL) {
      _Float16 const *a1 = static_cast<_Float16 const *>(P.a1.ptr) + gtile_offset(P.a1, bx, by, bz, it) +
                           (long long)row_ld * P.a1.d_cols + 8 * g;
#pragma unroll
      for (int j = 0; j < KS; j++) {
        ur[j] = *reinterpret_cast<uint4v const *>(a1 + 32 * j);
      }
    }
    // ---- one wait for all of it (direct-to-LDS loads and register loads do not complete in
    // one order, so nothing short of "all" says that a particular one has landed) ------------
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
#pragma unroll
    for (int j = 0; j < KS; j++) {
      asm volatile("" : "+v"(xr[j]));  // (no use of a fragment moves above the wait)
      if (PRO == PRO_SILU_MUL) {
        asm volatile("" : "+v"(ur[j]));
      }
      if (WCM) {
#pragma unroll
        for (int b = 0; b < STRIPS; b++) {
          asm volatile("" : "+v"(wr[b][j]));
        }
      }
    }
#pragma clang diagnostic pop
    // ---- activation fragments: rows past M are zero, prologue in registers -----------------
    half8 x[KS];
#pragma unroll
    for (int j = 0; j < KS; j++) {
      half8 v = __builtin_bit_cast(half8, xr[j]);
      if (PRO == PRO_EXP || PRO == PRO_SILU) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
          v[e] = static_cast<_Float16>(prologue(PRO, static_cast<float>(v[e])));
        }
      } else if (PRO == PRO_SILU_MUL) {
        half8 const u = __builtin_bit_cast(half8, ur[j]);
#pragma unroll
        for (int e = 0; e < 8; e++) {
          _Float16 const sg = static_cast<_Float16>(prologue(PRO_SILU, static_cast<float>(v[e])));
          v[e] = static_cast<_Float16>(static_cast<float>(sg) * static_cast<float>(u[e]));
        }
      }
      if (!row_ok) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
          v[e] = (_Float16)0.0f;
        }
      }
      x[j] = v;
    }
    // ---- lora inner product, transposed: d[r] = (X.A)[m = c][n = 4g + r] -------------------
    half4 dfrag = {(_Float16)0.0f, (_Float16)0.0f, (_Float16)0.0f, (_Float16)0.0f};
    if (LORA) {
      float4v d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < KS; j++) {
        half8 a;
        if (WCM) {
          a = __builtin_bit_cast(half8, wr[WCM ? NB : 0][j]);
        } else {
          _Float16 const *ap = strip[NB] + (32 * j + 8 * g) * 16 + tr_off;
          half4 const lo = lane_tr16(ap), hi = lane_tr16(ap + 64);
          a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
        d = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, x[j], d, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        dfrag[r] = static_cast<_Float16>(d[r]);
      }
    }
    // ---- products: o[r] = O[m = c][n = n0 + 4g + r] ----------------------------------------
#pragma unroll
    for (int b = 0; b < NB; b++) {
      float4v o = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < KS; j++) {
        half8 w;
        if (WCM) {
          w = __builtin_bit_cast(half8, wr[WCM ? b : 0][j]);
        } else {
          _Float16 const *wp = strip[b] + (32 * j + 8 * g) * 16 + tr_off;
          half4 const lo = lane_tr16(wp), hi = lane_tr16(wp + 64);
          w = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
        o = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, x[j], o, 0, 0, 0);
      }
      if (LORA) {
        half4 const w = WCM ? lb_frag : lane_tr16(lb_piece + (4 * g) * 16 + tr_off);  // B[k = 4g ..][n = c]
        o = __builtin_amdgcn_mfma_f32_16x16x16f16(w, dfrag, o, 0, 0, 0);
      }
      half4 p16;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        p16[r] = static_cast<_Float16>(o[r]);
      }
      *reinterpret_cast<half4 *>(slots + ((it * NB + b) * 16 + c) * 16 + 4 * g) = p16;
    }
  }
  __syncthreads();
  // ---- the saver: pieces added in iteration order, two neighbouring columns per thread ----
  typedef _Float16 half2v __attribute__((ext_vector_type(2)));
  for (int e = tid; e < NB * 128; e += blockDim.x) {
    int const b = e / 128, r = (e % 128) / 8, col = (e % 8) * 2;
    _Float16 const *sp = slots + (b * 16 + r) * 16 + col;
    float a0 = 0.0f, a1 = 0.0f;  // hold fp16 values between the adds
    int q = 0;
    for (; q + 8 <= F; q += 8) {
      half2v v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        v[u] = *reinterpret_cast<half2v const *>(sp + (q + u) * NB * 256);
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        a0 = static_cast<float>(static_cast<_Float16>(a0 + static_cast<float>(v[u][0])));
        a1 = static_cast<float>(static_cast<_Float16>(a1 + static_cast<float>(v[u][1])));
      }
    }
    for (; q < F; q++) {
      half2v const v = *reinterpret_cast<half2v const *>(sp + q * NB * 256);
      a0 = static_cast<float>(static_cast<_Float16>(a0 + static_cast<float>(v[0])));
      a1 = static_cast<float>(static_cast<_Float16>(a1 + static_cast<float>(v[1])));
    }
    if (16 * mt + r < M) {
      GTile const &ot = b == 0 ? P.o0 : P.o1;
      _Float16 *og = static_cast<_Float16 *>(const_cast<void *>(ot.ptr)) + gtile_offset(ot, bx, by, bz, 0);
      half2v out;
      out[0] = static_cast<_Float16>(a0);
      out[1] = static_cast<_Float16>(a1);
      *reinterpret_cast<half2v *>(og + (long long)(16 * mt + r) * ot.d_cols + n0 + col) = out;
    }
  }
}

}  // namespace mi355
