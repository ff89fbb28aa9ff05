// Kernel-level fp16 operators (the un-fused ops a kernel graph runs outside its
// customized ops).  Arithmetic is fp32 with one fp16 rounding per stored element, the rule
// the reference's generated programs follow (src/kernel/triton_code_gen.cc:246-268).
// Results are row-major; the matmul reads either storage order of its operands (as the
// reference's GEMM call does, src/kernel/cuda/matmul_kernel.cu:61-76), the element-wise
// operators and reductions index their inputs flat, so their callers hand them row-major
// buffers (mi355_f16_transpose makes one from a column-major tensor).
#include "common.h"

#include <algorithm>
#include <atomic>

namespace mi355 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;

__device__ __forceinline__ uint64_t mix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

// reference src/kernel/cuda/input_kernel.cu:29-38
__global__ void f16_fill_iota_kernel(_Float16 *x, size_t n, int last_dim) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    x[i] = static_cast<_Float16>(static_cast<float>(i % last_dim));
  }
}

__global__ void f16_fill_normal_kernel(_Float16 *x, size_t n, float std, uint64_t seed) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    uint64_t r = mix64(seed + i);
    float u1 = (static_cast<float>((r >> 40) & 0xffffff) + 1.0f) * (1.0f / 16777216.0f);
    float u2 = static_cast<float>((r >> 16) & 0xffffff) * (1.0f / 16777216.0f);
    float z = sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
    x[i] = static_cast<_Float16>(z * std);
  }
}

// The general-purpose GEMM: any shape, either storage order of the operands (element (r, c) of
// A at r * a_rs + c * a_cs, likewise B), unaligned bases.  64x64 output tile per workgroup,
// four wavefronts each owning a 32x32 quadrant, k advanced 32 at a time through LDS, both
// tiles staged k-contiguous with rows padded by 8 halfs.  What the streaming kernel below does
// not take (k not a multiple of 32, operands not reachable with 16-byte accesses) runs here.
__global__ __launch_bounds__(kThreads) void f16_matmul_kernel(_Float16 const *__restrict__ A,
                                                             _Float16 const *__restrict__ B,
                                                             _Float16 *__restrict__ C, int m,
                                                             int n, int k, int a_rs, int a_cs,
                                                             int b_rs, int b_cs) {
  constexpr int T = 64, TK = 32, LD = TK + 8;
  __shared__ __attribute__((aligned(16))) _Float16 As[T][LD];
  __shared__ __attribute__((aligned(16))) _Float16 Bs[T][LD];
  int const tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  int const row0 = blockIdx.y * T, col0 = blockIdx.x * T;
  size_t const b = blockIdx.z;
  A += b * (size_t)m * k;
  B += b * (size_t)k * n;
  C += b * (size_t)m * n;
  int const wr = (wave / 2) * 32, wc = (wave % 2) * 32;
  float16v acc;
#pragma unroll
  for (int i = 0; i < 16; i++) {
    acc[i] = 0.0f;
  }
  // a thread stages 8 elements of each tile per step, walking the direction that is
  // contiguous in memory: along k (8 consecutive k of one row) or along the rows / columns
  // (one k of 8 consecutive rows / columns)
  bool const a_along_k = a_cs == 1, b_along_k = b_rs == 1;
  for (int k0 = 0; k0 < k; k0 += TK) {
    {
      int const r = a_along_k ? tid / 4 : (tid % 8) * 8, kk = a_along_k ? (tid % 4) * 8 : tid / 8;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        int const rr = a_along_k ? r : r + j, kj = a_along_k ? kk + j : kk;
        int const gr = row0 + rr, gk = k0 + kj;
        As[rr][kj] = (gr < m && gk < k) ? A[(size_t)gr * a_rs + (size_t)gk * a_cs] : (_Float16)0.0f;
      }
    }
    {
      int const c = b_along_k ? tid / 4 : (tid % 8) * 8, kk = b_along_k ? (tid % 4) * 8 : tid / 8;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        int const cc = b_along_k ? c : c + j, kj = b_along_k ? kk + j : kk;
        int const gc = col0 + cc, gk = k0 + kj;
        Bs[cc][kj] = (gk < k && gc < n) ? B[(size_t)gk * b_rs + (size_t)gc * b_cs] : (_Float16)0.0f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < TK; ks += 16) {
      half8 a = *reinterpret_cast<half8 const *>(&As[wr + lane % 32][ks + 8 * (lane / 32)]);
      half8 bb = *reinterpret_cast<half8 const *>(&Bs[wc + lane % 32][ks + 8 * (lane / 32)]);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bb, acc, 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < 16; r++) {
    int row = row0 + wr + (r / 4) * 8 + (lane / 32) * 4 + (r % 4);
    int col = col0 + wc + lane % 32;
    if (row < m && col < n) {
      C[(size_t)row * n + col] = static_cast<_Float16>(acc[r]);
    }
  }
}

// ---------------------------------------------------------------------------------------
// Streaming GEMM for operands whose reduction index is contiguous: A [m][k] row-major and B
// column-major, i.e. B^T [n][k] -- the form every plan of the reference declares its weights in
// (cpp_examples/lora.cc:36-41).  C = A . B, fp32 accumulation, one fp16 rounding per element.
//
//  * a workgroup owns a BM x BN tile of C, its wavefronts WM x WN sub-tiles (256 x 256 with
//    eight wavefronts of 128 x 64, or 128 x 128 with four of 64 x 64 for smaller grids);
//  * k advances 32 at a time through a ring of four LDS stages.  A stage is BM + BN rows of 64
//    bytes, filled by direct-to-LDS loads (global_load_lds_dwordx4: no registers, no LDS store
//    instructions) issued three stages ahead; a wavefront waits for its own loads
//    (s_waitcnt vmcnt), one barrier per stage publishes everybody's;
//  * rows are 4 chunks of 16 bytes; chunk q of row r sits at position q ^ ((r >> 2) & 3), so the
//    sixteen rows a 16-lane read phase touches fall on sixteen different bank groups (the lane
//    -> global chunk map of the loads applies the swizzle, since a direct load writes its 64
//    chunks in lane order);
//  * v_mfma_f32_32x32x16_f16, operands one plain 16-byte LDS read per lane, all twelve operand
//    reads of a stage issued before its sixteen matrix instructions;
//  * the tile leaves through LDS as 16-byte row segments; rows and columns past the matrix are
//    clamped on load and masked on store (m and n are arbitrary, k a multiple of 32);
//  * workgroup ids are renumbered so that an XCD (whose 32 compute units share one L2) works on
//    a compact block of tiles: 4 tile rows deep, walked column by column.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ uint32_t gemm_lds_address(void const *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void const *)p;
}
__device__ __forceinline__ void gemm_dma16(_Float16 const *gbase, uint32_t lane_byte_offset, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_wave_base)), "v"(lane_byte_offset), "s"(gbase)
               : "m0", "memory");
}
template <int N>
__device__ __forceinline__ void gemm_wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
#pragma clang diagnostic pop

struct GemmArgs {
  _Float16 const *A, *Bt;  // [batch][m][k], [batch][n][k]
  _Float16 *C;             // [batch][m][n]
  int m, n, k;
  int tiles_m, tiles_n, tiles_per_batch;
  unsigned total;          // workgroups
  // k cut into `ksplit` ranges of `steps_per_split` steps of 32, one workgroup each (products
  // with few output tiles and a long k: skinny activations against a weight matrix): a range's
  // fp32 sums go to partial[split][batch][m][n] and f16_gemm_fold_kernel adds the ranges in
  // fp32 and rounds once
  int ksplit, steps_per_split;
  float *partial;
};

constexpr int kGemmStages = 4, kGemmBK = 32;

template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(64 * (BM / WM) * (BN / WN)) void f16_gemm_nt_kernel(GemmArgs const G) {
  constexpr int NW = (BM / WM) * (BN / WN), NT = 64 * NW;
  constexpr int STAGE_HALFS = (BM + BN) * kGemmBK;
  constexpr int AI = BM * 4 / NT, BI = BN * 4 / NT;  // direct loads per thread and stage
  constexpr int TM = WM / 32, TN = WN / 32;
  static_assert(BM * 4 % NT == 0 && BN * 4 % NT == 0, "a stage must split evenly over the threads");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  _Float16 *const ring = reinterpret_cast<_Float16 *>(lds);
  int const tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);

  // ---- which tile: XCD-aware renumbering, then groups of four tile rows -----------------
  unsigned id = blockIdx.x;
  if (G.total % 8 == 0) {
    id = (id % 8) * (G.total / 8) + id / 8;
  }
  int const split = (int)(id % (unsigned)G.ksplit);  // (the ranges of a tile sit next to each other)
  id /= (unsigned)G.ksplit;
  int const batch = (int)(id / (unsigned)G.tiles_per_batch);
  int const t = (int)(id % (unsigned)G.tiles_per_batch);
  int const per_group = 4 * G.tiles_n, group = t / per_group, first_m = 4 * group;
  int const gsz = (G.tiles_m - first_m) < 4 ? (G.tiles_m - first_m) : 4;
  int const tile_m = first_m + (t % per_group) % gsz, tile_n = (t % per_group) / gsz;
  int const row0 = tile_m * BM, col0 = tile_n * BN;
  _Float16 const *const Ab = G.A + (size_t)batch * G.m * G.k + (size_t)row0 * G.k;
  _Float16 const *const Bb = G.Bt + (size_t)batch * G.n * G.k + (size_t)col0 * G.k;

  // ---- this lane's share of a stage's loads (byte offsets from the tile's first element) --
  uint32_t a_off[AI], b_off[BI];
#pragma unroll
  for (int i = 0; i < AI; i++) {
    int const p = i * NT + tid, r = p / 4, pos = p % 4;
    int const rr = row0 + r < G.m ? r : G.m - 1 - row0;  // rows past the matrix re-read the last one
    a_off[i] = 2u * (uint32_t)(rr * G.k + 8 * (pos ^ ((r >> 2) & 3)));
  }
#pragma unroll
  for (int i = 0; i < BI; i++) {
    int const p = i * NT + tid, r = p / 4, pos = p % 4;
    int const rr = col0 + r < G.n ? r : G.n - 1 - col0;
    b_off[i] = 2u * (uint32_t)(rr * G.k + 8 * (pos ^ ((r >> 2) & 3)));
  }
  uint32_t const ring_addr = gemm_lds_address(ring);
  int const kt_first = split * G.steps_per_split;  // this workgroup's first step of 32 k
  auto issue = [&](int kt) {
    uint32_t const stage = ring_addr + 2u * (uint32_t)((kt % kGemmStages) * STAGE_HALFS);
    _Float16 const *ag = Ab + (size_t)(kt_first + kt) * kGemmBK, *bg = Bb + (size_t)(kt_first + kt) * kGemmBK;
#pragma unroll
    for (int i = 0; i < AI; i++) {
      gemm_dma16(ag, a_off[i], stage + 16u * (uint32_t)(i * NT + wave * 64));
    }
#pragma unroll
    for (int i = 0; i < BI; i++) {
      gemm_dma16(bg, b_off[i], stage + 2u * (uint32_t)(BM * kGemmBK) + 16u * (uint32_t)(i * NT + wave * 64));
    }
  };

  // ---- operand reads: row (lane % 32) of a 32-row block, chunk 2 s + lane / 32 of its row -----
  int const wm0 = (wave / (BN / WN)) * WM, wn0 = (wave % (BN / WN)) * WN;
  int const l32 = lane & 31, hi = lane >> 5, swz = (l32 >> 2) & 3;
  int const x0 = ((0 + hi) ^ swz) << 3, x1 = ((2 + hi) ^ swz) << 3;  // halfs, k steps 0 and 1
  int const a_lane = (wm0 + l32) * kGemmBK, b_lane = BM * kGemmBK + (wn0 + l32) * kGemmBK;

  float16v acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++) {
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
      for (int e = 0; e < 16; e++) {
        acc[i][j][e] = 0.0f;
      }
    }
  }

  int const k_steps = G.k / kGemmBK;
  int const KT = (k_steps - kt_first) < G.steps_per_split ? (k_steps - kt_first) : G.steps_per_split;
  constexpr int LPS = AI + BI;  // loads per thread and stage
#pragma unroll
  for (int st = 0; st < kGemmStages - 1; st++) {
    if (st < KT) {
      issue(st);
    }
  }
  // operand reads of k step `s` (16 k) of the stage in ring slot `slot`
  auto read_step = [&](int slot, int s, half8 (&af)[TM], half8 (&bf)[TN]) {
    _Float16 const *stage = ring + slot * STAGE_HALFS;
#pragma unroll
    for (int i = 0; i < TM; i++) {
      af[i] = *reinterpret_cast<half8 const *>(stage + a_lane + 32 * i * kGemmBK + (s ? x1 : x0));
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
      bf[j] = *reinterpret_cast<half8 const *>(stage + b_lane + 32 * j * kGemmBK + (s ? x1 : x0));
    }
  };
  auto multiply = [&](half8 const (&af)[TM], half8 const (&bf)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int j = 0; j < TN; j++) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
      }
    }
  };
  // stage `kt` has landed (this wavefront's share) when at most the stages issued after it --
  // up to stage kt + 2 by then -- are outstanding
  auto landed = [&](int kt) {
    int const later = (KT - 1 - kt) < 2 ? (KT - 1 - kt) : 2;
    if (later == 2) {
      gemm_wait_vm<2 * LPS>();
    } else if (later == 1) {
      gemm_wait_vm<LPS>();
    } else {
      gemm_wait_vm<0>();
    }
  };
  // The loop is skewed by half a stage so that every batch of operand reads is followed by
  // eight matrix instructions on operands that are already in registers: the second k step of
  // stage kt is read before the first one is multiplied, and the first k step of stage kt + 1
  // -- published by the barrier in the middle -- before the second one is.
  half8 a0[TM], b0[TN], a1[TM], b1[TN];
  landed(0);
  __syncthreads();
  if (kGemmStages - 1 < KT) {
    issue(kGemmStages - 1);
  }
  read_step(0, 0, a0, b0);
  for (int kt = 0; kt < KT; kt++) {
    int const slot = kt % kGemmStages;
    read_step(slot, 1, a1, b1);
    multiply(a0, b0);
    if (kt + 1 < KT) {
      landed(kt + 1);
      // (this wavefront's reads of stage kt are in registers before it lets the others go on)
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __syncthreads();  // stage kt + 1 is there for everybody; stage kt is in everybody's registers
      if (kt + kGemmStages < KT) {
        issue(kt + kGemmStages);  // into the slot stage kt leaves
      }
      read_step((kt + 1) % kGemmStages, 0, a0, b0);
    }
    multiply(a1, b1);
  }

  if (G.ksplit > 1) {
    // a k range's fp32 sums, straight from the accumulators (32 consecutive columns per row)
    int const batches = (int)(G.total / (unsigned)(G.ksplit * G.tiles_per_batch));
    float *const Pb = G.partial + ((size_t)split * batches + batch) * (size_t)G.m * G.n;
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int e = 0; e < 16; e++) {
          int const row = row0 + wm0 + 32 * i + 8 * (e / 4) + 4 * hi + (e % 4), col = col0 + wn0 + 32 * j + l32;
          if (row < G.m && col < G.n) {
            Pb[(size_t)row * G.n + col] = acc[i][j][e];
          }
        }
      }
    }
    return;
  }
  // ---- the tile leaves through LDS: each wavefront its own WM x WN piece -------------------
  __syncthreads();  // the last stage's operand reads are done everywhere
  constexpr int LDW = WN;
  _Float16 *const piece = ring + wave * WM * LDW;
  static_assert(NW * WM * LDW * 2 <= kGemmStages * STAGE_HALFS * 2, "pieces must fit the ring");
#pragma unroll
  for (int i = 0; i < TM; i++) {
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
      for (int e = 0; e < 16; e++) {
        // acc[e] = C[32 i + 8 (e / 4) + 4 (lane / 32) + e % 4][32 j + lane % 32]
        piece[(32 * i + 8 * (e / 4) + 4 * hi + (e % 4)) * LDW + 32 * j + l32] = static_cast<_Float16>(acc[i][j][e]);
      }
    }
  }
  // (a wavefront reads back only what it wrote: its own LDS operations complete in order)
  __builtin_amdgcn_wave_barrier();
  _Float16 *const Cb = G.C + (size_t)batch * G.m * G.n;
  constexpr int CPR = WN / 8;  // 16-byte chunks per row of the piece
  bool const vec = G.n % 8 == 0;
  for (int e = lane; e < WM * CPR; e += 64) {
    int const r = e / CPR, c8 = (e % CPR) * 8;
    int const row = row0 + wm0 + r, col = col0 + wn0 + c8;
    if (row < G.m && col < G.n) {
      half8 const v = *reinterpret_cast<half8 const *>(piece + r * LDW + c8);
      if (vec && col + 8 <= G.n) {
        *reinterpret_cast<half8 *>(Cb + (size_t)row * G.n + col) = v;
      } else {
        for (int x = 0; x < 8 && col + x < G.n; x++) {
          Cb[(size_t)row * G.n + col + x] = v[x];
        }
      }
    }
  }
}

// out[b][c][r] = in[b][r][c] through a 64 x 64 LDS tile: the row-major copy of a column-major
// tensor (or the other way round) for the operators that index their inputs flat.
__global__ __launch_bounds__(kThreads) void f16_transpose_kernel(_Float16 const *__restrict__ in,
                                                                _Float16 *__restrict__ out, int rows,
                                                                int cols) {
  __shared__ _Float16 tile[64][66];
  size_t const b = blockIdx.z;
  in += b * (size_t)rows * cols;
  out += b * (size_t)rows * cols;
  int const r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  for (int e = threadIdx.x; e < 64 * 64; e += kThreads) {
    int const r = e / 64, c = e % 64;
    if (r0 + r < rows && c0 + c < cols) {
      tile[r][c] = in[(size_t)(r0 + r) * cols + c0 + c];
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 64 * 64; e += kThreads) {
    int const c = e / 64, r = e % 64;
    if (r0 + r < rows && c0 + c < cols) {
      out[(size_t)(c0 + c) * rows + r0 + r] = tile[r][c];
    }
  }
}

// Element-wise operators move 16 bytes per lane; what is left over (fewer than 8 elements, or
// everything when a base is not 16-byte aligned) goes one element at a time.
__device__ __forceinline__ float f16_unary_value(int op, float x) {
  return (op == KN_EXP_OP) ? __expf(x) : x / (1.0f + __expf(-x));
}
__device__ __forceinline__ float f16_binary_value(int op, float x, float y) {
  return (op == KN_ADD_OP) ? x + y : (op == KN_MUL_OP) ? x * y : x / y;
}

__global__ void f16_unary_kernel(int op, _Float16 const *__restrict__ in,
                                 _Float16 *__restrict__ out, size_t n, int vec) {
  size_t const tid = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  size_t const stride = (size_t)gridDim.x * blockDim.x;
  size_t const n8 = vec ? n / 8 : 0;
  for (size_t i = tid; i < n8; i += stride) {
    half8 v = reinterpret_cast<half8 const *>(in)[i];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      v[j] = static_cast<_Float16>(f16_unary_value(op, static_cast<float>(v[j])));
    }
    reinterpret_cast<half8 *>(out)[i] = v;
  }
  for (size_t i = n8 * 8 + tid; i < n; i += stride) {
    out[i] = static_cast<_Float16>(f16_unary_value(op, static_cast<float>(in[i])));
  }
}

struct Dims4 {
  int nd;
  int d1[4], d2[4], od[4];
};

// The reference's broadcast rule, one element per thread (any shapes).
__global__ void f16_binary_kernel(int op, _Float16 const *__restrict__ in1,
                                  _Float16 const *__restrict__ in2, _Float16 *__restrict__ out,
                                  Dims4 D, size_t n) {
  size_t gid = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; gid < n; gid += stride) {
    size_t i = gid, s1 = 1, i1 = 0, s2 = 1, i2 = 0;
    for (int d = D.nd - 1; d >= 0; d--) {
      i1 += (i % D.d1[d]) * s1;
      i2 += (i % D.d2[d]) * s2;
      s1 *= D.d1[d];
      s2 *= D.d2[d];
      i /= D.od[d];
    }
    float x = static_cast<float>(in1[i1]), y = static_cast<float>(in2[i2]);
    out[gid] = static_cast<_Float16>(f16_binary_value(op, x, y));
  }
}

// The two shapes that carry the bytes: equal shapes (MODE 0), and a second operand with one
// value per row of the first (last dim 1, MODE 1: the division by row sums); rows are multiples
// of 8 elements, so a lane's eight elements share a row.
template <int MODE>
__global__ void f16_binary_vec_kernel(int op, _Float16 const *__restrict__ in1,
                                      _Float16 const *__restrict__ in2, _Float16 *__restrict__ out,
                                      size_t n8, int row8) {
  size_t const stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n8; i += stride) {
    half8 const a = reinterpret_cast<half8 const *>(in1)[i];
    half8 b;
    if (MODE == 0) {
      b = reinterpret_cast<half8 const *>(in2)[i];
    } else {
      _Float16 const y = in2[i / (size_t)row8];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        b[j] = y;
      }
    }
    half8 z;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      z[j] = static_cast<_Float16>(f16_binary_value(op, static_cast<float>(a[j]), static_cast<float>(b[j])));
    }
    reinterpret_cast<half8 *>(out)[i] = z;
  }
}

// Strided sum, the fingerprint kernel's definition (reduction_kernel.cu:86-107): one output per
// thread, `factor` terms `out_stride` apart.  Any shape.
__global__ void f16_reduce_kernel(_Float16 const *__restrict__ in, _Float16 *__restrict__ out,
                                  size_t n_out, int factor, int in_stride, int out_stride) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  if (i >= n_out) {
    return;
  }
  size_t base = (i / out_stride) * (size_t)in_stride + i % out_stride;
  float r = 0.0f;
  for (int k = 0; k < factor; k++) {
    r += static_cast<float>(in[base + (size_t)k * out_stride]);
  }
  out[i] = static_cast<_Float16>(r);
}

// The same with eight neighbouring outputs per thread (out_stride a multiple of 8): every term
// is one 16-byte load and neighbouring threads read neighbouring 16 bytes.
__global__ void f16_reduce_cols_kernel(_Float16 const *__restrict__ in, _Float16 *__restrict__ out,
                                       size_t n_out8, int factor, int in_stride, int out_stride) {
  size_t const i8 = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  if (i8 >= n_out8) {
    return;
  }
  size_t const i = i8 * 8;
  size_t const base = (i / out_stride) * (size_t)in_stride + i % out_stride;
  float r[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
  for (int k = 0; k < factor; k++) {
    half8 const v = *reinterpret_cast<half8 const *>(in + base + (size_t)k * out_stride);
#pragma unroll
    for (int j = 0; j < 8; j++) {
      r[j] += static_cast<float>(v[j]);
    }
  }
  half8 o;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    o[j] = static_cast<_Float16>(r[j]);
  }
  *reinterpret_cast<half8 *>(out + i) = o;
}

// Sums of runs of consecutive elements (out_stride 1): 16 lanes per run, 16 bytes per lane and
// step, the lanes' fp32 parts added across the group at the end; runs that are not a multiple
// of 8 elements (or not 16-byte aligned) finish one element at a time.
__global__ void f16_reduce_rows_kernel(_Float16 const *__restrict__ in,
                                       _Float16 *__restrict__ out, size_t n_out, int factor, int vec) {
  int const sub = threadIdx.x % 16;
  size_t const row = (blockIdx.x * (size_t)blockDim.x + threadIdx.x) / 16;
  float r = 0.0f;
  if (row < n_out) {
    _Float16 const *p = in + row * (size_t)factor;
    int const f8 = vec ? factor / 8 : 0;
    for (int k = sub; k < f8; k += 16) {
      half8 const v = reinterpret_cast<half8 const *>(p)[k];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        r += static_cast<float>(v[j]);
      }
    }
    for (int k = f8 * 8 + sub; k < factor; k += 16) {
      r += static_cast<float>(p[k]);
    }
  }
  for (int off = 8; off > 0; off >>= 1) {
    r += __shfl_xor(r, off, 64);
  }
  if (sub == 0 && row < n_out) {
    out[row] = static_cast<_Float16>(r);
  }
}

static inline int grid_for(size_t n) {
  size_t g = (n + kThreads - 1) / kThreads;
  return static_cast<int>(g < 1 ? 1 : (g > 8192 ? 8192 : g));
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_f16_fill_iota(void *x, size_t n, int last_dim) {
  MI355_REQUIRE_INIT();
  if (last_dim <= 0) {
    return fail(MI355_ERR_INVALID, "last_dim must be positive");
  }
  if (n == 0) {
    return MI355_OK;
  }
  f16_fill_iota_kernel<<<grid_for(n), kThreads, 0, state().stream()>>>(
      static_cast<_Float16 *>(x), n, last_dim);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_f16_fill_normal(void *x, size_t n, float std, uint64_t seed) {
  MI355_REQUIRE_INIT();
  if (n == 0) {
    return MI355_OK;
  }
  f16_fill_normal_kernel<<<grid_for(n), kThreads, 0, state().stream()>>>(
      static_cast<_Float16 *>(x), n, std, seed);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

namespace mi355 {

// C[i] = fp16(sum over the k ranges of partial[s][i]), added in fp32 in range order
__global__ void f16_gemm_fold_kernel(float const *__restrict__ partial, _Float16 *__restrict__ C, size_t n,
                                     int ksplit) {
  size_t const stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += stride) {
    float r = 0.0f;
    for (int s = 0; s < ksplit; s++) {
      r += partial[(size_t)s * n + i];
    }
    C[i] = static_cast<_Float16>(r);
  }
}

static int launch_transpose(_Float16 const *in, _Float16 *out, int batch, int rows, int cols) {
  dim3 grid((cols + 63) / 64, (rows + 63) / 64, batch);
  f16_transpose_kernel<<<grid, kThreads, 0, state().stream()>>>(in, out, rows, cols);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

template <int BM, int BN, int WM, int WN>
static int launch_gemm_nt(GemmArgs &G, int batch) {
  constexpr int threads = 64 * (BM / WM) * (BN / WN);
  constexpr int lds = kGemmStages * (BM + BN) * kGemmBK * 2;
  G.tiles_m = (G.m + BM - 1) / BM;
  G.tiles_n = (G.n + BN - 1) / BN;
  G.tiles_per_batch = G.tiles_m * G.tiles_n;
  long long const tiles = (long long)G.tiles_per_batch * batch;
  // Few tiles and a long k (2048 or more): cut k into ranges of at least 8 steps until there is
  // a workgroup for every compute unit, as far as the fp32 sums of the ranges fit this queue's
  // scratch ([16, 4096] . [4096, 4096]: 36 -> 13 us; 1024^3, 64 tiles, is faster unsplit).
  int const k_steps = G.k / kGemmBK;
  int ksplit = 1;
  if (tiles < 128 && k_steps >= 64 && state().scratch() != nullptr) {
    ksplit = (int)std::min<long long>((256 + tiles - 1) / tiles, k_steps / 8);
    size_t const per_range = (size_t)batch * G.m * G.n * sizeof(float);
    ksplit = (int)std::min<size_t>((size_t)ksplit, state().scratch_bytes / per_range);
    ksplit = std::max(ksplit, 1);
  }
  G.steps_per_split = (k_steps + ksplit - 1) / ksplit;
  G.ksplit = (k_steps + G.steps_per_split - 1) / G.steps_per_split;  // no empty range
  G.partial = static_cast<float *>(state().scratch());
  long long const total = tiles * G.ksplit;
  if (total > 2147483647LL) {
    return fail(MI355_ERR_UNSUPPORTED, "matmul has too many output tiles");
  }
  G.total = (unsigned)total;
  auto *fn = f16_gemm_nt_kernel<BM, BN, WM, WN>;
  static std::atomic<int> granted{0};  // per instantiation
  if (lds > 65536 && granted.load(std::memory_order_acquire) < lds) {
    MI355_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    granted.store(lds, std::memory_order_release);
  }
  fn<<<G.total, threads, lds, state().stream()>>>(G);
  MI355_HIP(hipGetLastError());
  if (G.ksplit > 1) {
    size_t const n = (size_t)batch * G.m * G.n;
    f16_gemm_fold_kernel<<<grid_for(n), kThreads, 0, state().stream()>>>(G.partial, G.C, n, G.ksplit);
    MI355_HIP(hipGetLastError());
  }
  return MI355_OK;
}

}  // namespace mi355

extern "C" int mi355_f16_matmul_layout(void const *A, void const *B, void *C, int batch, int m,
                                       int n, int k, int a_column_major, int b_column_major) {
  MI355_REQUIRE_INIT();
  if (batch < 0 || m < 0 || n < 0 || k < 0) {
    return fail(MI355_ERR_INVALID, "negative matmul extent");
  }
  if (batch == 0 || m == 0 || n == 0) {
    return MI355_OK;
  }
  if (batch > 65535) {
    return fail(MI355_ERR_UNSUPPORTED, "batch %d exceeds grid.z", batch);
  }
  if (state().f16_matmul_route == 1 && k > 0) {  // an empty sum is zeros from the kernel below
    return vendor_gemm(A, B, C, batch, m, n, k, a_column_major, b_column_major);
  }
  auto const *a = static_cast<_Float16 const *>(A);
  auto const *b = static_cast<_Float16 const *>(B);
  // The streaming kernel wants k contiguous in both operands (A row-major, B column-major) and
  // k in whole steps of 32.  An operand stored the other way round is first copied transposed
  // into this queue's plane memory (the fingerprint matmuls' workspace: work of one queue is
  // ordered, so the two never overlap); what does not fit there, or is not reachable with
  // 16-byte accesses, takes the general-purpose kernel.
  bool const aligned = ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0;
  size_t const a_bytes = a_column_major ? (size_t)batch * m * k * 2 : 0;
  size_t const b_bytes = b_column_major ? 0 : (size_t)batch * k * n * 2;
  size_t const a_room = (a_bytes + 255) & ~(size_t)255;
  bool const fits = state().planes() != nullptr && a_room + b_bytes <= state().planes_bytes;
  bool const fast = k >= kGemmBK && k % kGemmBK == 0 && aligned && fits &&
                    (size_t)std::max(m, n) * (size_t)k < ((size_t)1 << 30);
  if (fast) {
    if (a_column_major) {  // the buffer is [k][m] per matrix
      auto *at = reinterpret_cast<_Float16 *>(state().planes());
      if (int rc = launch_transpose(a, at, batch, k, m)) {
        return rc;
      }
      a = at;
    }
    if (!b_column_major) {  // the buffer is [k][n] per matrix
      auto *bt = reinterpret_cast<_Float16 *>(state().planes() + a_room);
      if (int rc = launch_transpose(b, bt, batch, k, n)) {
        return rc;
      }
      b = bt;
    }
    GemmArgs G{};
    G.A = a;
    G.Bt = b;
    G.C = static_cast<_Float16 *>(C);
    G.m = m;
    G.n = n;
    G.k = k;
    // 256 x 256 tiles once they alone fill the chip; 128 x 128 below that
    long long const big_tiles = (long long)((m + 255) / 256) * ((n + 255) / 256) * batch;
    return big_tiles >= 192 ? launch_gemm_nt<256, 256, 128, 64>(G, batch) : launch_gemm_nt<128, 128, 64, 64>(G, batch);
  }
  dim3 grid((n + 63) / 64, (m + 63) / 64, batch);
  f16_matmul_kernel<<<grid, kThreads, 0, state().stream()>>>(
      a, b, static_cast<_Float16 *>(C), m, n, k, a_column_major ? 1 : k, a_column_major ? m : 1,
      b_column_major ? 1 : n, b_column_major ? k : 1);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_f16_matmul(void const *A, void const *B, void *C, int batch, int m, int n,
                                int k) {
  return mi355_f16_matmul_layout(A, B, C, batch, m, n, k, 0, 0);
}

extern "C" int mi355_f16_transpose(void const *in, void *out, int batch, int rows, int cols) {
  MI355_REQUIRE_INIT();
  if (batch < 0 || rows < 0 || cols < 0) {
    return fail(MI355_ERR_INVALID, "negative transpose extent");
  }
  if (batch == 0 || rows == 0 || cols == 0) {
    return MI355_OK;
  }
  if (batch > 65535 || (rows + 63) / 64 > 65535) {
    return fail(MI355_ERR_UNSUPPORTED, "transpose grid out of range");
  }
  if (in == out) {
    return fail(MI355_ERR_INVALID, "transpose in place");
  }
  return launch_transpose(static_cast<_Float16 const *>(in), static_cast<_Float16 *>(out), batch, rows, cols);
}

extern "C" int mi355_f16_unary(int op, void const *in, void *out, size_t n) {
  MI355_REQUIRE_INIT();
  if (op != KN_EXP_OP && op != KN_SILU_OP) {
    return fail(MI355_ERR_UNSUPPORTED, "unary op %d", op);
  }
  if (n == 0) {
    return MI355_OK;
  }
  int const vec = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 ? 1 : 0;
  f16_unary_kernel<<<grid_for(vec ? (n + 7) / 8 : n), kThreads, 0, state().stream()>>>(
      op, static_cast<_Float16 const *>(in), static_cast<_Float16 *>(out), n, vec);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_f16_binary(int op, void const *in1, int const *dims1, void const *in2,
                                int const *dims2, void *out, int const *dims_out,
                                int num_dims) {
  MI355_REQUIRE_INIT();
  if (op != KN_ADD_OP && op != KN_MUL_OP && op != KN_DIV_OP) {
    return fail(MI355_ERR_UNSUPPORTED, "binary op %d", op);
  }
  if (num_dims < 1 || num_dims > 4) {
    return fail(MI355_ERR_INVALID, "num_dims %d out of range", num_dims);
  }
  Dims4 D{};
  D.nd = num_dims;
  size_t n = 1;
  for (int d = 0; d < num_dims; d++) {
    D.d1[d] = dims1[d];
    D.d2[d] = dims2[d];
    D.od[d] = dims_out[d];
    if (dims1[d] <= 0 || dims2[d] <= 0 || dims_out[d] <= 0 ||
        (dims1[d] != dims_out[d] && dims1[d] != 1) ||
        (dims2[d] != dims_out[d] && dims2[d] != 1)) {
      return fail(MI355_ERR_INVALID, "dim %d is not broadcastable", d);
    }
    n *= (size_t)dims_out[d];
  }
  // equal shapes, or one value of the second operand per row of the first: 16 bytes per lane
  bool same = true, row_scalar = num_dims >= 2 && dims2[num_dims - 1] == 1 && dims1[num_dims - 1] == dims_out[num_dims - 1];
  for (int d = 0; d < num_dims; d++) {
    same = same && dims1[d] == dims_out[d] && dims2[d] == dims_out[d];
    if (d < num_dims - 1) {
      row_scalar = row_scalar && dims1[d] == dims_out[d] && dims2[d] == dims_out[d];
    }
  }
  bool const aligned = ((reinterpret_cast<uintptr_t>(in1) | reinterpret_cast<uintptr_t>(out) |
                         (same ? reinterpret_cast<uintptr_t>(in2) : 0)) & 15) == 0;
  int const last = dims_out[num_dims - 1];
  auto const *x1 = static_cast<_Float16 const *>(in1);
  auto const *x2 = static_cast<_Float16 const *>(in2);
  auto *y = static_cast<_Float16 *>(out);
  if (aligned && same && n % 8 == 0) {
    f16_binary_vec_kernel<0><<<grid_for(n / 8), kThreads, 0, state().stream()>>>(op, x1, x2, y, n / 8, 1);
  } else if (aligned && row_scalar && last % 8 == 0 && last > 1) {
    f16_binary_vec_kernel<1><<<grid_for(n / 8), kThreads, 0, state().stream()>>>(op, x1, x2, y, n / 8, last / 8);
  } else {
    f16_binary_kernel<<<grid_for(n), kThreads, 0, state().stream()>>>(op, x1, x2, y, D, n);
  }
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_f16_reduce(void const *in, void *out, size_t n_out, int factor,
                                int in_stride, int out_stride) {
  MI355_REQUIRE_INIT();
  if (factor <= 0 || in_stride <= 0 || out_stride <= 0 ||
      (size_t)out_stride * factor != (size_t)in_stride) {
    return fail(MI355_ERR_INVALID, "reduction strides do not match the factor");
  }
  if (n_out == 0) {
    return MI355_OK;
  }
  hipStream_t st = state().stream();
  auto const *x = static_cast<_Float16 const *>(in);
  auto *y = static_cast<_Float16 *>(out);
  bool const aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  if (out_stride == 1 && factor >= 64) {
    int const vec = aligned && factor % 8 == 0 ? 1 : 0;
    size_t const blocks = (n_out * 16 + kThreads - 1) / kThreads;
    f16_reduce_rows_kernel<<<(unsigned)blocks, kThreads, 0, st>>>(x, y, n_out, factor, vec);
  } else if (aligned && out_stride % 8 == 0 && n_out % 8 == 0) {
    size_t const blocks = (n_out / 8 + kThreads - 1) / kThreads;
    f16_reduce_cols_kernel<<<(unsigned)blocks, kThreads, 0, st>>>(x, y, n_out / 8, factor, in_stride, out_stride);
  } else {
    size_t const blocks = (n_out + kThreads - 1) / kThreads;
    f16_reduce_kernel<<<(unsigned)blocks, kThreads, 0, st>>>(x, y, n_out, factor, in_stride, out_stride);
  }
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}
