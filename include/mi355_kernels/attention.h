// Device code of the fused, register-resident attention kernels (the attention family of
// thread-block graphs): attn_fused_kernel, attn_stream_kernel, attn_direct_kernel and the
// parameter block they take.  Header-only and free of host state so that two users share it:
// the backend library (attn_fused.hip recognises the family in a lowered program, chooses the
// kernel and its launch shape) and the programs Graph::generate_hip_program writes, which
// instantiate the chosen kernel with its literal template arguments and launch parameters.
//
// The reference emits its fast programs as Triton source (src/kernel/triton_code_gen.cc:
// 84-352); these kernels are what an emitted program of this backend runs instead.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernarg.h"

namespace mi355 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

// Two gfx950 data movers the throughput kernel is built on.
// lds_dma16: every lane fetches 16 bytes from its own global address
// (`gbase`, wave-uniform, plus its own byte offset); the wavefront's 64 chunks land in LDS
// at `lds_wave_base` + 16 * lane (wave-uniform, passed in m0), without passing through
// registers.  Completion is tracked by vmcnt.  Written as
// inline assembly on purpose: for the builtin the compiler makes the first LDS read after
// it wait for vmcnt(0) whenever it cannot prove the two do not alias, which serialises the
// transfer with the compute it is meant to run under.  The caller waits (`s_waitcnt
// vmcnt(0)`) before the barrier that publishes the data.  No other instruction of these
// kernels reads m0.
// lds_read_tr16: within each group of 16 lanes, lane r supplies the address of four
// consecutive halfs X[r][0..3]; lane i receives X[i / 4 + 4 * e][i % 4] for e = 0..3, i.e.
// the transposed operand an MFMA wants when the tile lies in LDS row-major in k.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ uint32_t lds_address(void const *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void const *)p;
}
__device__ __forceinline__ void lds_dma16(_Float16 const *gbase, uint32_t lane_byte_offset,
                                          uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_wave_base)), "v"(lane_byte_offset),
                 "s"(gbase)
               : "m0", "memory");
}
#pragma clang diagnostic pop
__device__ __forceinline__ half4 lds_read_tr16(_Float16 const *p) {
  typedef short short4v __attribute__((ext_vector_type(4)));
  short4v const v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (short4v __attribute__((address_space(3))) *)(__attribute__((address_space(3))) void *)(p));
  return __builtin_bit_cast(half4, v);
}

// Where a tile of a device tensor starts: the element offset is linear in the block
// coordinates and the for-loop iteration, so the host folds the plan's row / column / batch
// strides into one stride per coordinate (a handful of scalar multiplies per tile address
// instead of three sums of products; they sit on the path to the first load).
struct TileAddr {
  void const *ptr;
  int lin[4];  // elements per step of bx, by, bz and of the iteration (the host takes a plan on
               // these kernels only when every tile origin fits 31 bits: a tile address is then
               // four 32-bit multiplies, and the parameter block 240 bytes of scalar registers)
  int d_cols;  // row stride of the tensor
};

struct AttnParams {
  TileAddr q, k, v, o, r;  // r: row-sum output (form B only)
  int forloop_range;
  int split;   // workgroups per logical thread block
  int stages;  // for-loop iterations staged per barrier
  int lds_stage_bytes;
  int perm[3];  // grid dims from fastest to slowest varying in the renumbered workgroup id
  // extents of the launch grid in that order, their multiply-high division magics
  // (fast_div_magic: q = mulhi(id, magic), 0 stands for extent 1) and the magic of `split`
  unsigned perm_ext[3], perm_magic[3], split_magic;
  int rows;     // query rows of the last row group that exist (16, or 8 for an 8-row tile: the
                // missing rows are zeros in the Q fragment and are never stored)
  unsigned long long *trace;  // per-wavefront phase timestamps (attn_direct_kernel<.., TRACE>)
  // attn_direct_kernel: the row sums are stored r_copies times, r_copy_stride elements apart
  // (a plan whose blocks each take a few value columns and all store the same row sums runs
  // as one block with the whole value tile)
  int r_copies, r_copy_stride;
};

__device__ __forceinline__ long long tile_offset(TileAddr const &t, int bx, int by, int bz,
                                                 int it) {
  return (long long)(bx * t.lin[0] + by * t.lin[1] + bz * t.lin[2] + it * t.lin[3]);
}

// x[l] + x[l ^ 16] + x[l ^ 32] + x[l ^ 48] in every lane l: the sum over the four groups of 16
// lanes, in the order ((l, l ^ 16), (l ^ 32, l ^ 48)) that two shuffles would add them in.  The
// two lane-swap instructions of this part exchange rows of 16 lanes and halves of the
// wavefront between two registers in a few cycles; a shuffle is a trip through the LDS
// crossbar, and two of them in a row sit in the middle of the softmax's dependent chain.
// (Inline assembly: the compiler's own builtin for these instructions returns the first result
// twice here.  The wait states cover a vector write to either register just before.)
__device__ __forceinline__ float sum_lane_groups(float x) {
  float a = x, b = x;
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  float const pair = a + b;
  a = pair;
  b = pair;
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return a + b;
}

// Element offset of 16-byte chunk `chunk` of row `row` in a swizzled LDS tile whose
// rows hold LD halfs (LD a multiple of 64).
__device__ __forceinline__ int swz_chunk(int row, int chunk, int LD) {
  return row * LD + ((chunk ^ ((row ^ (row >> 3)) & 7)) << 3);
}

// A 4 x 8 patch of a tile whose columns are contiguous in memory: rows r..r+3,
// columns c..c+7, as four 16-byte words.
struct Patch {
  uint4v x[4];
};

__device__ __forceinline__ Patch load_patch(_Float16 const *__restrict__ src, int ld, int cblocks,
                                            int p) {
  int const cb = p % cblocks, rb = p / cblocks;
  _Float16 const *s = src + (long long)(4 * rb) * ld + 8 * cb;
  Patch q;
  q.x[0] = *reinterpret_cast<uint4v const *>(s);
  q.x[1] = *reinterpret_cast<uint4v const *>(s + ld);
  q.x[2] = *reinterpret_cast<uint4v const *>(s + 2 * (long long)ld);
  q.x[3] = *reinterpret_cast<uint4v const *>(s + 3 * (long long)ld);
  return q;
}

// The same patch addressed as (wavefront-uniform base) + (32-bit lane offset): the rows
// differ by the uniform leading dimension, so one lane offset serves all four loads.
__device__ __forceinline__ Patch load_patch_at(_Float16 const *__restrict__ base, uint32_t lane_off,
                                               int ld) {
  Patch q;
  q.x[0] = *reinterpret_cast<uint4v const *>(base + lane_off);
  q.x[1] = *reinterpret_cast<uint4v const *>(base + ld + lane_off);
  q.x[2] = *reinterpret_cast<uint4v const *>(base + 2 * (long long)ld + lane_off);
  q.x[3] = *reinterpret_cast<uint4v const *>(base + 3 * (long long)ld + lane_off);
  return q;
}

// Writes the patch transposed into a swizzled tile: dst row c + i holds source
// rows r..r+3 as four consecutive halfs, i < 8.  PAIRED reorders the eight 4-half groups
// of every 32-half block so that groups g and g + 4 sit side by side (slot 2g, 2g + 1):
// the sixteen bytes a lane needs as the B operand of P.V (keys 4g..4g+3 and
// 16+4g..16+4g+3, the key order the S^T accumulators leave P in) become one LDS read.
template <bool PAIRED = false>
__device__ __forceinline__ void store_patch_transposed(Patch const &q, _Float16 *__restrict__ dst,
                                                       int LD, int cblocks, int p) {
  int const cb = p % cblocks;
  int rb = p / cblocks;
  if (PAIRED) {
    rb = (rb & ~7) | ((rb & 3) << 1) | ((rb >> 2) & 1);
  }
#pragma unroll
  for (int w = 0; w < 4; w++) {
    uint2v even, odd;  // source columns 2w and 2w+1, rows 0..3
    // byte permute: selector bytes 0-3 pick from the second operand, 4-7 from the first
    even.x = __builtin_amdgcn_perm(q.x[1][w], q.x[0][w], 0x05040100u);
    even.y = __builtin_amdgcn_perm(q.x[3][w], q.x[2][w], 0x05040100u);
    odd.x = __builtin_amdgcn_perm(q.x[1][w], q.x[0][w], 0x07060302u);
    odd.y = __builtin_amdgcn_perm(q.x[3][w], q.x[2][w], 0x07060302u);
    int const row = 8 * cb + 2 * w;
    *reinterpret_cast<uint2v *>(dst + swz_chunk(row, rb >> 1, LD) + (rb & 1) * 4) = even;
    *reinterpret_cast<uint2v *>(dst + swz_chunk(row + 1, rb >> 1, LD) + (rb & 1) * 4) = odd;
  }
}

// Workgroups are dealt to the 8 XCDs round-robin by linear id, and each XCD has its
// own L2.  Renumber so that each XCD gets a contiguous run of ids, and unpack the id
// with the grid dims the K / V tiles do NOT depend on varying fastest (row slices
// first): workgroups that read the same K / V tiles then sit on one XCD and share
// one L2 instead of fetching the tiles once per XCD.
__device__ __forceinline__ void decode_block(AttnParams const &P, int &bx, int &by, int &bz,
                                             int &slice) {
  unsigned const ext[3] = {gridDim.x, gridDim.y, gridDim.z};
  unsigned const total = ext[0] * ext[1] * ext[2];
  unsigned id = blockIdx.x + ext[0] * (blockIdx.y + ext[1] * blockIdx.z);
  if (total % 8 == 0) {
    id = (id % 8) * (total / 8) + id / 8;
  }
  // divisions by the extents are multiply-highs with magics the host computed (exact while
  // id * extent < 2^32, which the host checks): this runs before the first load can go out
  unsigned digit[3];  // digit i of the id belongs to grid dim perm[i]
#pragma unroll
  for (int i = 0; i < 3; i++) {
    unsigned const e = P.perm_ext[i], m = P.perm_magic[i];
    unsigned const q = m == 0 ? id : __umulhi(id, m);
    digit[i] = id - q * e;
    id = q;
  }
  unsigned coord[3];  // (selects, no branches: this is on the path to the first load)
#pragma unroll
  for (int k = 0; k < 3; k++) {
    coord[k] = P.perm[0] == k ? digit[0] : (P.perm[1] == k ? digit[1] : digit[2]);
  }
  unsigned const b = P.split_magic == 0 ? coord[0] : __umulhi(coord[0], P.split_magic);
  bx = (int)b;
  slice = (int)(coord[0] - b * (unsigned)P.split);
  by = coord[1];
  bz = coord[2];
}

// Column-major K and V (template parameter CM of the kernels below): the K tile lies in memory and in LDS as K^T [NK keys][D], the V
// tile as V^T [DV][NK keys]: the reduction index of both matrix products is contiguous, and every
// operand is ONE plain 16-byte LDS read.  Key block j of S^T takes the keys
// 32 (j / 2) + 8 (c / 4) + 4 (j % 2) + c % 4 for c = 0 .. 15 (any 16 keys may form a block), so
// that the eight values of P a lane holds after blocks 2jj and 2jj + 1 are the eight CONSECUTIVE
// keys 32jj + 8g .. + 7: the keys its V^T operand read delivers.  16-byte chunks are swizzled so
// that the sixteen rows one read phase touches fall on sixteen different bank groups: chunk q of
// row r sits at position q ^ cm_key<row bytes>(r).
//   rows of 256 bytes (one row = all 64 banks): K^T rows with D = 128 read at the sixteen keys
//     above, key(r) = (r & 3) | ((r >> 3) & 3) << 2 (= c); V^T rows with NK = 128 read at sixteen
//     consecutive rows, key(r) = r & 15 (also for longer rows);
//   rows of 128 bytes (two rows per bank line, the row's parity picks the half): the key
//     permutes the eight chunks of the half: K^T with D = 64, key(r) = ((r >> 1) & 1) |
//     ((r >> 3) & 3) << 1 (= c >> 1); V^T with NK = 64, key(r) = (r >> 1) & 7.
template <int RowHalfs, bool IsK>
__device__ __forceinline__ constexpr int cm_swizzle_key(int r) {
  return IsK ? (RowHalfs == 128 ? ((r & 3) | (((r >> 3) & 3) << 2)) : (((r >> 1) & 1) | (((r >> 3) & 3) << 1)))
             : (RowHalfs >= 128 ? (r & 15) : ((r >> 1) & 7));
}

// RG row groups of 16 query rows, IP wavefronts per row group working on IP
// consecutive for-loop iterations.
template <int D, int NK, int DV, bool HAS_DIV, int RG, int IP, bool CM = false>
__global__ __launch_bounds__(64 * RG * IP) void attn_fused_kernel(AttnParams const P) {
  fetch_kernel_arguments<sizeof(AttnParams), 3>();  // every line of the block, one trip (decode_block reads gridDim.z)
  constexpr int LDO = DV + 8;
  constexpr int KB = NK / 16, DB = DV / 16, DK = D / 32;
  constexpr int NW = RG * IP, NT = 64 * NW;
  // staging work per for-loop iteration, in 4x8 patches: K patches then V patches.  The
  // patches of up to SG iterations form one list that ALL threads share out (a K or V
  // tile alone may have fewer patches than the workgroup has threads)
  constexpr int KP = (D / 4) * (NK / 8), VP = (NK / 4) * (DV / 8), PER_IT = KP + VP;
  // iterations whose loads are issued together: at most 8 patches = 32 x 16 B per thread
  constexpr int SG_RAW = 8 * NT / PER_IT;
  constexpr int SG = SG_RAW < 1 ? 1 : (SG_RAW > 4 ? 4 : SG_RAW);
  constexpr int IPT = (SG * PER_IT + NT - 1) / NT;  // patches per thread and load phase
  constexpr int SLOT_DW = DB * 2 + 1;  // one wavefront's iteration result, dwords per lane
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

  int const tid = threadIdx.x;
  int const lane = tid % 64, wave = tid / 64;
  int const rg = wave / IP, ip = wave % IP;
  int const g = lane / 16, c = lane % 16;
  int bx, by, bz, slice;
  decode_block(P, bx, by, bz, slice);
  int const row_base = (slice * RG + rg) * 16;  // first query row of this row group
  int const F = P.forloop_range;

  // Q fragments (B operand of S^T): Q[row c][32kk + 8g .. +7], loop invariant
  half8 qf[DK];
  {
    _Float16 const *q = static_cast<_Float16 const *>(P.q.ptr) + tile_offset(P.q, bx, by, bz, 0) +
                        (long long)(row_base + c) * P.q.d_cols + 8 * g;
#pragma unroll
    for (int kk = 0; kk < DK; kk++) {
      half8 z;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        z[e] = (_Float16)0.0f;
      }
      qf[kk] = c < P.rows ? *reinterpret_cast<half8 const *>(q + 32 * kk) : z;
    }
  }

  // for-loop accumulators of the row group, held by its first wavefront:
  // oacc[t][r] = O[row 4g + r][16t + c], fp16 like the reference's accumulators
  _Float16 oacc[DB][4];
  _Float16 racc = (_Float16)0.0f;
#pragma unroll
  for (int t = 0; t < DB; t++) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      oacc[t][r] = (_Float16)0.0f;
    }
  }

  unsigned char *const tail = lds + P.stages * P.lds_stage_bytes;
  _Float16 *const o_stage = reinterpret_cast<_Float16 *>(tail);
  uint32_t *const slots = reinterpret_cast<uint32_t *>(tail + RG * 16 * LDO * 2);

  for (int it0 = 0; it0 < F; it0 += P.stages) {
    int const n_st = (F - it0) < P.stages ? (F - it0) : P.stages;
    if (it0 > 0) {
      __syncthreads();  // previous chunk fully consumed
    }
    for (int s0 = 0; s0 < n_st; s0 += SG) {
      // phase 1: every load of up to SG iterations goes out before anything waits
      Patch pt[IPT];
#pragma unroll
      for (int i = 0; i < IPT; i++) {
        int const item = tid + i * NT;
        int const u = item / PER_IT, r = item % PER_IT;
        if (u < SG && s0 + u < n_st) {
          bool const is_k = r < KP;  // uniform per wavefront: KP is a multiple of 64
          TileAddr const &ta = is_k ? P.k : P.v;
          _Float16 const *src =
              static_cast<_Float16 const *>(ta.ptr) + tile_offset(ta, bx, by, bz, it0 + s0 + u);
          if (CM) {
            // column-major tiles need no transpose: item r is four consecutive 16-byte chunks
            // of K^T [NK][D] or V^T [DV][NK] (chunks per row are multiples of 4)
            int const cpr = is_k ? D / 8 : NK / 8, q = 4 * (is_k ? r : r - KP);
            _Float16 const *p4 = src + (long long)(q / cpr) * ta.d_cols + 8 * (q % cpr);
#pragma unroll
            for (int e = 0; e < 4; e++) {
              pt[i].x[e] = *reinterpret_cast<uint4v const *>(p4 + 8 * e);
            }
          } else {
            pt[i] = load_patch(src, ta.d_cols, is_k ? NK / 8 : DV / 8, is_k ? r : r - KP);
          }
        }
      }
      // phase 2: transpose in registers, write K^T [NK][D] and V^T [DV][NK]
#pragma unroll
      for (int i = 0; i < IPT; i++) {
        int const item = tid + i * NT;
        int const u = item / PER_IT, r = item % PER_IT;
        if (u < SG && s0 + u < n_st) {
          bool const is_k = r < KP;
          _Float16 *kt = reinterpret_cast<_Float16 *>(lds + (s0 + u) * P.lds_stage_bytes);
          if (CM) {
            int const cpr = is_k ? D / 8 : NK / 8, q = 4 * (is_k ? r : r - KP);
            int const row = q / cpr, pos = q % cpr;
            int const key = is_k ? cm_swizzle_key<D, true>(row) : cm_swizzle_key<NK, false>(row);
            _Float16 *dst = (is_k ? kt : kt + NK * D) + row * (is_k ? D : NK);
#pragma unroll
            for (int e = 0; e < 4; e++) {
              *reinterpret_cast<uint4v *>(dst + (((pos + e) ^ key) << 3)) = pt[i].x[e];
            }
          } else if (is_k) {
            store_patch_transposed(pt[i], kt, D, NK / 8, r);
          } else {
            store_patch_transposed<true>(pt[i], kt + NK * D, NK, DV / 8, r - KP);
          }
        }
      }
    }
    __syncthreads();
    // rounds of IP iterations: wavefront `ip` of each row group takes iteration r0 + ip
    for (int r0 = 0; r0 < n_st; r0 += IP) {
      int const s = r0 + ip;
      bool const active = s < n_st;
      _Float16 o16[DB][4];
      _Float16 r16 = (_Float16)0.0f;
      if (active) {
        _Float16 const *kt = reinterpret_cast<_Float16 const *>(lds + s * P.lds_stage_bytes);
        _Float16 const *vt = kt + NK * D;
        // ---- S^T = K^T . Q^T, exp, row sum ----------------------------------------
        // pk[jj][0..3]: eight keys of this lane's query row, packed fp16 (keys 4g..4g+3 of
        // key blocks 2jj and 2jj+1): the A operand of P.V as the accumulators leave it.
        // Roundings as the sequential program makes them: S to fp16, exp in fp32, the
        // result to fp16; the row sum adds the rounded values in fp32.
        uint32_t pk[KB / 2][4];
        float rs = 0.0f;
        half2v const ones = {(_Float16)1.0f, (_Float16)1.0f};
        constexpr float LOG2E = 1.44269504088896340736f;
#pragma unroll
        for (int j = 0; j < KB; j++) {
          float4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int kk = 0; kk < DK; kk++) {
            half8 a;
            if (CM) {
              // permuted key order inside a pair of blocks, see cm_swizzle_key
              int const row = 32 * (j >> 1) + 4 * (j & 1) + 8 * (c >> 2) + (c & 3);
              a = *reinterpret_cast<half8 const *>(
                  kt + row * D + (((4 * kk + g) ^ cm_swizzle_key<D, true>(8 * (c >> 2) + (c & 3))) << 3));
            } else {
              a = *reinterpret_cast<half8 const *>(kt + swz_chunk(16 * j + c, 4 * kk + g, D));
            }
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qf[kk], acc, 0, 0, 0);
          }
#pragma unroll
          for (int h = 0; h < 2; h++) {
            half2v const s2 = {static_cast<_Float16>(acc[2 * h]), static_cast<_Float16>(acc[2 * h + 1])};
            float const x0 = __builtin_amdgcn_exp2f(__builtin_fmaf(static_cast<float>(s2[0]), LOG2E, 0.0f));
            float const x1 = __builtin_amdgcn_exp2f(__builtin_fmaf(static_cast<float>(s2[1]), LOG2E, 0.0f));
            half2v const e2 = {static_cast<_Float16>(x0), static_cast<_Float16>(x1)};
            rs = __builtin_amdgcn_fdot2(e2, ones, rs, false);
            pk[j / 2][2 * (j & 1) + h] = __builtin_bit_cast(uint32_t, e2);
          }
        }
        rs = sum_lane_groups(rs);
        r16 = static_cast<_Float16>(rs);  // row-sum tile (fp16)
        if (HAS_DIV) {
          // one reciprocal per row, then multiplies: within an fp32 ulp of the division
          float const inv = __builtin_amdgcn_rcpf(static_cast<float>(r16));
#pragma unroll
          for (int jj = 0; jj < KB / 2; jj++) {
#pragma unroll
            for (int w = 0; w < 4; w++) {
              half2v const e2 = __builtin_bit_cast(half2v, pk[jj][w]);
              half2v const p2 = {static_cast<_Float16>(__builtin_fmaf(static_cast<float>(e2[0]), inv, 0.0f)),
                                 static_cast<_Float16>(__builtin_fmaf(static_cast<float>(e2[1]), inv, 0.0f))};
              pk[jj][w] = __builtin_bit_cast(uint32_t, p2);
            }
          }
        }
        // ---- O = P . V: the accumulators of S^T are the A operand as they stand ---
#pragma unroll
        for (int t = 0; t < DB; t++) {
          float4v o = {0.0f, 0.0f, 0.0f, 0.0f};
          int const vrow = 16 * t + c;
#pragma unroll
          for (int jj = 0; jj < KB / 2; jj++) {
            // paired key groups (see store_patch_transposed): one 16-byte read per operand
            half8 b;
            if (CM) {
              // V^T[16t + c][keys 32jj + 8g + 0..7]
              b = *reinterpret_cast<half8 const *>(vt + vrow * NK + (((4 * jj + g) ^ cm_swizzle_key<NK, false>(c)) << 3));
            } else {
              b = *reinterpret_cast<half8 const *>(vt + swz_chunk(vrow, 4 * jj + g, NK));
            }
            uint4v const a = {pk[jj][0], pk[jj][1], pk[jj][2], pk[jj][3]};
            o = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), b, o, 0, 0, 0);
          }
#pragma unroll
          for (int r = 0; r < 4; r++) {
            o16[t][r] = static_cast<_Float16>(o[r]);  // O tile (fp16)
          }
        }
      }
      if (IP > 1) {
        // hand the iteration's result to the row group's first wavefront
        if (ip > 0 && active) {
          uint32_t *slot = slots + ((rg * (IP - 1) + (ip - 1)) * SLOT_DW) * 64 + lane;
#pragma unroll
          for (int t = 0; t < DB; t++) {
            half2v lo = {o16[t][0], o16[t][1]}, hi = {o16[t][2], o16[t][3]};
            slot[(2 * t) * 64] = __builtin_bit_cast(uint32_t, lo);
            slot[(2 * t + 1) * 64] = __builtin_bit_cast(uint32_t, hi);
          }
          half2v rr = {r16, (_Float16)0.0f};
          slot[(2 * DB) * 64] = __builtin_bit_cast(uint32_t, rr);
        }
        __syncthreads();
      }
      if (ip == 0) {
        // add the round's results in iteration order, rounding to fp16 after each
        // add exactly as the sequential loop would
#pragma unroll
        for (int q = 0; q < IP; q++) {
          if (r0 + q < n_st) {
            if (q > 0) {
              uint32_t const *slot = slots + ((rg * (IP - 1) + (q - 1)) * SLOT_DW) * 64 + lane;
#pragma unroll
              for (int t = 0; t < DB; t++) {
                half2v lo = __builtin_bit_cast(half2v, slot[(2 * t) * 64]);
                half2v hi = __builtin_bit_cast(half2v, slot[(2 * t + 1) * 64]);
                o16[t][0] = lo[0];
                o16[t][1] = lo[1];
                o16[t][2] = hi[0];
                o16[t][3] = hi[1];
              }
              r16 = __builtin_bit_cast(half2v, slot[(2 * DB) * 64])[0];
            }
#pragma unroll
            for (int t = 0; t < DB; t++) {
#pragma unroll
              for (int r = 0; r < 4; r++) {
                oacc[t][r] = static_cast<_Float16>(static_cast<float>(oacc[t][r]) +
                                                   static_cast<float>(o16[t][r]));
              }
            }
            if (!HAS_DIV) {
              racc = static_cast<_Float16>(static_cast<float>(racc) + static_cast<float>(r16));
            }
          }
        }
      }
      if (IP > 1 && r0 + IP < n_st) {
        __syncthreads();  // slots are free again for the next round
      }
    }
  }

  // ---- store: through LDS so every lane writes a 16-byte row segment ----------------
  _Float16 *ow = o_stage + rg * 16 * LDO;
  if (ip == 0) {
#pragma unroll
    for (int t = 0; t < DB; t++) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        ow[(4 * g + r) * LDO + 16 * t + c] = oacc[t][r];
      }
    }
  }
  __syncthreads();
  if (ip == 0) {
    _Float16 *og = static_cast<_Float16 *>(const_cast<void *>(P.o.ptr)) +
                   tile_offset(P.o, bx, by, bz, 0) + (long long)row_base * P.o.d_cols;
    constexpr int CH = DV / 8;  // 16-byte chunks per row
    for (int e = lane; e < P.rows * CH; e += 64) {
      int rr = e / CH, cc = (e % CH) * 8;
      *reinterpret_cast<uint4v *>(og + (long long)rr * P.o.d_cols + cc) =
          *reinterpret_cast<uint4v const *>(ow + rr * LDO + cc);
    }
    if (!HAS_DIV && g == 0 && c < P.rows) {
      _Float16 *rgp = static_cast<_Float16 *>(const_cast<void *>(P.r.ptr)) +
                      tile_offset(P.r, bx, by, bz, 0);
      rgp[(long long)(row_base + c) * P.r.d_cols] = racc;
    }
  }
}

// Throughput variant for large problems: every wavefront owns RPW row groups of 16
// query rows (so each K / V operand fetched from LDS feeds RPW MFMAs) and walks all
// for-loop iterations itself.  K and V tiles are double-buffered in LDS in their global
// (row-major) layout: the next tiles stream from global memory straight into LDS while
// the current ones are on the matrix cores, and the MFMA operands are gathered with
// transposing LDS reads.  One barrier per iteration.
//
// LDS layout of a tile: 16-byte chunk p of row r is stored at chunk position
// p ^ 2 * key(r) of that row.  A transposing read is served 32 lanes at a time; those
// lanes touch eight rows (lane groups g, g + 1 and four rows each) and 32 bytes per row,
// and the LDS has 64 banks of 4 bytes, so the keys are chosen to send the eight 32-byte
// pieces to eight different bank groups:
//   rows of 256 bytes (V, DV = 128): the rows are keys 4g + c / 4 (+ multiples of 16), and
//     key(r) = r & 7 permutes the eight chunk pairs of the row;
//   rows of 128 bytes, two per bank line: the row's parity picks the half line, the key
//     permutes the four chunk pairs within it.  For K the rows are 8g + c / 4 (+ multiples
//     of 4 and 32) and key(r) = bit 1 of r | bit 3 of r << 1; for V with DV = 64 the rows
//     are 4g + c / 4 and key(r) = (r >> 1) & 3.
template <int RowHalfs, bool IsK>
__device__ __forceinline__ constexpr int stream_swizzle_key(int r) {
  return RowHalfs == 128 ? (r & 7) : (IsK ? (((r >> 1) & 1) | (((r >> 3) & 1) << 1)) : ((r >> 1) & 3));
}

// Key tiles wider than 64 keys (SPI strips of 64 keys per for-loop iteration; the form without the
// division only, which needs no whole row sum before P.V): the strips of an iteration go through
// the same pipeline one after the other, P.V and the row sums run on in fp32 across them and are
// rounded to fp16 and added to the for-loop accumulators once per ITERATION -- the roundings of
// the sequential program for that tile width, an eighth of the conversion work at SPI = 8.
// MSUM (the form without the division): the row sums are one more column block of P.V, against
// a B operand of ones, instead of a packed dot product and two cross-lane adds per key block on
// the vector pipe (v_dot2 shares the matrix pipe and stalls it more than the two MFMAs cost).
template <int D, int NK, int DV, bool HAS_DIV, int RG, int RPW, bool CM = false, int SPI = 1>
__global__ __launch_bounds__(64 * RG, 2) void attn_stream_kernel(AttnParams const P) {
  static_assert(SPI == 1 || !HAS_DIV, "strips of one iteration need the form without the division");
  constexpr bool MSUM = !HAS_DIV;
  constexpr int LDO = DV + 8;
  constexpr int KB = NK / 16, DB = DV / 16, DK = D / 32;
  constexpr int NT = 64 * RG;
  constexpr int KC = D * NK / 8, VC = NK * DV / 8;  // 16-byte chunks per tile
  constexpr int KI = KC / NT, VI = VC / NT;          // direct loads per wavefront and tile
  static_assert(KC % NT == 0 && VC % NT == 0, "tiles must split evenly over the wavefronts");
  static_assert(NK / 8 >= 8 && DV / 8 >= 8, "the chunk swizzle needs rows of 8 chunks");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  _Float16 *const buf = reinterpret_cast<_Float16 *>(lds);

  int const tid = threadIdx.x;
  int const lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
  int const g = lane / 16, c = lane % 16;
  int bx, by, bz, slice;
  decode_block(P, bx, by, bz, slice);
  // Transposing reads: lane (g, c) supplies row 8g + c / 4 (K, rows are d) or 4g + c / 4
  // (V, rows are keys) and halfs 4 * (c % 4) .. + 3 of a 16-column block.  The row's
  // swizzle key is the same for every block the lane reads, so the swizzled chunk of
  // column block x is 2 * (x ^ key) + (c % 4) / 2: one XOR with a compile-time constant
  // per fetch.
  static_assert(NK == 64, "the K swizzle assumes rows of 128 bytes");
  int const a4 = c >> 2, b4 = c & 3;
  int const k_lane = (8 * g + a4) * NK + ((b4 >> 1) << 3) + (b4 & 1) * 4;
  int const v_lane = (4 * g + a4) * DV + ((b4 >> 1) << 3) + (b4 & 1) * 4;
  int const sw_k = stream_swizzle_key<NK, true>(8 * g + a4) << 4;
  int const sw_v = stream_swizzle_key<DV, false>(4 * g + a4) << 4;
  // column-major tiles: this lane's K^T row inside a pair of key blocks (block parity adds 4)
  // and its V^T row inside a block of 16 value columns, with the rows' swizzle keys
  int const kc_row = 8 * a4 + b4, kc_key = cm_swizzle_key<D, true>(8 * a4 + b4);
  int const vc_key = cm_swizzle_key<NK, false>(c);
  int const row_base = (slice * RG + wave) * RPW * 16;
  int const F = P.forloop_range * SPI;  // passes: strips of 64 keys
  half8 qf[RPW][DK];
  {
    _Float16 const *q = static_cast<_Float16 const *>(P.q.ptr) + tile_offset(P.q, bx, by, bz, 0) +
                        (long long)(row_base + c) * P.q.d_cols + 8 * g;
#pragma unroll
    for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
      for (int kk = 0; kk < DK; kk++) {
        qf[rp][kk] = *reinterpret_cast<half8 const *>(q + (long long)(16 * rp) * P.q.d_cols + 32 * kk);
      }
    }
  }
  // fp16 accumulators, two per register: the per-iteration `acc + x` rounded to fp16
  // is one packed fp16 add (the exact sum of two fp16 numbers rounded once, which is
  // what adding in fp32 and rounding gives)
  half2v oacc[RPW][DB][2];
  // row-sum accumulators: lane (g, c) holds the sum of query row c (dot-product form: [0]), or of
  // rows 4g .. 4g + 3 (MSUM: the accumulator layout of the matrix instruction)
  _Float16 racc[RPW][MSUM ? 4 : 1];
  // running fp32 sums of the iteration in progress: P.V (SPI > 1 only; with one strip per
  // iteration they are transient) and, MSUM, the row sums
  float4v o_run[SPI > 1 ? DB : 1][RPW], s_run[RPW];
#pragma unroll
  for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
    for (int r = 0; r < (MSUM ? 4 : 1); r++) {
      racc[rp][r] = (_Float16)0.0f;
    }
    s_run[rp] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int t = 0; t < (SPI > 1 ? DB : 1); t++) {
      o_run[t][rp] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int t = 0; t < DB; t++) {
      oacc[rp][t][0] = half2v{(_Float16)0.0f, (_Float16)0.0f};
      oacc[rp][t][1] = half2v{(_Float16)0.0f, (_Float16)0.0f};
    }
  }

  _Float16 *const kbuf = buf;               // two K tiles [D][NK]
  _Float16 *const vbuf = buf + 2 * NK * D;  // two V tiles [NK][DV]
  uint32_t const lds_k = lds_address(kbuf), lds_v = lds_address(vbuf);
  // Direct load i of this wavefront fills LDS chunks 64 * (wave * KI + i) .. + 63 of the
  // tile; this lane's chunk is (row r, position pos) and comes from global chunk
  // pos ^ 2 * key(r) of row r (byte offsets from the tile's first element).
  uint32_t k_goff[KI], v_goff[VI];
#pragma unroll
  for (int i = 0; i < KI; i++) {
    int const q = (wave * KI + i) * 64 + lane;
    if (CM) {  // K^T: NK rows of D halfs
      int const r = q / (D / 8), pos = q % (D / 8);
      k_goff[i] = 2u * (uint32_t)(r * P.k.d_cols + 8 * (pos ^ cm_swizzle_key<D, true>(r)));
    } else {
      int const r = q / (NK / 8), pos = q % (NK / 8);
      k_goff[i] = 2u * (uint32_t)(r * P.k.d_cols + 8 * (pos ^ (2 * stream_swizzle_key<NK, true>(r))));
    }
  }
#pragma unroll
  for (int i = 0; i < VI; i++) {
    int const q = (wave * VI + i) * 64 + lane;
    if (CM) {  // V^T: DV rows of NK halfs
      int const r = q / (NK / 8), pos = q % (NK / 8);
      v_goff[i] = 2u * (uint32_t)(r * P.v.d_cols + 8 * (pos ^ cm_swizzle_key<NK, false>(r)));
    } else {
      int const r = q / (DV / 8), pos = q % (DV / 8);
      v_goff[i] = 2u * (uint32_t)(r * P.v.d_cols + 8 * (pos ^ (2 * stream_swizzle_key<DV, false>(r))));
    }
  }
  // (strip `it` is strip it % SPI of iteration it / SPI: 64 keys further is 64 columns of K and 64
  // rows of V, or 64 rows of K^T and 64 columns of V^T)
  auto fetch_k = [&](int it, int b) {
    _Float16 const *kg = static_cast<_Float16 const *>(P.k.ptr) + tile_offset(P.k, bx, by, bz, it / SPI) +
                         (CM ? (long long)(64 * (it % SPI)) * P.k.d_cols : (long long)(64 * (it % SPI)));
#pragma unroll
    for (int i = 0; i < KI; i++) {
      lds_dma16(kg, k_goff[i], lds_k + 2u * (uint32_t)(b * NK * D + (wave * KI + i) * 512));
    }
  };
  auto fetch_v = [&](int it, int b) {
    _Float16 const *vg = static_cast<_Float16 const *>(P.v.ptr) + tile_offset(P.v, bx, by, bz, it / SPI) +
                         (CM ? (long long)(64 * (it % SPI)) : (long long)(64 * (it % SPI)) * P.v.d_cols);
#pragma unroll
    for (int i = 0; i < VI; i++) {
      lds_dma16(vg, v_goff[i], lds_v + 2u * (uint32_t)(b * DV * NK + (wave * VI + i) * 512));
    }
  };
  // all direct loads of this wavefront have landed; the barrier that follows publishes them
  auto fetched = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };

  // P of one iteration, packed fp16: pk[rp][jj][0..3] = eight keys of this lane's query
  // row (keys 4g..4g+3 of key blocks 2jj and 2jj+1), the A operand of P.V.
  // One 16-key block of S^T = K^T . Q^T for the RPW row groups is made in three steps the
  // pipeline below places separately: operand fetch from LDS, the MFMA chain, and the
  // roundings the sequential program makes (S to fp16, exp in fp32, the result to fp16;
  // the row sum adds the rounded values in fp32).
  half2v const ones = {(_Float16)1.0f, (_Float16)1.0f};
  constexpr float LOG2E = 1.44269504088896340736f;
  auto s_fetch = [&](_Float16 const *kt, int j, half8 (&a)[DK]) {
#pragma unroll
    for (int kk = 0; kk < DK; kk++) {
      if (CM) {
        // K^T[key 32 (j / 2) + 8 (c / 4) + 4 (j % 2) + c % 4][32kk + 8g + 0..7]
        a[kk] = *reinterpret_cast<half8 const *>(kt + (32 * (j >> 1) + 4 * (j & 1) + kc_row) * D +
                                                 (((4 * kk + g) ^ kc_key) << 3));
      } else {
        // K[32kk + 8g + 0..7][16j + c]
        _Float16 const *ka = kt + k_lane + 32 * kk * NK + (sw_k ^ (j << 4));
        half4 const a_lo = lds_read_tr16(ka), a_hi = lds_read_tr16(ka + 4 * NK);
        a[kk] = __builtin_shufflevector(a_lo, a_hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
    }
  };
  auto s_mfma = [&](half8 const (&a)[DK], float4v (&acc)[RPW]) {
#pragma unroll
    for (int rp = 0; rp < RPW; rp++) {
      acc[rp] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int kk = 0; kk < DK; kk++) {
#pragma unroll
      for (int rp = 0; rp < RPW; rp++) {
        acc[rp] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[kk], qf[rp][kk], acc[rp], 0, 0, 0);
      }
    }
  };
  // Runs at raised wave priority: this is the only long stretch without matrix work, and
  // the other wavefronts of the SIMD have MFMAs to overlap with it.
  auto s_post = [&](float4v const (&acc)[RPW], int j, uint32_t (&pk)[RPW][KB / 2][4], float (&rs)[RPW]) {
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
      for (int h = 0; h < 2; h++) {
        float2v const f2 = {acc[rp][2 * h], acc[rp][2 * h + 1]};
        half2v const s2 = __builtin_convertvector(f2, half2v);  // one packed conversion
        float const x0 = __builtin_amdgcn_exp2f(__builtin_fmaf(static_cast<float>(s2[0]), LOG2E, 0.0f));
        float const x1 = __builtin_amdgcn_exp2f(__builtin_fmaf(static_cast<float>(s2[1]), LOG2E, 0.0f));
        half2v const e2 = {static_cast<_Float16>(x0), static_cast<_Float16>(x1)};
        if (!MSUM) {
          rs[rp] = __builtin_amdgcn_fdot2(e2, ones, rs[rp], false);
        }
        pk[rp][j / 2][2 * (j & 1) + h] = __builtin_bit_cast(uint32_t, e2);
      }
    }
    __builtin_amdgcn_s_setprio(0);
  };
  auto s_block = [&](_Float16 const *kt, int j, uint32_t (&pk)[RPW][KB / 2][4], float (&rs)[RPW]) {
    half8 a[DK];
    float4v acc[RPW];
    s_fetch(kt, j, a);
    s_mfma(a, acc);
    s_post(acc, j, pk, rs);
  };
  // After the last key block: the row sum across the four lane groups, then either the
  // normalisation of P (form with div) or the accumulation of the denominator.
  auto s_finish = [&](uint32_t (&pk)[RPW][KB / 2][4], float (&rs)[RPW]) {
    if (MSUM) {
      return;  // the row sums come out of the matrix cores with P.V
    }
#pragma unroll
    for (int rp = 0; rp < RPW; rp++) {
      rs[rp] = sum_lane_groups(rs[rp]);
      _Float16 const r16 = static_cast<_Float16>(rs[rp]);
      float const inv = __builtin_amdgcn_rcpf(static_cast<float>(r16));
#pragma unroll
      for (int jj = 0; jj < KB / 2; jj++) {
#pragma unroll
        for (int w = 0; w < 4; w++) {
          half2v const e2 = __builtin_bit_cast(half2v, pk[rp][jj][w]);
          // (a fused multiply-add with +0: maps to the mixed-precision FMA that reads and
          // writes fp16; exp values are positive, so the +0 changes nothing)
          half2v const p2 = {static_cast<_Float16>(__builtin_fmaf(static_cast<float>(e2[0]), inv, 0.0f)),
                             static_cast<_Float16>(__builtin_fmaf(static_cast<float>(e2[1]), inv, 0.0f))};
          pk[rp][jj][w] = __builtin_bit_cast(uint32_t, p2);
        }
      }
    }
  };
  // MSUM: the row sums of P(it) join the running sums; after an iteration's last strip they are
  // rounded to fp16 and added to the for-loop accumulators
  half8 ones8;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    ones8[e] = (_Float16)1.0f;
  }
  auto sum_mfma = [&](uint32_t const (&pk)[RPW][KB / 2][4], bool last_strip) {
    if (!MSUM) {
      return;
    }
#pragma unroll
    for (int jj = 0; jj < KB / 2; jj++) {
#pragma unroll
      for (int rp = 0; rp < RPW; rp++) {
        uint4v const a = {pk[rp][jj][0], pk[rp][jj][1], pk[rp][jj][2], pk[rp][jj][3]};
        s_run[rp] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), ones8, s_run[rp], 0, 0, 0);
      }
    }
    if (last_strip) {
#pragma unroll
      for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
          _Float16 const r16 = static_cast<_Float16>(s_run[rp][r]);
          racc[rp][MSUM ? r : 0] = static_cast<_Float16>(static_cast<float>(racc[rp][MSUM ? r : 0]) + static_cast<float>(r16));
        }
        s_run[rp] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
  };
  // Sixteen output columns of O += P . V for the RPW row groups: operand fetch, then the
  // MFMA chain and the fp16 accumulation.
  auto pv_fetch = [&](_Float16 const *vt, int t, half8 (&b)[KB / 2]) {
#pragma unroll
    for (int jj = 0; jj < KB / 2; jj++) {
      if (CM) {
        // V^T[16t + c][keys 32jj + 8g + 0..7]: the keys P holds (see the key order of S^T)
        b[jj] = *reinterpret_cast<half8 const *>(vt + (16 * t + c) * NK + (((4 * jj + g) ^ vc_key) << 3));
      } else {
        // V[32jj + 4g + 0..3][16t + c] and V[32jj + 16 + 4g + 0..3][16t + c]: the keys P holds
        _Float16 const *vb = vt + v_lane + 32 * jj * DV + (sw_v ^ (t << 4));
        half4 const b_lo = lds_read_tr16(vb), b_hi = lds_read_tr16(vb + 16 * DV);
        b[jj] = __builtin_shufflevector(b_lo, b_hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
    }
  };
  // (SPI > 1: `o` is the column block's running sum of the iteration, zeroed when the iteration's
  // last strip has been added to the accumulators; SPI == 1: a fresh sum per pass)
  auto pv_mfma = [&](half8 const (&b)[KB / 2], uint32_t const (&pk)[RPW][KB / 2][4], float4v (&o)[RPW]) {
    if (SPI == 1) {
#pragma unroll
      for (int rp = 0; rp < RPW; rp++) {
        o[rp] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
#pragma unroll
    for (int jj = 0; jj < KB / 2; jj++) {
#pragma unroll
      for (int rp = 0; rp < RPW; rp++) {
        uint4v const a = {pk[rp][jj][0], pk[rp][jj][1], pk[rp][jj][2], pk[rp][jj][3]};
        o[rp] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), b[jj], o[rp], 0,
                                                       0, 0);
      }
    }
  };
  auto pv_post = [&](float4v (&o)[RPW], int t, bool last_strip) {
    if (SPI > 1 && !last_strip) {
      return;
    }
#pragma unroll
    for (int rp = 0; rp < RPW; rp++) {
      half2v lo = {static_cast<_Float16>(o[rp][0]), static_cast<_Float16>(o[rp][1])};
      half2v hi = {static_cast<_Float16>(o[rp][2]), static_cast<_Float16>(o[rp][3])};
      oacc[rp][t][0] = oacc[rp][t][0] + lo;
      oacc[rp][t][1] = oacc[rp][t][1] + hi;
      if (SPI > 1) {
        o[rp] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
  };
  auto pv_block = [&](_Float16 const *vt, int t, uint32_t const (&pk)[RPW][KB / 2][4], bool last_strip) {
    half8 b[KB / 2];
    pv_fetch(vt, t, b);
    if (SPI > 1) {
      pv_mfma(b, pk, o_run[SPI > 1 ? t : 0]);
      pv_post(o_run[SPI > 1 ? t : 0], t, last_strip);
    } else {
      float4v o[RPW];
      pv_mfma(b, pk, o);
      pv_post(o, t, true);
    }
  };

  // The loop is skewed by one phase: pass `it` multiplies P(it) with V(it) while it
  // builds P(it + 1) from K(it + 1), so every pass has two independent instruction
  // streams (matrix-heavy P.V, conversion / exp-heavy S) to overlap.  K tiles and V
  // tiles are double-buffered separately: pass `it` reads K(it + 1) and V(it) and, at its
  // end, replaces K(it) by K(it + 2) and V(it - 1) by V(it + 1).
  fetch_k(0, 0);
  fetch_v(0, 0);
  if (F > 1) {
    fetch_k(1, 1);
  }
  fetched();
  __syncthreads();
  uint32_t pa[RPW][KB / 2][4], pb[RPW][KB / 2][4];  // P(it) and P(it + 1), roles alternate
  {
    float rs[RPW];
#pragma unroll
    for (int rp = 0; rp < RPW; rp++) {
      rs[rp] = 0.0f;
    }
#pragma unroll
    for (int j = 0; j < KB; j++) {
      s_block(kbuf, j, pa, rs);
    }
    s_finish(pa, rs);
  }
  __syncthreads();  // K(0) may be overwritten from here on
  // One skewed pass: P(it) . V(it) interleaved with building P(it + 1) from K(it + 1).
  // Within the pass the LDS operands of a step are requested one step ahead (before the
  // exp stretch or the MFMA chain that precedes their use), so their latency is covered
  // by this wavefront's own work; the scheduling barriers keep that order.
  constexpr int TPU = DB / KB;  // P.V column blocks per S block
  auto skewed_pass = [&](int it, uint32_t const (&pcur)[RPW][KB / 2][4],
                         uint32_t (&pnext)[RPW][KB / 2][4], bool last_strip) {
    _Float16 const *vt = vbuf + (it & 1) * DV * NK;
    _Float16 const *kt = kbuf + ((it + 1) & 1) * NK * D;
    float rs[RPW];
#pragma unroll
    for (int rp = 0; rp < RPW; rp++) {
      rs[rp] = 0.0f;
    }
    half8 ka[DK];
    s_fetch(kt, 0, ka);
#pragma unroll
    for (int u = 0; u < KB; u++) {
      float4v sacc[RPW];
      s_mfma(ka, sacc);
      half8 vb[TPU][KB / 2];
#pragma unroll
      for (int x = 0; x < TPU; x++) {
        pv_fetch(vt, u * TPU + x, vb[x]);
      }
      __builtin_amdgcn_sched_barrier(0);
      s_post(sacc, u, pnext, rs);
      if (u + 1 < KB) {
        s_fetch(kt, u + 1, ka);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (SPI > 1) {
#pragma unroll
        for (int x = 0; x < TPU; x++) {
          pv_mfma(vb[x], pcur, o_run[SPI > 1 ? u * TPU + x : 0]);
        }
        if (u == KB - 1) {
          sum_mfma(pcur, last_strip);
        }
#pragma unroll
        for (int x = 0; x < TPU; x++) {
          pv_post(o_run[SPI > 1 ? u * TPU + x : 0], u * TPU + x, last_strip);
        }
      } else {
        float4v o[TPU][RPW];
#pragma unroll
        for (int x = 0; x < TPU; x++) {
          pv_mfma(vb[x], pcur, o[x]);
        }
        if (u == KB - 1) {
          sum_mfma(pcur, true);
        }
#pragma unroll
        for (int x = 0; x < TPU; x++) {
          pv_post(o[x], u * TPU + x, true);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    s_finish(pnext, rs);
  };
  // Pass `it` starts by sending K(it + 2) after K(it) and V(it + 1) after V(it - 1) (both
  // last read in the previous pass); the transfers run under the whole pass.  Two passes
  // per trip, so that P(it) and P(it + 1) swap roles instead of being copied.
  int it = 0;
  for (; it + 3 < F; it += 2) {
    fetch_k(it + 2, 0);
    fetch_v(it + 1, 1);
    __builtin_amdgcn_sched_barrier(0);
    skewed_pass(0, pa, pb, (it & (SPI - 1)) == SPI - 1);
    fetched();
    __syncthreads();
    fetch_k(it + 3, 1);
    fetch_v(it + 2, 0);
    __builtin_amdgcn_sched_barrier(0);
    skewed_pass(1, pb, pa, ((it + 1) & (SPI - 1)) == SPI - 1);
    fetched();
    __syncthreads();
  }
  for (; it + 1 < F; it++) {  // at most two passes left before the last P . V
    if (it + 2 < F) {
      fetch_k(it + 2, it & 1);
    }
    fetch_v(it + 1, (it + 1) & 1);
    __builtin_amdgcn_sched_barrier(0);
    skewed_pass(it, pa, pb, (it & (SPI - 1)) == SPI - 1);
#pragma unroll
    for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
      for (int jj = 0; jj < KB / 2; jj++) {
#pragma unroll
        for (int w = 0; w < 4; w++) {
          pa[rp][jj][w] = pb[rp][jj][w];
        }
      }
    }
    fetched();
    __syncthreads();
  }
  {  // pass F - 1: the last P . V
    _Float16 const *vt = vbuf + (it & 1) * DV * NK;
#pragma unroll
    for (int t = 0; t < DB; t++) {
      pv_block(vt, t, pa, true);
    }
    sum_mfma(pa, true);
    __syncthreads();
  }

  // ---- store through LDS (the tile buffers are dead) ----------------------------------
  _Float16 *ow = buf + wave * RPW * 16 * LDO;
#pragma unroll
  for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
    for (int t = 0; t < DB; t++) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        ow[(16 * rp + 4 * g + r) * LDO + 16 * t + c] = oacc[rp][t][r >> 1][r & 1];
      }
    }
  }
  __syncthreads();
  {
    _Float16 *og = static_cast<_Float16 *>(const_cast<void *>(P.o.ptr)) +
                   tile_offset(P.o, bx, by, bz, 0) + (long long)row_base * P.o.d_cols;
    constexpr int CH = DV / 8;
    for (int e2 = lane; e2 < RPW * 16 * CH; e2 += 64) {
      int rr = e2 / CH, cc = (e2 % CH) * 8;
      *reinterpret_cast<uint4v *>(og + (long long)rr * P.o.d_cols + cc) =
          *reinterpret_cast<uint4v const *>(ow + rr * LDO + cc);
    }
    if (MSUM && c < 4) {
      // every lane of a group holds the sums of rows 4g .. 4g + 3: lane c < 4 stores row 4g + c
      _Float16 *rgp = static_cast<_Float16 *>(const_cast<void *>(P.r.ptr)) +
                      tile_offset(P.r, bx, by, bz, 0);
#pragma unroll
      for (int rp = 0; rp < RPW; rp++) {
        _Float16 const v = c == 0 ? racc[rp][0] : (c == 1 ? racc[rp][MSUM ? 1 : 0] : (c == 2 ? racc[rp][MSUM ? 2 : 0] : racc[rp][MSUM ? 3 : 0]));
        rgp[(long long)(row_base + 16 * rp + 4 * g + c) * P.r.d_cols] = v;
      }
    }
  }
}

// Direct-staging variant: one row group of (up to) 16 query rows per workgroup, IP wavefronts
// as iteration lanes.  Wavefront ip owns iterations ip, ip + IP, ip + 2 IP, ... and streams the
// K and V tile of each from global memory straight into ITS OWN LDS buffers, in their row-major
// layout (sixteen direct loads per tile pair: no registers, no transposing stores), NBUF tile
// pairs deep: while it multiplies one pair the next is in flight.  No workgroup barrier inside
// the loop: a wavefront waits for its own loads only (`s_waitcnt vmcnt`), so the workgroup is
// IP independent streams -- what a bandwidth-bound decode (8 or 16 query rows against a long
// key range) needs -- and with one iteration per wavefront (F <= IP) the shortest chain from
// launch to result.  MFMA operands are gathered with transposing LDS reads under the chunk
// swizzle of the throughput variant.  Arithmetic and rounding points are those of
// attn_fused_kernel.  Every iteration's fp16 result is kept (packed, in registers) until the
// wavefront has finished, then written to LDS (into its own, now dead, tile buffers); after
// ONE barrier all threads add the F results element by element in ITERATION order, rounding
// to fp16 after each add as the sequential loop does, and store straight from registers.
//
// The loads are inline assembly (see lds_dma16), so the compiler's own count of outstanding
// vector-memory operations knows nothing of them and the waits are written by hand.  Every
// load of this kernel is a direct-to-LDS load, the Q tile included: a wait for "all but the
// newest n" relies on loads completing in issue order, which holds among loads of one kind
// but not between direct-to-LDS loads and loads into registers (a register load issued after
// a tile's direct loads was seen to complete before them).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
#pragma clang diagnostic pop

// Key tiles of other widths ride on the same 64-key strips.  A wavefront's unit of work is
// max(one iteration, one strip of 64 keys):
//   SPI strips per iteration (key tiles of 128 / 256): the strips of an iteration are streamed
//     one after the other, the row sum and the fp32 P.V accumulators run across them and the
//     iteration's result is rounded once at its end (form without the division only: the
//     division needs the whole row sum before the first P.V);
//   IPS iterations per strip (key tiles of 32 / 16, whose tiles of consecutive iterations lie
//     side by side in memory -- the host checks the loader strides): one load of 64 keys, then
//     every 32- or 16-key slice gets its own exp / row sum / [division] / P.V and its own
//     rounded result.  Slices of 16 keys take the 16 x 16 x 16 matrix instruction.
// Column-major K and V (CM): the tiles are K^T [64 keys][64] and V^T [64][64 keys], swizzled and
// read as in attn_stream_kernel (one plain 16-byte LDS read per operand, keys of a pair of S^T
// blocks permuted so that P's eight values per lane are consecutive keys).  Slices of 16 keys
// (IPS == 4) need every block to be 16 consecutive keys: they keep the plain key order and fetch
// their V^T operand as two 8-byte reads.
template <int D, int NK, int DV, bool HAS_DIV, int IP, int RPW, int NBUF, int NIT, int SPI, int IPS,
          bool TRACE, bool CM>
__global__ __launch_bounds__(64 * IP) void attn_direct_kernel(AttnParams const) {
  // (the argument block is read by hand, all of it at once; decode_block reads gridDim.z, so
  // the block counts behind the arguments exist and are fetched with them)
  AttnParams const P = load_kernel_arguments<AttnParams, 3>();
  constexpr bool PERM = CM && IPS != 4;  // permuted key order inside pairs of S^T blocks
  static_assert(D == 64 && NK == 64 && DV == 64, "the chunk swizzles assume rows of 128 bytes");
  static_assert((SPI == 1 || IPS == 1) && (SPI == 1 || SPI == 2 || SPI == 4) &&
                    (IPS == 1 || IPS == 2 || IPS == 4) && !(HAS_DIV && SPI > 1),
                "strips per iteration or iterations per strip, not both");
  static_assert(NBUF == 1 || NBUF == 2, "one or two tile pairs per wavefront");
  constexpr int KB = NK / 16, DB = DV / 16, DK = D / 32;
  constexpr int KI = D * NK / 8 / 64, VI = NK * DV / 8 / 64;  // direct loads per tile
  constexpr int PAIR_HALFS = D * NK + NK * DV;                // one K tile + one V tile
  constexpr int ROWS = 16 * RPW;                              // query rows of one wavefront
  constexpr int Q_HALFS = ROWS * D;                           // this wavefront's copy of the Q tile
  constexpr int QI = Q_HALFS / 8 / 64;                        // direct loads of the Q tile
  constexpr int WAVE_HALFS = NBUF * PAIR_HALFS + Q_HALFS;
  constexpr int LDO = DV + 4;          // row stride of a result slot (halfs): 8-byte aligned rows
  constexpr int SLOT_HALFS = ROWS * LDO + ROWS;  // one iteration's O tile + its row sums
  // (the Q tile is in registers by then, so its region counts)
  static_assert(NIT * IPS * SLOT_HALFS <= WAVE_HALFS, "a wavefront's results must fit its own buffers");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

  unsigned long long t_start = 0, t_issued = 0, t_landed = 0, t_computed = 0, t_joined = 0;
  if (TRACE) {
    t_start = __builtin_amdgcn_s_memrealtime();
  }
  int const tid = threadIdx.x;
  int const lane = tid % 64, ip = __builtin_amdgcn_readfirstlane(tid / 64);
  int const g = lane / 16, c = lane % 16;
  int bx, by, bz, slice;
  decode_block(P, bx, by, bz, slice);
  int const row_base = slice * ROWS;
  int const rows = RPW == 1 ? P.rows : ROWS;  // rows that exist (only a lone row group may be short)
  int const F = P.forloop_range;
  int const units = F / IPS;                                     // units of work of the for-loop
  int const nit = ip < units ? (units - ip + IP - 1) / IP : 0;  // units of this wavefront

  _Float16 *const wbuf = reinterpret_cast<_Float16 *>(lds) + ip * WAVE_HALFS;
  uint32_t const lds_w = lds_address(wbuf);
  // Direct load i of a tile fills LDS chunks 64 i .. 64 i + 63: this lane's chunk is
  // (row 8 i + lane / 8, position lane % 8) and comes from global chunk pos ^ 2 * key(row) of
  // that row.  The swizzle keys depend on i only through its parity (K) or not at all (V), so
  // three lane offsets serve all sixteen loads and the row advance 8 i is added to the
  // wavefront-uniform base address.
  int const l3 = lane >> 3, pos = lane & 7;
  static_assert(stream_swizzle_key<NK, true>(8 + 5) == (stream_swizzle_key<NK, true>(5) | 2) &&
                    stream_swizzle_key<DV, false>(8 + 5) == stream_swizzle_key<DV, false>(5),
                "row advance by 8 flips bit 1 of the K key and leaves the V key unchanged");
  // (column-major tiles: the K^T key of row 8 i + l3 depends on i % 4, the V^T key on i % 2)
  uint32_t k_off[CM ? 4 : 2], v_offs[CM ? 2 : 1];
#pragma unroll
  for (int i = 0; i < (CM ? 4 : 2); i++) {
    int const key = CM ? cm_swizzle_key<D, true>(8 * i + l3) : 2 * stream_swizzle_key<NK, true>(8 * i + l3);
    k_off[i] = 2u * (uint32_t)(l3 * P.k.d_cols + 8 * (pos ^ key));
  }
#pragma unroll
  for (int i = 0; i < (CM ? 2 : 1); i++) {
    int const key = CM ? cm_swizzle_key<NK, false>(8 * i + l3) : 2 * stream_swizzle_key<DV, false>(l3);
    v_offs[i] = 2u * (uint32_t)(l3 * P.v.d_cols + 8 * (pos ^ key));
  }
  // strip `strip` (64 keys) of unit `unit`: the unit's first iteration names the tile origin;
  // 64 keys further is 64 columns of K and 64 rows of V (column-major: 64 rows of K^T, 64
  // columns of V^T)
  auto fetch = [&](int unit, int strip, int b) {
    _Float16 const *kg = static_cast<_Float16 const *>(P.k.ptr) + tile_offset(P.k, bx, by, bz, unit * IPS) +
                         (CM ? (long long)(64 * strip) * P.k.d_cols : (long long)(64 * strip));
    _Float16 const *vg = static_cast<_Float16 const *>(P.v.ptr) + tile_offset(P.v, bx, by, bz, unit * IPS) +
                         (CM ? (long long)(64 * strip) : (long long)(64 * strip) * P.v.d_cols);
    uint32_t const base = lds_w + 2u * (uint32_t)(b * PAIR_HALFS);
#pragma unroll
    for (int i = 0; i < KI; i++) {
      lds_dma16(kg + (long long)(8 * i) * P.k.d_cols, k_off[CM ? (i & 3) : (i & 1)],
                base + 1024u * (uint32_t)i);
    }
#pragma unroll
    for (int i = 0; i < VI; i++) {
      lds_dma16(vg + (long long)(8 * i) * P.v.d_cols, v_offs[CM ? (i & 1) : 0],
                base + 2u * (uint32_t)(D * NK) + 1024u * (uint32_t)i);
    }
  };
  // The Q tile (rows that do not exist re-read row 0 and are zeroed below), then the first
  // one or two tile pairs: everything this wavefront needs to start is in flight at once.
  // (A wavefront without an iteration loads nothing: no transfer may outlive its waits.)
  half8 qf[RPW][DK];
  if (nit > 0) {
    _Float16 const *qg = static_cast<_Float16 const *>(P.q.ptr) + tile_offset(P.q, bx, by, bz, 0) +
                         (long long)row_base * P.q.d_cols;
#pragma unroll
    for (int i = 0; i < QI; i++) {
      int const r = 8 * i + l3;
      uint32_t const off = 2u * (uint32_t)((r < rows ? r : 0) * P.q.d_cols + 8 * pos);
      lds_dma16(qg, off, lds_w + 2u * (uint32_t)(NBUF * PAIR_HALFS) + 1024u * (uint32_t)i);
    }
    fetch(ip, 0, 0);
  }
  // strips of this wavefront in the order it walks them: q = j * SPI + s (unit ip + j IP)
  int const nstrips = nit * SPI;
  if (NBUF == 2 && nstrips > 1) {
    fetch(ip + (1 / SPI) * IP, 1 % SPI, 1);
  }
  if (TRACE) {
    t_issued = __builtin_amdgcn_s_memrealtime();
  }
  int const a4 = c >> 2, b4 = c & 3;
  int const k_lane = (8 * g + a4) * NK + ((b4 >> 1) << 3) + (b4 & 1) * 4;
  int const v_lane = (4 * g + a4) * DV + ((b4 >> 1) << 3) + (b4 & 1) * 4;
  int const sw_k = stream_swizzle_key<NK, true>(8 * g + a4) << 4;
  int const sw_v = stream_swizzle_key<DV, false>(4 * g + a4) << 4;
  int const kc_row = 8 * a4 + b4, kc_key = cm_swizzle_key<D, true>(8 * a4 + b4);
  int const vc_key = cm_swizzle_key<NK, false>(c);
  // where this thread's share of the result goes (address arithmetic done while loads fly)
  constexpr int EPT = ROWS * DV / (64 * IP);  // elements per thread (16 rows: 8 / 4 / 2 for IP = 2 / 4 / 8)
  static_assert(EPT == 2 || EPT == 4 || EPT == 8, "2, 4 or 8 wavefronts");
  int const out_row = tid / (DV / EPT), out_col = (tid % (DV / EPT)) * EPT;
  _Float16 *og = static_cast<_Float16 *>(const_cast<void *>(P.o.ptr)) +
                 tile_offset(P.o, bx, by, bz, 0) +
                 (long long)(row_base + out_row) * P.o.d_cols + out_col;
  // (the address is made opaque here so that it IS computed here, while the wavefront waits for
  // its tiles: left alone the compiler computes it where it is used, after the last barrier)
  asm volatile("" : "+v"(og));

  // results of this wavefront's iterations, packed fp16: keep[j][rp][2t], [2t+1] =
  // O[row 16rp + c][16t + 4g + r] for r = 0,1 / 2,3; keep[j][rp][2 DB] = the row sum of row c
  uint32_t keep[NIT][IPS][RPW][2 * DB + 1];
  float4v o[RPW][DB];  // P.V accumulators of the iteration in progress (SPI > 1: across strips)
  float rs_run[RPW];   // its running row sums
#pragma unroll
  for (int q = 0; q < NIT * SPI; q++) {
    int const j = q / SPI, sidx = q % SPI;
    if (q < nstrips) {
      int const b = NBUF == 2 ? (q & 1) : 0;
      // the tile pair of iteration j (and everything older) has landed when at most the next
      // pair's loads are outstanding
      // (a pair's K loads go out before its V loads, and loads complete in order: the K tile,
      // and the Q tile before it, are there when the V loads are the oldest still outstanding;
      // the V tile is waited for where it is first read, after the S^T products are issued)
      if (NBUF == 2 && q + 1 < nstrips) {
        wait_vm<KI + 2 * VI>();
      } else {
        wait_vm<VI>();
      }
      if (q == 0) {
        // Q fragments (B operand of S^T): Q[row c][32kk + 8g .. +7]
        _Float16 const *ql = wbuf + NBUF * PAIR_HALFS + c * D + 8 * g;
#pragma unroll
        for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
          for (int kk = 0; kk < DK; kk++) {
            qf[rp][kk] = *reinterpret_cast<half8 const *>(ql + 16 * rp * D + 32 * kk);
            if (RPW == 1 && c >= rows) {
#pragma unroll
              for (int e = 0; e < 8; e++) {
                qf[rp][kk][e] = (_Float16)0.0f;
              }
            }
          }
        }
        if (TRACE) {
          t_landed = __builtin_amdgcn_s_memrealtime();
        }
      }
      _Float16 const *kt = wbuf + b * PAIR_HALFS;
      _Float16 const *vt = kt + D * NK;
      // Four phases, each with all of its independent work issued before anything waits:
      // every K operand read, the KB independent S^T accumulation chains interleaved, every
      // V operand read (their latency hides under the exp stretch), the DB independent P.V
      // chains interleaved.
      half8 ka[KB][DK];
#pragma unroll
      for (int jb = 0; jb < KB; jb++) {
#pragma unroll
        for (int kk = 0; kk < DK; kk++) {
          if (PERM) {
            // K^T[key 32 (jb / 2) + 8 (c / 4) + 4 (jb % 2) + c % 4][32kk + 8g + 0..7]
            ka[jb][kk] = *reinterpret_cast<half8 const *>(kt + (32 * (jb >> 1) + 4 * (jb & 1) + kc_row) * D +
                                                          (((4 * kk + g) ^ kc_key) << 3));
          } else if (CM) {
            // K^T[key 16jb + c][32kk + 8g + 0..7]
            ka[jb][kk] = *reinterpret_cast<half8 const *>(
                kt + (16 * jb + c) * D + (((4 * kk + g) ^ cm_swizzle_key<D, true>(16 * jb + c)) << 3));
          } else {
            // K[32kk + 8g + 0..7][16jb + c]
            _Float16 const *kp = kt + k_lane + 32 * kk * NK + (sw_k ^ (jb << 4));
            half4 const a_lo = lds_read_tr16(kp), a_hi = lds_read_tr16(kp + 4 * NK);
            ka[jb][kk] = __builtin_shufflevector(a_lo, a_hi, 0, 1, 2, 3, 4, 5, 6, 7);
          }
        }
      }
      float4v acc[RPW][KB];
#pragma unroll
      for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
        for (int jb = 0; jb < KB; jb++) {
          acc[rp][jb] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
        }
      }
#pragma unroll
      for (int kk = 0; kk < DK; kk++) {
#pragma unroll
        for (int jb = 0; jb < KB; jb++) {
#pragma unroll
          for (int rp = 0; rp < RPW; rp++) {
            acc[rp][jb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[jb][kk], qf[rp][kk], acc[rp][jb], 0, 0, 0);
          }
        }
      }
      if (NBUF == 2 && q + 1 < nstrips) {
        wait_vm<KI + VI>();
      } else {
        wait_vm<0>();
      }
      half8 vb[DB][KB / 2];
#pragma unroll
      for (int t = 0; t < DB; t++) {
#pragma unroll
        for (int jj = 0; jj < KB / 2; jj++) {
          if (PERM) {
            // V^T[16t + c][keys 32jj + 8g + 0..7]: the keys P holds under the permuted order
            vb[t][jj] = *reinterpret_cast<half8 const *>(vt + (16 * t + c) * NK + (((4 * jj + g) ^ vc_key) << 3));
          } else if (CM) {
            // V^T[16t + c][keys 32jj + 4g + 0..3] and [32jj + 16 + 4g + 0..3]: 8 bytes each
            _Float16 const *vrow = vt + (16 * t + c) * NK + 4 * (g & 1);
            half4 const b_lo = *reinterpret_cast<half4 const *>(vrow + (((4 * jj + (g >> 1)) ^ vc_key) << 3));
            half4 const b_hi = *reinterpret_cast<half4 const *>(vrow + (((4 * jj + 2 + (g >> 1)) ^ vc_key) << 3));
            vb[t][jj] = __builtin_shufflevector(b_lo, b_hi, 0, 1, 2, 3, 4, 5, 6, 7);
          } else {
            // V[32jj + 4g + 0..3][16t + c] and V[32jj + 16 + 4g + 0..3][16t + c]: the keys P holds
            _Float16 const *vp = vt + v_lane + 32 * jj * DV + (sw_v ^ (t << 4));
            half4 const b_lo = lds_read_tr16(vp), b_hi = lds_read_tr16(vp + 16 * DV);
            vb[t][jj] = __builtin_shufflevector(b_lo, b_hi, 0, 1, 2, 3, 4, 5, 6, 7);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      // exp of every 16-key block, packed fp16 as the next matrix instruction wants it, and
      // the blocks' row-sum parts (each lane: its four keys of the block)
      uint32_t pk[RPW][KB / 2][4];
      float rsb[RPW][KB];
      half2v const ones = {(_Float16)1.0f, (_Float16)1.0f};
      constexpr float LOG2E = 1.44269504088896340736f;
#pragma unroll
      for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
        for (int jb = 0; jb < KB; jb++) {
          float part = 0.0f;
#pragma unroll
          for (int h = 0; h < 2; h++) {
            // (pairs are rounded to fp16 by one packed conversion each)
            float2v const f2 = {acc[rp][jb][2 * h], acc[rp][jb][2 * h + 1]};
            half2v const s2 = __builtin_convertvector(f2, half2v);
            float2v const x2 = {__builtin_amdgcn_exp2f(__builtin_fmaf(static_cast<float>(s2[0]), LOG2E, 0.0f)),
                                __builtin_amdgcn_exp2f(__builtin_fmaf(static_cast<float>(s2[1]), LOG2E, 0.0f))};
            half2v const e2 = __builtin_convertvector(x2, half2v);
            part = __builtin_amdgcn_fdot2(e2, ones, part, false);
            pk[rp][jb / 2][2 * (jb & 1) + h] = __builtin_bit_cast(uint32_t, e2);
          }
          rsb[rp][jb] = part;
        }
      }
      // row sum of a slice (blocks jb0 .. jb0 + nb - 1 plus `carry`) over the four lane groups
      auto row_sum = [&](int rp, int jb0, int nb, float carry) {
        float rs = carry;
#pragma unroll
        for (int x = 0; x < KB; x++) {
          if (x >= jb0 && x < jb0 + nb) {
            rs += rsb[rp][x];
          }
        }
        return rs;
      };
      auto across = [&](float rs) {
        rs = sum_lane_groups(rs);
        return rs;
      };
      auto normalise = [&](int rp, int w0, int nw, _Float16 r16) {
        float const inv = __builtin_amdgcn_rcpf(static_cast<float>(r16));
#pragma unroll
        for (int w = 0; w < 4 * (KB / 2); w++) {
          if (w >= w0 && w < w0 + nw) {
            half2v const e2 = __builtin_bit_cast(half2v, pk[rp][w / 4][w % 4]);
            // (written as a fused multiply-add with +0 so that it maps to the mixed-precision
            // FMA that reads fp16 and writes fp16: exp values are positive, so adding +0 changes
            // nothing)
            half2v const p2 = {static_cast<_Float16>(__builtin_fmaf(static_cast<float>(e2[0]), inv, 0.0f)),
                               static_cast<_Float16>(__builtin_fmaf(static_cast<float>(e2[1]), inv, 0.0f))};
            pk[rp][w / 4][w % 4] = __builtin_bit_cast(uint32_t, p2);
          }
        }
      };
      auto store_result = [&](int sub, int rp, float4v const (&res)[DB], _Float16 r16) {
#pragma unroll
        for (int t = 0; t < DB; t++) {
          half2v const lo = __builtin_convertvector(float2v{res[t][0], res[t][1]}, half2v);
          half2v const hi = __builtin_convertvector(float2v{res[t][2], res[t][3]}, half2v);
          keep[j][sub][rp][2 * t] = __builtin_bit_cast(uint32_t, lo);
          keep[j][sub][rp][2 * t + 1] = __builtin_bit_cast(uint32_t, hi);
        }
        half2v const rr = {r16, (_Float16)0.0f};
        keep[j][sub][rp][2 * DB] = __builtin_bit_cast(uint32_t, rr);
      };
      // V^T is the first operand of every P.V instruction: the product comes out transposed,
      // which leaves a lane with four consecutive columns of one row,
      // res[t][r] = O[row c][16t + 4g + r]
      if (IPS == 1) {
#pragma unroll
        for (int rp = 0; rp < RPW; rp++) {
          rs_run[rp] = row_sum(rp, 0, KB, sidx == 0 ? 0.0f : rs_run[rp]);
        }
        _Float16 r16[RPW];
        if (sidx == SPI - 1) {
#pragma unroll
          for (int rp = 0; rp < RPW; rp++) {
            r16[rp] = static_cast<_Float16>(across(rs_run[rp]));
            if (HAS_DIV) {
              normalise(rp, 0, 4 * (KB / 2), r16[rp]);
            }
          }
        }
        if (sidx == 0) {
#pragma unroll
          for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
            for (int t = 0; t < DB; t++) {
              o[rp][t] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
            }
          }
        }
#pragma unroll
        for (int jj = 0; jj < KB / 2; jj++) {
#pragma unroll
          for (int t = 0; t < DB; t++) {
#pragma unroll
            for (int rp = 0; rp < RPW; rp++) {
              uint4v const a = {pk[rp][jj][0], pk[rp][jj][1], pk[rp][jj][2], pk[rp][jj][3]};
              o[rp][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vb[t][jj], __builtin_bit_cast(half8, a),
                                                                o[rp][t], 0, 0, 0);
            }
          }
        }
        if (sidx == SPI - 1) {
#pragma unroll
          for (int rp = 0; rp < RPW; rp++) {
            store_result(0, rp, o[rp], r16[rp]);
          }
        }
      } else if (IPS == 2) {
        // two iterations of 32 keys: blocks {0, 1} and {2, 3}, one matrix instruction each
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
#pragma unroll
          for (int rp = 0; rp < RPW; rp++) {
            _Float16 const r16 = static_cast<_Float16>(across(row_sum(rp, 2 * sub, 2, 0.0f)));
            if (HAS_DIV) {
              normalise(rp, 4 * sub, 4, r16);
            }
            float4v res[DB];
            uint4v const a = {pk[rp][sub][0], pk[rp][sub][1], pk[rp][sub][2], pk[rp][sub][3]};
#pragma unroll
            for (int t = 0; t < DB; t++) {
              res[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vb[t][sub], __builtin_bit_cast(half8, a),
                                                              float4v{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
            }
            store_result(sub, rp, res, r16);
          }
        }
      } else {
        // four iterations of 16 keys: one block each, the 16-deep matrix instruction
#pragma unroll
        for (int sub = 0; sub < 4; sub++) {
#pragma unroll
          for (int rp = 0; rp < RPW; rp++) {
            _Float16 const r16 = static_cast<_Float16>(across(row_sum(rp, sub, 1, 0.0f)));
            if (HAS_DIV) {
              normalise(rp, 2 * sub, 2, r16);
            }
            float4v res[DB];
            uint2v const a = {pk[rp][sub / 2][2 * (sub & 1)], pk[rp][sub / 2][2 * (sub & 1) + 1]};
#pragma unroll
            for (int t = 0; t < DB; t++) {
              // rows 32 (sub / 2) + 16 (sub & 1) + 4g .. + 3 of V: the low or the high half of
              // the operand read for the pair of blocks
              half4 const vh = (sub & 1) ? __builtin_shufflevector(vb[t][sub / 2], vb[t][sub / 2], 4, 5, 6, 7)
                                         : __builtin_shufflevector(vb[t][sub / 2], vb[t][sub / 2], 0, 1, 2, 3);
              res[t] = __builtin_amdgcn_mfma_f32_16x16x16f16(vh, __builtin_bit_cast(half4, a),
                                                             float4v{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
            }
            store_result(sub, rp, res, r16);
          }
        }
      }
      // every operand of this buffer is in registers: the next strip this buffer serves goes
      // out now (behind the one already in flight when there are two buffers)
      if (q + NBUF < nstrips) {
        int const qn = q + NBUF;
        // (nothing of this strip may still be on its way out of LDS when the transfers that
        // overwrite the buffer are issued, and the compiler may not move them up among the
        // matrix instructions: the operand reads' completion is what it would move them past)
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        fetch(ip + (qn / SPI) * IP, qn % SPI, b);
      }
    }
  }
  if (TRACE) {
    t_computed = __builtin_amdgcn_s_memrealtime();
  }
  // ---- results to LDS: iteration it = ip + j IP goes to slot j of this wavefront's buffers --
#pragma unroll
  for (int j = 0; j < NIT; j++) {
    if (j < nit) {
#pragma unroll
      for (int sub = 0; sub < IPS; sub++) {
        _Float16 *slot = wbuf + (j * IPS + sub) * SLOT_HALFS;
#pragma unroll
        for (int rp = 0; rp < RPW; rp++) {
#pragma unroll
          for (int t = 0; t < DB; t++) {
            uint2v const w = {keep[j][sub][rp][2 * t], keep[j][sub][rp][2 * t + 1]};
            *reinterpret_cast<uint2v *>(slot + (16 * rp + c) * LDO + 16 * t + 4 * g) = w;
          }
          if (g == 0) {
            slot[ROWS * LDO + 16 * rp + c] = __builtin_bit_cast(half2v, keep[j][sub][rp][2 * DB])[0];
          }
        }
      }
    }
  }
  __syncthreads();
  if (TRACE) {
    t_joined = __builtin_amdgcn_s_memrealtime();
  }
  // ---- ordered accumulation: every thread owns EPT consecutive columns of one row; the
  // slots of up to four iterations are read before their (dependent) adds ---------------
  {
    // fp16 sums, two per register: adding two fp16 numbers with one packed fp16 add gives their
    // exact sum rounded once, which is what adding in fp32 and rounding to fp16 gives
    half2v acc[EPT / 2];
#pragma unroll
    for (int e = 0; e < EPT / 2; e++) {
      acc[e] = half2v{(_Float16)0.0f, (_Float16)0.0f};
    }
    _Float16 const *all = reinterpret_cast<_Float16 const *>(lds) + out_row * LDO + out_col;
    // iteration `it` is slice it % IPS of unit it / IPS, which wavefront unit % IP kept as its
    // result number unit / IP
    auto slot_of = [&](int it) {
      int const unit = it / IPS;
      return all + (unit % IP) * WAVE_HALFS + ((unit / IP) * IPS + it % IPS) * SLOT_HALFS;
    };
    // (a slot no iteration filled holds whatever the tiles left there: it is read, never added)
    constexpr bool ALL = NIT == 1 && IPS == 1;  // one slot per wavefront: read them all at once
    constexpr int BATCH = ALL ? IP : 4;
    int const it_end = ALL ? IP : F;
#pragma unroll
    for (int it0 = 0; it0 < it_end; it0 += BATCH) {
      half2v v[BATCH][EPT / 2];
#pragma unroll
      for (int u = 0; u < BATCH; u++) {
        _Float16 const *src = slot_of(ALL ? it0 + u : (it0 + u < F ? it0 + u : 0));
#pragma unroll
        for (int e = 0; e < EPT / 2; e++) {
          v[u][e] = *reinterpret_cast<half2v const *>(src + 2 * e);
        }
      }
#pragma unroll
      for (int u = 0; u < BATCH; u++) {
        if (it0 + u < F) {
#pragma unroll
          for (int e = 0; e < EPT / 2; e++) {
            acc[e] = acc[e] + v[u][e];
          }
        }
      }
    }
    if (out_row < rows) {
      half2v out[EPT / 2];
#pragma unroll
      for (int e = 0; e < EPT / 2; e++) {
        out[e] = acc[e];
      }
      if (EPT == 8) {
        uint4v const w = {__builtin_bit_cast(uint32_t, out[0]), __builtin_bit_cast(uint32_t, out[1]),
                          __builtin_bit_cast(uint32_t, out[(EPT / 2 > 2) ? 2 : 0]),
                          __builtin_bit_cast(uint32_t, out[(EPT / 2 > 3) ? 3 : 0])};
        *reinterpret_cast<uint4v *>(og) = w;
      } else if (EPT == 4) {
        uint2v const w = {__builtin_bit_cast(uint32_t, out[0]),
                          __builtin_bit_cast(uint32_t, out[(EPT / 2 > 1) ? 1 : 0])};
        *reinterpret_cast<uint2v *>(og) = w;
      } else {
        *reinterpret_cast<uint32_t *>(og) = __builtin_bit_cast(uint32_t, out[0]);
      }
    }
    if (!HAS_DIV && tid < rows) {
      _Float16 const *sums = reinterpret_cast<_Float16 const *>(lds) + ROWS * LDO + tid;
      float ra = 0.0f;
      for (int it = 0; it < F; it++) {
        int const unit = it / IPS;
        _Float16 const v = sums[(unit % IP) * WAVE_HALFS + ((unit / IP) * IPS + it % IPS) * SLOT_HALFS];
        ra = static_cast<float>(static_cast<_Float16>(ra + static_cast<float>(v)));
      }
      _Float16 *rgp = static_cast<_Float16 *>(const_cast<void *>(P.r.ptr)) +
                      tile_offset(P.r, bx, by, bz, 0);
      for (int c = 0; c < P.r_copies; c++) {
        rgp[(long long)(row_base + tid) * P.r.d_cols + c * P.r_copy_stride] = static_cast<_Float16>(ra);
      }
    }
  }
  if (TRACE && lane == 0) {
    // start, loads issued, first tile pair landed, arithmetic done, joined, stores issued
    unsigned const wg = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    unsigned long long *t = P.trace + ((size_t)wg * IP + ip) * 6;
    t[0] = t_start;
    t[1] = t_issued;
    t[2] = t_landed;
    t[3] = t_computed;
    t[4] = t_joined;
    t[5] = __builtin_amdgcn_s_memrealtime();
  }
}

}  // namespace mi355
