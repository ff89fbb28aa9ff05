// Fingerprint matmul on the matrix cores (reference src/kernel/cuda/matmul_kernel.cu:145-173
// computes `r = (r + a*b) % 25651` per multiply-accumulate in one thread per output; the
// thread-block form is include/mirage/threadblock/cuda/matmul.h:773-804).
//
// (sum a*b) mod 25651 is fixed by its residues mod 227 and mod 113.  Every operand is first
// split, once per matrix, into two planes of signed bytes: the residue mod 227 recentred to
// [-113, 113] and the residue mod 113; A keeps its orientation [rows][k], B is transposed
// to [columns][k], k padded with zeros to a multiple of 64.  Both operands of
// v_mfma_i32_16x16x64_i8 then want the same thing: 16 consecutive k of one row per lane,
// one 16-byte load.  Planes are stored in blocks of 16 rows x 16 k
// (plane[row / 16][k / 16][row % 16][16 bytes]), so the 64 loads of a wavefront's operand
// fetch are one contiguous kilobyte and a strip of 16 rows is one stream along k.  A
// 16 x 16 x 64 step per residue is one matrix instruction; the int32 sums are exact
// (|sum| <= 113^2 * k, folded every 131072 k) and are recombined once per output with the
// reference's CRT multipliers (fp_from_residue_sums), so results are bit-identical.
//
// Two users.  Kernel-level matmuls: one submission takes many independent ones (those of a
// batch of candidate graphs): one launch splits all operands, one launch multiplies; a
// workgroup owns a 64 x 64 output tile (each wavefront a 32 x 32 quadrant over all of k)
// when its matmul has enough tiles to matter, otherwise a 32 x 32 tile whose k range the
// four wavefronts share, added up through LDS.  Fused tiled-matmul plans of customized
// operators (load A tile, load B tile, [exp / silu of a tile], matmul, [exp / silu of the
// product], accumulate over the for-loop, store): the operand TENSORS are split once per
// launch and every logical block reads its tiles from the planes through the plan's own
// strides; see fp_mfma_gemm_block.
#include "common.h"
#include "tb_program.h"

// fp_mfma_matmul_big_kernel loads registers by inline assembly and waits for them later: code
// compiled without optimisation stores every such register to scratch memory right after the
// load is issued, before its data is there.  Refuse to build that.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__OPTIMIZE__)
#error "fp_mfma.hip must be compiled with optimisation (-O1 or higher): its asynchronous register loads do not survive -O0"
#endif

#include <algorithm>
#include <atomic>
#include <vector>

namespace mi355 {

namespace {

constexpr int kThreads = 256;
constexpr int kMaxJobs = MI355_MAX_MATMULS;
typedef int v4i __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

// residue mod 227 as a signed byte congruent to it, residue mod 113 as it is
__device__ __forceinline__ uint32_t byte_p(uint32_t x) {
  uint32_t const r = x % FP_P;
  return (r > 113u ? r + 29u : r) & 0xffu;  // r - 227 = r + 29 (mod 256)
}
__device__ __forceinline__ uint32_t byte_q(uint32_t x) { return x % FP_Q; }

struct SplitJob {
  uint16_t const *src;   // [slabs][rows][cols], row-major
  int8_t *plane_p, *plane_q;
  int slabs, rows, cols;
  int kp;                // padded k of the planes
  int rp;                // plane rows per slab (a multiple of 16)
  int transpose;         // 0: plane rows = source rows, k = cols; 1: plane rows = source columns, k = rows
  int vec;               // source rows may be read 8 (plain) / 4 (transposed) values at a time
  int unary;             // TB_EXP_OP / TB_SILU_OP applied to every value first, 0: none
  unsigned first_block, blocks;
};
constexpr int kSplitPrograms = 24;  // matmuls / programs per splitting launch (3 KB of arguments)
struct SplitMany {
  SplitJob job[2 * kSplitPrograms];
  int count;
  FpTables tables;
};

__device__ __forceinline__ uint32_t prologue(FpTables const &t, int unary, uint32_t x) {
  return unary == 0 ? x : (unary == TB_EXP_OP ? fp_exp_value(t, x) : fp_silu_value(t, x));
}

__global__ __launch_bounds__(kThreads) void fp_split_planes_kernel(SplitMany const S) {
  __shared__ uint32_t tile[2][64][17];
  int j = 0;
  while (j + 1 < S.count && blockIdx.x >= S.job[j + 1].first_block) {
    j++;
  }
  SplitJob const &J = S.job[j];
  unsigned const block = blockIdx.x - J.first_block;
  int const tid = threadIdx.x;
  if (!J.transpose) {
    // unit = 16 consecutive k of one plane row; the 16 rows of a block go to 16 neighbouring
    // threads, which write one contiguous 256-byte block
    // (32-bit index arithmetic: a plane has fewer than 2^31 bytes, so fewer than 2^27 units)
    unsigned const chunks = (unsigned)J.kp / 16u, strips = (unsigned)J.rp / 16u;
    unsigned const units = (unsigned)J.slabs * (unsigned)J.rp * chunks;
    for (unsigned u = block * kThreads + tid; u < units; u += J.blocks * kThreads) {
      int const r = (int)(u % 16u);
      unsigned const blk = u / 16u;              // (slab, strip, chunk)
      unsigned const strip = blk / chunks;       // over slabs * rp / 16
      int const c = (int)(blk - strip * chunks);
      int const slab = (int)(strip / strips);
      int const row = (int)(strip - (unsigned)slab * strips) * 16 + r;
      int const k0 = c * 16;
      uint32_t v[16];
      if (row < J.rows) {
        uint16_t const *src = J.src + ((size_t)slab * J.rows + row) * J.cols + k0;
        if (J.vec && k0 + 16 <= J.cols) {
          uint4v const lo = *reinterpret_cast<uint4v const *>(src);
          uint4v const hi = *reinterpret_cast<uint4v const *>(src + 8);
#pragma unroll
          for (int i = 0; i < 4; i++) {
            v[2 * i] = lo[i] & 0xffffu;
            v[2 * i + 1] = lo[i] >> 16;
            v[8 + 2 * i] = hi[i] & 0xffffu;
            v[8 + 2 * i + 1] = hi[i] >> 16;
          }
        } else {
#pragma unroll
          for (int i = 0; i < 16; i++) {
            v[i] = k0 + i < J.cols ? src[i] : 0u;
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < 16; i++) {
          v[i] = 0u;
        }
      }
      if (J.unary != 0 && row < J.rows) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
          v[i] = k0 + i < J.cols ? prologue(S.tables, J.unary, v[i]) : 0u;  // the padding stays zero
        }
      }
      uint4v p, q;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        p[w] = byte_p(v[4 * w]) | (byte_p(v[4 * w + 1]) << 8) | (byte_p(v[4 * w + 2]) << 16) |
               (byte_p(v[4 * w + 3]) << 24);
        q[w] = byte_q(v[4 * w]) | (byte_q(v[4 * w + 1]) << 8) | (byte_q(v[4 * w + 2]) << 16) |
               (byte_q(v[4 * w + 3]) << 24);
      }
      *reinterpret_cast<uint4v *>(J.plane_p + (size_t)u * 16) = p;  // u = ((strip * chunks + c) * 16 + r)
      *reinterpret_cast<uint4v *>(J.plane_q + (size_t)u * 16) = q;
    }
    return;
  }
  // transposed: tiles of 64 k (source rows) x 64 n (source columns) through LDS
  int const tiles_k = J.kp / 64, tiles_n = (J.cols + 63) / 64;
  int const tiles = J.slabs * tiles_k * tiles_n;
  int const kq = tid / 16, ng = tid % 16;      // patch read: k = 4 kq .. +3, n = 4 ng .. +3
  int const out_n = tid % 64, out_c = tid / 64;  // chunk written: row out_n, k = 16 out_c .. +15
  for (int t = block; t < tiles; t += J.blocks) {
    int const slab = t / (tiles_k * tiles_n);
    int const k0 = (t / tiles_n) % tiles_k * 64, n0 = (t % tiles_n) * 64;
    uint16_t const *src = J.src + (size_t)slab * J.rows * J.cols;
    uint32_t v[4][4];  // [k][n]
#pragma unroll
    for (int r = 0; r < 4; r++) {
      int const k = k0 + 4 * kq + r, n = n0 + 4 * ng;
      if (J.vec && k < J.rows && n + 4 <= J.cols) {
        uint2 const w = *reinterpret_cast<uint2 const *>(src + (size_t)k * J.cols + n);
        v[r][0] = w.x & 0xffffu;
        v[r][1] = w.x >> 16;
        v[r][2] = w.y & 0xffffu;
        v[r][3] = w.y >> 16;
      } else {
#pragma unroll
        for (int c = 0; c < 4; c++) {
          v[r][c] = (k < J.rows && n + c < J.cols) ? src[(size_t)k * J.cols + n + c] : 0u;
        }
      }
    }
    if (J.unary != 0) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
          bool const inside = k0 + 4 * kq + r < J.rows && n0 + 4 * ng + c < J.cols;
          v[r][c] = inside ? prologue(S.tables, J.unary, v[r][c]) : 0u;
        }
      }
    }
#pragma unroll
    for (int c = 0; c < 4; c++) {
      tile[0][4 * ng + c][kq] = byte_p(v[0][c]) | (byte_p(v[1][c]) << 8) | (byte_p(v[2][c]) << 16) |
                                (byte_p(v[3][c]) << 24);
      tile[1][4 * ng + c][kq] = byte_q(v[0][c]) | (byte_q(v[1][c]) << 8) | (byte_q(v[2][c]) << 16) |
                                (byte_q(v[3][c]) << 24);
    }
    __syncthreads();
    if (n0 + out_n < J.rp) {  // rows past the last column hold zeros
      size_t const strip = (size_t)slab * (J.rp / 16) + (n0 + out_n) / 16;
      size_t const at = ((strip * (J.kp / 16) + k0 / 16 + out_c) * 16 + out_n % 16) * 16;
      uint4v p, q;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        p[w] = tile[0][out_n][4 * out_c + w];
        q[w] = tile[1][out_n][4 * out_c + w];
      }
      *reinterpret_cast<uint4v *>(J.plane_p + at) = p;
      *reinterpret_cast<uint4v *>(J.plane_q + at) = q;
    }
    __syncthreads();
  }
}

struct GemmJob {
  int8_t const *a_p, *a_q;    // blocked planes, mp rows per batch
  int8_t const *bt_p, *bt_q;  // blocked planes, np rows per batch
  uint16_t *out;              // [batch][m][n]
  int batch, m, n, kp;
  int mp, np;                 // m, n rounded up to 16
  int shared_k;               // 1: 32 x 32 tile per workgroup, wavefronts share k
  int tiles_m, tiles_n;       // tiles of 32 (shared k), 64, or 128 (fp_mfma_matmul_big_kernel) rows / columns
  int xcd_order;              // see tile_of_workgroup
  uint32_t magic_per_batch, magic_width;  // division magics of tiles_m * tiles_n and 8 * tiles_n
  unsigned first_block;
};
struct GemmMany {
  GemmJob job[kMaxJobs];
  int count;
};
static_assert(sizeof(GemmMany) <= 4096, "kernel arguments are limited to 4 KB");

__device__ __forceinline__ int fold_signed(int v, int mod) { return v % mod; }

// Four consecutive outputs of row `row` from column `col` on, from their residue sums.
__device__ __forceinline__ void store_outputs(uint16_t *out, int m, int n, bool whole4, int row, int col,
                                              v4i const &sp, v4i const &sq) {
  if (row >= m || col >= n) {
    return;
  }
  uint32_t z[4];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    z[e] = fp_from_residue_sums(sp[e], sq[e]);
  }
  uint16_t *dst = out + (size_t)row * n + col;
  if (whole4 && (reinterpret_cast<uintptr_t>(dst) & 7) == 0) {
    uint2 w;
    w.x = z[0] | (z[1] << 16);
    w.y = z[2] | (z[3] << 16);
    *reinterpret_cast<uint2 *>(dst) = w;
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++) {
      if (col + e < n) {
        dst[e] = (uint16_t)z[e];
      }
    }
  }
}

// Workgroup t of a job -> (batch, tile row, tile column).  Workgroups go to the 8 XCDs round
// robin, so XCD x gets the contiguous range of positions [x * total / 8, ...) of the tile order:
// the tiles that run together on one XCD are neighbours and share operand strips in that XCD's
// L2.  The order walks eight tile rows at a time, column after column within them.  Divisions
// by the job's tile counts are multiply-highs with magics from the host (a workgroup's first
// loads wait for this arithmetic).  The host decides per job whether this order or the plain
// one (row after row) is used.
__device__ __forceinline__ void tile_of_workgroup(GemmJob const &J, unsigned t, int *b, int *tm, int *tn) {
  unsigned const per_batch = (unsigned)(J.tiles_m * J.tiles_n);
  if (!J.xcd_order) {
    *b = (int)(t / per_batch);
    t %= per_batch;
    *tm = (int)(t / (unsigned)J.tiles_n);
    *tn = (int)(t % (unsigned)J.tiles_n);
    return;
  }
  unsigned const total = per_batch * (unsigned)J.batch;
  unsigned const x = t % 8, slot = t / 8, base = total / 8, rem = total % 8;
  unsigned const pos = x * base + min(x, rem) + slot;
  unsigned const bb = J.magic_per_batch ? __umulhi(pos, J.magic_per_batch) : pos;
  unsigned const l = pos - bb * per_batch;
  unsigned const width = 8u * (unsigned)J.tiles_n;
  unsigned const group = __umulhi(l, J.magic_width), within = l - group * width;
  int const first = (int)group * 8, rows = min(J.tiles_m - first, 8);
  *b = (int)bb;
  if (rows == 8) {
    *tm = first + (int)(within & 7u);
    *tn = (int)(within >> 3);
  } else {  // the last rows of a tile count that is no multiple of eight
    *tm = first + (int)(within % (unsigned)rows);
    *tn = (int)(within / (unsigned)rows);
  }
}

__global__ __launch_bounds__(kThreads) void fp_mfma_matmul_kernel(GemmMany const G) {
  __shared__ int part[4][32][64];  // shared-k reduction: [wavefront][register][lane]
  int j = 0;
  while (j + 1 < G.count && blockIdx.x >= G.job[j + 1].first_block) {
    j++;
  }
  GemmJob const &J = G.job[j];
  int const tid = threadIdx.x, wave = tid / 64, lane = tid % 64, r = lane % 16, g = lane / 16;
  unsigned t = blockIdx.x - J.first_block;
  int const per_batch = J.tiles_m * J.tiles_n;
  int const steps = J.kp / 64;
  int b, row0, col0, s_begin, s_end;
  if (J.shared_k) {
    b = (int)(t / per_batch);
    t %= per_batch;
    row0 = (int)(t / J.tiles_n) * 32;
    col0 = (int)(t % J.tiles_n) * 32;
    s_begin = (int)((long long)steps * wave / 4);
    s_end = (int)((long long)steps * (wave + 1) / 4);
  } else {
    int tm, tn;
    tile_of_workgroup(J, t, &b, &tm, &tn);
    row0 = tm * 64 + (wave / 2) * 32;
    col0 = tn * 64 + (wave % 2) * 32;
    s_begin = 0;
    s_end = steps;
  }
  // a strip past the edge reads the last strip; its results are not stored
  size_t a_off[2], b_off[2];
  size_t const strip_bytes = (size_t)J.kp * 16;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    size_t const sa = ((size_t)b * J.mp + min(row0 + 16 * i, J.mp - 16)) / 16;
    size_t const sb = ((size_t)b * J.np + min(col0 + 16 * i, J.np - 16)) / 16;
    a_off[i] = sa * strip_bytes + g * 256 + r * 16;
    b_off[i] = sb * strip_bytes + g * 256 + r * 16;
  }
  // acc[res][i][jn]: rows of the MFMA result are columns of C (B^T is the first operand), so a
  // lane ends up with four consecutive columns of one row of C
  v4i acc[2][2][2];
#pragma unroll
  for (int e = 0; e < 8; e++) {
    acc[e / 4][(e / 2) % 2][e % 2] = v4i{0, 0, 0, 0};
  }
  // operands of two steps are in flight while a third is multiplied
  struct Operands {
    v4i ap[2], aq[2], bp[2], bq[2];
  } o0, o1;
  auto fetch = [&](Operands &o, int s) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      o.ap[i] = *reinterpret_cast<v4i const *>(J.a_p + a_off[i] + (size_t)s * 1024);
      o.aq[i] = *reinterpret_cast<v4i const *>(J.a_q + a_off[i] + (size_t)s * 1024);
      o.bp[i] = *reinterpret_cast<v4i const *>(J.bt_p + b_off[i] + (size_t)s * 1024);
      o.bq[i] = *reinterpret_cast<v4i const *>(J.bt_q + b_off[i] + (size_t)s * 1024);
    }
  };
  auto multiply = [&](Operands const &o, int s) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
#pragma unroll
      for (int jn = 0; jn < 2; jn++) {
        acc[0][i][jn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(o.bp[jn], o.ap[i], acc[0][i][jn], 0, 0, 0);
        acc[1][i][jn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(o.bq[jn], o.aq[i], acc[1][i][jn], 0, 0, 0);
      }
    }
    if (((s - s_begin) & 2047) == 2047) {  // 2048 steps x 64 k x 113^2 < 2^31
#pragma unroll
      for (int i = 0; i < 2; i++) {
#pragma unroll
        for (int jn = 0; jn < 2; jn++) {
#pragma unroll
          for (int e = 0; e < 4; e++) {
            acc[0][i][jn][e] = fold_signed(acc[0][i][jn][e], (int)FP_P);
            acc[1][i][jn][e] = fold_signed(acc[1][i][jn][e], (int)FP_Q);
          }
        }
      }
    }
  };
  if (s_begin < s_end) {
    fetch(o0, s_begin);
  }
  if (s_begin + 1 < s_end) {
    fetch(o1, s_begin + 1);
  }
  for (int s = s_begin; s < s_end; s += 2) {
    multiply(o0, s);
    if (s + 2 < s_end) {
      fetch(o0, s + 2);
    }
    if (s + 1 < s_end) {
      multiply(o1, s + 1);
      if (s + 3 < s_end) {
        fetch(o1, s + 3);
      }
    }
  }
  uint16_t *out = J.out + (size_t)b * J.m * J.n;
  bool const whole4 = J.n % 4 == 0;
  auto store = [&](int i, int jn, v4i const &sp, v4i const &sq) {
    store_outputs(out, J.m, J.n, whole4, row0 + 16 * i + r, col0 + 16 * jn + 4 * g, sp, sq);
  };
  if (!J.shared_k) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
#pragma unroll
      for (int jn = 0; jn < 2; jn++) {
        store(i, jn, acc[0][i][jn], acc[1][i][jn]);
      }
    }
    return;
  }
  // shared k: every wavefront leaves its folded sums, wavefront w finishes sub-tile w
#pragma unroll
  for (int i = 0; i < 2; i++) {
#pragma unroll
    for (int jn = 0; jn < 2; jn++) {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        part[wave][(i * 2 + jn) * 8 + e][lane] = fold_signed(acc[0][i][jn][e], (int)FP_P);
        part[wave][(i * 2 + jn) * 8 + 4 + e][lane] = fold_signed(acc[1][i][jn][e], (int)FP_Q);
      }
    }
  }
  __syncthreads();
  v4i sp = {0, 0, 0, 0}, sq = {0, 0, 0, 0};
#pragma unroll
  for (int w = 0; w < 4; w++) {
#pragma unroll
    for (int e = 0; e < 4; e++) {
      sp[e] += part[w][wave * 8 + e][lane];
      sq[e] += part[w][wave * 8 + 4 + e][lane];
    }
  }
  store(wave / 2, wave % 2, sp, sq);
}

// ---- large kernel-level matmuls: 128 x 128 tiles, operand strips shared through LDS ------
// Every lane fetches 16 bytes from `gbase` (wave-uniform) + its own byte offset; the wavefront's
// 64 chunks land in LDS at `lds_wave_base` + 16 * lane without passing through registers
// (completion is counted by vmcnt).  Inline assembly so that the compiler does not make the
// next LDS read wait for the transfer; the caller waits before the barrier that publishes it.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void plane_dma16(int8_t const *gbase, uint32_t lane_byte_offset,
                                            uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_wave_base)), "v"(lane_byte_offset), "s"(gbase)
               : "m0", "memory");
}
#pragma clang diagnostic pop

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
// A 16-byte load whose latency the compiler knows nothing of: `dst` holds the data only after
// landed<N>() on it (N = transfers issued after this one that may still be in flight).  Both
// stand in the same straight-line piece of code, so the compiler has no reason to move or
// copy `dst` in between, and only landed values are carried round a loop.  A kernel that uses
// this must not spill registers (a spill of `dst` before its wait would save stale data): the
// one below builds with 235 vector registers and no scratch memory.
__device__ __forceinline__ void plane_load16(v4i &dst, int8_t const *gbase, uint32_t lane_byte_offset) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(lane_byte_offset), "s"(gbase) : "memory");
}
template <int N>
__device__ __forceinline__ void landed(v4i (&b)[4]) {
  asm volatile("s_waitcnt vmcnt(%4)" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void landed(v4i (&b)[2]) {
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(b[0]), "+v"(b[1]) : "n"(N) : "memory");
}
#pragma clang diagnostic pop

constexpr int kBigStage = 16384;  // A of one 64-k step: (mod 227, mod 113) x 8 strips x 1 KB
constexpr int kBigStages = 4;
constexpr int kBigLdsBytes = kBigStages * kBigStage;
constexpr long long kBigMinTiles = 256;  // tiles of fp_mfma_matmul_big_kernel from here on (256 compute units)
constexpr int kBigMaxK = 2048 * 64;

// A workgroup owns a 128 x TN output tile, TN = 128 or (for matmuls with too few of those) 64;
// wavefront w works in one residue field (w & 1) on one half of the tile's columns (w >> 1):
// with TN = 128, 128 x 64 sums and 32 matrix instructions per step of 64 k.  Operand blocks are 1 KB (16 plane rows x 64 k, contiguous in the blocked planes, lane
// l's operand of v_mfma_i32_16x16x64_i8 is bytes [16 l, 16 l + 16) of it).  The 16 A blocks of
// a step (8 row strips x 2 residues) are needed by two wavefronts each: they are copied to LDS
// three steps ahead (four stages of 16 KB), 4 transfers per wavefront, and read from there one
// step ahead.  The 4 B^T blocks a wavefront needs are needed by nobody else: it loads them
// straight into registers, one step ahead.  Against one 64 x 64 tile per workgroup with
// operands read straight from L2 by every wavefront, a tile's operands cross L2 -> compute
// unit once per 128 x 128 instead of once per 32 x 32 quadrant.  Two workgroups per compute
// unit.  The host sends matmuls of at most kBigMaxK k here: 2048 steps x 64 k x 113^2 < 2^31,
// so the int32 sums need no fold on the way.
template <int TN>  // columns of the tile: 128 or 64
__global__ __launch_bounds__(kThreads, 2) void fp_mfma_matmul_big_kernel(GemmMany const G) {
  constexpr int NB = TN / 32;  // B^T blocks (16 columns each) per wavefront
  extern __shared__ __attribute__((aligned(16))) int8_t big_lds[];
  int j = 0;
  while (j + 1 < G.count && blockIdx.x >= G.job[j + 1].first_block) {
    j++;
  }
  GemmJob const &J = G.job[j];
  int const tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
  int const r = lane % 16, g = lane / 16;
  int const res = wave & 1, half = wave >> 1;
  int b, tm, tn;
  tile_of_workgroup(J, blockIdx.x - J.first_block, &b, &tm, &tn);
  int const row0 = tm * 128, col0 = tn * TN + half * (TN / 2);
  int const steps = J.kp / 64;
  uint32_t const strip_bytes = (uint32_t)J.kp * 16u;
  // this wavefront copies 4 of the 16 A blocks of a step: residue wave / 2, strips 4 (wave % 2) ..
  int8_t const *a_plane = (wave / 2 == 0 ? J.a_p : J.a_q) + (size_t)b * (size_t)J.mp * (size_t)J.kp;
  int8_t const *b_plane = (res == 0 ? J.bt_p : J.bt_q) + (size_t)b * (size_t)J.np * (size_t)J.kp;
  uint32_t a_off[4], b_off[NB];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a_off[i] = (uint32_t)(min(row0 + 16 * ((wave % 2) * 4 + i), J.mp - 16) / 16) * strip_bytes + (uint32_t)lane * 16u;
  }
#pragma unroll
  for (int i = 0; i < NB; i++) {
    b_off[i] = (uint32_t)(min(col0 + 16 * i, J.np - 16) / 16) * strip_bytes + (uint32_t)lane * 16u;
  }
  uint32_t const lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void const *)big_lds;
  // Transfers are issued for every step up to three past the last one (the last step's data
  // again, into a stage / registers nobody reads any more): the queue of outstanding transfers
  // then looks the same at every wait and the waits need no conditions.
  auto issue_a = [&](int s) {
    int8_t const *src = a_plane + (size_t)min(s, steps - 1) * 1024;
    uint32_t const dst = lds0 + (uint32_t)((s % kBigStages) * kBigStage + wave * 4096);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      plane_dma16(src, a_off[i], dst + (uint32_t)i * 1024u);
    }
  };
  auto issue_b = [&](int s, v4i (&buf)[NB]) {
    int8_t const *src = b_plane + (size_t)min(s, steps - 1) * 1024;
#pragma unroll
    for (int i = 0; i < NB; i++) {
      plane_load16(buf[i], src, b_off[i]);
    }
  };
  v4i acc[8][NB];
#pragma unroll
  for (int e = 0; e < 8 * NB; e++) {
    acc[e / NB][e % NB] = v4i{0, 0, 0, 0};
  }
  // A: three steps ahead through the four LDS stages.  B^T: one step ahead in registers; a
  // load and the wait for it stand in the same iteration, and only values that have landed
  // are carried round the loop (the compiler knows nothing of the loads' latency).
  v4i cur[NB], next[NB], a[8], a_next[8];
  issue_a(0);
  issue_a(1);
  issue_b(0, cur);
  issue_a(2);
  landed<4>(cur);  // A(0), A(1) and B(0) are there; A(2) may still be on its way
  __syncthreads();
  {
    int8_t const *stage = big_lds + res * 8192 + lane * 16;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      a[i] = *reinterpret_cast<v4i const *>(stage + i * 1024);
    }
  }
  // one step: multiplies (a_now, b_now) while the next step's operands arrive in (a_new, b_new);
  // the loop runs it twice with the register sets swapped, so nothing is copied
  auto step = [&](int s, v4i (&a_now)[8], v4i (&b_now)[NB], v4i (&a_new)[8], v4i (&b_new)[NB]) {
    if (s > 0) {
      __syncthreads();  // A(s + 1) is in LDS; everyone has the stage of step s - 1 in registers
    }
    issue_b(s + 1, b_new);
    issue_a(s + 3);
    int8_t const *stage = big_lds + ((s + 1) % kBigStages) * kBigStage + res * 8192 + lane * 16;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      a_new[i] = *reinterpret_cast<v4i const *>(stage + i * 1024);
    }
    __builtin_amdgcn_sched_barrier(0);  // the next step's operands are on their way before ...
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
      for (int jn = 0; jn < NB; jn++) {
        acc[i][jn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b_now[jn], a_now[i], acc[i][jn], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);  // ... this step's products, and awaited after them
    landed<4>(b_new);  // B(s + 1) and, issued before it, A(s + 2)
  };
  for (int s = 0; s < steps; s += 2) {
    step(s, a, cur, a_next, next);
    if (s + 1 < steps) {
      step(s + 1, a_next, next, a, cur);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the transfers past the last step
  // The two wavefronts of a column half hold the sums mod 227 and mod 113 of the same outputs:
  // each hands the other one half of its rows (through LDS, lane for lane) and finishes the half
  // it keeps.
  __syncthreads();
  v4i *mine = reinterpret_cast<v4i *>(big_lds) + wave * 1024, *theirs = reinterpret_cast<v4i *>(big_lds) + (wave ^ 1) * 1024;
  // (row strips 4 - 7 given away by the mod 227 wavefront, 0 - 3 by the mod 113 one; written
  // with constant register indices under a wave-uniform branch)
  if (res == 0) {
#pragma unroll
    for (int e = 0; e < 4 * NB; e++) {
      mine[e * 64 + lane] = acc[4 + e / NB][e % NB];
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4 * NB; e++) {
      mine[e * 64 + lane] = acc[e / NB][e % NB];
    }
  }
  __syncthreads();
  uint16_t *out = J.out + (size_t)b * J.m * J.n;
  bool const whole4 = J.n % 4 == 0;
  if (res == 0) {
#pragma unroll
    for (int e = 0; e < 4 * NB; e++) {
      store_outputs(out, J.m, J.n, whole4, row0 + (e / NB) * 16 + r, col0 + (e % NB) * 16 + 4 * g,
                    acc[e / NB][e % NB], theirs[e * 64 + lane]);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4 * NB; e++) {
      store_outputs(out, J.m, J.n, whole4, row0 + (4 + e / NB) * 16 + r, col0 + (e % NB) * 16 + 4 * g,
                    theirs[e * 64 + lane], acc[4 + e / NB][e % NB]);
    }
  }
}

// ---- fused tiled-matmul plans (load A tile, load B tile, matmul, accumulate, store) -------
// One workgroup: logical block (bx, by, bz), part `split` of the for-loop.  The for-loop's
// k tiles, 16 k at a time, form one sequence of chunks; a matrix instruction takes four
// of them (one per 16-lane group), so tiles of 16 or 32 k pair up across iterations.  Tile
// origins come from the plan's own strides, as byte strides into the blocked planes.  A
// wavefront owns 32 x 32 outputs at a time; a tile with fewer than three such pieces shares
// its chunk sequence between wavefronts and adds their sums through `part`.  (bx, by) is the
// first of pl_group[0] x pl_group[1] logical blocks whose tiles the workgroup treats as one
// tile of gy * m rows and gx * n columns: strip s of its rows belongs to block by + s / (m / 16).
template <bool EPI>  // an operator is applied to every iteration's product
__device__ __forceinline__ void fp_mfma_gemm_block(DevProgram const &P, FpTables const &tbl, int *part,
                                                   uint16_t const *exp_lds, int bx, int by, int bz,
                                                   int split) {
  // Everything read from the program record is the same for all lanes; in a multi-program launch
  // the record sits in LDS, where the compiler cannot know that, so the values are made scalar
  // here (`uni`) and the address arithmetic below runs on the scalar unit.  Divisions are 32-bit
  // (products of loop counts and split numbers are small) or multiply-highs with host magics.
  auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
  auto uni_ptr = [](auto *ptr) {
    unsigned long long const v = reinterpret_cast<unsigned long long>(ptr);
    unsigned const lo = __builtin_amdgcn_readfirstlane((unsigned)v);
    unsigned const hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return reinterpret_cast<decltype(ptr)>(((unsigned long long)hi << 32) | lo);
  };
  auto udiv = [](unsigned v, uint32_t magic) { return magic == 0 ? v : __umulhi(v, magic); };
  DevOp const &la = P.ops[P.fg[0]], &lb = P.ops[P.fg[1]], &so = P.ops[P.num_ops - 1];
  int const bm = uni(P.t[la.dst].rows), kt = uni(P.t[la.dst].cols), bn = uni(P.t[lb.dst].cols);
  int const group_x = uni(P.pl_group[0]), group_y = uni(P.pl_group[1]);
  int const m = bm * group_y, n = bn * group_x;    // the grouped tile
  int const spb_m = bm / 16, spb_n = bn / 16;      // strips per block
  uint32_t const magic_m = (uint32_t)uni((int)P.pl_magic[0]), magic_n = (uint32_t)uni((int)P.pl_magic[1]);
  int const cpi = kt / 16;  // chunks per iteration
  int const F = uni(P.forloop_range), splits = uni(P.splits);
  bx = uni(bx);
  by = uni(by);
  bz = uni(bz);
  split = uni(split);
  int const it_begin = (int)((unsigned)(F * split) / (unsigned)splits);
  int const it_end = (int)((unsigned)(F * (split + 1)) / (unsigned)splits);
  // An operator applied to every iteration's product: an iteration is a whole number of steps
  // (k tiles of 16, 32 or 48 take one step in which only the first one, two or three lane
  // groups hold a chunk; longer k tiles are multiples of 64); after its last step the two sums
  // become a fingerprint value, the operator is applied and the result added to a running sum.
  int const epi = EPI ? uni(P.fp_unary[2]) : 0;
  int const cps = EPI && cpi < 4 ? cpi : 4;  // chunks per step
  int const spi = EPI && cpi >= 4 ? cpi / 4 : 1;    // steps per iteration (with an operator)
  int const Q = (it_end - it_begin) * cpi, steps = (Q + cps - 1) / cps;
  int const tid = threadIdx.x, wave = uni(tid / 64), lane = tid % 64, r = lane % 16, g = lane / 16;
  int const pl_a0 = uni(P.pl_a[0]), pl_a1 = uni(P.pl_a[1]), pl_a2 = uni(P.pl_a[2]), pl_a3 = uni(P.pl_a[3]),
            pl_a4 = uni(P.pl_a[4]);
  int const pl_b0 = uni(P.pl_b[0]), pl_b1 = uni(P.pl_b[1]), pl_b2 = uni(P.pl_b[2]), pl_b3 = uni(P.pl_b[3]),
            pl_b4 = uni(P.pl_b[4]);
  int const a0 = bx * pl_a0 + by * pl_a1 + bz * pl_a2 + it_begin * pl_a3;
  int const b0 = bx * pl_b0 + by * pl_b1 + bz * pl_b2 + it_begin * pl_b3;
  int const a_it = pl_a3, b_it = pl_b3;
  int const dq_it = cps / cpi, dq_c = cps % cpi;
  int const mt_n = (n + 31) / 32, mt = ((m + 31) / 32) * mt_n;
  int const ways_log2 = mt >= 3 ? 0 : (mt == 2 ? 1 : 2);  // wavefronts sharing one piece's chunks
  int const ways = 1 << ways_log2;
  int const so_io = uni(so.io);
  uint16_t *const gout = uni_ptr(splits > 1 ? P.part[so_io] + (long long)split * P.part_stride[so_io]
                                            : static_cast<uint16_t *>(P.out[so_io]));
  // element offset of the output tile of logical block (bx + dx, by + dy, bz): linear in the
  // block coordinates
  int const so_cols = uni(so.d_cols);
  long long const o_x = uni(so.g_bs[0]) + (long long)uni(so.row_bs[0]) * so_cols + uni(so.col_bs[0]);
  long long const o_y = uni(so.g_bs[1]) + (long long)uni(so.row_bs[1]) * so_cols + uni(so.col_bs[1]);
  long long const o_z = uni(so.g_bs[2]) + (long long)uni(so.row_bs[2]) * so_cols + uni(so.col_bs[2]);
  long long const o_base = bx * o_x + by * o_y + bz * o_z;
  auto out_origin = [&](int dx, int dy) { return o_base + dx * o_x + dy * o_y; };
  int8_t const *const pa = uni_ptr(P.pl[0]), *const qa = uni_ptr(P.pl[1]), *const pb = uni_ptr(P.pl[2]),
                      *const qb = uni_ptr(P.pl[3]);
  for (int t = wave >> ways_log2; t < mt; t += 4) {
    int const ks = wave & (ways - 1);
    // wavefronts that share a piece split its steps, by whole iterations if there is an
    // operator on the products
    int const units = EPI ? it_end - it_begin : steps, per_unit = EPI ? spi : 1;
    int const s_begin = ((units * ks) >> ways_log2) * per_unit;
    int const s_end = ((units * (ks + 1)) >> ways_log2) * per_unit;
    int const t_row = (int)((unsigned)t / (unsigned)mt_n);
    int const row_m = t_row * 32, col_n = (t - t_row * mt_n) * 32;
    int const i1 = row_m + 16 < m ? 1 : 0, j1 = col_n + 16 < n ? 1 : 0;
    int a_base[2], b_base[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
      int const sa = row_m / 16 + (i ? i1 : 0), sb = col_n / 16 + (i ? j1 : 0);
      int const sa_blk = (int)udiv((unsigned)sa, magic_m), sb_blk = (int)udiv((unsigned)sb, magic_n);
      a_base[i] = a0 + sa_blk * pl_a1 + (sa - sa_blk * spb_m) * pl_a4 + r * 16;
      b_base[i] = b0 + sb_blk * pl_b0 + (sb - sb_blk * spb_n) * pl_b4 + r * 16;
    }
    // this lane's chunk of step s: number cps s + g of the sequence (none if g >= cps)
    int q = cps * s_begin + g;
    int itr = (int)((unsigned)(cps * s_begin) / (unsigned)cpi), c = cps * s_begin - itr * cpi + g;
#pragma unroll
    for (int wrap = 0; wrap < 4; wrap++) {  // g <= 3 chunks further on
      if (c >= cpi) {
        c -= cpi;
        itr++;
      }
    }
    // operands of two steps are in flight while a third is multiplied
    struct Operands {
      v4i ap[2], aq[2], bp[2], bq[2];
    } o0, o1;
    auto fetch = [&](Operands &o) {
      bool const valid = g < cps && q < Q;
      int const oa = itr * a_it + c * 256, ob = itr * b_it + c * 256;
      v4i const zero = {0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < 2; i++) {
        o.ap[i] = valid ? *reinterpret_cast<v4i const *>(pa + a_base[i] + oa) : zero;
        o.aq[i] = valid ? *reinterpret_cast<v4i const *>(qa + a_base[i] + oa) : zero;
        o.bp[i] = valid ? *reinterpret_cast<v4i const *>(pb + b_base[i] + ob) : zero;
        o.bq[i] = valid ? *reinterpret_cast<v4i const *>(qb + b_base[i] + ob) : zero;
      }
      q += cps;
      itr += dq_it;
      c += dq_c;
      if (c >= cpi) {
        c -= cpi;
        itr++;
      }
    };
    v4i acc[2][2][2];
#pragma unroll
    for (int e = 0; e < 8; e++) {
      acc[e / 4][(e / 2) % 2][e % 2] = v4i{0, 0, 0, 0};
    }
    uint32_t run[4][4];  // running sums of the operator's results, [2 i + jn][e]
#pragma unroll
    for (int e = 0; e < 16; e++) {
      run[e / 4][e % 4] = 0;
    }
    int until = spi, folds = 0;
    auto multiply = [&](Operands const &o, int s) {
#pragma unroll
      for (int i = 0; i < 2; i++) {
#pragma unroll
        for (int jn = 0; jn < 2; jn++) {
          acc[0][i][jn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(o.bp[jn], o.ap[i], acc[0][i][jn], 0, 0, 0);
          acc[1][i][jn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(o.bq[jn], o.aq[i], acc[1][i][jn], 0, 0, 0);
        }
      }
      if constexpr (EPI) {
        if (--until == 0) {  // the iteration's product is complete
          until = spi;
          bool const fold = (++folds & 32767) == 0;  // 32768 values below 25651 fit 32 bits
#pragma unroll
          for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int jn = 0; jn < 2; jn++) {
#pragma unroll
              for (int e = 0; e < 4; e++) {
                uint32_t &sum = run[2 * i + jn][e];
                if (epi == TB_EXP_OP) {
                  // exp reads only the value's residue modulo 113, which is the second sum's
                  sum += exp_lds[static_cast<uint32_t>(acc[1][i][jn][e]) % FP_Q];
                } else {
                  sum += fp_silu_value(tbl, fp_from_residue_sums(acc[0][i][jn][e], acc[1][i][jn][e]));
                }
                sum = fold ? sum % FP_PQ : sum;
                acc[0][i][jn][e] = 0;
                acc[1][i][jn][e] = 0;
              }
            }
          }
        }
      } else if (((s - s_begin) & 2047) == 2047) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
          for (int jn = 0; jn < 2; jn++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
              acc[0][i][jn][e] = fold_signed(acc[0][i][jn][e], (int)FP_P);
              acc[1][i][jn][e] = fold_signed(acc[1][i][jn][e], (int)FP_Q);
            }
          }
        }
      }
    };
    if (s_begin < s_end) {
      fetch(o0);
    }
    if (s_begin + 1 < s_end) {
      fetch(o1);
    }
    for (int s = s_begin; s < s_end; s += 2) {
      multiply(o0, s);
      if (s + 2 < s_end) {
        fetch(o0);
      }
      if (s + 1 < s_end) {
        multiply(o1, s + 1);
        if (s + 3 < s_end) {
          fetch(o1);
        }
      }
    }
    auto store_values = [&](int i, int jn, uint32_t const (&z)[4]) {
      if (i > i1 || jn > j1) {
        return;
      }
      uint2 w;
      w.x = z[0] | (z[1] << 16);
      w.y = z[2] | (z[3] << 16);
      // strip -> logical block of the grouped tile by multiply-high (magics from the host)
      int const srow = row_m / 16 + i, scol = col_n / 16 + jn;
      int const dy = (int)udiv((unsigned)srow, magic_m), dx = (int)udiv((unsigned)scol, magic_n);
      int const row = (srow - dy * spb_m) * 16 + r, col = (scol - dx * spb_n) * 16 + 4 * g;
      *reinterpret_cast<uint2 *>(gout + out_origin(dx, dy) + (long long)row * so_cols + col) = w;
    };
    auto store = [&](int i, int jn, v4i const &sp, v4i const &sq) {
      uint32_t z[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        z[e] = fp_from_residue_sums(sp[e], sq[e]);
      }
      store_values(i, jn, z);
    };
    if constexpr (EPI) {
      // the running sums are fingerprint values already
      if (ways > 1 && ks != 0) {
#pragma unroll
        for (int e = 0; e < 16; e++) {
          part[(wave * 32 + e) * 64 + lane] = (int)(run[e / 4][e % 4] % FP_PQ);
        }
      }
      if (ways > 1) {
        __syncthreads();
      }
      if (ks == 0) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
          for (int jn = 0; jn < 2; jn++) {
            uint32_t z[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
              z[e] = run[2 * i + jn][e] % FP_PQ;
            }
            for (int w = 1; w < ways; w++) {
#pragma unroll
              for (int e = 0; e < 4; e++) {
                z[e] += (uint32_t)part[((wave + w) * 32 + (2 * i + jn) * 4 + e) * 64 + lane];
              }
            }
#pragma unroll
            for (int e = 0; e < 4; e++) {
              z[e] %= FP_PQ;
            }
            store_values(i, jn, z);
          }
        }
      }
      continue;
    }
    if (ways == 1) {
#pragma unroll
      for (int i = 0; i < 2; i++) {
#pragma unroll
        for (int jn = 0; jn < 2; jn++) {
          store(i, jn, acc[0][i][jn], acc[1][i][jn]);
        }
      }
      continue;
    }
    // shared chunk sequence: every wavefront but the piece's first leaves its folded sums
    if (ks != 0) {
#pragma unroll
      for (int i = 0; i < 2; i++) {
#pragma unroll
        for (int jn = 0; jn < 2; jn++) {
#pragma unroll
          for (int e = 0; e < 4; e++) {
            part[(wave * 32 + (i * 2 + jn) * 8 + e) * 64 + lane] = fold_signed(acc[0][i][jn][e], (int)FP_P);
            part[(wave * 32 + (i * 2 + jn) * 8 + 4 + e) * 64 + lane] = fold_signed(acc[1][i][jn][e], (int)FP_Q);
          }
        }
      }
    }
    __syncthreads();
    if (ks == 0) {
#pragma unroll
      for (int i = 0; i < 2; i++) {
#pragma unroll
        for (int jn = 0; jn < 2; jn++) {
          v4i sp, sq;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            sp[e] = fold_signed(acc[0][i][jn][e], (int)FP_P);
            sq[e] = fold_signed(acc[1][i][jn][e], (int)FP_Q);
          }
          for (int w = 1; w < ways; w++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
              sp[e] += part[((wave + w) * 32 + (i * 2 + jn) * 8 + e) * 64 + lane];
              sq[e] += part[((wave + w) * 32 + (i * 2 + jn) * 8 + 4 + e) * 64 + lane];
            }
          }
          store(i, jn, sp, sq);
        }
      }
    }
  }
}

// exp table premultiplied by the CRT lift, as exp_fp(x) = (3^(x mod 113) * 25425) mod 25651
__device__ __forceinline__ void load_exp_table(FpTables const &tbl, uint16_t *exp_lds) {
  if (threadIdx.x < FP_Q) {
    exp_lds[threadIdx.x] = static_cast<uint16_t>((tbl.exp_tbl[threadIdx.x] * FP_Q_MUL_P_MOD_1) % FP_PQ);
  }
  __syncthreads();
}

__global__ __launch_bounds__(kThreads) void fp_mfma_gemm_kernel(DevProgram const P, FpTables const tbl) {
  __shared__ int part[kFpMfmaLdsBytes / 4];
  __shared__ uint16_t exp_lds[128];
  if (P.fp_unary[2] == TB_EXP_OP) {
    load_exp_table(tbl, exp_lds);
  }
  int const gx = P.grid[0] / P.pl_group[0];
  if (P.fp_unary[2] != 0) {
    fp_mfma_gemm_block<true>(P, tbl, part, exp_lds, (blockIdx.x % gx) * P.pl_group[0], blockIdx.y * P.pl_group[1],
                             blockIdx.z, blockIdx.x / gx);
  } else {
    fp_mfma_gemm_block<false>(P, tbl, part, exp_lds, (blockIdx.x % gx) * P.pl_group[0], blockIdx.y * P.pl_group[1],
                              blockIdx.z, blockIdx.x / gx);
  }
}

// Many programs in one launch: workgroup -> program by a prefix table, the program record
// copied to LDS above the wavefront sums.
__global__ __launch_bounds__(kThreads) void fp_mfma_gemm_multi_kernel(
    DevProgram const *__restrict__ progs, int const *__restrict__ first_block, int n,
    FpTables const tbl) {
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
  uint4v *dst = reinterpret_cast<uint4v *>(lds + kFpMfmaLdsBytes);
  for (int i = threadIdx.x; i < (int)(sizeof(DevProgram) / 16); i += kThreads) {
    dst[i] = src[i];
  }
  __syncthreads();
  DevProgram const &P = *reinterpret_cast<DevProgram const *>(lds + kFpMfmaLdsBytes);
  uint16_t *exp_lds = reinterpret_cast<uint16_t *>(lds + kFpMfmaLdsBytes + sizeof(DevProgram));
  if (P.fp_unary[2] == TB_EXP_OP) {
    load_exp_table(tbl, exp_lds);
  }
  int v = w - first_block[lo];
  int const gx = P.grid[0] / P.pl_group[0], gy = P.grid[1] / P.pl_group[1];
  int const x = v % (gx * P.splits);
  v /= gx * P.splits;
  if (P.fp_unary[2] != 0) {
    fp_mfma_gemm_block<true>(P, tbl, reinterpret_cast<int *>(lds), exp_lds, (x % gx) * P.pl_group[0],
                             (v % gy) * P.pl_group[1], v / gy, x / gx);
  } else {
    fp_mfma_gemm_block<false>(P, tbl, reinterpret_cast<int *>(lds), exp_lds, (x % gx) * P.pl_group[0],
                              (v % gy) * P.pl_group[1], v / gy, x / gx);
  }
}

inline size_t round_up(size_t v, size_t to) { return (v + to - 1) / to * to; }

}  // namespace

// Splitting launches for `count` jobs (their first_block fields are filled in here).
static int launch_split_jobs(SplitJob *jobs, int count, hipStream_t stream) {
  for (int done = 0; done < count; done += 2 * kSplitPrograms) {
    int const group = std::min(count - done, 2 * kSplitPrograms);
    SplitMany S{};
    unsigned blocks = 0;
    for (int j = 0; j < group; j++) {
      jobs[done + j].first_block = blocks;
      blocks += jobs[done + j].blocks;
      S.job[j] = jobs[done + j];
    }
    S.count = group;
    S.tables = tables();
    fp_split_planes_kernel<<<blocks, kThreads, 0, stream>>>(S);
    MI355_HIP(hipGetLastError());
  }
  return MI355_OK;
}

// Whether one matmul can take the matrix-core path, and the bytes of planes it needs.
static bool mfma_matmul_fits(int batch, int m, int n, int k, size_t *plane_bytes) {
  if (batch <= 0 || m <= 0 || n <= 0 || k <= 0) {
    return false;
  }
  size_t const kp = round_up((size_t)k, 64);
  size_t const rows = (size_t)batch * (round_up((size_t)m, 16) + round_up((size_t)n, 16));
  if (rows * kp > ((size_t)1 << 31)) {
    return false;
  }
  *plane_bytes = 2 * rows * kp;  // two residues; every plane is a multiple of 64 bytes
  return true;
}

// Enqueues matmuls [0, count) whose planes fit the queue's plane memory together.
static int launch_mfma_group(uint16_t const *const *A, uint16_t const *const *B, uint16_t *const *C,
                             int const *batch, int const *m, int const *n, int const *k, int count) {
  std::vector<SplitJob> jobs((size_t)(2 * count));
  GemmMany G{}, Big{}, Narrow{};  // jobs of the 64 x 64 / 32 x 32 kernel, of the 128 x 128 and 128 x 64 kernels
  char *planes = state().planes();
  size_t used = 0;
  unsigned gemm_blocks = 0, big_blocks = 0, narrow_blocks = 0;
  for (int e = 0; e < count; e++) {
    int const kp = (int)round_up((size_t)k[e], 64);
    int const mp = (int)round_up((size_t)m[e], 16), np = (int)round_up((size_t)n[e], 16);
    size_t const a_plane = (size_t)batch[e] * mp * kp, b_plane = (size_t)batch[e] * np * kp;
    int8_t *a_p = reinterpret_cast<int8_t *>(planes + used);
    int8_t *a_q = a_p + a_plane;
    int8_t *bt_p = a_q + a_plane;
    int8_t *bt_q = bt_p + b_plane;
    used += 2 * (a_plane + b_plane);
    SplitJob &sa = jobs[(size_t)(2 * e)], &sb = jobs[(size_t)(2 * e + 1)];
    sa = SplitJob{};
    sb = SplitJob{};
    sa.src = A[e];
    sa.plane_p = a_p;
    sa.plane_q = a_q;
    sa.slabs = batch[e];
    sa.rows = m[e];
    sa.cols = k[e];
    sa.kp = kp;
    sa.rp = mp;
    sa.transpose = 0;
    sa.vec = k[e] % 8 == 0 && (reinterpret_cast<uintptr_t>(A[e]) & 15) == 0;
    size_t const a_units = (size_t)batch[e] * mp * (kp / 16);
    sa.blocks = (unsigned)std::min<size_t>((a_units + kThreads - 1) / kThreads, 1024);
    sb.src = B[e];
    sb.plane_p = bt_p;
    sb.plane_q = bt_q;
    sb.slabs = batch[e];
    sb.rows = k[e];
    sb.cols = n[e];
    sb.kp = kp;
    sb.rp = np;
    sb.transpose = 1;
    sb.vec = n[e] % 4 == 0 && (reinterpret_cast<uintptr_t>(B[e]) & 7) == 0;
    size_t const b_tiles = (size_t)batch[e] * (kp / 64) * ((n[e] + 63) / 64);
    sb.blocks = (unsigned)std::min<size_t>(b_tiles, 1024);
    GemmJob g{};
    g.a_p = a_p;
    g.a_q = a_q;
    g.bt_p = bt_p;
    g.bt_q = bt_q;
    g.out = C[e];
    g.batch = batch[e];
    g.m = m[e];
    g.n = n[e];
    g.kp = kp;
    g.mp = mp;
    g.np = np;
    long long const tiles64 = (long long)((m[e] + 63) / 64) * ((n[e] + 63) / 64) * batch[e];
    long long const tiles128 = (long long)((m[e] + 127) / 128) * ((n[e] + 127) / 128) * batch[e];
    long long const tiles128x64 = (long long)((m[e] + 127) / 128) * ((n[e] + 63) / 64) * batch[e];
    // 128 x 128 tiles once there is one for every compute unit (a tile's plane offsets are
    // 32-bit there); below that 128 x 64 tiles if there is one of those for every compute unit
    // (1536^3: 26.7 us against 33.2 on 64 x 64 tiles; 1536 x 2048 x 1024: 23.2 against 25.7 on
    // 128 x 128; from 256 wide tiles on the narrow ones are no faster or slower)
    bool const fits_big = state().fp_big_tiles && state().fp_big_tiles_ok && kp <= kBigMaxK &&
                          (size_t)std::max(mp, np) * (size_t)kp < ((size_t)1 << 31);
    bool const narrow = fits_big && tiles128 < kBigMinTiles && tiles128x64 >= kBigMinTiles;
    bool const large = fits_big && (tiles128 >= kBigMinTiles || narrow);
    g.shared_k = !large && tiles64 < 64;
    int const edge = large ? 128 : (g.shared_k ? 32 : 64);
    int const edge_n = narrow ? 64 : edge;
    g.tiles_m = (m[e] + edge - 1) / edge;
    g.tiles_n = (n[e] + edge_n - 1) / edge_n;
    unsigned const blocks = (unsigned)((long long)g.tiles_m * g.tiles_n * batch[e]);
    // Measured with the split launch in front, as it runs: the XCD-aware order pays once the
    // tiles no longer all run at once (8 x 1024^3: 40 against 49 us); for fewer it costs a
    // microsecond although it halves the bytes fetched (1024^3 on 64 x 64 tiles: 16.6 against
    // 15.1 us).  The magics are exact while dividend * divisor < 2^32 (dividends: below `blocks`).
    g.xcd_order = large && !narrow && blocks >= 512u && blocks < 65536u;
    g.magic_per_batch = fast_div_magic(g.tiles_m * g.tiles_n);
    g.magic_width = fast_div_magic(8 * g.tiles_n);
    if (narrow) {
      g.first_block = narrow_blocks;
      narrow_blocks += blocks;
      Narrow.job[Narrow.count++] = g;
    } else if (large) {
      g.first_block = big_blocks;
      big_blocks += blocks;
      Big.job[Big.count++] = g;
    } else {
      g.first_block = gemm_blocks;
      gemm_blocks += blocks;
      G.job[G.count++] = g;
    }
  }
  hipStream_t st = state().stream();
  if (int rc = launch_split_jobs(jobs.data(), 2 * count, st)) {
    return rc;
  }
  if (G.count > 0) {
    fp_mfma_matmul_kernel<<<gemm_blocks, kThreads, 0, st>>>(G);
    MI355_HIP(hipGetLastError());
  }
  if (Big.count > 0 || Narrow.count > 0) {
    static std::atomic<int> granted{0};
    if (granted.load(std::memory_order_acquire) < kBigLdsBytes) {
      MI355_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(fp_mfma_matmul_big_kernel<128>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kBigLdsBytes));
      MI355_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(fp_mfma_matmul_big_kernel<64>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kBigLdsBytes));
      granted.store(kBigLdsBytes, std::memory_order_release);
    }
    if (Big.count > 0) {
      fp_mfma_matmul_big_kernel<128><<<big_blocks, kThreads, kBigLdsBytes, st>>>(Big);
      MI355_HIP(hipGetLastError());
    }
    if (Narrow.count > 0) {
      fp_mfma_matmul_big_kernel<64><<<narrow_blocks, kThreads, kBigLdsBytes, st>>>(Narrow);
      MI355_HIP(hipGetLastError());
    }
  }
  return MI355_OK;
}

extern "C" int mi355_fp_matmul(uint16_t const *A, uint16_t const *B, uint16_t *C, int batch, int m,
                               int n, int k);

bool mfma_matmul_pays(int batch, int m, int n, int k) {
  size_t need = 0;
  return !state().fp_vector_dot_only && mfma_matmul_fits(batch, m, n, k, &need) && need <= state().planes_bytes &&
         (double)batch * m * n * k >= (double)(1 << 27);
}

int launch_mfma_matmul(uint16_t const *A, uint16_t const *B, uint16_t *C, int batch, int m, int n,
                       int k) {
  return launch_mfma_group(&A, &B, &C, &batch, &m, &n, &k, 1);
}

// fp_mfma_matmul_big_kernel prefetches B^T with loads that land in registers behind the
// compiler's back (plane_load16 / landed): correct as long as the compiler neither spills nor
// copies those registers between the load and its wait, which the build checks for (no
// scratch, the recorded occupancy) but cannot prove.  So the kernels are also checked where
// they run: one product that takes the 128 x 128 tiles and one that takes the 128 x 64 tiles,
// 8 k steps each, against the 64 x 64-tile kernel that uses ordinary loads.  The ring makes
// the results bit-identical; on a difference the 128-row kernels stay off for this process.
extern "C" int mi355_fp_big_tiles_check(int *passed) {
  MI355_REQUIRE_INIT();
  State &s = state();
  constexpr int M = 2048, N = 2048, NN = 1024, K = 512;
  size_t const a_elems = (size_t)M * K, b_elems = (size_t)K * N, c_elems = (size_t)M * N,
               cn_elems = (size_t)M * NN;
  uint16_t *buf = nullptr;
  MI355_HIP(hipMalloc(reinterpret_cast<void **>(&buf), (a_elems + b_elems + 2 * c_elems + 2 * cn_elems) * 2));
  uint16_t *A = buf, *B = A + a_elems, *C1 = B + b_elems, *C2 = C1 + c_elems, *D1 = C2 + c_elems,
           *D2 = D1 + cn_elems;
  std::vector<uint16_t> host(a_elems + b_elems);
  uint64_t x = 0x9E3779B97F4A7C15ull;
  for (uint16_t &v : host) {
    x = x * 6364136223846793005ull + 1442695040888963407ull;
    v = (uint16_t)((x >> 33) % FP_PQ);
  }
  int rc = MI355_OK, eq_big = 0, eq_narrow = 0;
  int const asked = s.fp_big_tiles, ok_before = s.fp_big_tiles_ok;
  auto run = [&](int big, uint16_t *c, uint16_t *d) {
    s.fp_big_tiles = big;
    s.fp_big_tiles_ok = 1;
    if (rc == MI355_OK) {
      rc = mi355_fp_matmul(A, B, c, 1, M, N, K);
    }
    if (rc == MI355_OK) {
      rc = mi355_fp_matmul(A, B, d, 1, M, NN, K);  // the first K x NN elements of B, as a matrix
    }
  };
  if (hipMemcpy(A, host.data(), host.size() * 2, hipMemcpyHostToDevice) != hipSuccess) {
    rc = fail(MI355_ERR_HIP, "self-check upload failed");
  }
  run(1, C1, D1);
  run(0, C2, D2);
  s.fp_big_tiles = asked;
  s.fp_big_tiles_ok = ok_before;
  if (rc == MI355_OK) {
    rc = mi355_fp_equal(C1, C2, c_elems, &eq_big);
  }
  if (rc == MI355_OK) {
    rc = mi355_fp_equal(D1, D2, cn_elems, &eq_narrow);
  }
  hipError_t const freed = hipFree(buf);
  if (rc != MI355_OK) {
    return rc;
  }
  MI355_HIP(freed);
  s.fp_big_tiles_ok = (eq_big && eq_narrow) ? 1 : 0;
  if (!s.fp_big_tiles_ok) {
    fprintf(stderr,
            "mi355: the 128-row fingerprint matmul kernels disagree with the 64 x 64-tile kernel on this "
            "device (128 x 128 tiles %s, 128 x 64 tiles %s); large matmuls keep 64 x 64 tiles\n",
            eq_big ? "equal" : "DIFFER", eq_narrow ? "equal" : "DIFFER");
  }
  if (passed != nullptr) {
    *passed = s.fp_big_tiles_ok;
  }
  return MI355_OK;
}

extern "C" int mi355_fp_matmul_many(uint16_t const *const *A, uint16_t const *const *B,
                                    uint16_t *const *C, int const *batch, int const *m,
                                    int const *n, int const *k, int count) {
  MI355_REQUIRE_INIT();
  if (count < 0 || (count > 0 && (A == nullptr || B == nullptr || C == nullptr || batch == nullptr ||
                                  m == nullptr || n == nullptr || k == nullptr))) {
    return fail(MI355_ERR_INVALID, "bad matmul list (count %d)", count);
  }
  for (int e = 0; e < count; e++) {
    if (batch[e] < 0 || m[e] < 0 || n[e] < 0 || k[e] < 0) {
      return fail(MI355_ERR_INVALID, "matmul %d: negative extent", e);
    }
    bool const any_output = (long long)batch[e] * m[e] * n[e] > 0;
    if (any_output && (C[e] == nullptr || (k[e] > 0 && (A[e] == nullptr || B[e] == nullptr)))) {
      return fail(MI355_ERR_INVALID, "matmul %d: null matrix", e);
    }
  }
  // consecutive matmuls whose planes fit the queue's plane memory go out together; one that
  // cannot take this path at all (no k, planes too large) goes through the single entry point
  int begin = 0;
  while (begin < count) {
    size_t need = 0;
    if (state().fp_vector_dot_only ||
        !mfma_matmul_fits(batch[begin], m[begin], n[begin], k[begin], &need) ||
        need > state().planes_bytes) {
      if (int rc = mi355_fp_matmul(A[begin], B[begin], C[begin], batch[begin], m[begin], n[begin], k[begin])) {
        return rc;
      }
      begin++;
      continue;
    }
    int end = begin + 1;
    size_t total = need;
    while (end < count && end - begin < kMaxJobs) {
      size_t more = 0;
      if (!mfma_matmul_fits(batch[end], m[end], n[end], k[end], &more) ||
          total + more > state().planes_bytes) {
        break;
      }
      total += more;
      end++;
    }
    if (int rc = launch_mfma_group(A + begin, B + begin, C + begin, batch + begin, m + begin,
                                   n + begin, k + begin, end - begin)) {
      return rc;
    }
    begin = end;
  }
  return MI355_OK;
}

// ---- fused tiled-matmul plans, host side ---------------------------------------------------
static bool multiple_of_16(int const *v, int count) {
  for (int i = 0; i < count; i++) {
    if (v[i] % 16 != 0) {
      return false;
    }
  }
  return true;
}

bool fp_mfma_gemm_fits(DevProgram &P, PlanExtents const &ext, size_t *plane_bytes) {
  if (P.fused != 4 || state().fp_vector_dot_only || state().planes() == nullptr) {
    return false;
  }
  DevOp const &la = P.ops[P.fg[0]], &lb = P.ops[P.fg[1]];
  int const m = P.t[la.dst].rows, kt = P.t[la.dst].cols, n = P.t[lb.dst].cols;
  if (m % 16 != 0 || n % 16 != 0 || kt % 16 != 0 || (P.fp_unary[2] != 0 && kt > 48 && kt % 64 != 0)) {
    return false;
  }
  size_t total = 0;
  DevOp const *ops[2] = {&la, &lb};
  for (int which = 0; which < 2; which++) {
    DevOp const &op = *ops[which];
    long long const matrix = (long long)op.d_rows * op.d_cols;
    long long const elems = ext.in_elems[op.io];
    if (!multiple_of_16(op.row_bs, 3) || !multiple_of_16(op.col_bs, 3) || op.row_fs % 16 != 0 ||
        op.col_fs % 16 != 0 || matrix <= 0 || elems <= 0 || elems % matrix != 0 || op.g_fs % matrix != 0 ||
        op.g_bs[0] % matrix != 0 || op.g_bs[1] % matrix != 0 || op.g_bs[2] % matrix != 0) {
      return false;
    }
    long long const slabs = elems / matrix;
    // plane rows: A keeps its rows, B^T has one row per column of B; k the other extent
    long long const rows = which == 0 ? op.d_rows : op.d_cols, k = which == 0 ? op.d_cols : op.d_rows;
    long long const rp = (rows + 15) / 16 * 16, kp = (k + 63) / 64 * 64;
    if (slabs * rp * kp > ((long long)1 << 26)) {  // a plane stays addressable by a 32-bit offset
      return false;
    }
    P.pl_geo[3 * which] = (int)slabs;
    P.pl_geo[3 * which + 1] = (int)rp;
    P.pl_geo[3 * which + 2] = (int)kp;
    total += (size_t)(2 * slabs * rp * kp);
  }
  *plane_bytes = total;
  return true;
}

void fp_mfma_plane_bytes(DevProgram const &P, size_t *a_bytes, size_t *b_bytes) {
  *a_bytes = 2 * (size_t)P.pl_geo[0] * P.pl_geo[1] * P.pl_geo[2];
  *b_bytes = 2 * (size_t)P.pl_geo[3] * P.pl_geo[4] * P.pl_geo[5];
}

void fp_mfma_gemm_bind(DevProgram &P, char *planes, int min_blocks) {
  size_t a_bytes, b_bytes;
  fp_mfma_plane_bytes(P, &a_bytes, &b_bytes);
  fp_mfma_gemm_bind(P, planes, planes + a_bytes, 0, min_blocks);
}

void fp_mfma_gemm_bind(DevProgram &P, char *a_planes, char *b_planes, int shared, int min_blocks) {
  DevOp const &la = P.ops[P.fg[0]], &lb = P.ops[P.fg[1]];
  size_t const a_plane = (size_t)P.pl_geo[0] * P.pl_geo[1] * P.pl_geo[2];
  size_t const b_plane = (size_t)P.pl_geo[3] * P.pl_geo[4] * P.pl_geo[5];
  P.pl[0] = reinterpret_cast<int8_t *>(a_planes);
  P.pl[1] = P.pl[0] + a_plane;
  P.pl[2] = reinterpret_cast<int8_t *>(b_planes);
  P.pl[3] = P.pl[2] + b_plane;
  P.pl_shared = shared;
  // A: strips follow rows, chunks follow columns
  {
    long long const matrix = (long long)la.d_rows * la.d_cols;
    int const strip = P.pl_geo[2] * 16, per_slab = P.pl_geo[1] / 16;
    auto stride = [&](int g, int row, int col) {
      return (int)(((long long)(g / matrix) * per_slab + row / 16) * strip + (col / 16) * 256);
    };
    for (int d = 0; d < 3; d++) {
      P.pl_a[d] = stride(la.g_bs[d], la.row_bs[d], la.col_bs[d]);
    }
    P.pl_a[3] = stride(la.g_fs, la.row_fs, la.col_fs);
    P.pl_a[4] = strip;
  }
  // B^T: strips follow columns of B, chunks follow its rows
  {
    long long const matrix = (long long)lb.d_rows * lb.d_cols;
    int const strip = P.pl_geo[5] * 16, per_slab = P.pl_geo[4] / 16;
    auto stride = [&](int g, int row, int col) {
      return (int)(((long long)(g / matrix) * per_slab + col / 16) * strip + (row / 16) * 256);
    };
    for (int d = 0; d < 3; d++) {
      P.pl_b[d] = stride(lb.g_bs[d], lb.row_bs[d], lb.col_bs[d]);
    }
    P.pl_b[3] = stride(lb.g_fs, lb.row_fs, lb.col_fs);
    P.pl_b[4] = strip;
  }
  P.fg[5] = 1;
  P.lds_bytes = kFpMfmaLdsBytes;
  // group neighbouring blocks of small tiles up to 64 x 64 outputs per workgroup, as long as
  // the program keeps `min_blocks` workgroups (a few hundred when it is launched by itself, a
  // few when many programs share the launch)
  P.pl_group[0] = P.pl_group[1] = 1;
  int const m = P.t[la.dst].rows, n = P.t[lb.dst].cols;
  P.pl_magic[0] = fast_div_magic(m / 16);
  P.pl_magic[1] = fast_div_magic(n / 16);
  if (P.pl_a[0] == 0 && P.pl_b[1] == 0) {
    long long blocks = (long long)P.grid[0] * P.grid[1] * P.grid[2];
    auto grow = [&](int which, int tile) {
      int &g = P.pl_group[which];
      while (tile * g * 2 <= 64 && P.grid[which] % (g * 2) == 0 && blocks / 2 >= min_blocks) {
        g *= 2;
        blocks /= 2;
      }
    };
    grow(1, m);
    grow(0, n);
  }
}

int fp_mfma_split_programs(DevProgram const *const *progs, int n, hipStream_t stream) {
  std::vector<SplitJob> jobs;
  jobs.reserve((size_t)(2 * n));
  for (int e = 0; e < n; e++) {
    DevProgram const &P = *progs[e];
    DevOp const *ops[2] = {&P.ops[P.fg[0]], &P.ops[P.fg[1]]};
    for (int which = 0; which < 2; which++) {
      if (P.pl_shared & (1 << which)) {
        continue;  // an earlier program of this launch splits the same tensor into these planes
      }
      DevOp const &op = *ops[which];
      jobs.emplace_back();
      SplitJob &j = jobs.back();
      j = SplitJob{};
      j.src = static_cast<uint16_t const *>(P.in[op.io]);
      j.plane_p = P.pl[2 * which];
      j.plane_q = P.pl[2 * which + 1];
      j.slabs = P.pl_geo[3 * which];
      j.rows = op.d_rows;
      j.cols = op.d_cols;
      j.rp = P.pl_geo[3 * which + 1];
      j.kp = P.pl_geo[3 * which + 2];
      j.transpose = which;
      j.unary = P.fp_unary[which];
      size_t work;
      if (which == 0) {
        j.vec = op.d_cols % 8 == 0 && (reinterpret_cast<uintptr_t>(j.src) & 15) == 0;
        work = ((size_t)j.slabs * j.rp * (j.kp / 16) + kThreads - 1) / kThreads;
      } else {
        j.vec = op.d_cols % 4 == 0 && (reinterpret_cast<uintptr_t>(j.src) & 7) == 0;
        work = (size_t)j.slabs * (j.kp / 64) * ((op.d_cols + 63) / 64);
      }
      j.blocks = (unsigned)std::min<size_t>(work, 1024);
    }
  }
  return launch_split_jobs(jobs.data(), (int)jobs.size(), stream);
}

int launch_fp_mfma_gemm(DevProgram const &P, hipStream_t stream) {
  DevProgram const *one = &P;
  if (int rc = fp_mfma_split_programs(&one, 1, stream)) {
    return rc;
  }
  dim3 grid(P.grid[0] / P.pl_group[0] * P.splits, P.grid[1] / P.pl_group[1], P.grid[2]);
  fp_mfma_gemm_kernel<<<grid, kThreads, 0, stream>>>(P, tables());
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

int launch_fp_mfma_gemm_multi(DevProgram const *progs, int const *first_block, int n, int blocks,
                              hipStream_t stream) {
  int const lds_total = kFpMfmaLdsBytes + (int)sizeof(DevProgram) + 256;  // sums, record, exp table
  fp_mfma_gemm_multi_kernel<<<blocks, kThreads, lds_total, stream>>>(progs, first_block, n, tables());
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

}  // namespace mi355
