// Device program of one customized op: what the host-side lowering hands to
// the interpreter kernels.  Built from an mi355_plan (the reference's flat-int
// NewKernelParams bytecode) by compile_plan(): operands are resolved to tensor
// records, every tensor gets a physical LDS placement from a liveness scan
// (the plan's own offsets only name tensors: they are a bump allocation with no
// reuse and would not fit the larger plans into 160 KB), loop-invariant loads
// are hoisted, and each tensor gets the LDS layout its consumers want.
#pragma once

#include "mi355_abi.h"
#include <hip/hip_runtime_api.h>
#include <cstdint>
#include <string>

namespace mi355 {

constexpr int kMaxTensors = 24;
constexpr int kTableBytes = 1024;  // fingerprint tables at the bottom of LDS

enum DevOpKind : int {
  DOP_LOAD = 1,
  DOP_MATMUL = 2,
  DOP_UNARY = 3,
  DOP_BINARY = 4,
  DOP_REDUCE = 5,
  DOP_CONCAT = 6,
  DOP_OUTPUT = 7,
};

// A 2-D tile in LDS: element (r, c) lives at byte offset off + 2 * (r*rs + c*cs).
struct DevTensor {
  int off;
  int rows, cols;
  int rs, cs;
  uint32_t mcols, mcpr;  // division magics of cols and cols / 8 (see fast_div_magic)
};

// q = e / d as one multiply-high: magic = ceil(2^32 / d), exact while e * d < 2^32;
// 0 stands for d == 1.
inline uint32_t fast_div_magic(int d) {
  return d <= 1 ? 0u : (uint32_t)((((uint64_t)1 << 32) + (uint64_t)d - 1) / (uint64_t)d);
}

struct DevOp {
  int kind;
  int sub;             // UNARY / BINARY: the TB_* operator code; LOAD / OUTPUT (fp16): 1 = the device tensor
                       // is DmemColumnMajor, element (r, c) of its [d_rows, d_cols] matrix at
                       // c * d_rows + r (fingerprint tensors are always row-major)
  int src0, src1, dst; // tensor ids (-1 when unused)
  int io;              // LOAD: input slot; OUTPUT: output slot
  int hoist;           // LOAD: loop invariant, executed at iteration 0 only
  int vec8;            // LOAD / OUTPUT: 16-byte accesses usable on both the global and LDS side
  int galign;          // LOAD / OUTPUT: every row segment (column segment of a column-major tensor)
                       // is 16-byte aligned in global memory
  int row_bs[3], col_bs[3], row_fs, col_fs;  // block / for-loop strides of the tile origin
  int g_bs[3], g_fs;                         // block / for-loop strides of the batch offset
  int d_rows, d_cols;                        // matrix shape of the device tensor
  int red_deg, red_inner;                    // REDUCE (flat row-major rule of the reference)
  int cat_a, cat_b, cat_inner;               // CONCAT
  int mm_kc;  // MATMUL, uint16 interpreter: k chunk of the packed-residue path, 0 = scalar path
  int mm_mb;  // MATMUL, matrix-core variant (sub == 1): rows of A packed at a time
  // division magics.  MATMUL: kc / 4, n / 2, n / 4.  REDUCE: inner.  CONCAT: inner, a + b.
  // LOAD of a column-major tensor: the tile's rows, rows / 8.
  uint32_t mg0, mg1, mg2;
};

struct alignas(16) DevProgram {
  int num_ops, num_tensors;
  int forloop_range;
  int lds_bytes;  // dynamic LDS the interpreter requests (tables included)
  int fused;      // fp16: 1 / 2 / 3 = run by the fused attention / GEMM / combine kernel; uint16:
                  // 4 = run by the fused fingerprint matmul kernel; 0 = the interpreter
  int fg[6];      // fused fingerprint matmul: loader of A, loader of B, k chunk, register tiles per
                  // thread, thread groups sharing a tile's k range (small tiles), 1 = matrix-core
                  // route (the operand tensors are read from residue planes, see pl / pl_geo)
  // matrix-core route: signed-byte residue planes of the two operand tensors in 16 x 16 blocks
  // (A mod 227, A mod 113, B^T mod 227, B^T mod 113) and their geometry: A slabs, A plane rows
  // per slab, A padded k; B slabs, B^T plane rows per slab, B padded k
  int8_t *pl[4];
  int pl_geo[6];
  // byte offset of a tile's first block in the A / B^T planes = bx * [0] + by * [1] + bz * [2] +
  // iteration * [3]; [4] = bytes of one strip of 16 plane rows
  int pl_a[5], pl_b[5];
  // a workgroup of the matrix-core route takes pl_group[0] x pl_group[1] neighbouring logical
  // blocks (along grid x / y) when A does not move with x and B not with y: their tiles form
  // one larger tile whose operand strips are fetched once
  int pl_group[2];
  // element-wise operators around the matmul (TB_EXP_OP, TB_SILU_OP or 0): [0] / [1] applied
  // to the A / B tile before it (on the matrix-core route once per element, while the operand
  // tensor is split into planes), [2] applied to every iteration's product before the saver
  // adds it up.  Only the matrix-core route runs a program that has any of them.
  int fp_unary[3];
  uint32_t pl_magic[2];  // division magics of m / 16 and n / 16 (strips per logical block)
  int pl_shared;  // bit 0 / 1: the A / B^T planes belong to an earlier program of the launch
                  // (same operand tensor, same prologue): this program does not split them
  int grid[3];
  int mm_off;  // uint16 interpreter: LDS offset of the matmul residue scratch
  // uint16 interpreter, split for-loop: workgroup (split, block) runs iterations
  // [F*split/splits, F*(split+1)/splits) and stores its sums to part[o] + split*part_elems[o];
  // a second launch adds the splits (exact in the ring).  splits == 1: stores go to out[].
  int splits;
  long long part_elems[MI355_MAX_DMEM_OUTPUTS];
  long long part_stride[MI355_MAX_DMEM_OUTPUTS];  // part_elems rounded up to 8
  uint16_t *part[MI355_MAX_DMEM_OUTPUTS];
  DevTensor t[kMaxTensors];
  DevOp ops[MI355_MAX_OPERATORS];
  void const *in[MI355_MAX_DMEM_INPUTS];
  void *out[MI355_MAX_DMEM_OUTPUTS];
};

struct PlanExtents {
  long long in_elems[MI355_MAX_DMEM_INPUTS];   // 1 + largest element index read
  long long out_elems[MI355_MAX_DMEM_OUTPUTS]; // 1 + largest element index written
};

// Fused register-resident kernels for recognised graph shapes (attn_fused.hip).
// Returns 1 when `prog` was recognised and launched, 0 when it is not of that
// family, a negative error code on failure.
int try_launch_attention(DevProgram const &prog);
bool attention_applicable(DevProgram const &prog);
int try_launch_gemm(DevProgram const &prog);  // gemm_fused.hip, same convention
bool gemm_applicable(DevProgram const &prog);
int try_launch_combine(DevProgram const &prog);  // combine_fused.hip, same convention
bool combine_applicable(DevProgram const &prog);

// Lowers `plan` for the uint16 interpreter (f16 == false: plain row-major tiles)
// or the fp16 interpreter (f16 == true: padded rows, B operands k-contiguous).
// Returns MI355_OK or an error code with `err` set.
// Fused fingerprint matmul family (fp_gemm_fused.hip): recognise (marks the program and
// replaces its LDS need), launch one program, launch many (programs and prefix table in
// device memory, `staging_bytes` = the largest member's LDS need).
bool fp_gemm_applicable(DevProgram &P);
int launch_fp_gemm(DevProgram const &P, hipStream_t stream);
int launch_fp_gemm_multi(DevProgram const *progs, int const *first_block, int n, int blocks, int tpt,
                         int staging_bytes, hipStream_t stream);

// Matrix-core route of the same family (fp_mfma.hip).  fp_mfma_gemm_fits: whether a program
// already marked fused = 4 can take it, and the bytes of residue planes it needs;
// fp_mfma_gemm_bind: places the planes at `planes` and marks the program; the launches split
// the operand tensors of the bound programs into their planes first (fp_mfma_split_programs).
bool fp_mfma_gemm_fits(DevProgram &P, PlanExtents const &ext, size_t *plane_bytes);
void fp_mfma_gemm_bind(DevProgram &P, char *planes, int min_blocks);
// The same with the two operands' planes at places of their own (`a_planes`: both planes of A,
// `b_planes`: both of B^T) and `shared` as in DevProgram::pl_shared; fp_mfma_plane_bytes gives
// the bytes each side needs once fp_mfma_gemm_fits has filled in the geometry.
void fp_mfma_gemm_bind(DevProgram &P, char *a_planes, char *b_planes, int shared, int min_blocks);
void fp_mfma_plane_bytes(DevProgram const &P, size_t *a_bytes, size_t *b_bytes);
int fp_mfma_split_programs(DevProgram const *const *progs, int n, hipStream_t stream);
int launch_fp_mfma_gemm(DevProgram const &P, hipStream_t stream);
int launch_fp_mfma_gemm_multi(DevProgram const *progs, int const *first_block, int n, int blocks,
                              hipStream_t stream);
constexpr int kFpMfmaLdsBytes = 32768;  // wavefront sums of a tile whose k range is shared
inline bool fp_needs_matrix_cores(DevProgram const &p) {
  return (p.fp_unary[0] | p.fp_unary[1] | p.fp_unary[2]) != 0;
}
// Workgroups a fused matmul program is launched with (grouped blocks count once).
inline long long fp_program_blocks(DevProgram const &p) {
  long long const gx = p.fused == 4 && p.fg[5] ? p.pl_group[0] : 1, gy = p.fused == 4 && p.fg[5] ? p.pl_group[1] : 1;
  return (long long)(p.grid[0] / gx) * p.splits * (p.grid[1] / gy) * p.grid[2];
}

// ---- source emission of the fused families (emit_hip.cc) ---------------------------------------
// While a sink is installed on the calling thread, try_launch_attention / _gemm / _combine go
// through their whole choice of kernel and launch shape and then PRINT the launches they would
// make -- the kernel template with its literal arguments, grid, LDS and the parameter block
// with literal values, as statements of a C++ function body -- instead of making them.  The
// printed code names the kernels of include/mi355_kernels/*.h.  Device pointers bound to the
// program while printing are tags that print as `in[i]`, `out[i]` or `scratch`.
// True when a saver of `P` writes a column-major device tensor: the fused kernels store rows,
// such a program runs on the interpreter.
inline bool has_column_major_saver(DevProgram const &P) {
  for (int o = 0; o < P.num_ops; o++) {
    if (P.ops[o].kind == DOP_OUTPUT && P.ops[o].sub == 1) {
      return true;
    }
  }
  return false;
}

struct EmitSink {
  std::string text;          // statements of the launcher body
  unsigned headers = 0;      // bit 0: attention.h, bit 1: gemm.h, bit 2: combine.h
  size_t scratch_bytes = 0;  // workspace the printed launches share (0: none)
};
EmitSink *&emit_sink();
constexpr uintptr_t kEmitInBase = 0x100000, kEmitOutBase = 0x200000, kEmitScratch = 0x300000, kEmitStep = 0x1000;
constexpr size_t kEmitScratchBytes = (size_t)64 << 20;  // what a printed program may ask for
inline void *emit_in_tag(int i) { return reinterpret_cast<void *>(kEmitInBase + kEmitStep * (uintptr_t)i); }
inline void *emit_out_tag(int i) { return reinterpret_cast<void *>(kEmitOutBase + kEmitStep * (uintptr_t)i); }
std::string emit_pointer(void const *p);  // "in[2]", "out[0]", "scratch", "nullptr"
std::string emit_fmt(char const *f, ...);
// One printed launch: `params` declares the parameter block `P`.
void emit_launch(EmitSink &sink, char const *kernel, std::string const &template_args, dim3 grid, int threads,
                 int lds, std::string const &params);

// `declared_layouts`: fp16 loader tiles take the LDS layout the plan declares for them
// (see MI355_OPT_PLAN_SMEM_LAYOUT) instead of the one their consumers want.
int compile_plan(mi355_plan const &plan, bool f16, int max_lds, DevProgram &prog,
                 PlanExtents &ext, std::string &err, bool declared_layouts = false);

}  // namespace mi355
