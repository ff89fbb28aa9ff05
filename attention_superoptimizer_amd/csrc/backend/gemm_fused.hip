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
// the MFMAs.  Two kernels.  gemm_lanes_kernel (further down) runs a plan in ONE launch with
// the output tile cut into 16 x 16 pieces, one workgroup each, whose wavefronts take the
// for-loop's iterations side by side; it serves the launch-bound members.  gemm_fused_kernel
// cuts the for-loop instead and needs a second launch to add the ranges.  Its design:
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
//
// This file is the host side (recognition, choice of kernel and launch shape, the launch or,
// for Graph::generate_hip_program, its source text); the kernels are in
// include/mi355_kernels/gemm.h, which generated programs include as well.
#include "common.h"
#include "tb_program.h"
#include <algorithm>
#include <string>

#include "mi355_kernels/gemm.h"

namespace mi355 {

// ---------------------------------------------------------------------------------------
// host: recognise the family and launch
// ---------------------------------------------------------------------------------------
namespace {

// (a column-major tensor -- DevOp::sub == 1 on its loader -- holds element (r, c) at
// c * d_rows + r: a step along the rows is one element, a step along the columns d_rows, and
// `d_cols` of the result is that leading dimension)
// The tile origin of a loader / saver as one stride per block coordinate and per iteration.
// `fits` is cleared when an origin could leave 31 bits (the kernels multiply and add these
// strides in 32 bits): `extents` = the grid and the for-loop range.
GTile gtile(DevOp const &op, void const *ptr, int const (&extents)[4], bool &fits) {
  GTile t;
  t.ptr = ptr;
  bool const cm = op.kind == DOP_LOAD && op.sub == 1;
  long long const rstep = cm ? 1 : op.d_cols, cstep = cm ? op.d_rows : 1;
  long long lin[4];
  for (int i = 0; i < 3; i++) {
    lin[i] = op.g_bs[i] + op.row_bs[i] * rstep + op.col_bs[i] * cstep;
  }
  lin[3] = op.g_fs + op.row_fs * rstep + op.col_fs * cstep;
  long long reach = 0;
  for (int i = 0; i < 4; i++) {
    long long const a = lin[i] < 0 ? -lin[i] : lin[i];
    if (a >= (1LL << 31)) {
      fits = false;
    }
    reach += a * (extents[i] > 0 ? extents[i] - 1 : 0);
    t.lin[i] = (int)lin[i];
  }
  if (reach >= (1LL << 31)) {
    fits = false;
  }
  t.d_cols = cm ? op.d_rows : op.d_cols;
  return t;
}

// The parameter blocks as C++ source (for programs that Graph::generate_hip_program writes).
std::string literal(GTile const &t) {
  return emit_fmt("mi355::GTile{%s, {%d, %d, %d, %d}, %d}", emit_pointer(t.ptr).c_str(), t.lin[0], t.lin[1],
                  t.lin[2], t.lin[3], t.d_cols);
}
std::string literal(GemmParams const &A, char const *var) {
  std::string t = emit_fmt("    mi355::GemmParams %s{};\n", var);
  char const *names[8] = {"a0", "a1", "b0", "b1", "la", "lb", "o0", "o1"};
  GTile const *tiles[8] = {&A.a0, &A.a1, &A.b0, &A.b1, &A.la, &A.lb, &A.o0, &A.o1};
  for (int i = 0; i < 8; i++) {
    t += emit_fmt("    %s.%s = ", var, names[i]) + literal(*tiles[i]) + ";\n";
  }
  t += emit_fmt("    %s.M = %d;\n    %s.KT = %d;\n    %s.forloop_range = %d;\n    %s.ksplit = %d;\n", var, A.M, var,
                A.KT, var, A.forloop_range, var, A.ksplit);
  t += emit_fmt("    %s.scratch = static_cast<_Float16 *>(%s);\n", var, emit_pointer(A.scratch).c_str());
  return t;
}
std::string literal(LaneParams const &L) {
  std::string t = literal(L.g, "G") + "    mi355::LaneParams P{};\n    P.g = G;\n";
  t += emit_fmt("    P.gx = %d;\n    P.gy = %d;\n    P.blocks = %d;\n    P.mtiles = %d;\n    P.slot_base = %d;\n", L.gx,
                L.gy, L.blocks, L.mtiles, L.slot_base);
  t += emit_fmt("    P.m_group = %uu;\n    P.m_pieces = %uu;\n    P.m_gx = %uu;\n    P.m_gy = %uu;\n", L.m_group,
                L.m_pieces, L.m_gx, L.m_gy);
  return t;
}
char const *tf(bool b) { return b ? "true" : "false"; }

struct GMatch {
  int pro, nb;
  bool lora;
  int a0, a1, b0, b1, la, lb;  // load op indices (-1 when absent)
  int o0, o1;                  // output op indices
  int M, KT;
  // every weight-side operand (b0, b1, la, lb) is a DmemColumnMajor tensor, as the reference's
  // plans declare their weights (cpp_examples/lora.cc:36-41): k is contiguous in memory
  bool wcm;
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
  if (has_column_major_saver(P)) {
    return false;
  }
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
  // activations row-major; the weight-side operands all in one storage order
  G.wcm = P.ops[G.b0].sub == 1;
  for (int i : {G.a0, G.a1}) {
    if (i >= 0 && P.ops[i].sub == 1) {
      return false;
    }
  }
  for (int i : {G.b0, G.b1, G.la, G.lb}) {
    if (i >= 0 && (P.ops[i].sub == 1) != G.wcm) {
      return false;
    }
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

template <int MT, int NB, int PRO, bool LORA, bool WCM>
int launch_kt(GemmParams const &A, dim3 grid, int lds) {
  if (EmitSink *sink = emit_sink()) {
    sink->headers |= 2u;
    int const ktmax = A.KT <= 64 ? 64 : (A.KT <= 256 ? 256 : 512);
    emit_launch(*sink, "gemm_fused_kernel", emit_fmt("%d, %d, %d, %s, %d, %s", MT, NB, PRO, tf(LORA), ktmax, tf(WCM)), grid,
                256, lds, literal(A, "P"));
    return 1;
  }
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
    return go(gemm_fused_kernel<MT, NB, PRO, LORA, 64, WCM>);
  }
  if (A.KT <= 256) {
    return go(gemm_fused_kernel<MT, NB, PRO, LORA, 256, WCM>);
  }
  return go(gemm_fused_kernel<MT, NB, PRO, LORA, 512, WCM>);
}

// gemm_lanes_kernel for this plan, or 0 when it is not the better choice (see the rule in
// try_launch_lanes); k extents 64 / 128 / 256.
template <int NB, int PRO, bool LORA, bool WCM>
int launch_lanes_kt(LaneParams const &L, int grid, int threads, int lds) {
  if (EmitSink *sink = emit_sink()) {
    if (!(L.g.KT == 64 || L.g.KT == 128 || L.g.KT == 256)) {
      return 0;
    }
    sink->headers |= 2u;
    emit_launch(*sink, "gemm_lanes_kernel", emit_fmt("%d, %d, %d, %s, %s", L.g.KT, NB, PRO, tf(LORA), tf(WCM)),
                dim3(grid, 1, 1), threads, lds, literal(L));
    return 1;
  }
  State &s = state();
  auto go = [&](auto *fn) -> int {
    if (lds > 65536) {
      MI355_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(fn),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    }
    fn<<<grid, threads, lds, s.stream()>>>(L);
    MI355_HIP(hipGetLastError());
    return 1;
  };
  switch (L.g.KT) {
    case 64:
      return go(gemm_lanes_kernel<64, NB, PRO, LORA, WCM>);
    case 128:
      return go(gemm_lanes_kernel<128, NB, PRO, LORA, WCM>);
    case 256:
      return go(gemm_lanes_kernel<256, NB, PRO, LORA, WCM>);
    default:
      return 0;
  }
}

int try_launch_lanes(DevProgram const &P, GMatch const &G, GemmParams const &A) {
  State &s = state();
  if (s.gemm_mode == 1 || !(G.KT == 64 || G.KT == 128 || G.KT == 256)) {
    return 0;
  }
  long long const blocks = (long long)P.grid[0] * P.grid[1] * P.grid[2];
  int const mtiles = (G.M + 15) / 16, S = 4 * mtiles, F = P.forloop_range;
  long long const groups = (blocks + 7) / 8;
  // (the kernel decodes the flat id with multiply-high magics: exact while id x divisor < 2^32)
  long long const widest = std::max<long long>(8 * S, std::max(P.grid[0], P.grid[1]));
  if (groups * 8 * S * widest >= (1LL << 32)) {
    return 0;
  }
  // By itself only where the launch, not the traffic, sets the time (weights of a few MB): a
  // 16-column strip uses 32 bytes of every 128-byte line it pulls into a compute unit's L1, and
  // every piece re-reads the activation rows, so the L2 -> L1 traffic is 4-5 x the bytes of the
  // plan (measured on the LoRA plan: 202 MB of requests for 34 MB), which is what bounds a plan
  // of tens of MB; the range-splitting kernel moves whole lines once.
  // With column-major weights a piece's columns are whole lines of its own, read straight into
  // registers, so the first cost is gone; measured on the configurations of the benchmark the one
  // launch then also wins for the two-weight plan (gated MLP, first half, 235 MB: 45.8 against
  // 49.0 us) but not for the others (LoRA, 34 MB: 14.0 against 12.4 us; gated MLP, second half,
  // 117 MB: 36.2 against 24.7 us), where each wavefront's loads of its activation rows and of the
  // lora A tile outnumber its weight loads.
  long long const weight_bytes = blocks * F * (long long)(G.nb * G.KT * 64 + (G.lora ? G.KT * 16 : 0)) * 2;
  bool const two_weights_cm = G.wcm && G.nb == 2 && blocks * S <= 4096;
  if (s.gemm_mode == 0 && !two_weights_cm && (blocks * S > 1024 || weight_bytes > (8LL << 20))) {
    return 0;
  }
  int const strips = G.nb + (G.lora ? 1 : 0);
  int const wave_bytes = G.wcm ? 0 : strips * G.KT * 32 + (G.lora ? 512 : 0);
  int const slot_bytes = F * G.nb * 512;
  int ip = F < 16 ? F : 16;
  while (ip > 1 && ip * wave_bytes + slot_bytes > s.max_lds) {
    ip = (ip + 1) / 2;
  }
  if (ip * wave_bytes + slot_bytes > s.max_lds) {
    return 0;
  }
  LaneParams L{};
  L.g = A;
  L.gx = P.grid[0];
  L.gy = P.grid[1];
  L.blocks = (int)blocks;
  L.mtiles = mtiles;
  L.slot_base = ip * wave_bytes;
  L.m_group = fast_div_magic(8 * 4 * mtiles);
  L.m_pieces = fast_div_magic(4 * mtiles);
  L.m_gx = fast_div_magic(P.grid[0]);
  L.m_gy = fast_div_magic(P.grid[1]);
  int const lds = ip * wave_bytes + slot_bytes, grid = (int)(groups * 8 * S);
  int rc = 0;
#define MI355_LANES_CASE(NBV, PROV, LORAV)                                  \
  if (G.nb == NBV && G.pro == PROV && G.lora == LORAV) {                    \
    rc = G.wcm ? launch_lanes_kt<NBV, PROV, LORAV, true>(L, grid, ip * 64, lds)   \
               : launch_lanes_kt<NBV, PROV, LORAV, false>(L, grid, ip * 64, lds); \
  }
  MI355_LANES_CASE(1, PRO_NONE, false)
  MI355_LANES_CASE(1, PRO_EXP, false)
  MI355_LANES_CASE(1, PRO_SILU, false)
  MI355_LANES_CASE(2, PRO_NONE, false)
  MI355_LANES_CASE(1, PRO_SILU_MUL, false)
  MI355_LANES_CASE(1, PRO_NONE, true)
#undef MI355_LANES_CASE
  if (rc == 1) {
    s.last().kernel_id = MI355_KERNEL_F16_GEMM;
    s.last().workgroups = grid;
    s.last().threads = ip * 64;
    s.last().lds_bytes = lds;
    s.last().row_split = S;
  }
  return rc;
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
  int const extents[4] = {P.grid[0], P.grid[1], P.grid[2], P.forloop_range};
  bool fits = true;
  auto in_tile = [&](int i) { return gtile(P.ops[i], P.in[P.ops[i].io], extents, fits); };
  A.a0 = in_tile(G.a0);
  A.a1 = G.a1 >= 0 ? in_tile(G.a1) : A.a0;
  A.b0 = in_tile(G.b0);
  A.b1 = G.b1 >= 0 ? in_tile(G.b1) : A.b0;
  A.la = G.la >= 0 ? in_tile(G.la) : A.a0;
  A.lb = G.lb >= 0 ? in_tile(G.lb) : A.a0;
  A.o0 = gtile(P.ops[G.o0], P.out[P.ops[G.o0].io], extents, fits);
  A.o1 = G.o1 >= 0 ? gtile(P.ops[G.o1], P.out[P.ops[G.o1].io], extents, fits) : A.o0;
  if (!fits) {
    return 0;  // a tensor of more than 2^31 elements: the generic interpreter takes the plan
  }
  A.M = G.M;
  A.KT = G.KT;
  A.forloop_range = P.forloop_range;
  if (int const rc = try_launch_lanes(P, G, A)) {
    return rc;
  }
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
  EmitSink *const sink = emit_sink();
  if (ksplit > 1 && (scratch_elems * 2 > (long long)(sink ? kEmitScratchBytes : s.scratch_bytes))) {
    ksplit = 1;
  }
  A.ksplit = ksplit;
  A.scratch = static_cast<_Float16 *>(s.scratch());
  if (sink) {  // a printed program allocates the workspace itself
    A.scratch = ksplit > 1 ? reinterpret_cast<_Float16 *>(kEmitScratch) : nullptr;
    if (ksplit > 1) {
      sink->scratch_bytes = std::max<size_t>(sink->scratch_bytes, (size_t)scratch_elems * 2);
    }
  }
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
    rc = G.wcm ? launch_kt<MTV, NBV, PROV, LORAV, true>(A, grid, lds)                 \
               : launch_kt<MTV, NBV, PROV, LORAV, false>(A, grid, lds);               \
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
  if (rc == 1 && ksplit > 1 && sink) {
    emit_launch(*sink, "gemm_combine_kernel", emit_fmt("%d", G.nb), dim3(P.grid[0], P.grid[1], P.grid[2]), 256, 0,
                literal(A, "P"));
  } else if (rc == 1 && ksplit > 1) {
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
