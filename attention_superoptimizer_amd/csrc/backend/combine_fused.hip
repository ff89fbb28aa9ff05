// Fused kernel for the "fold the partial results and divide" family of thread-block
// graphs: the second operator of the reference's split-KV attention plans
// (cpp_examples/multi_head_attn_prefill.cc:75-98 and its siblings) and of the programs its
// search records for them.  With N the partial numerators (S pieces of X columns per row, side
// by side or one per for-loop iteration) and D the partial denominators (SD per row, or the
// finished one), the members differ in where the division sits:
//
//   sum, then divide   O[r][x] = fp16( fp16(sum_s N[r][s X + x]) / d[r] )
//                      (loader, loader, reduction_to_dimx, [reduction], div, saver)
//   divide, then sum   O[r][x] = fp16( sum_s fp16(N[r][s X + x] / d[r]) )
//                      (loader, loader, [reduction], div, reduction_to_dimx, saver)
//   divide, then the saver's for-loop accumulation
//                      O[r][x] = acc_F,  acc_i = fp16(acc_{i-1} + fp16(N_i[r][x] / d[r]))
//                      (loader, loader, [reduction], div, saver; any for-loop range)
//
// with d[r] = fp16(sum_s D[r][s]) (or D[r] itself when the plan has no reduction over it).
// Nothing is reused, so nothing goes through LDS: each thread folds eight (or, for tiles of
// 4 columns, four) output columns of one row with vector loads and stores.  Sums run in
// fp32 over s = 0, 1, ... and are rounded to fp16 where the thread-block graph materialises a
// tile, the division is IEEE fp32.
#include "common.h"
#include <algorithm>
#include "tb_program.h"

#include <string>

#include "mi355_kernels/combine.h"

namespace mi355 {

namespace {

CTile ctile(DevOp const &op, void const *ptr) {
  CTile t;
  t.ptr = ptr;
  for (int i = 0; i < 3; i++) {
    t.lin[i] = op.g_bs[i] + (long long)op.row_bs[i] * op.d_cols + op.col_bs[i];
  }
  t.d_cols = op.d_cols;
  return t;
}

struct CMatch {
  int ln, ld, out;  // op indices: numerator loader, denominator loader, saver
  int rows, X, S, SD, mode, vec;
  long long step;
};

bool aligned(CTile const &t, int vec) {
  if ((reinterpret_cast<uintptr_t>(t.ptr) & (2 * vec - 1)) != 0 || t.d_cols % vec != 0) {
    return false;
  }
  for (int i = 0; i < 3; i++) {
    if (t.lin[i] % vec != 0) {
      return false;
    }
  }
  return true;
}

bool cmatch(DevProgram const &P, CMatch &M) {
  // (inputs are read and the result stored as row-major matrices: a column-major one takes
  // the interpreter)
  if (has_column_major_saver(P)) {
    return false;
  }
  for (int o = 0; o < P.num_ops && P.ops[o].kind == DOP_LOAD; o++) {
    if (P.ops[o].sub == 1) {
      return false;
    }
  }
  int const last = P.num_ops - 1, F = P.forloop_range;
  if (P.num_ops < 4 || P.num_ops > 6 || P.ops[0].kind != DOP_LOAD || P.ops[1].kind != DOP_LOAD ||
      P.ops[last].kind != DOP_OUTPUT) {
    return false;
  }
  DevOp const &out = P.ops[last];
  auto loader_of = [&](int tensor) { return P.ops[0].dst == tensor ? 0 : (P.ops[1].dst == tensor ? 1 : -1); };
  auto producer = [&](int tensor) {  // a middle statement writing `tensor`, or -1
    for (int o = 2; o < last; o++) {
      if (P.ops[o].dst == tensor) {
        return o;
      }
    }
    return -1;
  };
  // the one division
  int dv = -1;
  for (int o = 2; o < last; o++) {
    if (P.ops[o].kind == DOP_BINARY && P.ops[o].sub == TB_DIV_OP) {
      if (dv >= 0) {
        return false;
      }
      dv = o;
    }
  }
  if (dv < 0) {
    return false;
  }
  int used = 1;
  // its divisor: a one-column tile, loaded as such or folded from the SD columns of a loaded tile
  int ld = loader_of(P.ops[dv].src1), SD = 1;
  if (ld < 0) {
    int const rd = producer(P.ops[dv].src1);
    if (rd < 0 || P.ops[rd].kind != DOP_REDUCE || P.ops[rd].red_inner != 1) {
      return false;
    }
    ld = loader_of(P.ops[rd].src0);
    if (ld < 0) {
      return false;
    }
    SD = P.ops[rd].red_deg;
    used++;
  }
  DevTensor const &td = P.t[P.ops[ld].dst], &tden = P.t[P.ops[dv].src1];
  if (td.cols != SD || tden.cols != 1 || tden.rows != td.rows) {
    return false;
  }
  // a fold over S pieces of X columns
  auto to_dimx = [&](DevOp const &r, int &S, int &X) {
    DevTensor const &ti = P.t[r.src0], &to = P.t[r.dst];
    S = r.red_deg;
    X = r.red_inner;
    return r.kind == DOP_REDUCE && to.rows == ti.rows && to.cols == X && ti.cols == S * X && S >= 1;
  };
  int ln = loader_of(P.ops[dv].src0), S = 1, X = 0, mode;
  if (ln < 0) {
    // sum, then divide
    int const rn = producer(P.ops[dv].src0);
    if (rn < 0 || !to_dimx(P.ops[rn], S, X) || out.src0 != P.ops[dv].dst || F != 1) {
      return false;
    }
    ln = loader_of(P.ops[rn].src0);
    mode = SUM_THEN_DIV;
    used++;
  } else if (out.src0 == P.ops[dv].dst) {
    // divide, then the saver accumulates over the for-loop
    mode = DIV_THEN_SAVE;
    S = F;
    X = P.t[P.ops[ln].dst].cols;
  } else {
    // divide, then sum
    int const rn = producer(out.src0);
    if (rn < 0 || !to_dimx(P.ops[rn], S, X) || P.ops[rn].src0 != P.ops[dv].dst || F != 1) {
      return false;
    }
    mode = DIV_THEN_SUM;
    used++;
  }
  if (ln < 0 || ln == ld || used != P.num_ops - 3) {
    return false;
  }
  DevOp const &opn = P.ops[ln], &opd = P.ops[ld];
  DevTensor const &tn = P.t[opn.dst], &to = P.t[out.src0];
  int const pieces = mode == DIV_THEN_SAVE ? 1 : S;
  if (tn.rows != td.rows || tn.cols != pieces * X || to.rows != tn.rows || to.cols != X ||
      P.t[P.ops[dv].dst].cols != (mode == SUM_THEN_DIV ? X : tn.cols)) {
    return false;
  }
  // the divisor does not move with the for-loop; the numerator may (one piece an iteration)
  // (the strides of a single iteration mean nothing)
  if (F > 1 && (opd.row_fs != 0 || opd.col_fs != 0 || opd.g_fs != 0)) {
    return false;
  }
  M.step = mode != DIV_THEN_SAVE ? X
           : F > 1 ? (long long)opn.g_fs + (long long)opn.row_fs * opn.d_cols + opn.col_fs
                   : 0;
  M.vec = X % 8 == 0 ? 8 : (X % 4 == 0 ? 4 : 0);
  if (M.vec == 0 || M.step % M.vec != 0 || !aligned(ctile(opn, P.in[opn.io]), M.vec) ||
      !aligned(ctile(out, P.out[out.io]), M.vec)) {
    return false;
  }
  M.ln = ln;
  M.ld = ld;
  M.out = last;
  M.rows = tn.rows;
  M.X = X;
  M.S = S;
  M.SD = SD;
  M.mode = mode;
  return true;
}

}  // namespace

bool combine_applicable(DevProgram const &P) {
  CMatch M;
  return cmatch(P, M);
}

int try_launch_combine(DevProgram const &P) {
  CMatch M;
  if (!cmatch(P, M)) {
    return 0;
  }
  State &s = state();
  CombineParams A{};
  A.n = ctile(P.ops[M.ln], P.in[P.ops[M.ln].io]);
  A.d = ctile(P.ops[M.ld], P.in[P.ops[M.ld].io]);
  A.o = ctile(P.ops[M.out], P.out[P.ops[M.out].io]);
  A.rows = M.rows;
  A.X = M.X;
  A.S = M.S;
  A.SD = M.SD;
  A.step = M.step;
  A.mxv = fast_div_magic(M.X / M.vec);
  dim3 grid(P.grid[0], P.grid[1], P.grid[2]);
  // a fold of a few MB is a chain of trips to the L2 (deep batches pay); a larger one runs at
  // the memory's rate (four pieces in flight per thread: 7.4 against 14.6 us on 34 MB)
  long long const piece_bytes = (long long)grid.x * grid.y * grid.z * M.rows * M.X * 2;
  // (whole batches only: what is left over is folded piece by piece)
  int const batch = piece_bytes * M.S <= (4LL << 20) && std::max(M.S, M.SD) >= 16 ? 16 : 4;
  if (EmitSink *sink = emit_sink()) {
    // the launch as C++ source (for programs that Graph::generate_hip_program writes)
    auto tile = [](CTile const &t) {
      return emit_fmt("mi355::CTile{%s, {%lldLL, %lldLL, %lldLL}, %d}", emit_pointer(t.ptr).c_str(), t.lin[0], t.lin[1],
                      t.lin[2], t.d_cols);
    };
    std::string lit = "    mi355::CombineParams P{};\n";
    lit += "    P.n = " + tile(A.n) + ";\n    P.d = " + tile(A.d) + ";\n    P.o = " + tile(A.o) + ";\n";
    lit += emit_fmt("    P.rows = %d;\n    P.X = %d;\n    P.S = %d;\n    P.SD = %d;\n    P.step = %lldLL;\n    P.mxv = %uu;\n",
                    A.rows, A.X, A.S, A.SD, A.step, A.mxv);
    sink->headers |= 4u;
    emit_launch(*sink, "combine_fused_kernel", emit_fmt("%d, %d, %d", M.vec == 8 ? 8 : 4, M.mode, batch), grid, 256, 0, lit);
    return 1;
  }
  hipStream_t const q = s.stream();
#define MI355_COMBINE_CASE(VECV, MODEV, BATCHV)                                  \
  if ((M.vec == 8 ? 8 : 4) == VECV && M.mode == MODEV && batch == BATCHV) {      \
    combine_fused_kernel<VECV, MODEV, BATCHV><<<grid, 256, 0, q>>>(A);           \
  }
  MI355_COMBINE_CASE(8, SUM_THEN_DIV, 4)
  MI355_COMBINE_CASE(8, DIV_THEN_SUM, 4)
  MI355_COMBINE_CASE(8, DIV_THEN_SAVE, 4)
  MI355_COMBINE_CASE(4, SUM_THEN_DIV, 4)
  MI355_COMBINE_CASE(4, DIV_THEN_SUM, 4)
  MI355_COMBINE_CASE(4, DIV_THEN_SAVE, 4)
  MI355_COMBINE_CASE(8, SUM_THEN_DIV, 16)
  MI355_COMBINE_CASE(8, DIV_THEN_SUM, 16)
  MI355_COMBINE_CASE(8, DIV_THEN_SAVE, 16)
  MI355_COMBINE_CASE(4, SUM_THEN_DIV, 16)
  MI355_COMBINE_CASE(4, DIV_THEN_SUM, 16)
  MI355_COMBINE_CASE(4, DIV_THEN_SAVE, 16)
#undef MI355_COMBINE_CASE
  MI355_HIP(hipGetLastError());
  s.last().kernel_id = MI355_KERNEL_F16_COMBINE;
  s.last().workgroups = (int)(grid.x * grid.y * grid.z);
  s.last().threads = 256;
  s.last().lds_bytes = 0;
  s.last().row_split = 1;
  return 1;
}

}  // namespace mi355
