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
//  * one wavefront owns 16 query rows for one for-loop iteration at a time.  A
//    workgroup is RG row groups x IP iteration lanes: the IP wavefronts of a row
//    group work on IP consecutive iterations at once and hand their fp16 results to
//    the group's first wavefront, which adds them in iteration order (the order the
//    sequential loop would use).  A logical thread block's rows are split over as
//    many workgroups as it takes to fill the chip: the plan's grid is a lower bound
//    on parallelism, not the launch shape;
//  * S is produced TRANSPOSED (S^T = K^T.Q^T) with 16x16x32 fp16 MFMA, so that each
//    lane ends up holding four consecutive keys of one query row — exactly the
//    A-operand layout of the next MFMA.  exp, the row sum (two cross-lane adds) and
//    the normalisation happen on those accumulator registers; P.V consumes them
//    directly;
//  * K tiles arrive [head_dim][keys] and V tiles [keys][dv], both with the MFMA's
//    reduction index strided in memory, so they are transposed once while being
//    staged into LDS (four 16-byte global reads -> eight 8-byte LDS writes per 4x8
//    patch) and every operand fetch is one contiguous LDS read.  LDS rows are
//    unpadded; 16-byte chunks are XOR-swizzled with (row ^ row>>3) & 7, which makes
//    both the transposing writes and the operand reads spread over all banks;
//  * as many for-loop iterations as fit are staged per barrier, and every load of
//    a staging step is issued before the first one is waited for;
//  * the for-loop accumulators live in VGPRs (fp16-rounded each iteration, as the
//    reference's generated programs do) and are written once, through LDS, as full
//    16-byte row segments.
//
// This file is the host side: it recognises the family in a lowered program, chooses kernel
// and launch shape and either launches or, for Graph::generate_hip_program, prints the launch
// as source.  The kernels are in include/mi355_kernels/attention.h, which generated
// programs include as well.
#include "common.h"
#include "tb_program.h"
#include <atomic>
#include <cstdlib>
#include <string>

#include "mi355_kernels/attention.h"

namespace mi355 {

// ---------------------------------------------------------------------------------------
// host: recognise the family in a lowered program and launch
// ---------------------------------------------------------------------------------------
namespace {

// (a column-major tensor -- DevOp::sub == 1 on its loader -- holds element (r, c) at
// c * d_rows + r: a step along the rows is one element, a step along the columns d_rows, and
// `d_cols` of the result is that leading dimension)
// `fits` is cleared when a tile origin could leave 31 bits (the kernels multiply and add the
// strides in 32 bits); `extents` = the plan's grid and its for-loop range.
TileAddr tile_addr(DevOp const &op, void const *ptr, int const (&extents)[4], bool &fits) {
  TileAddr t;
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

// The parameter block as C++ source (for programs that Graph::generate_hip_program writes).
std::string literal(TileAddr const &t) {
  return emit_fmt("mi355::TileAddr{%s, {%d, %d, %d, %d}, %d}", emit_pointer(t.ptr).c_str(), t.lin[0], t.lin[1],
                  t.lin[2], t.lin[3], t.d_cols);
}
std::string literal(AttnParams const &A) {
  std::string t = "    mi355::AttnParams P{};\n";
  t += "    P.q = " + literal(A.q) + ";\n    P.k = " + literal(A.k) + ";\n    P.v = " + literal(A.v) + ";\n";
  t += "    P.o = " + literal(A.o) + ";\n    P.r = " + literal(A.r) + ";\n";
  t += emit_fmt("    P.forloop_range = %d;\n    P.split = %d;\n    P.stages = %d;\n    P.lds_stage_bytes = %d;\n",
                A.forloop_range, A.split, A.stages, A.lds_stage_bytes);
  for (int i = 0; i < 3; i++) {
    t += emit_fmt("    P.perm[%d] = %d;\n    P.perm_ext[%d] = %uu;\n    P.perm_magic[%d] = %uu;\n", i, A.perm[i], i,
                  A.perm_ext[i], i, A.perm_magic[i]);
  }
  t += emit_fmt("    P.split_magic = %uu;\n    P.rows = %d;\n    P.trace = nullptr;\n    P.r_copies = %d;\n"
                "    P.r_copy_stride = %d;\n", A.split_magic, A.rows, A.r_copies, A.r_copy_stride);
  return t;
}
char const *tf(bool b) { return b ? "true" : "false"; }

struct Match {
  int q, k, v;        // load op indices
  int out_o, out_r;   // output op indices (out_r < 0 in form A)
  bool has_div;
  int m, D, NK, DV;
  // K and V are both DmemColumnMajor (the layout every attention plan of the reference declares,
  // e.g. cpp_examples/group_query_attn_inc_decode.cc:41-44): K [D][keys] is then stored key by key
  // with the head dim contiguous, V [keys][DV] column by column with the keys contiguous, so both
  // tiles arrive with the MFMA's reduction index contiguous and no read transposes anything
  bool kv_colmajor;
};

// `pieces`: the value tile may be narrower than 16 bytes (checked by merge_column_pieces)
bool match(DevProgram const &P, Match &M, bool pieces = false) {
  if (has_column_major_saver(P) || P.num_ops < 9 || P.ops[0].kind != DOP_LOAD || P.ops[1].kind != DOP_LOAD ||
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
  // query tiles of whole 16-row groups, or a single group of 8 rows (padded with zero rows)
  if (tk.rows != M.D || tv.rows != M.NK || (M.m % 16 != 0 && M.m != 8)) {
    return false;
  }
  // Q must be loop invariant; all tiles reachable with 16-byte accesses
  DevOp const &lq = P.ops[M.q];
  if (lq.row_fs != 0 || lq.col_fs != 0 || lq.g_fs != 0) {
    return false;
  }
  // Q row-major; K and V in one storage order (a mixed pair takes the interpreter)
  if (lq.sub == 1 || P.ops[M.k].sub != P.ops[M.v].sub) {
    return false;
  }
  M.kv_colmajor = P.ops[M.k].sub == 1;
  if (!lq.galign || !P.ops[M.k].galign ||
      (!pieces && (!P.ops[M.v].galign || !P.ops[M.out_o].galign))) {
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

// A plan that cuts the value columns into pieces along one grid dimension -- every block of
// that dimension loads the same Q and K tiles, takes DV / G columns of V, stores its columns of
// the result and, in the row-sum form, its own copy of the same row sums -- computes the scores
// G times.  Column j of the result depends on column j of V only, so the G blocks are one block
// with the whole value tile: Q gets that program (grid dimension `g` of extent 1, V and the
// result 64 columns wide, the row sums stored G times).  False when P is not of this shape.
bool merge_column_pieces(DevProgram const &P, Match &M, DevProgram &Q, int &copies, int &copy_stride) {
  if (!match(P, M, true) || M.DV >= 64 || 64 % M.DV != 0) {
    return false;
  }
  int const G = 64 / M.DV;
  DevOp const &lq = P.ops[M.q], &lk = P.ops[M.k], &lv = P.ops[M.v], &oo = P.ops[M.out_o];
  for (int g = 0; g < 3; g++) {
    if (P.grid[g] != G) {
      continue;
    }
    auto free_of = [&](DevOp const &op) { return !op.row_bs[g] && !op.col_bs[g] && !op.g_bs[g]; };
    auto pieced = [&](DevOp const &op) { return !op.row_bs[g] && !op.g_bs[g] && op.col_bs[g] == M.DV; };
    if (!free_of(lq) || !free_of(lk) || !pieced(lv) || !pieced(oo)) {
      continue;
    }
    copies = 1;
    copy_stride = 0;
    if (M.out_r >= 0) {
      DevOp const &orr = P.ops[M.out_r];
      if (orr.row_bs[g] || orr.g_bs[g]) {
        continue;
      }
      copies = G;
      copy_stride = orr.col_bs[g];
    }
    Q = P;
    Q.grid[g] = 1;
    Q.ops[M.v].col_bs[g] = 0;
    Q.ops[M.out_o].col_bs[g] = 0;
    if (M.out_r >= 0) {
      Q.ops[M.out_r].col_bs[g] = 0;
    }
    // 16-byte reachability of the widened tiles
    for (int o : {M.v, M.out_o}) {
      DevOp &d = Q.ops[o];
      if (d.kind == DOP_LOAD && d.sub == 1) {
        // column-major V: a wider tile is more columns, i.e. more rows of V^T, each as
        // reachable with 16-byte accesses as before
        if (!d.galign) {
          return false;
        }
        Q.t[d.dst].cols = 64;
        continue;
      }
      bool al = d.d_cols % 8 == 0 && d.col_fs % 8 == 0 && d.g_fs % 8 == 0;
      for (int e = 0; e < 3; e++) {
        al = al && d.col_bs[e] % 8 == 0 && d.g_bs[e] % 8 == 0;
      }
      if (!al) {
        return false;
      }
      d.galign = d.vec8 = 1;
      Q.t[d.dst].cols = 64;
    }
    void const *vp = P.in[lv.io], *op = P.out[oo.io];
    if (((reinterpret_cast<uintptr_t>(vp) | reinterpret_cast<uintptr_t>(op)) & 15) != 0) {
      return false;
    }
    M.DV = 64;
    return true;
  }
  return false;
}

template <bool HAS_DIV, bool CM, int IP, int RPW, int NBUF, int NIT, int SPI, int IPS>
int launch_direct_one(AttnParams const &A, dim3 grid, int lds, bool dry) {
  if (dry) {
    return 1;  // the question was only whether this shape is built
  }
  if (EmitSink *sink = emit_sink()) {
    sink->headers |= 1u;
    emit_launch(*sink, "attn_direct_kernel",
                emit_fmt("64, 64, 64, %s, %d, %d, %d, %d, %d, %d, false, %s", tf(HAS_DIV), IP, RPW, NBUF, NIT, SPI, IPS,
                         tf(CM)),
                grid, 64 * IP, lds, literal(A));
    return 1;
  }
  auto go = [&](auto *fn) -> int {
    static std::atomic<int> granted{0};  // per instantiation
    if (lds > 65536 && lds > granted) {
      MI355_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(fn),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, state().max_lds));
      granted = state().max_lds;
    }
    fn<<<grid, 64 * IP, lds, state().stream()>>>(A);
    MI355_HIP(hipGetLastError());
    return 1;
  };
  if (SPI == 1 && IPS == 1 && A.trace != nullptr) {
    return go(attn_direct_kernel<64, 64, 64, HAS_DIV, IP, RPW, NBUF, NIT, SPI, IPS, SPI == 1 && IPS == 1, CM>);
  }
  return go(attn_direct_kernel<64, 64, 64, HAS_DIV, IP, RPW, NBUF, NIT, SPI, IPS, false, CM>);
}

// The shape of a direct-staging launch: `ip` wavefronts of `rpw` row groups each, `nbuf` tile
// pairs per wavefront, up to `nit` units of work per wavefront, `spi` strips per iteration or
// `ips` iterations per strip.
struct DirectShape {
  int ip = 0, rpw = 1, nbuf = 1, nit = 1, spi = 1, ips = 1;
  int code() const { return ((((ip * 10 + rpw) * 10 + nbuf) * 10 + nit) * 10 + spi) * 10 + ips; }
};

// 0: no instantiation for this shape
template <bool HAS_DIV, bool CM>
int launch_direct(AttnParams const &A, dim3 grid, DirectShape const &d, int lds, bool dry = false) {
#define MI355_DIRECT(IPV, RPWV, NBUFV, NITV, SPIV, IPSV) \
  case ((((IPV * 10 + RPWV) * 10 + NBUFV) * 10 + NITV) * 10 + SPIV) * 10 + IPSV: \
    return launch_direct_one<HAS_DIV, CM, IPV, RPWV, NBUFV, NITV, SPIV, IPSV>(A, grid, lds, dry);
  switch (d.code()) {
    // one 64-key tile per iteration
    MI355_DIRECT(2, 1, 1, 1, 1, 1)
    MI355_DIRECT(4, 1, 1, 1, 1, 1)
    MI355_DIRECT(8, 1, 1, 1, 1, 1)
    MI355_DIRECT(4, 2, 1, 1, 1, 1)
    MI355_DIRECT(4, 1, 2, 2, 1, 1)
    MI355_DIRECT(4, 1, 2, 4, 1, 1)
    MI355_DIRECT(4, 1, 2, 8, 1, 1)
    MI355_DIRECT(4, 1, 1, 2, 1, 1)
    MI355_DIRECT(4, 1, 1, 4, 1, 1)
    MI355_DIRECT(4, 1, 1, 8, 1, 1)
    MI355_DIRECT(8, 1, 1, 2, 1, 1)
    MI355_DIRECT(8, 1, 1, 4, 1, 1)
    // key tiles of 32 and 16: two / four iterations per strip
    MI355_DIRECT(4, 1, 1, 1, 1, 2)
    MI355_DIRECT(4, 2, 1, 1, 1, 2)
    MI355_DIRECT(8, 1, 1, 1, 1, 2)
    MI355_DIRECT(8, 1, 1, 2, 1, 2)
    MI355_DIRECT(4, 1, 1, 1, 1, 4)
    MI355_DIRECT(4, 2, 1, 1, 1, 4)
    MI355_DIRECT(8, 1, 1, 1, 1, 4)
    default: break;
  }
  if constexpr (!HAS_DIV) {
    switch (d.code()) {
      // key tiles of 128 and 256: two / four strips per iteration (no division inside)
      MI355_DIRECT(4, 1, 1, 1, 2, 1)
      MI355_DIRECT(8, 1, 1, 1, 2, 1)
      MI355_DIRECT(8, 1, 1, 2, 2, 1)
      MI355_DIRECT(8, 1, 1, 4, 2, 1)
      MI355_DIRECT(4, 1, 1, 1, 4, 1)
      MI355_DIRECT(8, 1, 1, 1, 4, 1)
      MI355_DIRECT(8, 1, 1, 2, 4, 1)
      MI355_DIRECT(8, 1, 1, 4, 4, 1)
      default: break;
    }
  }
#undef MI355_DIRECT
  return 0;
}

template <int D, int NK, int DV, bool HAS_DIV, int RG, int IP, bool CM>
int launch_one(AttnParams const &A, dim3 grid, int lds) {
  if (EmitSink *sink = emit_sink()) {
    sink->headers |= 1u;
    emit_launch(*sink, "attn_fused_kernel", emit_fmt("%d, %d, %d, %s, %d, %d, %s", D, NK, DV, tf(HAS_DIV), RG, IP, tf(CM)),
                grid, 64 * RG * IP, lds, literal(A));
    return 1;
  }
  auto *fn = attn_fused_kernel<D, NK, DV, HAS_DIV, RG, IP, CM>;
  static std::atomic<int> granted{0};  // per instantiation
  if (lds > 65536 && lds > granted) {
    MI355_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(fn),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, state().max_lds));
    granted = state().max_lds;
  }
  fn<<<grid, 64 * RG * IP, lds, state().stream()>>>(A);
  MI355_HIP(hipGetLastError());
  return 1;
}

template <int D, int NK, int DV, bool HAS_DIV, bool CM>
int launch_waves(AttnParams const &A, dim3 grid, int rg, int ip, int lds) {
  switch (rg * 16 + ip) {
    case 1 * 16 + 1: return launch_one<D, NK, DV, HAS_DIV, 1, 1, CM>(A, grid, lds);
    case 1 * 16 + 2: return launch_one<D, NK, DV, HAS_DIV, 1, 2, CM>(A, grid, lds);
    case 1 * 16 + 4: return launch_one<D, NK, DV, HAS_DIV, 1, 4, CM>(A, grid, lds);
    case 1 * 16 + 8: return launch_one<D, NK, DV, HAS_DIV, 1, 8, CM>(A, grid, lds);
    case 2 * 16 + 1: return launch_one<D, NK, DV, HAS_DIV, 2, 1, CM>(A, grid, lds);
    case 2 * 16 + 2: return launch_one<D, NK, DV, HAS_DIV, 2, 2, CM>(A, grid, lds);
    case 2 * 16 + 4: return launch_one<D, NK, DV, HAS_DIV, 2, 4, CM>(A, grid, lds);
    case 4 * 16 + 1: return launch_one<D, NK, DV, HAS_DIV, 4, 1, CM>(A, grid, lds);
    case 4 * 16 + 2: return launch_one<D, NK, DV, HAS_DIV, 4, 2, CM>(A, grid, lds);
    default: return 0;
  }
}

template <int D, int NK, int DV>
int launch_shape(AttnParams const &A, bool has_div, bool cm, dim3 grid, int rg, int ip, int lds) {
  if (cm) {
    return has_div ? launch_waves<D, NK, DV, true, true>(A, grid, rg, ip, lds)
                   : launch_waves<D, NK, DV, false, true>(A, grid, rg, ip, lds);
  }
  return has_div ? launch_waves<D, NK, DV, true, false>(A, grid, rg, ip, lds)
                 : launch_waves<D, NK, DV, false, false>(A, grid, rg, ip, lds);
}

template <int D, int NK, int DV, bool HAS_DIV, int RG, int RPW, bool CM, int SPI = 1>
int launch_stream_one(AttnParams const &A, dim3 grid, int lds) {
  if (EmitSink *sink = emit_sink()) {
    sink->headers |= 1u;
    emit_launch(*sink, "attn_stream_kernel",
                emit_fmt("%d, %d, %d, %s, %d, %d, %s, %d", D, NK, DV, tf(HAS_DIV), RG, RPW, tf(CM), SPI), grid, 64 * RG,
                lds, literal(A));
    return 1;
  }
  auto *fn = attn_stream_kernel<D, NK, DV, HAS_DIV, RG, RPW, CM, SPI>;
  if (lds > 65536) {
    MI355_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(fn),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  }
  fn<<<grid, 64 * RG, lds, state().stream()>>>(A);
  MI355_HIP(hipGetLastError());
  return 1;
}

template <int D, int NK, int DV, bool CM>
int launch_stream(AttnParams const &A, bool has_div, dim3 grid, int rg, int lds, bool wide = false, int spi = 1) {
  if (spi > 1) {  // wider key tiles: four wavefronts of 32 rows, the form without the division
    if (has_div || rg != 4 || wide) {
      return 0;
    }
    switch (spi) {
      case 2: return launch_stream_one<D, NK, DV, false, 4, 2, CM, 2>(A, grid, lds);
      case 4: return launch_stream_one<D, NK, DV, false, 4, 2, CM, 4>(A, grid, lds);
      case 8: return launch_stream_one<D, NK, DV, false, 4, 2, CM, 8>(A, grid, lds);
      default: return 0;
    }
  }
  if constexpr (D == 64) {
    if (wide) {  // four wavefronts of 64 rows
      return has_div ? launch_stream_one<D, NK, DV, true, 4, 4, CM>(A, grid, lds)
                     : launch_stream_one<D, NK, DV, false, 4, 4, CM>(A, grid, lds);
    }
  }
  if (has_div) {
    return rg == 4 ? launch_stream_one<D, NK, DV, true, 4, 2, CM>(A, grid, lds)
                   : launch_stream_one<D, NK, DV, true, 2, 2, CM>(A, grid, lds);
  }
  return rg == 4 ? launch_stream_one<D, NK, DV, false, 4, 2, CM>(A, grid, lds)
                 : launch_stream_one<D, NK, DV, false, 2, 2, CM>(A, grid, lds);
}

}  // namespace

// Fills the division magics decode_block uses for this launch grid; false when an id times an
// extent could leave 32 bits (the magics are exact only below that).
static bool set_grid_magics(AttnParams &A, dim3 grid) {
  unsigned const ext[3] = {grid.x, grid.y, grid.z};
  unsigned long long const total = (unsigned long long)grid.x * grid.y * grid.z;
  for (int i = 0; i < 3; i++) {
    unsigned const e = ext[A.perm[i]];
    if (total * e >= (1ull << 32)) {
      return false;
    }
    A.perm_ext[i] = e;
    A.perm_magic[i] = fast_div_magic((int)e);
  }
  if ((unsigned long long)grid.x * (unsigned)A.split >= (1ull << 32)) {
    return false;
  }
  A.split_magic = fast_div_magic(A.split);
  return true;
}

// Shapes the register-transposed and the throughput variants are built for.
static bool shape_supported(Match const &M) {
  return (M.m % 16 == 0 || M.m == 8) &&
         ((M.D == 64 && M.DV == 64 && (M.NK == 64 || M.NK == 128 || M.NK == 256)) ||
          (M.D == 128 && M.DV == 128 && M.NK == 64));
}

// Whether (and in which shape) the direct-staging variant takes the plan: head size 64,
// key tiles of 16 ... 256 on 64-key strips.
static bool choose_direct(DevProgram const &P, Match const &M, DirectShape &d, int &lds) {
  State &s = state();
  if (M.D != 64 || M.DV != 64 || s.attention_mode == 3 || !(M.m % 16 == 0 || M.m == 8)) {
    return false;
  }
  int const F = P.forloop_range;
  d = DirectShape{};
  if (M.NK == 16 || M.NK == 32) {
    // consecutive iterations' tiles must lie side by side: K advances by NK columns, V by NK rows
    DevOp const &lk = P.ops[M.k], &lv = P.ops[M.v];
    d.ips = 64 / M.NK;
    if (lk.col_fs != M.NK || lk.row_fs != 0 || lk.g_fs != 0 || lv.row_fs != M.NK || lv.col_fs != 0 ||
        lv.g_fs != 0 || F % d.ips != 0) {
      return false;
    }
  } else if (M.NK == 128 || M.NK == 256) {
    d.spi = M.NK / 64;
    if (M.has_div) {
      return false;
    }
  } else if (M.NK != 64) {
    return false;
  }
  int const units = F / d.ips;
  int const groups = (M.m + 15) / 16;
  long long const blocks = (long long)P.grid[0] * P.grid[1] * P.grid[2];
  auto round_nit = [](int per) { return per <= 1 ? 1 : (per <= 2 ? 2 : (per <= 4 ? 4 : 8)); };
  if ((groups == 1 && units > 1) || units > 8) {
    // a lone row group (or a loop too long for a wavefront per unit: then every row group is
    // a workgroup of its own): eight lanes with a tile pair each; four when the grid is large
    // enough to put two workgroups on every compute unit; or (DIRECT_LANES = 4, whole-tile
    // iterations only) four lanes with two tile pairs each
    int const per8 = (units + 7) / 8, per4 = (units + 3) / 4;
    if (s.direct_lanes == 4 && d.spi == 1 && d.ips == 1 && per4 <= 8 && units > 4) {
      d.ip = 4;
      d.nbuf = 2;
      d.nit = round_nit(per4) < 2 ? 2 : round_nit(per4);
    } else if (units <= 4 && d.spi == 1) {
      d.ip = units <= 2 ? 2 : 4;
      if (d.ips > 1) {
        d.ip = 4;
      }
    } else if (s.direct_lanes == 0 && blocks >= 512 && units > 4 && per4 <= 8 && d.spi == 1 && d.ips == 1) {
      // enough blocks for two workgroups on every compute unit: four single-buffered lanes (half
      // the LDS), so that one workgroup streams while its neighbour starts up or adds up its
      // results (the HBM-bound decode: 5.75 -> 6.3 TB/s)
      d.ip = 4;
      d.nit = round_nit(per4);
    } else {
      d.ip = 8;
      d.nit = round_nit(per8);
    }
  } else if (units >= 1 && units <= 8 && (groups > 1 || units == 1)) {
    // every unit on a wavefront of its own, one slab of one or two row groups per workgroup
    d.ip = units <= 2 && d.ips == 1 && d.spi == 1 ? 2 : (units <= 4 ? 4 : 8);
    if (d.ip == 4 && d.spi == 1 && groups % 2 == 0 && blocks * (groups / 2) >= 256 && s.direct_lanes != 1) {
      d.rpw = 2;
    }
    if (d.ip == 2 && units == 1) {
      return false;  // a single iteration: nothing to hand over, the other variants serve it
    }
  } else {
    return false;
  }
  int const pair_bytes = (64 * 64 + 64 * 64) * 2;
  lds = d.ip * (d.nbuf * pair_bytes + d.rpw * 16 * M.D * 2);  // + a Q tile per wavefront
  if (lds > s.max_lds || (long long)P.grid[0] * (groups / d.rpw) > 2147483647LL) {
    return false;
  }
  AttnParams none{};
  return (M.has_div ? launch_direct<true, false>(none, dim3(1, 1, 1), d, lds, true)
                    : launch_direct<false, false>(none, dim3(1, 1, 1), d, lds, true)) == 1;
}

// Whether (and in which shape) the throughput variant takes the plan: query tiles of whole
// 64- or 128-row slabs, enough of them to fill the chip twice over, a for-loop long enough to
// pipeline; key tiles of 64 keys, or (the form without the division, 128-row slabs) of 128 / 256 /
// 512 keys walked as strips of 64.
struct StreamShape {
  int rgs = 0, spi = 1;
  bool wide = false;
};
static bool choose_stream(DevProgram const &P, Match const &M, StreamShape &st) {
  State &s = state();
  st = StreamShape{};
  if (s.attention_mode == 1 || s.attention_mode == 3) {
    return false;
  }
  long long const blocks_all = (long long)P.grid[0] * P.grid[1] * P.grid[2];
  int const slabs = M.m / 32;
  st.rgs = (M.m % 128 == 0) ? 4 : ((M.m % 64 == 0) ? 2 : 0);
  bool const heads = (M.D == 64 && M.DV == 64) || (M.D == 128 && M.DV == 128);
  if (st.rgs == 0 || !heads) {
    return false;
  }
  if (M.NK == 128 || M.NK == 256 || M.NK == 512) {
    st.spi = M.NK / 64;
    if (M.has_div || st.rgs != 4) {
      return false;
    }
  } else if (M.NK != 64) {
    return false;
  }
  // (64-key tiles on a small grid are better served by the latency variants; wider key tiles
  // have no other kernel, so they take this one whatever the grid)
  if (s.attention_mode != 2 && st.spi == 1 &&
      !(P.forloop_range >= 2 && blocks_all * (slabs / st.rgs) >= 512)) {
    return false;
  }
  // Head size 64 with 256-row query tiles and enough of them for two wavefronts per SIMD:
  // wavefronts of 64 rows (half the LDS operand reads per MFMA; at head size 64 the registers
  // still fit two wavefronts per SIMD).  Measured on the 32-group x 16,384-key decode plan:
  // 68.8 -> 67.0 us.
  st.wide = st.spi == 1 && M.D == 64 && M.m % 256 == 0 &&
            (s.attention_mode == 2 || blocks_all * (M.m / 64) >= 2048);
  if (st.wide) {
    st.rgs = 8;
  }
  return true;
}

bool attention_applicable(DevProgram const &P) {
  Match M;
  DirectShape d;
  StreamShape st;
  int lds = 0;
  if (match(P, M) && (shape_supported(M) || choose_stream(P, M, st) || choose_direct(P, M, d, lds))) {
    return true;
  }
  DevProgram merged;
  int copies = 1, stride = 0;
  return merge_column_pieces(P, M, merged, copies, stride) && choose_direct(merged, M, d, lds);
}

int try_launch_attention(DevProgram const &P0) {
  Match M;
  DevProgram merged;
  DevProgram const *run = &P0;
  int r_copies = 1, r_copy_stride = 0;
  // as the plan states it, or (value tiles narrower than 64 columns) with its column pieces merged
  bool pieces = !match(P0, M);
  if (!pieces) {
    DirectShape probe;
    StreamShape probe_stream;
    int probe_lds = 0;
    pieces = !shape_supported(M) && !choose_stream(P0, M, probe_stream) &&
             !choose_direct(P0, M, probe, probe_lds);
  }
  if (pieces) {
    if (!merge_column_pieces(P0, M, merged, r_copies, r_copy_stride)) {
      return 0;
    }
    run = &merged;
  }
  DevProgram const &P = *run;
  DirectShape dshape;
  int direct_lds = 0;
  bool const direct = choose_direct(P, M, dshape, direct_lds);
  StreamShape stream_probe;
  bool const stream = !pieces && choose_stream(P, M, stream_probe);
  if (!direct && !stream && (pieces || !shape_supported(M))) {
    return 0;  // (only the direct-staging variant stores copies of the row sums)
  }
  State &s = state();
  AttnParams A;
  A.r_copies = r_copies;
  A.r_copy_stride = r_copy_stride;
  int const extents[4] = {P.grid[0], P.grid[1], P.grid[2], P.forloop_range};
  bool fits = true;
  A.q = tile_addr(P.ops[M.q], P.in[P.ops[M.q].io], extents, fits);
  A.k = tile_addr(P.ops[M.k], P.in[P.ops[M.k].io], extents, fits);
  A.v = tile_addr(P.ops[M.v], P.in[P.ops[M.v].io], extents, fits);
  A.o = tile_addr(P.ops[M.out_o], P.out[P.ops[M.out_o].io], extents, fits);
  A.r = M.out_r >= 0 ? tile_addr(P.ops[M.out_r], P.out[P.ops[M.out_r].io], extents, fits) : A.o;
  if (!fits) {
    return 0;  // a tensor of more than 2^31 elements: the generic interpreter takes the plan
  }
  A.forloop_range = P.forloop_range;
  A.rows = M.m < 16 ? M.m : 16;
  A.trace = nullptr;
  {
    // grid dims the K / V tiles do not depend on vary fastest in the workgroup id
    int n = 0;
    bool dep[3];
    for (int d = 0; d < 3; d++) {
      DevOp const &lk = P.ops[M.k], &lv = P.ops[M.v];
      dep[d] = lk.row_bs[d] || lk.col_bs[d] || lk.g_bs[d] || lv.row_bs[d] || lv.col_bs[d] || lv.g_bs[d];
    }
    for (int d = 0; d < 3; d++) {
      if (!dep[d]) {
        A.perm[n++] = d;
      }
    }
    for (int d = 0; d < 3; d++) {
      if (dep[d]) {
        A.perm[n++] = d;
      }
    }
  }
  // ---- throughput variant
  {
    StreamShape st;
    if (!pieces && choose_stream(P, M, st)) {
      int const slabs = M.m / 32, rgs = st.rgs;
      A.split = slabs / rgs;
      A.stages = 2;
      A.lds_stage_bytes = (64 * M.D + M.DV * 64) * 2;  // one strip of 64 keys of K and of V
      int const out_bytes = rgs * 32 * (M.DV + 8) * 2;
      int lds = 2 * A.lds_stage_bytes;
      lds = lds > out_bytes ? lds : out_bytes;
      if (lds <= s.max_lds && (long long)P.grid[0] * A.split <= 2147483647LL) {
        dim3 grid(P.grid[0] * A.split, P.grid[1], P.grid[2]);
        if (!set_grid_magics(A, grid)) {
          return 0;
        }
        int rc;
        if (M.kv_colmajor) {
          rc = M.D == 64 ? launch_stream<64, 64, 64, true>(A, M.has_div, grid, rgs, lds, st.wide, st.spi)
                         : launch_stream<128, 64, 128, true>(A, M.has_div, grid, rgs, lds, false, st.spi);
        } else {
          rc = M.D == 64 ? launch_stream<64, 64, 64, false>(A, M.has_div, grid, rgs, lds, st.wide, st.spi)
                         : launch_stream<128, 64, 128, false>(A, M.has_div, grid, rgs, lds, false, st.spi);
        }
        if (rc == 1) {
          s.last().kernel_id = MI355_KERNEL_F16_ATTENTION;
          s.last().workgroups = grid.x * grid.y * grid.z;
          s.last().threads = st.wide ? 256 : rgs * 64;
          s.last().lds_bytes = lds;
          s.last().row_split = A.split;
        }
        if (rc != 0) {
          return rc;
        }
      }
    }
  }

  // ---- direct-staging variant (attention mode 3 keeps the register-transposed staging):
  // head size 64, key tiles of 16 ... 256, in two situations.
  // (a) Every unit of work (an iteration, or a 64-key strip of several) has a wavefront of
  //     its own.  A wavefront takes two row groups when that still puts a workgroup on every
  //     compute unit: each K / V operand read from LDS then feeds two MFMAs and half as many
  //     wavefronts stream the tiles (C2: 256 workgroups of 4 wavefronts x 32 rows; the
  //     L2 -> LDS traffic and the LDS reads, both per-CU bandwidth limits at this size, halve).
  // (b) A lone row group (decode: 8 or 16 query rows) with a longer for-loop: eight
  //     wavefronts that each stream every eighth unit through a tile pair of their own, or
  //     (DIRECT_LANES = 4) four wavefronts with two tile pairs each.
  if (direct) {
    int const groups = (M.m + 15) / 16;
    AttnParams B = A;
    B.split = groups / dshape.rpw;
    B.trace = s.phase_trace;
    dim3 const direct_grid(P.grid[0] * B.split, P.grid[1], P.grid[2]);
    if (set_grid_magics(B, direct_grid)) {
      if (B.trace != nullptr && (size_t)direct_grid.x * direct_grid.y * direct_grid.z * dshape.ip * 6 * 8 >
                                    s.phase_trace_bytes) {
        B.trace = nullptr;
      }
      int const rc = M.kv_colmajor
                         ? (M.has_div ? launch_direct<true, true>(B, direct_grid, dshape, direct_lds)
                                      : launch_direct<false, true>(B, direct_grid, dshape, direct_lds))
                         : (M.has_div ? launch_direct<true, false>(B, direct_grid, dshape, direct_lds)
                                      : launch_direct<false, false>(B, direct_grid, dshape, direct_lds));
      if (rc != 0) {
        if (rc == 1) {
          s.last().kernel_id = MI355_KERNEL_F16_ATTENTION;
          s.last().workgroups = direct_grid.x * direct_grid.y * direct_grid.z;
          s.last().threads = dshape.ip * 64;
          s.last().lds_bytes = direct_lds;
          s.last().row_split = B.split;
        }
        return rc;
      }
    }
    if (pieces || !shape_supported(M)) {
      return 0;
    }
  }

  if (pieces || !shape_supported(M)) {
    return 0;  // (a shape only the throughput variant is built for)
  }
  // Row groups per workgroup: up to 4, fewer when that is what it takes to put a
  // workgroup on every compute unit.  Iteration lanes: whatever is left of 8
  // wavefronts, at most the for-loop range.
  int const groups = (M.m + 15) / 16;
  int rg = groups % 4 == 0 ? 4 : (groups % 2 == 0 ? 2 : 1);
  long long const blocks = (long long)P.grid[0] * P.grid[1] * P.grid[2];
  while (rg > 1 && blocks * (groups / rg) < 256) {
    rg /= 2;
  }
  int ip = 1;
  while (ip * 2 * rg <= 8 && ip * 2 <= P.forloop_range) {
    ip *= 2;
  }
  A.split = groups / rg;
  if ((long long)P.grid[0] * A.split > 2147483647LL) {
    return 0;
  }
  int const stage_bytes = (M.NK * M.D + M.DV * M.NK) * 2;
  int const tail_bytes = rg * 16 * (M.DV + 8) * 2 + rg * (ip - 1) * (M.DV / 8 + 1) * 64 * 4;
  int stages = (96 * 1024 - tail_bytes) / stage_bytes;
  stages = stages < 1 ? 1 : (stages > P.forloop_range ? P.forloop_range : stages);
  if (stages >= ip) {
    stages -= stages % ip;  // whole rounds per staging step
  } else {
    ip = 1;
    while (ip * 2 <= stages) {
      ip *= 2;
    }
    stages = ip;
  }
  A.stages = stages;
  A.lds_stage_bytes = stage_bytes;
  int lds = stages * stage_bytes + tail_bytes;
  if (lds > s.max_lds) {
    return 0;
  }
  dim3 grid(P.grid[0] * A.split, P.grid[1], P.grid[2]);
  int const nw = rg * ip;
  int rc = 0;
  if (!set_grid_magics(A, grid)) {
    return 0;
  }
  if (M.D == 64 && M.NK == 64) {
    rc = launch_shape<64, 64, 64>(A, M.has_div, M.kv_colmajor, grid, rg, ip, lds);
  } else if (M.D == 64 && M.NK == 128) {
    rc = launch_shape<64, 128, 64>(A, M.has_div, M.kv_colmajor, grid, rg, ip, lds);
  } else if (M.D == 64 && M.NK == 256) {
    rc = launch_shape<64, 256, 64>(A, M.has_div, M.kv_colmajor, grid, rg, ip, lds);
  } else {
    rc = launch_shape<128, 64, 128>(A, M.has_div, M.kv_colmajor, grid, rg, ip, lds);
  }
  if (rc == 1) {
    s.last().kernel_id = MI355_KERNEL_F16_ATTENTION;
    s.last().workgroups = grid.x * grid.y * grid.z;
    s.last().threads = nw * 64;
    s.last().lds_bytes = lds;
    s.last().row_split = A.split;
  }
  return rc;
}

}  // namespace mi355
