// Host-side lowering of an mi355_plan (the reference's NewKernelParams bytecode,
// produced by threadblock::Graph::get_new_kernel_params, reference
// src/threadblock/graph.cc:68-432) into a DevProgram for the interpreter kernels.
#include "common.h"
#include "tb_program.h"

#include <algorithm>
#include <cstring>
#include <map>
#include <vector>

namespace mi355 {

namespace {

struct TensorInfo {
  int rows = 0, cols = 0;
  int def_op = 0, last_use = 0;
  bool persistent = false;
  bool as_a = false, as_b = false;
  int declared = 299;  // loader tiles: the plan's stensor layout word (SmemUnknownLayout otherwise)
  bool dmem_colmajor = false;  // loader tiles (fp16): the device tensor is stored column by column
  int bytes = 0;
};

// Declared thread-block layouts (values of the reference's include/mirage/layout.h:37-47):
// 200 / 202-204 are the row-major family, 201 / 205-207 the column-major one; the
// TensorOpMultiplicand_Crosswise{16,32,64} members pad by 4 / 8 / 16 halfs.
constexpr int kDmemColumnMajor = 101;  // include/mirage/layout.h:28-34
bool declared_known(int l) { return l >= 200 && l <= 207; }
bool declared_column_major(int l) { return l == 201 || (l >= 205 && l <= 207); }
int declared_pad(int l) {
  switch (l) {
    case 202: case 205: return 4;
    case 203: case 206: return 8;
    case 204: case 207: return 16;
    default: return 0;
  }
}

std::string fmt(char const *f, ...) {
  char buf[256];
  va_list ap;
  va_start(ap, f);
  vsnprintf(buf, sizeof(buf), f, ap);
  va_end(ap);
  return buf;
}

int round_up(int x, int a) { return (x + a - 1) / a * a; }

}  // namespace

static int compile_plan_padded(mi355_plan const &plan, bool f16, int pad, int max_lds,
                               DevProgram &prog, PlanExtents &ext, std::string &err,
                               bool declared_layouts);

int compile_plan(mi355_plan const &plan, bool f16, int max_lds, DevProgram &prog,
                 PlanExtents &ext, std::string &err, bool declared_layouts) {
  // fp16 tiles are padded by 8 halfs per row to spread 16-byte reads over the LDS
  // banks; a graph that only fits unpadded runs unpadded
  int rc = compile_plan_padded(plan, f16, 8, max_lds, prog, ext, err, declared_layouts);
  if (rc == MI355_ERR_UNSUPPORTED && f16 && prog.lds_bytes > max_lds) {
    rc = compile_plan_padded(plan, f16, 0, max_lds, prog, ext, err, declared_layouts);
  }
  return rc;
}

static int compile_plan_padded(mi355_plan const &plan, bool f16, int pad, int max_lds,
                               DevProgram &prog, PlanExtents &ext, std::string &err,
                               bool declared_layouts) {
  memset(&prog, 0, sizeof(prog));
  memset(&ext, 0, sizeof(ext));
  if (plan.num_operators < 1 || plan.num_operators > MI355_MAX_OPERATORS ||
      plan.num_parameters < 0 || plan.num_parameters > MI355_MAX_PARAMETERS ||
      plan.num_dmem_inputs < 0 || plan.num_dmem_inputs > MI355_MAX_DMEM_INPUTS ||
      plan.num_dmem_outputs < 0 || plan.num_dmem_outputs > MI355_MAX_DMEM_OUTPUTS) {
    err = "plan counts out of range";
    return MI355_ERR_INVALID;
  }
  for (int g = 0; g < 3; g++) {
    if (plan.grid_dim[g] < 1) {
      err = "grid_dim must be positive";
      return MI355_ERR_INVALID;
    }
    prog.grid[g] = plan.grid_dim[g];
  }
  if (plan.grid_dim[1] > 65535 || plan.grid_dim[2] > 65535) {
    err = "grid_dim.y/z exceed 65535";
    return MI355_ERR_UNSUPPORTED;
  }
  if (plan.forloop_range < 1) {
    err = "forloop_range must be positive";
    return MI355_ERR_INVALID;
  }
  int const F = plan.forloop_range;
  prog.forloop_range = F;
  prog.num_ops = plan.num_operators;

  std::vector<TensorInfo> T;
  std::map<int, int> by_offset;  // plan smem offset -> tensor id (latest definition)
  auto lookup = [&](int voff, int op) -> int {
    auto it = by_offset.find(voff);
    if (it == by_offset.end()) {
      return -1;
    }
    T[it->second].last_use = op;
    return it->second;
  };
  auto define = [&](int voff, int rows, int cols, int op) -> int {
    if ((int)T.size() >= kMaxTensors) {
      return -1;
    }
    TensorInfo ti;
    ti.rows = rows;
    ti.cols = cols;
    ti.def_op = op;
    ti.last_use = op;
    T.push_back(ti);
    by_offset[voff] = (int)T.size() - 1;
    return (int)T.size() - 1;
  };

  int const *P = plan.parameters;
  int pi = 0, n_in = 0, n_out = 0;
  int const out_start = plan.num_operators - plan.num_dmem_outputs;
  for (int o = 0; o < plan.num_operators; o++) {
    DevOp &d = prog.ops[o];
    d.src0 = d.src1 = d.dst = -1;
    int const t = plan.operator_types[o];
    auto need = [&](int n) { return pi + n <= plan.num_parameters; };
    if (t == TB_INPUT_OP) {
      if (!need(19) || n_in >= plan.num_dmem_inputs || o != n_in) {
        err = "input loader out of place or truncated";
        return MI355_ERR_INVALID;
      }
      int const *q = P + pi;
      pi += 19;
      d.kind = DOP_LOAD;
      d.io = n_in++;
      for (int g = 0; g < 3; g++) {
        d.row_bs[g] = q[g];
        d.col_bs[g] = q[3 + g];
        d.g_bs[g] = q[8 + g];
      }
      d.row_fs = q[6];
      d.col_fs = q[7];
      d.g_fs = q[11];
      d.d_rows = q[12];
      d.d_cols = q[13];
      int rows = q[14], cols = q[15];
      if (rows < 1 || cols < 1 || d.d_rows < 1 || d.d_cols < 1) {
        err = "input tile shape must be positive";
        return MI355_ERR_INVALID;
      }
      d.dst = define(q[18], rows, cols, o);
      if (d.dst >= 0) {
        T[d.dst].declared = q[17];
        T[d.dst].dmem_colmajor = f16 && q[16] == kDmemColumnMajor;
      }
      d.hoist = (F == 1) || (d.row_fs == 0 && d.col_fs == 0 && d.g_fs == 0);
      // The fp16 data of a DmemColumnMajor tensor is stored column by column (element (r, c)
      // of a [R, C] matrix at c * R + r), as the reference's fp16 loader reads it
      // (include/mirage/threadblock/cuda/input_loader.h:221-247); fingerprint buffers are
      // row-major whatever the declaration (input_loader.h:457-467).
      bool const colmajor = f16 && q[16] == kDmemColumnMajor;
      d.sub = colmajor ? 1 : 0;
      long long max_row = (long long)(F - 1) * d.row_fs + rows - 1;
      long long max_col = (long long)(F - 1) * d.col_fs + cols - 1;
      long long max_g = (long long)(F - 1) * d.g_fs;
      // 16-byte pieces run along the contiguous direction: columns, or rows when column-major
      bool al = colmajor ? (rows % 8 == 0 && d.d_rows % 8 == 0 && d.row_fs % 8 == 0 && d.g_fs % 8 == 0)
                         : (cols % 8 == 0 && d.d_cols % 8 == 0 && d.col_fs % 8 == 0 && d.g_fs % 8 == 0);
      for (int g = 0; g < 3; g++) {
        long long b = plan.grid_dim[g] - 1;
        if (d.row_bs[g] < 0 || d.col_bs[g] < 0 || d.g_bs[g] < 0) {
          err = "negative loader stride";
          return MI355_ERR_INVALID;
        }
        max_row += b * d.row_bs[g];
        max_col += b * d.col_bs[g];
        max_g += b * d.g_bs[g];
        al = al && (colmajor ? d.row_bs[g] : d.col_bs[g]) % 8 == 0 && d.g_bs[g] % 8 == 0;
      }
      if (d.row_fs < 0 || d.col_fs < 0 || d.g_fs < 0) {
        err = "negative loader stride";
        return MI355_ERR_INVALID;
      }
      if (max_row >= d.d_rows || max_col >= d.d_cols) {
        err = fmt("input %d: tile walks outside its %dx%d matrix", d.io, d.d_rows, d.d_cols);
        return MI355_ERR_INVALID;
      }
      d.vec8 = al ? 1 : 0;
      d.galign = d.vec8;
      ext.in_elems[d.io] = colmajor ? max_g + max_col * d.d_rows + max_row + 1
                                    : max_g + max_row * d.d_cols + max_col + 1;
    } else if (t == TB_OUTPUT_OP) {
      if (!need(17) || o < out_start) {
        err = "output saver out of place or truncated";
        return MI355_ERR_INVALID;
      }
      int const *q = P + pi;
      pi += 17;
      d.kind = DOP_OUTPUT;
      d.io = n_out++;
      for (int g = 0; g < 3; g++) {
        d.row_bs[g] = q[g];
        d.col_bs[g] = q[3 + g];
        d.g_bs[g] = q[6 + g];
      }
      d.d_rows = q[9];
      d.d_cols = q[10];
      int rows = q[11], cols = q[12];
      d.src0 = lookup(q[15], o);
      if (d.src0 < 0 || T[d.src0].rows != rows || T[d.src0].cols != cols) {
        err = "output saver input does not name a tile of its shape";
        return MI355_ERR_INVALID;
      }
      d.dst = define(q[16], rows, cols, o);
      // a DmemColumnMajor result is stored column by column, as the reference's fp16 saver does
      // (include/mirage/threadblock/cuda/output_saver.h:252-290); element by element here
      bool const colmajor = f16 && q[13] == kDmemColumnMajor;
      d.sub = colmajor ? 1 : 0;
      long long max_row = rows - 1, max_col = cols - 1, max_g = 0;
      bool al = !colmajor && cols % 8 == 0 && d.d_cols % 8 == 0;
      for (int g = 0; g < 3; g++) {
        long long b = plan.grid_dim[g] - 1;
        if (d.row_bs[g] < 0 || d.col_bs[g] < 0 || d.g_bs[g] < 0) {
          err = "negative saver stride";
          return MI355_ERR_INVALID;
        }
        max_row += b * d.row_bs[g];
        max_col += b * d.col_bs[g];
        max_g += b * d.g_bs[g];
        al = al && d.col_bs[g] % 8 == 0 && d.g_bs[g] % 8 == 0;
      }
      if (max_row >= d.d_rows || max_col >= d.d_cols) {
        err = fmt("output %d: tile walks outside its %dx%d matrix", d.io, d.d_rows, d.d_cols);
        return MI355_ERR_INVALID;
      }
      d.vec8 = al ? 1 : 0;
      d.galign = d.vec8;
      ext.out_elems[d.io] = colmajor ? max_g + max_col * d.d_rows + max_row + 1
                                     : max_g + max_row * d.d_cols + max_col + 1;
    } else if (t == TB_MATMUL_OP) {
      if (!need(6)) {
        err = "matmul truncated";
        return MI355_ERR_INVALID;
      }
      int m = P[pi], n = P[pi + 1], k = P[pi + 2];
      d.kind = DOP_MATMUL;
      d.src0 = lookup(P[pi + 3], o);
      d.src1 = lookup(P[pi + 4], o);
      if (d.src0 < 0 || d.src1 < 0 || T[d.src0].rows != m || T[d.src0].cols != k ||
          T[d.src1].rows != k || T[d.src1].cols != n || m < 1 || n < 1 || k < 1) {
        err = "matmul operands do not match m, n, k";
        return MI355_ERR_INVALID;
      }
      T[d.src0].as_a = true;
      T[d.src1].as_b = true;
      d.dst = define(P[pi + 5], m, n, o);
      pi += 6;
    } else if (t == TB_EXP_OP || t == TB_SILU_OP) {
      if (!need(2)) {
        err = "unary truncated";
        return MI355_ERR_INVALID;
      }
      d.kind = DOP_UNARY;
      d.sub = t;
      d.src0 = lookup(P[pi], o);
      if (d.src0 < 0 || T[d.src0].rows * T[d.src0].cols != P[pi + 1]) {
        err = "unary operand does not match its element count";
        return MI355_ERR_INVALID;
      }
      d.dst = d.src0;  // in place (reference src/threadblock/element_unary.cc:46)
      pi += 2;
    } else if (t == TB_ADD_OP || t == TB_MUL_OP || t == TB_DIV_OP) {
      if (!need(9)) {
        err = "binary truncated";
        return MI355_ERR_INVALID;
      }
      int const *q = P + pi;
      pi += 9;
      if (q[0] != 1 || q[3] != 1) {
        err = "binary operands with a leading dim > 1 are not supported";
        return MI355_ERR_UNSUPPORTED;
      }
      d.kind = DOP_BINARY;
      d.sub = t;
      d.src0 = lookup(q[6], o);
      d.src1 = lookup(q[7], o);
      if (d.src0 < 0 || d.src1 < 0 || T[d.src0].rows != q[1] || T[d.src0].cols != q[2] ||
          T[d.src1].rows != q[4] || T[d.src1].cols != q[5]) {
        err = "binary operands do not match their shapes";
        return MI355_ERR_INVALID;
      }
      int rows = std::max(q[1], q[4]), cols = std::max(q[2], q[5]);
      if ((q[1] != rows && q[1] != 1) || (q[4] != rows && q[4] != 1) ||
          (q[2] != cols && q[2] != 1) || (q[5] != cols && q[5] != 1)) {
        err = "binary operands are not broadcastable";
        return MI355_ERR_INVALID;
      }
      d.dst = define(q[8], rows, cols, o);
    } else if (t >= TB_REDUCTION_0_OP && t <= TB_REDUCTION_2_TO_DIMX_OP) {
      if (!need(5)) {
        err = "reduction truncated";
        return MI355_ERR_INVALID;
      }
      int n_o = P[pi], deg = P[pi + 1], inner = P[pi + 2];
      d.kind = DOP_REDUCE;
      d.src0 = lookup(P[pi + 3], o);
      if (d.src0 < 0 || n_o < 1 || deg < 1 || inner < 1) {
        err = "reduction operand missing";
        return MI355_ERR_INVALID;
      }
      int R = T[d.src0].rows, C = T[d.src0].cols;
      int orows, ocols;
      if (n_o % R == 0 && inner == n_o / R && (long long)inner * deg == C) {
        orows = R;  // reduce along columns down to `inner` columns
        ocols = inner;
      } else if (inner == n_o && n_o % C == 0 && (long long)(n_o / C) * deg == R) {
        orows = n_o / C;  // reduce along rows
        ocols = C;
      } else {
        err = "reduction shape is not a row or column reduction of a 2-D tile";
        return MI355_ERR_UNSUPPORTED;
      }
      d.red_deg = deg;
      d.red_inner = inner;
      d.dst = define(P[pi + 4], orows, ocols, o);
      pi += 5;
    } else if (t >= TB_CONCAT_0_OP && t <= TB_CONCAT_2_OP) {
      if (!need(7)) {
        err = "concat truncated";
        return MI355_ERR_INVALID;
      }
      int n_o = P[pi], a = P[pi + 1], b = P[pi + 2], inner = P[pi + 3];
      d.kind = DOP_CONCAT;
      d.src0 = lookup(P[pi + 4], o);
      d.src1 = lookup(P[pi + 5], o);
      if (d.src0 < 0 || d.src1 < 0) {
        err = "concat operand missing";
        return MI355_ERR_INVALID;
      }
      TensorInfo const &A = T[d.src0], &B = T[d.src1];
      int orows, ocols;
      if (inner == 1 && A.cols == a && B.cols == b && A.rows == B.rows) {
        orows = A.rows;
        ocols = a + b;
      } else if (inner == A.cols && A.cols == B.cols && A.rows == a && B.rows == b) {
        orows = a + b;
        ocols = A.cols;
      } else {
        err = "concat is not along the rows or columns of a 2-D tile";
        return MI355_ERR_UNSUPPORTED;
      }
      if (n_o != orows * ocols) {
        err = "concat element count mismatch";
        return MI355_ERR_INVALID;
      }
      d.cat_a = a;
      d.cat_b = b;
      d.cat_inner = inner;
      d.dst = define(P[pi + 6], orows, ocols, o);
      pi += 7;
    } else {
      err = fmt("unsupported thread-block operator %d", t);
      return MI355_ERR_UNSUPPORTED;
    }
    if (d.dst < 0) {
      err = "too many tensors in one thread-block graph";
      return MI355_ERR_UNSUPPORTED;
    }
  }
  if (pi != plan.num_parameters || n_in != plan.num_dmem_inputs ||
      n_out != plan.num_dmem_outputs) {
    err = "parameter stream does not match the operator list";
    return MI355_ERR_INVALID;
  }

  // A loader whose tile an operator overwrites in place (exp / silu) runs every iteration even
  // when its origin does not move with the for-loop: the reference reloads every input tile in
  // every iteration (customized_kernel.cu:51-56, 323-328), so iteration i must see f(tile), not
  // f applied i + 1 times to what iteration 0 loaded.
  if (F > 1) {
    for (int o = 0; o < prog.num_ops; o++) {
      DevOp const &u = prog.ops[o];
      if (u.kind != DOP_UNARY) {
        continue;
      }
      for (int l = 0; l < prog.num_ops; l++) {
        if (prog.ops[l].kind == DOP_LOAD && prog.ops[l].dst == u.dst) {
          prog.ops[l].hoist = 0;
        }
      }
    }
  }

  // ---- layouts ---------------------------------------------------------------
  prog.num_tensors = (int)T.size();
  for (int i = 0; i < prog.num_tensors; i++) {
    DevTensor &dt = prog.t[i];
    TensorInfo &ti = T[i];
    dt.rows = ti.rows;
    dt.cols = ti.cols;
    if (!f16) {
      dt.rs = ti.cols;
      dt.cs = 1;
      ti.bytes = round_up(ti.rows * ti.cols * 2, 16);
    } else {
      // every tile row-major with padded rows, as it is loaded (the matrix-core B operand is
      // gathered with transposing LDS reads) -- unless the plan's declaration rules
      // A tile of a column-major device tensor stays column-major in LDS (16-byte pieces
      // then move as they are, and a matmul reads it k-contiguous as its B operand) unless
      // a matmul wants it as its A operand.
      bool column_major = ti.dmem_colmajor && !ti.as_a;
      int p = pad;
      if (declared_layouts && declared_known(ti.declared)) {
        column_major = declared_column_major(ti.declared);
        p = pad == 0 ? 0 : declared_pad(ti.declared);
      }
      if (column_major) {
        dt.rs = 1;
        dt.cs = ti.rows >= 8 ? round_up(ti.rows, 8) + p : ti.rows;
        ti.bytes = round_up(dt.cs * ti.cols * 2, 16);
      } else {
        dt.cs = 1;
        dt.rs = ti.cols >= 8 ? round_up(ti.cols, 8) + p : ti.cols;
        ti.bytes = round_up(dt.rs * ti.rows * 2, 16);
      }
    }
  }
  // persistent tiles: accumulators and hoisted loads stay live over the whole loop
  for (int o = 0; o < prog.num_ops; o++) {
    DevOp const &d = prog.ops[o];
    if (d.kind == DOP_OUTPUT || (d.kind == DOP_LOAD && d.hoist)) {
      T[d.dst].persistent = true;
    }
    if (d.kind == DOP_OUTPUT && F == 1) {
      T[d.dst].bytes = 0;  // a single iteration stores straight from its input tile
    }
  }
  // ---- LDS placement: persistent tiles first, the rest by first fit over their
  // [definition, last use] interval inside one iteration
  int top = kTableBytes;
  for (int i = 0; i < prog.num_tensors; i++) {
    if (T[i].persistent) {
      prog.t[i].off = top;
      top += T[i].bytes;
    }
  }
  int const base = top;
  int peak = top;
  struct Live {
    int off, bytes, id;
  };
  std::vector<Live> live;
  for (int o = 0; o < prog.num_ops; o++) {
    for (int i = 0; i < prog.num_tensors; i++) {
      if (T[i].persistent || T[i].def_op != o) {
        continue;
      }
      // an element-wise result may overwrite an operand of the same shape and
      // layout that dies here: every thread reads element e before writing it
      DevOp const &d = prog.ops[o];
      if (d.kind == DOP_BINARY && d.dst == i) {
        int alias = -1;
        for (int src : {d.src0, d.src1}) {
          if (alias < 0 && src >= 0 && !T[src].persistent && T[src].last_use == o &&
              T[src].rows == T[i].rows && T[src].cols == T[i].cols &&
              prog.t[src].rs == prog.t[i].rs && prog.t[src].cs == prog.t[i].cs) {
            alias = src;
          }
        }
        bool done = false;
        if (alias >= 0) {
          for (Live &l : live) {
            if (l.id == alias) {
              prog.t[i].off = l.off;
              l.id = i;
              done = true;
              break;
            }
          }
        }
        if (done) {
          continue;
        }
      }
      std::sort(live.begin(), live.end(), [](Live const &a, Live const &b) { return a.off < b.off; });
      int off = base;
      for (Live const &l : live) {
        if (off + T[i].bytes <= l.off) {
          break;
        }
        off = std::max(off, l.off + l.bytes);
      }
      prog.t[i].off = off;
      live.push_back(Live{off, T[i].bytes, i});
      peak = std::max(peak, off + T[i].bytes);
    }
    live.erase(std::remove_if(live.begin(), live.end(),
                              [&](Live const &l) { return T[l.id].last_use <= o; }),
               live.end());
  }
  prog.lds_bytes = peak;
  if (peak > max_lds) {
    err = fmt("thread-block graph needs %d bytes of LDS, the device offers %d", peak, max_lds);
    return MI355_ERR_UNSUPPORTED;
  }
  prog.mm_off = peak;
  prog.splits = 1;
  for (int o = 0; o < prog.num_ops; o++) {
    prog.ops[o].mm_kc = 0;
  }
  if (!f16 && max_lds <= (1 << 20)) {  // not for a lowering that only sizes the plan
    // Residue scratch of the packed matmul path: two fields x (m + 4 + n) x kc bytes for
    // a k chunk of kc.  Each matmul takes the largest chunk that still fits; one that
    // cannot get even 16 keeps the scalar path.
    int const device_lds = max_lds;
    int const vector_dot_only = state().fp_vector_dot_only;
    int scratch = 0;
    for (int o = 0; o < prog.num_ops; o++) {
      DevOp &d = prog.ops[o];
      if (d.kind != DOP_MATMUL) {
        continue;
      }
      int const m = prog.t[d.src0].rows, k = prog.t[d.src0].cols, n = prog.t[d.src1].cols;
      if (m % 4 != 0 || n % 4 != 0 || k % 4 != 0) {
        continue;
      }
      // Matrix-core variant (signed-byte residues, swizzled rows, no padding): tiles whose m
      // and n are multiples of 16, k chunks that are powers of two from 64; A may be packed in
      // row blocks (a power-of-two fraction of m, at least 16 rows) when the whole tile does
      // not fit beside B^T.  `sub` = 1 selects it; preferred over the vector-dot path, which
      // takes whatever chunk still fits otherwise.
      d.sub = 0;
      d.mm_mb = 0;
      if (vector_dot_only == 0 && m % 16 == 0 && n % 16 == 0) {
        int top = 64;
        while (top * 2 <= k) {
          top *= 2;
        }
        for (int kc = top; kc >= 64 && kc <= k && d.sub == 0; kc /= 2) {
          if (k % kc != 0) {
            continue;
          }
          for (int mb = m; mb >= 16 && mb % 16 == 0 && m % mb == 0; mb /= 2) {
            int const need = 2 * kc * (mb + n);
            if (peak + need <= device_lds) {
              d.mm_kc = kc;
              d.mm_mb = mb;
              d.sub = 1;
              scratch = std::max(scratch, need);
              break;
            }
          }
        }
      }
      for (int kc = k; d.sub == 0 && (kc >= 16 || kc == k); kc /= 2) {
        if (kc % 4 != 0 || k % kc != 0) {
          break;
        }
        int const need = 2 * kc * (m + 4 + n);
        if (peak + need <= device_lds) {
          d.mm_kc = kc;
          scratch = std::max(scratch, need);
          break;
        }
      }
    }
    prog.lds_bytes = peak + scratch;
  }
  for (int i = 0; i < prog.num_tensors; i++) {
    prog.t[i].mcols = fast_div_magic(prog.t[i].cols);
    prog.t[i].mcpr = fast_div_magic(prog.t[i].cols / 8);
  }
  for (int o = 0; o < prog.num_ops; o++) {
    DevOp &d = prog.ops[o];
    d.mg0 = d.mg1 = d.mg2 = 0;
    if (d.kind == DOP_MATMUL) {
      int const n = prog.t[d.src1].cols;
      d.mg0 = fast_div_magic(d.mm_kc / 4);
      d.mg1 = fast_div_magic(n / 2);
      d.mg2 = fast_div_magic(n / 4);
    } else if (d.kind == DOP_LOAD && d.sub == 1) {
      // a column-major tensor is walked as the row-major matrix of its transpose
      d.mg0 = fast_div_magic(prog.t[d.dst].rows);
      d.mg1 = fast_div_magic(prog.t[d.dst].rows / 8);
    } else if (d.kind == DOP_REDUCE) {
      d.mg0 = fast_div_magic(d.red_inner);
    } else if (d.kind == DOP_CONCAT) {
      d.mg0 = fast_div_magic(d.cat_inner);
      d.mg1 = fast_div_magic(d.cat_a + d.cat_b);
    }
  }
  // LDS writes of 16 bytes need 8-element row strides on the destination
  for (int o = 0; o < prog.num_ops; o++) {
    DevOp &d = prog.ops[o];
    if (d.kind == DOP_LOAD && f16) {
      // (for a column-major device tensor the 16-byte pieces run down a column of the tile)
      DevTensor const &t = prog.t[d.dst];
      int const along = d.sub == 1 ? t.rs : t.cs, across = d.sub == 1 ? t.cs : t.rs;
      if (along != 1 || across % 8 != 0) {
        d.vec8 = d.vec8 ? 2 : 0;  // 2: vector global read, scalar LDS scatter
      }
    }
    if (d.kind == DOP_OUTPUT && f16 && (prog.t[d.dst].cs != 1 || prog.t[d.dst].rs % 8 != 0)) {
      d.vec8 = 0;
    }
  }
  return MI355_OK;
}

}  // namespace mi355
