// Fused kernel for the "fold the partial results and divide" family of thread-block
// graphs: the second operator of the reference's split-KV attention plans
// (cpp_examples/multi_head_attn_prefill.cc:75-98 and its siblings),
//
//   O[r][x] = fp16( fp16(sum_s N[r][s*X + x]) / fp16(sum_s D[r][s]) )
//
// i.e. loader, loader, reduction_to_dimx over the partial numerators, reduction over the
// partial denominators, div, saver, with a for-loop of one iteration.  Nothing is reused,
// so nothing goes through LDS: each thread folds eight output columns of one row with
// 16-byte loads and stores.  Sums run in fp32 over s = 0, 1, ... and are rounded to fp16
// where the thread-block graph materialises a tile, the division is IEEE fp32.
#include "common.h"
#include "tb_program.h"

namespace mi355 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));

struct CTile {
  void const *ptr;
  int row_bs[3], col_bs[3], g_bs[3];
  int d_cols;
};

struct CombineParams {
  CTile n, d, o;
  int rows;  // tile rows
  int X, S;  // output columns, partial results folded
  uint32_t mx8;  // division magic of X / 8
};

__device__ __forceinline__ long long ctile_origin(CTile const &t) {
  int const bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  long long const row0 = (long long)bx * t.row_bs[0] + (long long)by * t.row_bs[1] +
                         (long long)bz * t.row_bs[2];
  long long const col0 = (long long)bx * t.col_bs[0] + (long long)by * t.col_bs[1] +
                         (long long)bz * t.col_bs[2];
  long long const base = (long long)bx * t.g_bs[0] + (long long)by * t.g_bs[1] +
                         (long long)bz * t.g_bs[2];
  return base + row0 * t.d_cols + col0;
}

__global__ __launch_bounds__(256) void combine_fused_kernel(CombineParams const P) {
  _Float16 const *n = static_cast<_Float16 const *>(P.n.ptr) + ctile_origin(P.n);
  _Float16 const *d = static_cast<_Float16 const *>(P.d.ptr) + ctile_origin(P.d);
  _Float16 *o = static_cast<_Float16 *>(const_cast<void *>(P.o.ptr)) + ctile_origin(P.o);
  int const x8 = P.X / 8, items = P.rows * x8;
  for (int e = threadIdx.x; e < items; e += 256) {
    int const r = P.mx8 ? (int)__umulhi((uint32_t)e, P.mx8) : e;
    int const x = (e - r * x8) * 8;
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    float den = 0.0f;
    _Float16 const *nr = n + (long long)r * P.n.d_cols + x;
    _Float16 const *dr = d + (long long)r * P.d.d_cols;
    for (int s = 0; s < P.S; s++) {
      half8 v = *reinterpret_cast<half8 const *>(nr + (long long)s * P.X);
#pragma unroll
      for (int j = 0; j < 8; j++) {
        acc[j] += static_cast<float>(v[j]);
      }
      den += static_cast<float>(dr[s]);
    }
    float const den16 = static_cast<float>(static_cast<_Float16>(den));
    half8 out;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      float const num16 = static_cast<float>(static_cast<_Float16>(acc[j]));
      out[j] = static_cast<_Float16>(num16 / den16);
    }
    *reinterpret_cast<half8 *>(o + (long long)r * P.o.d_cols + x) = out;
  }
}

namespace {

CTile ctile(DevOp const &op, void const *ptr) {
  CTile t;
  t.ptr = ptr;
  for (int i = 0; i < 3; i++) {
    t.row_bs[i] = op.row_bs[i];
    t.col_bs[i] = op.col_bs[i];
    t.g_bs[i] = op.g_bs[i];
  }
  t.d_cols = op.d_cols;
  return t;
}

struct CMatch {
  int ln, ld, out;  // op indices: numerator loader, denominator loader, saver
  int rows, X, S;
};

bool aligned16(CTile const &t) {
  if ((reinterpret_cast<uintptr_t>(t.ptr) & 15) != 0 || t.d_cols % 8 != 0) {
    return false;
  }
  for (int i = 0; i < 3; i++) {
    if (t.col_bs[i] % 8 != 0 || t.g_bs[i] % 8 != 0) {
      return false;
    }
  }
  return true;
}

bool cmatch(DevProgram const &P, CMatch &M) {
  if (P.forloop_range != 1 || P.num_ops != 6) {
    return false;
  }
  DevOp const &l0 = P.ops[0], &l1 = P.ops[1], &r0 = P.ops[2], &r1 = P.ops[3], &dv = P.ops[4],
              &out = P.ops[5];
  if (l0.kind != DOP_LOAD || l1.kind != DOP_LOAD || r0.kind != DOP_REDUCE ||
      r1.kind != DOP_REDUCE || dv.kind != DOP_BINARY || dv.sub != TB_DIV_OP ||
      out.kind != DOP_OUTPUT) {
    return false;
  }
  // either reduction may come first; the numerator is the one the div takes as src0
  DevOp const *rn = nullptr, *rd = nullptr;
  for (DevOp const *r : {&r0, &r1}) {
    if (r->dst == dv.src0) {
      rn = r;
    } else if (r->dst == dv.src1) {
      rd = r;
    }
  }
  if (rn == nullptr || rd == nullptr || out.src0 != dv.dst) {
    return false;
  }
  DevOp const *ln = nullptr, *ld = nullptr;
  for (DevOp const *l : {&l0, &l1}) {
    if (l->dst == rn->src0) {
      ln = l;
    } else if (l->dst == rd->src0) {
      ld = l;
    }
  }
  if (ln == nullptr || ld == nullptr) {
    return false;
  }
  DevTensor const &tn = P.t[ln->dst], &td = P.t[ld->dst], &to = P.t[dv.dst];
  int const S = rn->red_deg, X = rn->red_inner;
  if (tn.cols != S * X || td.rows != tn.rows || td.cols != S || rd->red_deg != S ||
      rd->red_inner != 1 || P.t[rn->dst].rows != tn.rows || P.t[rn->dst].cols != X ||
      P.t[rd->dst].rows != tn.rows || P.t[rd->dst].cols != 1 || to.rows != tn.rows ||
      to.cols != X || X % 8 != 0 || S < 1) {
    return false;
  }
  if (!aligned16(ctile(*ln, P.in[ln->io])) || !aligned16(ctile(out, P.out[out.io]))) {
    return false;
  }
  M.ln = (int)(ln - P.ops);
  M.ld = (int)(ld - P.ops);
  M.out = 5;
  M.rows = tn.rows;
  M.X = X;
  M.S = S;
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
  A.mx8 = fast_div_magic(M.X / 8);
  dim3 grid(P.grid[0], P.grid[1], P.grid[2]);
  combine_fused_kernel<<<grid, 256, 0, s.stream()>>>(A);
  MI355_HIP(hipGetLastError());
  s.last().kernel_id = MI355_KERNEL_F16_COMBINE;
  s.last().workgroups = (int)(grid.x * grid.y * grid.z);
  s.last().threads = 256;
  s.last().lds_bytes = 0;
  s.last().row_split = 1;
  return 1;
}

}  // namespace mi355
