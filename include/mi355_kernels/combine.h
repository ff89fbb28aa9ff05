// Device code of combine_fused_kernel (the second operator of the split-KV attention plans: fold
// partial numerators and denominators, divide) and its parameter block.  Header-only and free of
// host state: combine_fused.hip recognises the family and chooses the launch, the programs
// Graph::generate_hip_program writes instantiate the same template (where the reference emits
// Triton source, src/kernel/triton_code_gen.cc:84-352).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernarg.h"

namespace mi355 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));

// Where a block's tile starts: linear in the block coordinates, so the host folds the plan's
// row / column / batch strides into one element stride per coordinate.
struct CTile {
  void const *ptr;
  long long lin[3];
  int d_cols;
};

enum { SUM_THEN_DIV = 0, DIV_THEN_SUM = 1, DIV_THEN_SAVE = 2 };

struct CombineParams {
  CTile n, d, o;
  int rows;        // tile rows
  int X, S, SD;    // output columns, numerator pieces folded, denominators folded
  long long step;  // elements from one numerator piece to the next
  uint32_t mxv;    // division magic of X / VEC
};

__device__ __forceinline__ long long ctile_origin(CTile const &t) {
  return (long long)blockIdx.x * t.lin[0] + (long long)blockIdx.y * t.lin[1] + (long long)blockIdx.z * t.lin[2];
}

// BATCH: pieces a thread keeps in flight: 16 for a small fold (latency sets its time), 4 for a
// large one (bandwidth does, and sixteen pieces a power of two apart in flight per thread halve
// the rate).
template <int VEC, int MODE, int BATCH>
__global__ __launch_bounds__(256) void combine_fused_kernel(CombineParams const) {
  CombineParams const P = load_kernel_arguments<CombineParams, 0>();  // the whole block, one trip
  typedef _Float16 halfv __attribute__((ext_vector_type(VEC)));
  _Float16 const *n = static_cast<_Float16 const *>(P.n.ptr) + ctile_origin(P.n);
  _Float16 const *d = static_cast<_Float16 const *>(P.d.ptr) + ctile_origin(P.d);
  _Float16 *o = static_cast<_Float16 *>(const_cast<void *>(P.o.ptr)) + ctile_origin(P.o);
  int const xv = P.X / VEC, items = P.rows * xv;
  for (int e = threadIdx.x; e < items; e += 256) {
    int const r = P.mxv ? (int)__umulhi((uint32_t)e, P.mxv) : e;
    int const x = (e - r * xv) * VEC;
    _Float16 const *nr = n + (long long)r * P.n.d_cols + x;
    _Float16 const *dr = d + (long long)r * P.d.d_cols;
    // Whole batches of pieces are loaded together and consumed in order afterwards: piece by
    // piece (a load, its wait, an add) a fold of 16 denominators and 16 numerator pieces is 32
    // trips to the L2 in a row, several microseconds for a kilobyte of data.  The first
    // numerator batch is in flight while the denominators are added; what is left over after
    // the whole batches is folded piece by piece.
    halfv v[BATCH];
    auto load_pieces = [&](int s0) {
      _Float16 const *first = nr + s0 * P.step;
#pragma unroll
      for (int u = 0; u < BATCH; u++) {
        v[u] = *reinterpret_cast<halfv const *>(first + u * P.step);
      }
    };
    halfv lone = {};  // (a fold of fewer pieces than a batch: its first piece, loaded as early)
    if (P.S >= BATCH) {
      load_pieces(0);
    } else if (P.S > 0) {
      lone = *reinterpret_cast<halfv const *>(nr);
    }
    float den = 0.0f;
    int sd = 0;
    for (; sd + BATCH <= P.SD; sd += BATCH) {
      _Float16 dv[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; u++) {
        dv[u] = dr[sd + u];
      }
#pragma unroll
      for (int u = 0; u < BATCH; u++) {
        den += static_cast<float>(dv[u]);
      }
    }
    for (; sd < P.SD; sd++) {
      den += static_cast<float>(dr[sd]);
    }
    float const den16 = static_cast<float>(static_cast<_Float16>(den));
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      acc[j] = 0.0f;
    }
    auto add_piece = [&](halfv const &piece) {
#pragma unroll
      for (int j = 0; j < VEC; j++) {
        float const t = static_cast<float>(piece[j]);
        if (MODE == SUM_THEN_DIV) {
          acc[j] += t;
        } else if (MODE == DIV_THEN_SUM) {
          acc[j] += static_cast<float>(static_cast<_Float16>(t / den16));
        } else {
          acc[j] = static_cast<float>(
              static_cast<_Float16>(acc[j] + static_cast<float>(static_cast<_Float16>(t / den16))));
        }
      }
    };
    int sn = 0;
    for (; sn + BATCH <= P.S; sn += BATCH) {
      if (sn > 0) {
        load_pieces(sn);
      }
#pragma unroll
      for (int u = 0; u < BATCH; u++) {
        add_piece(v[u]);
      }
    }
#pragma unroll 4
    for (; sn < P.S; sn++) {
      add_piece(sn == 0 ? lone : *reinterpret_cast<halfv const *>(nr + sn * P.step));
    }
    halfv out;
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      float const sum16 = static_cast<float>(static_cast<_Float16>(acc[j]));
      out[j] = static_cast<_Float16>(MODE == SUM_THEN_DIV ? sum16 / den16 : sum16);
    }
    *reinterpret_cast<halfv *>(o + (long long)r * P.o.d_cols + x) = out;
  }
}

}  // namespace mi355
