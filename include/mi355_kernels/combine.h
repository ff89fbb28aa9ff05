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

template <int VEC, int MODE>
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
    float den = 0.0f;
    for (int s = 0; s < P.SD; s++) {
      den += static_cast<float>(dr[s]);
    }
    float const den16 = static_cast<float>(static_cast<_Float16>(den));
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      acc[j] = 0.0f;
    }
#pragma unroll 4
    for (int s = 0; s < P.S; s++) {
      halfv const v = *reinterpret_cast<halfv const *>(nr + s * P.step);
#pragma unroll
      for (int j = 0; j < VEC; j++) {
        float const t = static_cast<float>(v[j]);
        if (MODE == SUM_THEN_DIV) {
          acc[j] += t;
        } else if (MODE == DIV_THEN_SUM) {
          acc[j] += static_cast<float>(static_cast<_Float16>(t / den16));
        } else {
          acc[j] = static_cast<float>(
              static_cast<_Float16>(acc[j] + static_cast<float>(static_cast<_Float16>(t / den16))));
        }
      }
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
