// Second route of the kernel-level fp16 matmul: the vendor library's GEMM.
//
// The reference runs a kernel-level matmul on the vendor's BLAS
// (cublasGemmStridedBatchedEx, src/kernel/cuda/matmul_kernel.cu:86-131); this is the same
// call on this machine: rocblas_gemm_strided_batched_ex with fp16 operands and results and
// fp32 accumulation.  rocBLAS is opened at run time (dlopen), so the backend neither links
// nor needs it unless MI355_OPT_F16_MATMUL_ROUTE asks for it, and a machine without the
// library gets an error naming it rather than a different kernel.
//
// rocBLAS counts in column-major matrices.  A row-major [m, k] buffer is a column-major
// [k, m] one, so the row-major product C = A . B is computed as C^T = B^T . A^T:
//   first operand   B's buffer: column-major storage of B ([n][k], k contiguous) is a
//                   column-major [k, n] matrix, taken transposed (ld k); row-major storage
//                   ([k][n]) is a column-major [n, k] matrix, taken as it is (ld n)
//   second operand  A's buffer: row-major storage ([m][k]) is a column-major [k, m] matrix,
//                   taken as it is (ld k); column-major storage ([k][m]) is a column-major
//                   [m, k] matrix, taken transposed (ld m)
//   result          column-major [n, m] with ld n = the row-major [m, n] buffer of C
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <mutex>

#include "common.h"

namespace mi355 {
namespace {

// the part of rocBLAS's C API this file calls (rocblas.h: rocblas-functions.h,
// rocblas-auxiliary.h); enumerators by their published values
using handle_t = void *;
constexpr int kOpNone = 111, kOpTranspose = 112;    // rocblas_operation
constexpr int kF16 = 150, kF32 = 151;               // rocblas_datatype f16_r, f32_r
constexpr int kAlgoStandard = 0;                    // rocblas_gemm_algo
constexpr int kAtomicsNotAllowed = 0;               // rocblas_atomics_mode
using create_fn = int (*)(handle_t *);
using destroy_fn = int (*)(handle_t);
using set_stream_fn = int (*)(handle_t, hipStream_t);
using set_atomics_fn = int (*)(handle_t, int);
using gemm_fn = int (*)(handle_t, int, int, int32_t, int32_t, int32_t, void const *, void const *, int,
                        int32_t, int64_t, void const *, int, int32_t, int64_t, void const *,
                        void const *, int, int32_t, int64_t, void *, int, int32_t, int64_t, int32_t,
                        int, int, int32_t, uint32_t);

struct Vendor {
  std::mutex mu;
  bool tried = false;
  void *lib = nullptr;
  create_fn create = nullptr;
  destroy_fn destroy = nullptr;
  set_stream_fn set_stream = nullptr;
  set_atomics_fn set_atomics = nullptr;
  gemm_fn gemm = nullptr;
  handle_t handles[MI355_NUM_QUEUES] = {};  // one per backend queue, bound to its stream
};
Vendor g_vendor;

int open_library(Vendor &v) {
  if (v.tried) {
    return v.gemm != nullptr ? MI355_OK : fail(MI355_ERR_UNSUPPORTED, "rocBLAS could not be loaded");
  }
  v.tried = true;
  for (char const *name : {"librocblas.so.5", "/opt/rocm/lib/librocblas.so.5", "librocblas.so"}) {
    v.lib = dlopen(name, RTLD_NOW | RTLD_LOCAL);
    if (v.lib != nullptr) {
      break;
    }
  }
  if (v.lib == nullptr) {
    return fail(MI355_ERR_UNSUPPORTED, "rocBLAS could not be loaded: %s", dlerror());
  }
  v.create = reinterpret_cast<create_fn>(dlsym(v.lib, "rocblas_create_handle"));
  v.destroy = reinterpret_cast<destroy_fn>(dlsym(v.lib, "rocblas_destroy_handle"));
  v.set_stream = reinterpret_cast<set_stream_fn>(dlsym(v.lib, "rocblas_set_stream"));
  v.set_atomics = reinterpret_cast<set_atomics_fn>(dlsym(v.lib, "rocblas_set_atomics_mode"));
  gemm_fn const gemm = reinterpret_cast<gemm_fn>(dlsym(v.lib, "rocblas_gemm_strided_batched_ex"));
  if (v.create == nullptr || v.destroy == nullptr || v.set_stream == nullptr || v.set_atomics == nullptr ||
      gemm == nullptr) {
    return fail(MI355_ERR_UNSUPPORTED, "rocBLAS lacks an entry point this backend calls");
  }
  v.gemm = gemm;
  return MI355_OK;
}

}  // namespace

int vendor_gemm(void const *A, void const *B, void *C, int batch, int m, int n, int k, int a_column_major,
                int b_column_major) {
  Vendor &v = g_vendor;
  handle_t h = nullptr;
  {
    std::lock_guard<std::mutex> lock(v.mu);
    if (int rc = open_library(v)) {
      return rc;
    }
    handle_t &slot = v.handles[tls_queue];
    if (slot == nullptr) {
      handle_t fresh = nullptr;
      if (int st = v.create(&fresh)) {
        return fail(MI355_ERR_HIP, "rocblas_create_handle failed (status %d)", st);
      }
      // results must not depend on the order in which workgroups finish
      int st = v.set_stream(fresh, state().stream());
      if (st == 0) {
        st = v.set_atomics(fresh, kAtomicsNotAllowed);
      }
      if (st != 0) {
        v.destroy(fresh);
        return fail(MI355_ERR_HIP, "rocBLAS handle set-up failed (status %d)", st);
      }
      slot = fresh;
    }
    h = slot;
  }
  float const alpha = 1.0f, beta = 0.0f;
  int const st = v.gemm(h, b_column_major ? kOpTranspose : kOpNone, a_column_major ? kOpTranspose : kOpNone, n, m, k,
                        &alpha, B, kF16, b_column_major ? k : n, (int64_t)k * n, A, kF16, a_column_major ? m : k,
                        (int64_t)m * k, &beta, C, kF16, n, (int64_t)m * n, C, kF16, n, (int64_t)m * n, batch, kF32,
                        kAlgoStandard, 0, 0);
  if (st != 0) {
    return fail(MI355_ERR_HIP, "rocblas_gemm_strided_batched_ex failed (status %d) for [%d x %d x %d] x %d", st, m,
                n, k, batch);
  }
  return MI355_OK;
}

int vendor_gemm_release() {
  Vendor &v = g_vendor;
  std::lock_guard<std::mutex> lock(v.mu);
  for (handle_t &h : v.handles) {
    if (h != nullptr) {
      v.destroy(h);
      h = nullptr;
    }
  }
  return MI355_OK;
}

}  // namespace mi355
