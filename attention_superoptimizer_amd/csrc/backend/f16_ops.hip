// Kernel-level fp16 operators (the un-fused ops a kernel graph runs outside its
// customized ops).  Arithmetic is fp32 with one fp16 rounding per stored element, the rule
// the reference's generated programs follow (src/kernel/triton_code_gen.cc:246-268).
// Results are row-major; the matmul reads either storage order of its operands (as the
// reference's GEMM call does, src/kernel/cuda/matmul_kernel.cu:61-76), the element-wise
// operators and reductions index their inputs flat, so their callers hand them row-major
// buffers (mi355_f16_transpose makes one from a column-major tensor).
#include "common.h"

namespace mi355 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;

__device__ __forceinline__ uint64_t mix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

// reference src/kernel/cuda/input_kernel.cu:29-38
__global__ void f16_fill_iota_kernel(_Float16 *x, size_t n, int last_dim) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    x[i] = static_cast<_Float16>(static_cast<float>(i % last_dim));
  }
}

__global__ void f16_fill_normal_kernel(_Float16 *x, size_t n, float std, uint64_t seed) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    uint64_t r = mix64(seed + i);
    float u1 = (static_cast<float>((r >> 40) & 0xffffff) + 1.0f) * (1.0f / 16777216.0f);
    float u2 = static_cast<float>((r >> 16) & 0xffffff) * (1.0f / 16777216.0f);
    float z = sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
    x[i] = static_cast<_Float16>(z * std);
  }
}

// Batched GEMM on the matrix cores, any shape and either storage order of the operands
// (element (r, c) of A at r * a_rs + c * a_cs, likewise B): 64x64 output tile per workgroup,
// four wavefronts each owning a 32x32 quadrant, k advanced 32 at a time through LDS, both
// tiles staged k-contiguous with rows padded by 8 halfs.  The general-purpose kernel: ragged
// extents, unaligned bases.
__global__ __launch_bounds__(kThreads) void f16_matmul_kernel(_Float16 const *__restrict__ A,
                                                             _Float16 const *__restrict__ B,
                                                             _Float16 *__restrict__ C, int m,
                                                             int n, int k, int a_rs, int a_cs,
                                                             int b_rs, int b_cs) {
  constexpr int T = 64, TK = 32, LD = TK + 8;
  __shared__ __attribute__((aligned(16))) _Float16 As[T][LD];
  __shared__ __attribute__((aligned(16))) _Float16 Bs[T][LD];
  int const tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  int const row0 = blockIdx.y * T, col0 = blockIdx.x * T;
  size_t const b = blockIdx.z;
  A += b * (size_t)m * k;
  B += b * (size_t)k * n;
  C += b * (size_t)m * n;
  int const wr = (wave / 2) * 32, wc = (wave % 2) * 32;
  float16v acc;
#pragma unroll
  for (int i = 0; i < 16; i++) {
    acc[i] = 0.0f;
  }
  // a thread stages 8 elements of each tile per step, walking the direction that is
  // contiguous in memory: along k (8 consecutive k of one row) or along the rows / columns
  // (one k of 8 consecutive rows / columns)
  bool const a_along_k = a_cs == 1, b_along_k = b_rs == 1;
  for (int k0 = 0; k0 < k; k0 += TK) {
    {
      int const r = a_along_k ? tid / 4 : (tid % 8) * 8, kk = a_along_k ? (tid % 4) * 8 : tid / 8;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        int const rr = a_along_k ? r : r + j, kj = a_along_k ? kk + j : kk;
        int const gr = row0 + rr, gk = k0 + kj;
        As[rr][kj] = (gr < m && gk < k) ? A[(size_t)gr * a_rs + (size_t)gk * a_cs] : (_Float16)0.0f;
      }
    }
    {
      int const c = b_along_k ? tid / 4 : (tid % 8) * 8, kk = b_along_k ? (tid % 4) * 8 : tid / 8;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        int const cc = b_along_k ? c : c + j, kj = b_along_k ? kk + j : kk;
        int const gc = col0 + cc, gk = k0 + kj;
        Bs[cc][kj] = (gk < k && gc < n) ? B[(size_t)gk * b_rs + (size_t)gc * b_cs] : (_Float16)0.0f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < TK; ks += 16) {
      half8 a = *reinterpret_cast<half8 const *>(&As[wr + lane % 32][ks + 8 * (lane / 32)]);
      half8 bb = *reinterpret_cast<half8 const *>(&Bs[wc + lane % 32][ks + 8 * (lane / 32)]);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bb, acc, 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < 16; r++) {
    int row = row0 + wr + (r / 4) * 8 + (lane / 32) * 4 + (r % 4);
    int col = col0 + wc + lane % 32;
    if (row < m && col < n) {
      C[(size_t)row * n + col] = static_cast<_Float16>(acc[r]);
    }
  }
}

// out[b][c][r] = in[b][r][c] through a 64 x 64 LDS tile: the row-major copy of a column-major
// tensor (or the other way round) for the operators that index their inputs flat.
__global__ __launch_bounds__(kThreads) void f16_transpose_kernel(_Float16 const *__restrict__ in,
                                                                _Float16 *__restrict__ out, int rows,
                                                                int cols) {
  __shared__ _Float16 tile[64][66];
  size_t const b = blockIdx.z;
  in += b * (size_t)rows * cols;
  out += b * (size_t)rows * cols;
  int const r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  for (int e = threadIdx.x; e < 64 * 64; e += kThreads) {
    int const r = e / 64, c = e % 64;
    if (r0 + r < rows && c0 + c < cols) {
      tile[r][c] = in[(size_t)(r0 + r) * cols + c0 + c];
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 64 * 64; e += kThreads) {
    int const c = e / 64, r = e % 64;
    if (r0 + r < rows && c0 + c < cols) {
      out[(size_t)(c0 + c) * rows + r0 + r] = tile[r][c];
    }
  }
}

__global__ void f16_unary_kernel(int op, _Float16 const *__restrict__ in,
                                 _Float16 *__restrict__ out, size_t n) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    float x = static_cast<float>(in[i]);
    float y = (op == KN_EXP_OP) ? __expf(x) : x / (1.0f + __expf(-x));
    out[i] = static_cast<_Float16>(y);
  }
}

struct Dims4 {
  int nd;
  int d1[4], d2[4], od[4];
};

__global__ void f16_binary_kernel(int op, _Float16 const *__restrict__ in1,
                                  _Float16 const *__restrict__ in2, _Float16 *__restrict__ out,
                                  Dims4 D, size_t n) {
  size_t gid = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; gid < n; gid += stride) {
    size_t i = gid, s1 = 1, i1 = 0, s2 = 1, i2 = 0;
    for (int d = D.nd - 1; d >= 0; d--) {
      i1 += (i % D.d1[d]) * s1;
      i2 += (i % D.d2[d]) * s2;
      s1 *= D.d1[d];
      s2 *= D.d2[d];
      i /= D.od[d];
    }
    float x = static_cast<float>(in1[i1]), y = static_cast<float>(in2[i2]);
    float z = (op == KN_ADD_OP) ? x + y : (op == KN_MUL_OP) ? x * y : x / y;
    out[gid] = static_cast<_Float16>(z);
  }
}

__global__ void f16_reduce_kernel(_Float16 const *__restrict__ in, _Float16 *__restrict__ out,
                                  size_t n_out, int factor, int in_stride, int out_stride) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  if (i >= n_out) {
    return;
  }
  size_t base = (i / out_stride) * (size_t)in_stride + i % out_stride;
  float r = 0.0f;
  for (int k = 0; k < factor; k++) {
    r += static_cast<float>(in[base + (size_t)k * out_stride]);
  }
  out[i] = static_cast<_Float16>(r);
}

__global__ void f16_reduce_rows_kernel(_Float16 const *__restrict__ in,
                                       _Float16 *__restrict__ out, size_t n_out, int factor) {
  int const lane = threadIdx.x % 64;
  size_t row = (blockIdx.x * (size_t)blockDim.x + threadIdx.x) / 64;
  if (row >= n_out) {
    return;
  }
  _Float16 const *p = in + row * (size_t)factor;
  float r = 0.0f;
  for (int k = lane; k < factor; k += 64) {
    r += static_cast<float>(p[k]);
  }
  for (int off = 32; off > 0; off >>= 1) {
    r += __shfl_down(r, off, 64);
  }
  if (lane == 0) {
    out[row] = static_cast<_Float16>(r);
  }
}

static inline int grid_for(size_t n) {
  size_t g = (n + kThreads - 1) / kThreads;
  return static_cast<int>(g < 1 ? 1 : (g > 8192 ? 8192 : g));
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_f16_fill_iota(void *x, size_t n, int last_dim) {
  MI355_REQUIRE_INIT();
  if (last_dim <= 0) {
    return fail(MI355_ERR_INVALID, "last_dim must be positive");
  }
  if (n == 0) {
    return MI355_OK;
  }
  f16_fill_iota_kernel<<<grid_for(n), kThreads, 0, state().stream()>>>(
      static_cast<_Float16 *>(x), n, last_dim);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_f16_fill_normal(void *x, size_t n, float std, uint64_t seed) {
  MI355_REQUIRE_INIT();
  if (n == 0) {
    return MI355_OK;
  }
  f16_fill_normal_kernel<<<grid_for(n), kThreads, 0, state().stream()>>>(
      static_cast<_Float16 *>(x), n, std, seed);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_f16_matmul_layout(void const *A, void const *B, void *C, int batch, int m,
                                       int n, int k, int a_column_major, int b_column_major) {
  MI355_REQUIRE_INIT();
  if (batch < 0 || m < 0 || n < 0 || k < 0) {
    return fail(MI355_ERR_INVALID, "negative matmul extent");
  }
  if (batch == 0 || m == 0 || n == 0) {
    return MI355_OK;
  }
  if (batch > 65535) {
    return fail(MI355_ERR_UNSUPPORTED, "batch %d exceeds grid.z", batch);
  }
  dim3 grid((n + 63) / 64, (m + 63) / 64, batch);
  f16_matmul_kernel<<<grid, kThreads, 0, state().stream()>>>(
      static_cast<_Float16 const *>(A), static_cast<_Float16 const *>(B),
      static_cast<_Float16 *>(C), m, n, k, a_column_major ? 1 : k, a_column_major ? m : 1,
      b_column_major ? 1 : n, b_column_major ? k : 1);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_f16_matmul(void const *A, void const *B, void *C, int batch, int m, int n,
                                int k) {
  return mi355_f16_matmul_layout(A, B, C, batch, m, n, k, 0, 0);
}

extern "C" int mi355_f16_transpose(void const *in, void *out, int batch, int rows, int cols) {
  MI355_REQUIRE_INIT();
  if (batch < 0 || rows < 0 || cols < 0) {
    return fail(MI355_ERR_INVALID, "negative transpose extent");
  }
  if (batch == 0 || rows == 0 || cols == 0) {
    return MI355_OK;
  }
  if (batch > 65535 || (rows + 63) / 64 > 65535) {
    return fail(MI355_ERR_UNSUPPORTED, "transpose grid out of range");
  }
  if (in == out) {
    return fail(MI355_ERR_INVALID, "transpose in place");
  }
  dim3 grid((cols + 63) / 64, (rows + 63) / 64, batch);
  f16_transpose_kernel<<<grid, kThreads, 0, state().stream()>>>(
      static_cast<_Float16 const *>(in), static_cast<_Float16 *>(out), rows, cols);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_f16_unary(int op, void const *in, void *out, size_t n) {
  MI355_REQUIRE_INIT();
  if (op != KN_EXP_OP && op != KN_SILU_OP) {
    return fail(MI355_ERR_UNSUPPORTED, "unary op %d", op);
  }
  if (n == 0) {
    return MI355_OK;
  }
  f16_unary_kernel<<<grid_for(n), kThreads, 0, state().stream()>>>(
      op, static_cast<_Float16 const *>(in), static_cast<_Float16 *>(out), n);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_f16_binary(int op, void const *in1, int const *dims1, void const *in2,
                                int const *dims2, void *out, int const *dims_out,
                                int num_dims) {
  MI355_REQUIRE_INIT();
  if (op != KN_ADD_OP && op != KN_MUL_OP && op != KN_DIV_OP) {
    return fail(MI355_ERR_UNSUPPORTED, "binary op %d", op);
  }
  if (num_dims < 1 || num_dims > 4) {
    return fail(MI355_ERR_INVALID, "num_dims %d out of range", num_dims);
  }
  Dims4 D{};
  D.nd = num_dims;
  size_t n = 1;
  for (int d = 0; d < num_dims; d++) {
    D.d1[d] = dims1[d];
    D.d2[d] = dims2[d];
    D.od[d] = dims_out[d];
    if (dims1[d] <= 0 || dims2[d] <= 0 || dims_out[d] <= 0 ||
        (dims1[d] != dims_out[d] && dims1[d] != 1) ||
        (dims2[d] != dims_out[d] && dims2[d] != 1)) {
      return fail(MI355_ERR_INVALID, "dim %d is not broadcastable", d);
    }
    n *= (size_t)dims_out[d];
  }
  f16_binary_kernel<<<grid_for(n), kThreads, 0, state().stream()>>>(
      op, static_cast<_Float16 const *>(in1), static_cast<_Float16 const *>(in2),
      static_cast<_Float16 *>(out), D, n);
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}

extern "C" int mi355_f16_reduce(void const *in, void *out, size_t n_out, int factor,
                                int in_stride, int out_stride) {
  MI355_REQUIRE_INIT();
  if (factor <= 0 || in_stride <= 0 || out_stride <= 0 ||
      (size_t)out_stride * factor != (size_t)in_stride) {
    return fail(MI355_ERR_INVALID, "reduction strides do not match the factor");
  }
  if (n_out == 0) {
    return MI355_OK;
  }
  hipStream_t st = state().stream();
  if (out_stride == 1 && factor >= 64) {
    size_t blocks = (n_out * 64 + kThreads - 1) / kThreads;
    f16_reduce_rows_kernel<<<(unsigned)blocks, kThreads, 0, st>>>(
        static_cast<_Float16 const *>(in), static_cast<_Float16 *>(out), n_out, factor);
  } else {
    size_t blocks = (n_out + kThreads - 1) / kThreads;
    f16_reduce_kernel<<<(unsigned)blocks, kThreads, 0, st>>>(
        static_cast<_Float16 const *>(in), static_cast<_Float16 *>(out), n_out, factor,
        in_stride, out_stride);
  }
  MI355_HIP(hipGetLastError());
  return MI355_OK;
}
