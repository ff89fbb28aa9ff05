// gfx950_rates: the three stand-alone rate measurements the fused attention kernels' design
// notes rest on.  No inputs; prints one table per section.
//
//   1. co-issue: how much of the sum (matrix time + vector time) disappears when every MFMA of
//      a wavefront is followed by four independent vector instructions of one kind, and whether
//      two wavefronts of a SIMD (one with only MFMAs, one with only vector work) overlap at all;
//   2. LDS read throughput per compute unit for the transposing read the attention kernels
//      gather their K / V operands with, and for plain 8- and 16-byte reads;
// One workgroup per compute unit (256 workgroups), registers and LDS only: no global memory in
// the timed loops.
#include <hip/hip_runtime.h>

#include <cstdio>

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int2v __attribute__((ext_vector_type(2)));

#define CHECK(call)                                                        \
  do {                                                                     \
    hipError_t e_ = (call);                                                \
    if (e_ != hipSuccess) {                                                \
      fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));    \
      return 1;                                                            \
    }                                                                      \
  } while (0)

enum { V_FMA = 0, V_EXP = 1, V_CVT_PK = 2, V_DOT2 = 3, V_PK_ADD = 4 };

template <int KIND>
__device__ __forceinline__ void vector4(float (&x)[8], half2v (&h)[8], int base) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int const j = base + i;
    if (KIND == V_FMA) {
      x[j] = __builtin_fmaf(x[j], 1.0001f, 0.5f);
    } else if (KIND == V_EXP) {
      x[j] = __builtin_amdgcn_exp2f(x[j]);
    } else if (KIND == V_CVT_PK) {
      float2v const f = {x[j], x[j]};
      h[j] = __builtin_convertvector(f, half2v);
      asm volatile("" : "+v"(h[j]));
    } else if (KIND == V_DOT2) {
      x[j] = __builtin_amdgcn_fdot2(h[j], h[(j + 1) & 7], x[j], false);
    } else {
      h[j] = h[j] + h[(j + 4) & 7];
    }
  }
}

// MODE 0: MFMAs only, 1: vector instructions only, 2: 1 MFMA : 4 vector instructions interleaved,
// 3: even wavefronts MFMAs only, odd wavefronts vector only (two wavefronts per SIMD)
template <int KIND, int MODE>
__global__ __launch_bounds__(512) void coissue_kernel(float *out, int iters) {
  int const wave = threadIdx.x / 64;
  half8 a, b;
  for (int i = 0; i < 8; i++) {
    a[i] = (_Float16)(threadIdx.x * 0.001f);
    b[i] = (_Float16)(i * 0.01f);
  }
  float4v c0 = {0, 0, 0, 0}, c1 = c0;
  float x[8];
  half2v h[8];
  for (int i = 0; i < 8; i++) {
    x[i] = threadIdx.x * 0.001f + i;
    h[i] = half2v{(_Float16)(i * 0.1f), (_Float16)0.5f};
  }
  // (wavefronts of a workgroup go to the four SIMDs in turn: wavefronts w and w + 4 share one)
  bool const mfma = MODE == 0 || MODE == 2 || (MODE == 3 && wave < 4);
  bool const vec = MODE == 1 || MODE == 2 || (MODE == 3 && wave >= 4);
  if (mfma && vec) {
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int u = 0; u < 4; u++) {
        c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c0, 0, 0, 0);
        vector4<KIND>(x, h, 0);
        c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c1, 0, 0, 0);
        vector4<KIND>(x, h, 4);
      }
    }
  } else if (mfma) {
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int u = 0; u < 4; u++) {
        c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c1, 0, 0, 0);
      }
    }
  } else {
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int u = 0; u < 4; u++) {
        vector4<KIND>(x, h, 0);
        vector4<KIND>(x, h, 4);
      }
    }
  }
  float r = c0[0] + c1[1];
  for (int i = 0; i < 8; i++) {
    r += x[i] + static_cast<float>(h[i][0]);
  }
  if (r == 12345.678f) {
    out[threadIdx.x] = r;
  }
}

// KIND 0: ds_read_b64_tr_b16, 1: ds_read_b64, 2: ds_read_b128; 8 wavefronts, each on its own 4 KB
template <int KIND>
__global__ __launch_bounds__(512) void lds_read_kernel(float *out, int iters) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[65536];
  for (int i = threadIdx.x; i < 16384; i += blockDim.x) {
    reinterpret_cast<int *>(lds)[i] = i;
  }
  __syncthreads();
  int const lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  // transposing read: 16 lanes cover 4 rows x 32 bytes of a tile with 128-byte rows
  int const a4 = (lane % 16) / 4, b4 = lane % 4, g = lane / 16;
  unsigned const tr_off = wave * 4096 + (8 * g + a4) * 128 + b4 * 8;
  unsigned const lin8 = wave * 4096 + lane * 8, lin16 = wave * 4096 + lane * 16;
  int acc = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 8; u++) {
      unsigned const o = (u * 1024 + it * 32) & 0x3fff;
      if (KIND == 0) {
        short4v const v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (short4v __attribute__((address_space(3))) *)(__attribute__((address_space(3))) void *)(
                lds + ((tr_off + o) & 0xfff8)));
        acc += v[0] + v[3];
      } else if (KIND == 1) {
        int2v const v = *reinterpret_cast<int2v const *>(lds + ((lin8 + o) & 0xfff8));
        acc += v[0] + v[1];
      } else {
        int4v const v = *reinterpret_cast<int4v const *>(lds + ((lin16 + o) & 0xfff0));
        acc += v[0] + v[3];
      }
    }
  }
  if (acc == 123456789) {
    out[threadIdx.x] = acc;
  }
}

template <typename F>
static float time_us(F launch) {
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  launch();
  (void)hipDeviceSynchronize();
  (void)hipEventRecord(e0);
  for (int r = 0; r < 5; r++) {
    launch();
  }
  (void)hipEventRecord(e1);
  (void)hipEventSynchronize(e1);
  float ms = 0.0f;
  (void)hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return ms * 200.0f;  // per launch
}

constexpr int kIters = 20000;

template <int KIND>
static void coissue_row(float *d, char const *name) {
  float const m = time_us([&] { coissue_kernel<KIND, 0><<<256, 256>>>(d, kIters); });
  float const v = time_us([&] { coissue_kernel<KIND, 1><<<256, 256>>>(d, kIters); });
  float const b = time_us([&] { coissue_kernel<KIND, 2><<<256, 256>>>(d, kIters); });
  printf("  %-18s MFMA only %7.1f us   vector only %7.1f us   interleaved %7.1f us   saved against the sum %5.1f %%\n",
         name, m, v, b, 100.0f * (m + v - b) / (m + v));
}

template <int KIND>
static void lds_row(float *d, char const *name, int bytes_per_lane) {
  float const us = time_us([&] { lds_read_kernel<KIND><<<256, 512>>>(d, kIters); });
  double const instr = 8.0 * 8 * kIters;  // per compute unit: 8 wavefronts x 8 reads x iterations
  printf("  %-20s %8.1f us   %.2f ns per wavefront instruction per compute unit   %.1f B/ns per compute unit\n", name,
         us, us * 1e3 / instr, bytes_per_lane * 64 * instr / (us * 1e3));
}

int main() {
  float *d = nullptr;
  CHECK(hipMalloc(&d, 4096));
  printf("1. co-issue, one wavefront per SIMD: per iteration 8 v_mfma_f32_16x16x32_f16 (two chains) and 32 vector "
         "instructions of one kind, %d iterations\n", kIters);
  coissue_row<V_FMA>(d, "v_fma_f32");
  coissue_row<V_EXP>(d, "v_exp_f32");
  coissue_row<V_CVT_PK>(d, "v_cvt_pk_f16_f32");
  coissue_row<V_DOT2>(d, "v_dot2_f32_f16");
  coissue_row<V_PK_ADD>(d, "v_pk_add_f16");
  {
    float const m = time_us([&] { coissue_kernel<V_FMA, 0><<<256, 256>>>(d, kIters); });
    float const v = time_us([&] { coissue_kernel<V_FMA, 1><<<256, 256>>>(d, kIters); });
    float const two = time_us([&] { coissue_kernel<V_FMA, 3><<<256, 512>>>(d, kIters); });
    float const mm = time_us([&] { coissue_kernel<V_FMA, 0><<<256, 512>>>(d, kIters); });
    float const vv = time_us([&] { coissue_kernel<V_FMA, 1><<<256, 512>>>(d, kIters); });
    float const both = time_us([&] { coissue_kernel<V_FMA, 2><<<256, 512>>>(d, kIters); });
    printf("   two wavefronts per SIMD: one MFMA-only and one v_fma-only %7.1f us (one of them alone: %7.1f and %7.1f;"
           " two MFMA-only %7.1f, two v_fma-only %7.1f); both interleaved %7.1f us\n", two, m, v, mm, vv, both);
  }
  printf("2. LDS reads, 8 wavefronts per compute unit issuing back to back\n");
  lds_row<0>(d, "ds_read_b64_tr_b16", 8);
  lds_row<1>(d, "ds_read_b64", 8);
  lds_row<2>(d, "ds_read_b128", 16);
  CHECK(hipFree(d));
  return 0;
}
