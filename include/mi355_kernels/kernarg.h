// Early fetch of the kernel-argument block, for kernels whose run time is a few microseconds.
//
// The host writes a launch's argument block just before the launch, so every line of it is
// cold when the first wavefront asks for it, and the compiler loads each field where it is
// first needed: a latency-bound kernel with a parameter block of a few hundred bytes makes
// two or three trips to memory in a row before it can form its first address.
// fetch_kernel_arguments<BYTES>() issues one scalar load per 64-byte line of the block, all at
// once at the top of the kernel, and waits for them: one trip, after which every field comes
// from the scalar cache.  The loaded words are not used (they all go to one register), and the
// wait is part of the same statement, so no load is in flight where the compiler could hand
// that register to something else.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mi355 {

// Offset of the last word of a kernel's argument block: BYTES of explicit arguments and, when
// the kernel reads gridDim or blockDim, the words the compiler keeps right behind them (8-byte
// aligned): the block counts x, y, z, then a word with the workgroup's sizes x and y.
// HIDDEN_WORDS = how many of these words the kernel is known to read up to (1 = gridDim.x, 2 =
// .x and .y, 3 = all of gridDim, 4 = blockDim.x as well): they are part of its block exactly
// when it reads them.
template <int BYTES, int HIDDEN_WORDS>
constexpr int kernarg_last_word() {
  static_assert(BYTES % 4 == 0 && BYTES >= 4 && HIDDEN_WORDS >= 0 && HIDDEN_WORDS <= 4, "words of 4 bytes");
  return HIDDEN_WORDS == 0 ? BYTES - 4 : (BYTES + 7) / 8 * 8 + 4 * HIDDEN_WORDS - 4;
}

// Loads go to the first word of every 64 bytes and to the block's last word (the block may
// start anywhere in a line, so its tail can lie one line further than its last multiple of
// 64); none reaches past the block.
template <int BYTES, int HIDDEN_WORDS>
__device__ __forceinline__ void fetch_kernel_arguments() {
  constexpr int last = kernarg_last_word<BYTES, HIDDEN_WORDS>();
  static_assert(last <= 512, "nine loads cover 576 bytes");
#define MI355_KERNARG_AT(i) "i"(64 * (i) < last ? 64 * (i) : last)
  auto const *block = __builtin_amdgcn_kernarg_segment_ptr();
  uint32_t unused;
  asm volatile(
      "s_load_dword %0, %1, %2\n\t"
      "s_load_dword %0, %1, %3\n\t"
      "s_load_dword %0, %1, %4\n\t"
      "s_load_dword %0, %1, %5\n\t"
      "s_load_dword %0, %1, %6\n\t"
      "s_load_dword %0, %1, %7\n\t"
      "s_load_dword %0, %1, %8\n\t"
      "s_load_dword %0, %1, %9\n\t"
      "s_load_dword %0, %1, %10\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&s"(unused)
      : "s"(block), MI355_KERNARG_AT(0), MI355_KERNARG_AT(1), MI355_KERNARG_AT(2), MI355_KERNARG_AT(3),
        MI355_KERNARG_AT(4), MI355_KERNARG_AT(5), MI355_KERNARG_AT(6), MI355_KERNARG_AT(7), MI355_KERNARG_AT(8)
      : "memory");
#undef MI355_KERNARG_AT
}

// The same for an argument block of any size (job tables of a few KB that a workgroup searches
// entry by entry: every entry in a new line would be a trip of its own): a loop of scalar loads,
// one per 64 bytes and one to the last word, then one wait.  BYTES: the explicit arguments, or
// any prefix of them that ends on a word.
template <int BYTES>
__device__ __forceinline__ void fetch_kernel_arguments_large() {
  static_assert(BYTES % 4 == 0 && BYTES > 64 && BYTES <= 4096, "an argument block of up to 4 KB");
  auto const *block = __builtin_amdgcn_kernarg_segment_ptr();
  uint32_t unused, offset;
  asm volatile(
      "s_mov_b32 %1, 0\n"
      ".Lkernarg_line%=:\n\t"
      "s_load_dword %0, %2, %1\n\t"
      "s_add_u32 %1, %1, 64\n\t"
      "s_cmp_lt_u32 %1, %3\n\t"
      "s_cbranch_scc1 .Lkernarg_line%=\n\t"
      "s_load_dword %0, %2, %3\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&s"(unused), "=&s"(offset)
      : "s"(block), "i"(BYTES - 4)
      : "scc", "memory");
}

// The whole argument block of a kernel whose only parameter is one T, read into scalar
// registers by loads issued together: the kernel then makes one trip for its arguments instead
// of one per place where the compiler first needs a field.  For blocks of 320 bytes (five
// loads of 64), of 240 (64, 64, 64, 32, 16) and of 152 (64, 64, 16, 8); a larger block does not
// fit the scalar registers
// beside the kernel's own values and takes fetch_kernel_arguments.  The block counts behind
// the arguments are touched as above.
typedef uint32_t kernarg_words16 __attribute__((ext_vector_type(16)));
typedef uint32_t kernarg_words8 __attribute__((ext_vector_type(8)));
typedef uint32_t kernarg_words4 __attribute__((ext_vector_type(4)));
typedef uint32_t kernarg_words2 __attribute__((ext_vector_type(2)));
template <typename T, int HIDDEN_WORDS>
__device__ __forceinline__ T load_kernel_arguments() {
  static_assert((sizeof(T) == 320 || sizeof(T) == 240 || sizeof(T) == 152) && alignof(T) <= 8,
                "a block size this was written for");
  auto const *block = __builtin_amdgcn_kernarg_segment_ptr();
  constexpr int last = kernarg_last_word<(int)sizeof(T), HIDDEN_WORDS>();
  uint32_t unused;
  T t;
  if constexpr (sizeof(T) == 320) {
    struct {
      kernarg_words16 w[5];
    } regs;
    asm volatile(
        "s_load_dwordx16 %0, %6, 0x0\n\t"
        "s_load_dwordx16 %1, %6, 0x40\n\t"
        "s_load_dwordx16 %2, %6, 0x80\n\t"
        "s_load_dwordx16 %3, %6, 0xc0\n\t"
        "s_load_dwordx16 %4, %6, 0x100\n\t"
        "s_load_dword %5, %6, %7\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&s"(regs.w[0]), "=&s"(regs.w[1]), "=&s"(regs.w[2]), "=&s"(regs.w[3]), "=&s"(regs.w[4]), "=&s"(unused)
        : "s"(block), "i"(last)
        : "memory");
    static_assert(sizeof(regs) == sizeof(T), "no padding");
    __builtin_memcpy(&t, &regs, sizeof(T));
  } else if constexpr (sizeof(T) == 240) {
    struct {
      kernarg_words16 w[3];
      kernarg_words8 x;
      kernarg_words4 y;
    } regs;
    asm volatile(
        "s_load_dwordx16 %0, %6, 0x0\n\t"
        "s_load_dwordx16 %1, %6, 0x40\n\t"
        "s_load_dwordx16 %2, %6, 0x80\n\t"
        "s_load_dwordx8 %3, %6, 0xc0\n\t"
        "s_load_dwordx4 %4, %6, 0xe0\n\t"
        "s_load_dword %5, %6, %7\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&s"(regs.w[0]), "=&s"(regs.w[1]), "=&s"(regs.w[2]), "=&s"(regs.x), "=&s"(regs.y), "=&s"(unused)
        : "s"(block), "i"(last)
        : "memory");
    static_assert(sizeof(regs) >= sizeof(T), "registers for the whole block");
    __builtin_memcpy(&t, &regs, sizeof(T));
  } else {
    struct {
      kernarg_words16 w[2];
      kernarg_words4 x;
      kernarg_words2 y;
    } regs;
    asm volatile(
        "s_load_dwordx16 %0, %5, 0x0\n\t"
        "s_load_dwordx16 %1, %5, 0x40\n\t"
        "s_load_dwordx4 %2, %5, 0x80\n\t"
        "s_load_dwordx2 %3, %5, 0x90\n\t"
        "s_load_dword %4, %5, %6\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&s"(regs.w[0]), "=&s"(regs.w[1]), "=&s"(regs.x), "=&s"(regs.y), "=&s"(unused)
        : "s"(block), "i"(last)
        : "memory");
    static_assert(sizeof(regs) >= sizeof(T), "registers for the whole block");
    __builtin_memcpy(&t, &regs, sizeof(T));
  }
  return t;
}

}  // namespace mi355
