# Compiles one HIP source for the device only with the compiler's resource report switched on and
# fails when a named kernel uses scratch memory, spills vector registers or runs fewer than
# OCCUPANCY wavefronts per SIMD.
#
#   cmake -DHIP_COMPILER=... -DSOURCE=... -DKERNELS=a;b -DOCCUPANCY=2 -DFLAGS=... -DSTAMP=...
#         -P check_kernel_resources.cmake
#
# For kernels whose inline-assembly loads land in registers behind the compiler's back
# (fp_mfma_matmul_big_kernel): a register spilled between such a load and its wait would save
# stale data, so a build that spills must not produce a library.  Same rule as
# attention_superoptimizer_amd/build.py (NO_SPILL_KERNELS).
separate_arguments(FLAG_LIST UNIX_COMMAND "${FLAGS}")
execute_process(
  COMMAND ${HIP_COMPILER} -x hip --offload-arch=gfx950 --cuda-device-only -O3 -std=c++17 ${FLAG_LIST}
          -Rpass-analysis=kernel-resource-usage -c ${SOURCE} -o ${STAMP}.o
  RESULT_VARIABLE rc
  ERROR_VARIABLE remarks
  OUTPUT_QUIET)
if(NOT rc EQUAL 0)
  message(FATAL_ERROR "resource check: ${SOURCE} does not compile:\n${remarks}")
endif()
# one chunk of text per kernel: from its "Function Name:" remark to the next
string(REPLACE "Function Name:" "\;" chunks "${remarks}")
string(REPLACE ";" "|" chunks "${chunks}")
string(REPLACE "\\|" ";" chunks "${chunks}")
foreach(kernel IN LISTS KERNELS)
  set(found 0)
  foreach(chunk IN LISTS chunks)
    string(FIND "${chunk}" "${kernel}" at)
    if(at EQUAL -1)
      continue()
    endif()
    # the chunk starts with the mangled name; the kernel's name must be in that first line
    string(REGEX MATCH "^[^\n]*" first_line "${chunk}")
    string(FIND "${first_line}" "${kernel}" at)
    if(at EQUAL -1)
      continue()
    endif()
    math(EXPR found "${found} + 1")
    if(NOT chunk MATCHES "ScratchSize \\[bytes/lane\\]: 0[^0-9]")
      message(FATAL_ERROR "resource check: ${kernel} uses scratch memory:\n${chunk}")
    endif()
    if(NOT chunk MATCHES "VGPRs Spill: 0[^0-9]")
      message(FATAL_ERROR "resource check: ${kernel} spills vector registers:\n${chunk}")
    endif()
    if(OCCUPANCY)
      string(REGEX MATCH "Occupancy \\[waves/SIMD\\]: ([0-9]+)" occ "${chunk}")
      if(NOT occ OR CMAKE_MATCH_1 LESS OCCUPANCY)
        message(FATAL_ERROR "resource check: ${kernel} runs fewer than ${OCCUPANCY} wavefronts per SIMD:\n${chunk}")
      endif()
    endif()
  endforeach()
  if(found EQUAL 0)
    message(FATAL_ERROR "resource check: the compiler reported nothing for ${kernel}")
  endif()
  message(STATUS "resource check: ${kernel}: ${found} instantiation(s), no scratch, no spills")
endforeach()
file(REMOVE ${STAMP}.o)
file(WRITE ${STAMP} "ok\n")
