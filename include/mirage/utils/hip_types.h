// dim3 / int3 / int2 as HIP defines them (the reference takes them from CUDA's
// <vector_types.h>), plus a fail-loudly check used by the host runtime.
#pragma once

#include <hip/hip_runtime_api.h>
#include <hip/hip_vector_types.h>

#include <cstdio>
#include <cstdlib>

#define MIRAGE_CHECK(cond, msg)                                                   \
  do {                                                                            \
    if (!(cond)) {                                                                \
      std::fprintf(stderr, "mirage: %s (%s) at %s:%d\n", msg, #cond, __FILE__,    \
                   __LINE__);                                                     \
      std::abort();                                                               \
    }                                                                             \
  } while (0)
