// Process-wide device arena (reference include/mirage/kernel/device_memory_manager.h:28-53):
// one allocation made by the backend at first use, handed out by a bump pointer
// and returned strictly last-in-first-out.  Every tensor gets a data buffer and
// a fingerprint buffer, each rounded to 16 bytes.  Default size 10 GiB
// (environment MIRAGE_ARENA_BYTES overrides).  With MIRAGE_HOST_ONLY=1 and no
// GPU the manager hands out addresses only, so graph construction and plan
// lowering can be exercised on a CPU-only machine; any device work then aborts.
#pragma once

#include "mirage/kernel/device_tensor.h"
#include <sys/types.h>
#include <utility>
#include <vector>

namespace mirage {
namespace kernel {

class DeviceMemoryManager {
public:
  static DeviceMemoryManager *singleton;
  DeviceMemoryManager(void);
  ~DeviceMemoryManager(void);
  bool allocate(DTensor &tensor, bool allocate_fingerprint = true);
  bool free(DTensor &tensor);
  static DeviceMemoryManager *get_instance();

  char *base_ptr;
  off_t offset;
  size_t total_size;
  std::vector<std::pair<void *, size_t>> allocated_tensors;
  // device copies of the fingerprint lookup tables (owned by the backend)
  mirage::type::FPType *exp_lookup_table;
  mirage::type::FPType *div_p_lookup_table;
  mirage::type::FPType *div_q_lookup_table;
  bool device_ready;  // false in host-only mode
};

// Aborts with a clear message unless a GPU backend is attached.
void require_device(char const *what);

}  // namespace kernel
}  // namespace mirage
