// The device arena: bookkeeping on the host, memory and lookup tables owned by
// the backend (mi355_init).  Reference src/kernel/device_memory_manager.cu:26-145.
#include "mirage/kernel/device_memory_manager.h"
#include "mi355_abi.h"
#include "mirage/utils/hip_types.h"

#include <cstdlib>
#include <cstring>

namespace mirage {
namespace kernel {

DeviceMemoryManager *DeviceMemoryManager::singleton = nullptr;

static size_t round16(size_t n) { return (n + 15) / 16 * 16; }

DeviceMemoryManager::DeviceMemoryManager()
    : base_ptr(nullptr), offset(0), total_size((size_t)10 * 1024 * 1024 * 1024),
      exp_lookup_table(nullptr), div_p_lookup_table(nullptr), div_q_lookup_table(nullptr),
      device_ready(false) {
  if (char const *env = std::getenv("MIRAGE_ARENA_BYTES")) {
    total_size = std::strtoull(env, nullptr, 10);
  }
  void *base = nullptr;
  int rc = mi355_init(total_size, &base);
  if (rc == MI355_OK) {
    base_ptr = static_cast<char *>(base);
    void const *e = nullptr, *p = nullptr, *q = nullptr;
    MIRAGE_CHECK(mi355_get_tables(&e, &p, &q) == MI355_OK, mi355_last_error());
    exp_lookup_table = static_cast<mirage::type::FPType *>(const_cast<void *>(e));
    div_p_lookup_table = static_cast<mirage::type::FPType *>(const_cast<void *>(p));
    div_q_lookup_table = static_cast<mirage::type::FPType *>(const_cast<void *>(q));
    device_ready = true;
    return;
  }
  char const *host_only = std::getenv("MIRAGE_HOST_ONLY");
  if (rc == MI355_ERR_NO_DEVICE && host_only != nullptr && std::strcmp(host_only, "1") == 0) {
    // addresses only: a fake, never dereferenced base
    base_ptr = reinterpret_cast<char *>(static_cast<uintptr_t>(1) << 40);
    return;
  }
  std::fprintf(stderr, "mirage: cannot initialise the MI355X backend: %s\n", mi355_last_error());
  std::abort();
}

DeviceMemoryManager::~DeviceMemoryManager() {
  if (device_ready) {
    mi355_shutdown();
  }
}

bool DeviceMemoryManager::allocate(DTensor &tensor, bool allocate_fingerprint) {
  MIRAGE_CHECK(offset % 16 == 0, "arena offset lost its alignment");
  size_t bytes = round16(tensor.data_size());
  tensor.data_ptr = base_ptr + offset;
  allocated_tensors.push_back({tensor.data_ptr, bytes});
  offset += bytes;
  tensor.fp_ptr = nullptr;
  if (allocate_fingerprint) {
    bytes = round16(tensor.fingerprint_size());
    tensor.fp_ptr = reinterpret_cast<mirage::type::FPType *>(base_ptr + offset);
    allocated_tensors.push_back({tensor.fp_ptr, bytes});
    offset += bytes;
  }
  MIRAGE_CHECK((size_t)offset <= total_size, "device arena exhausted");
  return true;
}

bool DeviceMemoryManager::free(DTensor &tensor) {
  // strictly last-in-first-out
  if (tensor.fp_ptr != nullptr) {
    MIRAGE_CHECK(!allocated_tensors.empty() && allocated_tensors.back().first == tensor.fp_ptr,
                 "tensors must be freed in reverse allocation order");
    offset -= allocated_tensors.back().second;
    allocated_tensors.pop_back();
  }
  MIRAGE_CHECK(!allocated_tensors.empty() && allocated_tensors.back().first == tensor.data_ptr,
               "tensors must be freed in reverse allocation order");
  offset -= allocated_tensors.back().second;
  allocated_tensors.pop_back();
  return true;
}

DeviceMemoryManager *DeviceMemoryManager::get_instance() {
  if (singleton == nullptr) {
    singleton = new DeviceMemoryManager();
  }
  return singleton;
}

void require_device(char const *what) {
  if (!DeviceMemoryManager::get_instance()->device_ready) {
    std::fprintf(stderr, "mirage: %s needs the MI355X backend, but the runtime is in host-only mode\n",
                 what);
    std::abort();
  }
}

}  // namespace kernel
}  // namespace mirage
