// SPDX-License-Identifier: Apache-2.0
/**
 * @file   hip_mem_allocator.cpp
 * @brief  HipMemAllocator (see hip_mem_allocator.h).
 */
#include "hip_mem_allocator.h"

#include <cstdlib>
#include <stdexcept>

#include "hipq_host.h"

namespace nntrainer {

void HipMemAllocator::alloc(void **ptr, size_t size, size_t /*alignment*/) {
  if (!ptr)
    throw std::invalid_argument("[HipMemAllocator] null result pointer");
  if (size == 0)
    size = 1; /* the default allocator logs and allocates nothing useful; a valid pointer is kinder */
  if (hipq_host::runtime_available()) {
    void *p = nullptr;
    const int rc = hipq_host_alloc(&p, size);
    if (rc == HIPQ_OK) {
      std::lock_guard<std::mutex> lock(mtx);
      pinned.insert(p);
      *ptr = p;
      return;
    }
    /* a pool larger than the system lets a process page-lock (a multi-GB model): ordinary memory
     * serves as well, its tensors cross through the library's page-locked staging instead */
    if (rc != HIPQ_ERR_OUT_OF_MEMORY)
      hipq_host::check(rc, "hipq_host_alloc");
  }
  *ptr = std::calloc(size, 1);
  if (!*ptr)
    throw std::bad_alloc();
}

void HipMemAllocator::free(void *ptr) {
  if (!ptr)
    return;
  {
    std::lock_guard<std::mutex> lock(mtx);
    auto it = pinned.find(ptr);
    if (it == pinned.end()) {
      std::free(ptr);
      return;
    }
    pinned.erase(it);
  }
  hipq_host::check(hipq_host_free(ptr), "hipq_host_free");
}

} // namespace nntrainer
