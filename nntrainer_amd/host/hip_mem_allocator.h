// SPDX-License-Identifier: Apache-2.0
/**
 * @file   hip_mem_allocator.h
 * @brief  The allocator the HIP context gives the framework's memory pool: page-locked host
 *         memory, so that tensors cross to the GPU by DMA without a staging copy.
 *
 * A context publishes its allocator through ContextData (nntrainer/context.h:46-57); ClContext
 * sets the default calloc-based one (cl_context.cpp:83). MemAllocator's interface is alloc, free
 * and getName (nntrainer/mem_allocator.h:24-33).
 */
#ifndef HIPQ_HIP_MEM_ALLOCATOR_H
#define HIPQ_HIP_MEM_ALLOCATOR_H

#include <mutex>
#include <string>
#include <unordered_set>

#include "nntr_api.h"

namespace nntrainer {

class HipMemAllocator : public MemAllocator {
public:
  HipMemAllocator() = default;
  ~HipMemAllocator() override = default;
  /** zero-filled like the default allocator's calloc; `alignment` is met by any page-locked
   *  allocation (page aligned). Without a usable device, or when the runtime cannot page-lock
   *  that much, the memory is ordinary host memory: the framework must still be able to build
   *  and inspect a model, and pageable tensors cross through the library's own staging. */
  void alloc(void **ptr, size_t size, size_t alignment) override;
  void free(void *ptr) override;
  std::string getName() override { return "gpu"; }

private:
  std::mutex mtx;
  std::unordered_set<void *> pinned; /* what came from the device runtime and must return to it */
};

} // namespace nntrainer

#endif /* HIPQ_HIP_MEM_ALLOCATOR_H */
