// Compile-only check: a native consumer written against the reference's shipped header
// (common/csrc/managed_memory/managed_mem.h, included as "managed_mem.h" by
// pcieThrough/csrc/host/gather_torch.cpp:8 and multi_layer_block_transfer_torch.cpp:9)
// must build unchanged against the header shipped here. Every call below is one the
// reference's own sources make (file:line beside it); nothing here is run.
#include "managed_mem.h"

#include <torch/extension.h>

namespace consumer {

// gather_torch.cpp:50-51, multi_layer_block_transfer_torch.cpp:77-78
void* device_side_of(at::Tensor& hostTensor) {
    auto& hmm = managed_memory::HostRegisteredMemoryManager::GetInstance();
    void* hostPtr = hostTensor.data_ptr();
    return hmm.getDevicePtr(hostPtr);
}

// managed_mem.cpp:305-323 (what register_ptr does with the manager)
void* register_range(void* ptr, size_t size) {
    auto& hmm = managed_memory::HostRegisteredMemoryManager::GetInstance();
    managed_memory::RegisteredMemoryRecord* record = hmm.registerHostPtr(ptr, size);
    if (record == nullptr) {
        return nullptr;
    }
    return reinterpret_cast<void*>(record->devptr);
}

// managed_mem.cpp:325-334, 366-370, mem_alloc.cpp:49-57
int drop_range(void* ptr, torch::Tensor& tensor) {
    auto& hmm = managed_memory::HostRegisteredMemoryManager::GetInstance();
    size_t known = hmm.getRecordSize(ptr);
    (void)known;
    unregister_tensor(tensor);
    return hmm.aclUnregisterHostPtr(ptr);
}

// pybind.cpp:7-11 binds these three by address
using RegisterTensorFn = void* (*)(torch::Tensor&);
using GetDevicePtrFn = uintptr_t (*)(uintptr_t);
RegisterTensorFn bound_host_register = &register_tensor;
GetDevicePtrFn bound_get_device_ptr = &get_device_ptr;

// mem_alloc.cpp:17-64 (allocation + deleter of alloc_numa_pinned_tensor)
uintptr_t pinned(std::size_t bytes, int node) {
    uintptr_t p = alloc_pinned_numa_ptr(bytes, node);
    if (p != 0) free_pinned_numa_ptr(reinterpret_cast<void*>(p));
    void* again = register_ptr(reinterpret_cast<void*>(p), bytes);
    (void)again;
    return static_cast<uintptr_t>(unregister_ptr(reinterpret_cast<void*>(p)));
}

void everything_off() { managed_memory::HostRegisteredMemoryManager::GetInstance().unregisterAll(); }

}  // namespace consumer
