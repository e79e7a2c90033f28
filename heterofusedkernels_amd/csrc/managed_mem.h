// C++ face of libmanaged_memory.so for native code that links it directly
// (the torch op library does). Source-compatible with what callers use of the
// reference's common/csrc/managed_memory/managed_mem.h:9-88: the record struct, the
// manager's registerHostPtr / aclUnregisterHostPtr / getDevicePtr / getRecordSize /
// unregisterAll, and the free functions register_ptr, unregister_ptr, register_tensor,
// unregister_tensor, get_device_ptr. The vendor-specific second registration path
// (halRegisterHostPtr and the driver-version probe, managed_mem.h:48-71) has no
// counterpart. The extern "C" form is in hfk_managed_memory.h.
//
// The library itself does not depend on torch. register_tensor / unregister_tensor are
// therefore defined in this header, for translation units that can see torch's headers
// (every caller of the reference's header can: it includes them unconditionally).
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <shared_mutex>

#if !defined(HFK_MANAGED_MEM_NO_TORCH) && defined(__has_include)
#if __has_include(<torch/extension.h>)
#define HFK_MANAGED_MEM_HAS_TORCH 1
#include <torch/extension.h>
#endif
#endif

namespace managed_memory {

struct RegisteredMemoryRecord {
    uintptr_t ptr;     // host start address
    uintptr_t devptr;  // address kernels use for the same bytes
    size_t buffSize;
    int32_t device;    // HIP device current at registration, -1 if unknown
    int32_t kind;      // hfk_mm_kind
};

class HostRegisteredMemoryManager {
public:
    static HostRegisteredMemoryManager& GetInstance();

    HostRegisteredMemoryManager(const HostRegisteredMemoryManager&) = delete;
    HostRegisteredMemoryManager& operator=(const HostRegisteredMemoryManager&) = delete;

    // Returns the (new or already existing) record, nullptr on failure (lastError() says why;
    // memory that is not pinned yet is refused with HFK_MM_ERR_NOT_PINNED).
    RegisteredMemoryRecord* registerHostPtr(void* hostPtr, size_t bufferSize);
    // Records a mapping established by the caller; no HIP call.
    RegisteredMemoryRecord* adoptMapping(void* hostPtr, void* devPtr, size_t bufferSize, int32_t device,
                                         int32_t kind);
    int unregisterHostPtr(void* hostPtr);
    // The reference's name for the same call (managed_mem.h:52).
    int aclUnregisterHostPtr(void* hostPtr) { return unregisterHostPtr(hostPtr); }
    void* getDevicePtr(const void* hostPtr) const;
    size_t getRecordSize(const void* hostPtr) const;
    size_t recordCount() const;
    void unregisterAll();
    // Status of the last failed registerHostPtr on this thread (hfk_mm_status or hipError_t).
    static int lastError();

private:
    HostRegisteredMemoryManager() = default;
    ~HostRegisteredMemoryManager();

    // Record containing addr, or nullptr. Caller holds the lock.
    RegisteredMemoryRecord* findContaining(uintptr_t addr) const;
    bool overlapsOther(uintptr_t start, size_t size) const;

    mutable std::map<uintptr_t, RegisteredMemoryRecord> records_;  // keyed by host start address
    mutable std::shared_mutex mux_;
};

}  // namespace managed_memory

// Free functions with the reference's names (managed_mem.cpp:305-334,372-375).
void* register_ptr(void* ptr, size_t size);
int unregister_ptr(void* ptr);
uintptr_t get_device_ptr(uintptr_t ptr);
// The reference's allocator entry points (common/csrc/mem_alloc.h:8-10): zero-filled pinned,
// device-mapped memory bound to numaNode (< 0: no binding), 0 on failure.
uintptr_t alloc_pinned_numa_ptr(std::size_t size, int numaNode);
void free_pinned_numa_ptr(void* ptr);

#if defined(HFK_MANAGED_MEM_HAS_TORCH)
// Registers a pinned CPU tensor and returns its device-visible address; any other tensor is
// rejected with the reference's message (managed_mem.cpp:336-364). torch answers is_pinned()
// through its device hooks, which say "not pinned" until torch has initialised the device, so
// that is done first (where no usable GPU exists the tensor check below reports the problem).
inline void* register_tensor(torch::Tensor& tensor) {
    if (tensor.device().is_cpu()) {
        try {
            at::globalContext().lazyInitDevice(c10::DeviceType::CUDA);
        } catch (const c10::Error&) {
        }
    }
    if (!tensor.device().is_cpu() || !tensor.is_pinned()) {
        TORCH_CHECK(false, "Invalid device. Device must be CPU and tensor must be pinned.");
    }
    void* dev = register_ptr(tensor.data_ptr(), tensor.nbytes());
    TORCH_CHECK(dev != nullptr, "Failed to register memory");
    return dev;
}

// Drops the tensor's record (managed_mem.cpp:366-370).
inline void unregister_tensor(torch::Tensor& tensor) { (void)unregister_ptr(tensor.data_ptr()); }
#endif
