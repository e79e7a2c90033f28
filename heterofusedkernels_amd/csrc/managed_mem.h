// C++ face of libmanaged_memory.so for native code that links it directly
// (the torch op library does). Same role and method names as the reference's
// common/csrc/managed_memory/managed_mem.h:20-88, minus the vendor-specific
// second registration path; the extern "C" form is in hfk_managed_memory.h.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <shared_mutex>

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

    // Returns the (new or already existing) record, nullptr on failure.
    const RegisteredMemoryRecord* registerHostPtr(void* hostPtr, size_t bufferSize);
    // Records a mapping established by the caller; no HIP call.
    const RegisteredMemoryRecord* adoptMapping(void* hostPtr, void* devPtr, size_t bufferSize,
                                               int32_t device, int32_t kind);
    int unregisterHostPtr(void* hostPtr);
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
    const RegisteredMemoryRecord* findContaining(uintptr_t addr) const;
    bool overlapsOther(uintptr_t start, size_t size) const;

    std::map<uintptr_t, RegisteredMemoryRecord> records_;  // keyed by host start address
    mutable std::shared_mutex mux_;
};

}  // namespace managed_memory

// Free functions with the reference's names (managed_mem.cpp:305-334,372-375).
void* register_ptr(void* ptr, size_t size);
int unregister_ptr(void* ptr);
uintptr_t get_device_ptr(uintptr_t ptr);
