// libmanaged_memory.so: registry of device-visible host ranges + pinned NUMA allocator.
#include "managed_mem.h"

#include <hip/hip_runtime_api.h>
#include <sched.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <cctype>
#include <cerrno>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iterator>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "hfk_managed_memory.h"

namespace managed_memory {

namespace {
thread_local int t_last_error = 0;

// Swallow the sticky error a failed HIP call leaves behind so that it is not
// reported by an unrelated later call.
void drop_hip_error() { (void)hipGetLastError(); }
}  // namespace

HostRegisteredMemoryManager& HostRegisteredMemoryManager::GetInstance() {
    // Leaked on purpose: records may be released from tensor deleters that run
    // during interpreter shutdown, after static destructors would have fired.
    static HostRegisteredMemoryManager* instance = new HostRegisteredMemoryManager();
    return *instance;
}

HostRegisteredMemoryManager::~HostRegisteredMemoryManager() { unregisterAll(); }

int HostRegisteredMemoryManager::lastError() { return t_last_error; }

RegisteredMemoryRecord* HostRegisteredMemoryManager::findContaining(uintptr_t addr) const {
    auto it = records_.upper_bound(addr);
    if (it == records_.begin()) return nullptr;
    --it;
    RegisteredMemoryRecord& r = it->second;
    return (addr - r.ptr < r.buffSize) ? &r : nullptr;
}

bool HostRegisteredMemoryManager::overlapsOther(uintptr_t start, size_t size) const {
    // Only neighbours can overlap because stored ranges are disjoint.
    auto next = records_.lower_bound(start);
    if (next != records_.end() && next->first - start < size) return true;
    if (next != records_.begin()) {
        auto prev = std::prev(next);
        if (start - prev->second.ptr < prev->second.buffSize) return true;
    }
    return false;
}

RegisteredMemoryRecord* HostRegisteredMemoryManager::adoptMapping(void* hostPtr, void* devPtr,
                                                                        size_t bufferSize, int32_t device,
                                                                        int32_t kind) {
    if (hostPtr == nullptr || devPtr == nullptr || bufferSize == 0) {
        t_last_error = HFK_MM_ERR_BAD_ARGUMENT;
        return nullptr;
    }
    const uintptr_t start = reinterpret_cast<uintptr_t>(hostPtr);
    const std::unique_lock<std::shared_mutex> guard(mux_);
    auto hit = records_.find(start);
    if (hit != records_.end()) {
        // Same start again: idempotent. A longer range over memory this library does not
        // own (it was pinned elsewhere and may have been re-used at a new size) grows the
        // record, provided it still ends before the next one.
        RegisteredMemoryRecord& r = hit->second;
        if (bufferSize > r.buffSize && r.kind == HFK_MM_KIND_ADOPTED && kind == HFK_MM_KIND_ADOPTED) {
            auto next = std::next(hit);
            if (next == records_.end() || next->first - start >= bufferSize) r.buffSize = bufferSize;
        }
        return &r;
    }
    if (overlapsOther(start, bufferSize)) {
        t_last_error = HFK_MM_ERR_OVERLAP;
        return nullptr;
    }
    auto ins = records_.emplace(
        start, RegisteredMemoryRecord{start, reinterpret_cast<uintptr_t>(devPtr), bufferSize, device, kind});
    return &ins.first->second;
}

RegisteredMemoryRecord* HostRegisteredMemoryManager::registerHostPtr(void* hostPtr, size_t bufferSize) {
    if (hostPtr == nullptr || bufferSize == 0) {
        t_last_error = HFK_MM_ERR_BAD_ARGUMENT;
        return nullptr;
    }
    const uintptr_t start = reinterpret_cast<uintptr_t>(hostPtr);
    {
        const std::shared_lock<std::shared_mutex> guard(mux_);
        auto hit = records_.find(start);
        if (hit != records_.end() && bufferSize <= hit->second.buffSize) return &hit->second;  // idempotent
        // A range inside an existing record is already device-visible.
        RegisteredMemoryRecord* outer = findContaining(start);
        if (outer != nullptr && start + bufferSize <= outer->ptr + outer->buffSize) return outer;
    }

    int device = -1;
    if (hipGetDevice(&device) != hipSuccess) {
        drop_hip_error();
        device = -1;
    }

    // The memory must be pinned already (hipHostMalloc, torch's pinned allocator, or a
    // hipHostRegister the caller made itself): it is adopted through hipHostGetDevicePointer.
    // This library never pins existing pageable memory. The runtime call that does so is refused
    // on some platforms (and the error it leaves is reported by an unrelated later call), so a
    // caller whose platform allows it registers the range itself and then hands it over; everyone
    // else allocates with hfk_mm_alloc_pinned / alloc_numa_pinned_tensor.
    hipPointerAttribute_t attr;
    std::memset(&attr, 0, sizeof(attr));
    hipError_t e = hipPointerGetAttributes(&attr, hostPtr);
    if (e != hipSuccess) drop_hip_error();
    if (e != hipSuccess || attr.type != hipMemoryTypeHost) {
        t_last_error = HFK_MM_ERR_NOT_PINNED;
        return nullptr;
    }
    void* devPtr = nullptr;
    e = hipHostGetDevicePointer(&devPtr, hostPtr, 0);
    if (e != hipSuccess || devPtr == nullptr) {
        drop_hip_error();
        t_last_error = e != hipSuccess ? static_cast<int>(e) : HFK_MM_ERR_BAD_ARGUMENT;
        return nullptr;
    }
    return adoptMapping(hostPtr, devPtr, bufferSize, device, HFK_MM_KIND_ADOPTED);
}

int HostRegisteredMemoryManager::unregisterHostPtr(void* hostPtr) {
    if (hostPtr == nullptr) return HFK_MM_ERR_BAD_ARGUMENT;
    const std::unique_lock<std::shared_mutex> guard(mux_);
    records_.erase(reinterpret_cast<uintptr_t>(hostPtr));   // never registered: nothing to undo
    return HFK_MM_OK;   // the pinning itself belongs to whoever made it (the allocator here, or the caller)
}

void HostRegisteredMemoryManager::unregisterAll() {
    const std::unique_lock<std::shared_mutex> guard(mux_);
    records_.clear();
}

void* HostRegisteredMemoryManager::getDevicePtr(const void* hostPtr) const {
    if (hostPtr == nullptr) return nullptr;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(hostPtr);
    const std::shared_lock<std::shared_mutex> guard(mux_);
    const RegisteredMemoryRecord* r = findContaining(addr);
    return r ? reinterpret_cast<void*>(r->devptr + (addr - r->ptr)) : nullptr;
}

size_t HostRegisteredMemoryManager::getRecordSize(const void* hostPtr) const {
    if (hostPtr == nullptr) return 0;
    const std::shared_lock<std::shared_mutex> guard(mux_);
    const RegisteredMemoryRecord* r = findContaining(reinterpret_cast<uintptr_t>(hostPtr));
    return r ? r->buffSize : 0;
}

size_t HostRegisteredMemoryManager::recordCount() const {
    const std::shared_lock<std::shared_mutex> guard(mux_);
    return records_.size();
}

}  // namespace managed_memory

using managed_memory::HostRegisteredMemoryManager;

void* register_ptr(void* ptr, size_t size) {
    const auto* rec = HostRegisteredMemoryManager::GetInstance().registerHostPtr(ptr, size);
    if (rec == nullptr) return nullptr;
    const uintptr_t off = reinterpret_cast<uintptr_t>(ptr) - rec->ptr;
    return reinterpret_cast<void*>(rec->devptr + off);
}

int unregister_ptr(void* ptr) { return HostRegisteredMemoryManager::GetInstance().unregisterHostPtr(ptr); }

uintptr_t get_device_ptr(uintptr_t ptr) {
    return reinterpret_cast<uintptr_t>(
        HostRegisteredMemoryManager::GetInstance().getDevicePtr(reinterpret_cast<const void*>(ptr)));
}

// The reference's allocator entry points (common/csrc/mem_alloc.cpp:66-115) under their own names.
uintptr_t alloc_pinned_numa_ptr(std::size_t size, int numaNode) {
    void* p = nullptr;
    if (hfk_mm_alloc_pinned(size, numaNode, 0, &p) != HFK_MM_OK) return 0;
    return reinterpret_cast<uintptr_t>(p);
}

void free_pinned_numa_ptr(void* ptr) {
    if (ptr != nullptr) (void)hfk_mm_free_pinned(ptr);
}

// ---------------------------------------------------------------------------
// NUMA placement. The memory policy syscalls are used directly so the library
// has no libnuma dependency.
// ---------------------------------------------------------------------------
namespace {

constexpr int kMpolDefault = 0;
constexpr int kMpolBind = 2;
constexpr unsigned long kMaxNodes = 1024;
constexpr size_t kMaskWords = kMaxNodes / (8 * sizeof(unsigned long));

long sys_get_mempolicy(int* mode, unsigned long* mask, unsigned long maxnode) {
    return syscall(SYS_get_mempolicy, mode, mask, maxnode, nullptr, 0ul);
}

long sys_set_mempolicy(int mode, const unsigned long* mask, unsigned long maxnode) {
    return syscall(SYS_set_mempolicy, mode, mask, maxnode);
}

// Binds this thread's future page allocations to one node for its lifetime.
class ScopedNodeBinding {
public:
    explicit ScopedNodeBinding(int node) {
        if (node < 0 || static_cast<unsigned long>(node) >= kMaxNodes) return;
        if (sys_get_mempolicy(&saved_mode_, saved_mask_, kMaxNodes) != 0) return;
        unsigned long mask[kMaskWords] = {0};
        mask[node / (8 * sizeof(unsigned long))] = 1ul << (node % (8 * sizeof(unsigned long)));
        if (sys_set_mempolicy(kMpolBind, mask, kMaxNodes) == 0) active_ = true;
    }
    ~ScopedNodeBinding() {
        if (!active_) return;
        if (saved_mode_ == kMpolDefault) (void)sys_set_mempolicy(kMpolDefault, nullptr, 0);
        else (void)sys_set_mempolicy(saved_mode_, saved_mask_, kMaxNodes);
    }
    bool active() const { return active_; }

private:
    bool active_ = false;
    int saved_mode_ = kMpolDefault;
    unsigned long saved_mask_[kMaskWords] = {0};
};

// Zero-fills freshly pinned memory. hipHostMalloc returns at once and the pages are faulted in
// (and pinned) by their first touch, which is what takes the time: 2.8 GB/s from one thread,
// 14 GB/s from eight, 19 GB/s from sixteen (measured; once touched, one thread writes 99 GB/s).
// So a large range is touched by several threads, each under the same node binding as the
// caller because a memory policy is per thread and the first touch decides where a page lands.
void zero_fill(void* p, size_t bytes, int numa_node) {
    constexpr size_t kPerThreadMin = 128u << 20;
    constexpr size_t kAlign = 2u << 20;
    unsigned cpus = 1;
    cpu_set_t set;
    if (sched_getaffinity(0, sizeof(set), &set) == 0) cpus = static_cast<unsigned>(CPU_COUNT(&set));
    size_t parts = bytes / kPerThreadMin;
    if (parts > 8) parts = 8;
    if (parts > cpus) parts = cpus;
    if (parts < 2) {
        std::memset(p, 0, bytes);
        return;
    }
    size_t per = (bytes / parts + kAlign - 1) / kAlign * kAlign;
    auto fill_part = [=](size_t i) {
        const size_t lo = i * per;
        if (lo >= bytes) return;
        const size_t n = lo + per < bytes ? per : bytes - lo;
        ScopedNodeBinding bind(numa_node);
        std::memset(static_cast<char*>(p) + lo, 0, n);
    };
    std::vector<std::thread> workers;
    size_t started = 1;  // part 0 is this thread's
    try {
        for (; started < parts; ++started) workers.emplace_back(fill_part, started);
    } catch (...) {
        // no more threads to be had: this thread does the rest
    }
    fill_part(0);
    for (size_t i = started; i < parts; ++i) fill_part(i);
    for (auto& w : workers) w.join();
}

}  // namespace

extern "C" {

int hfk_mm_register(void* host_ptr, size_t bytes, void** dev_ptr_out) {
    if (host_ptr == nullptr || bytes == 0) return HFK_MM_ERR_BAD_ARGUMENT;
    void* dev = register_ptr(host_ptr, bytes);
    if (dev == nullptr) {
        const int err = HostRegisteredMemoryManager::lastError();
        return err != 0 ? err : HFK_MM_ERR_BAD_ARGUMENT;
    }
    if (dev_ptr_out) *dev_ptr_out = dev;
    return HFK_MM_OK;
}

int hfk_mm_adopt(void* host_ptr, void* dev_ptr, size_t bytes, int device) {
    const auto* rec = HostRegisteredMemoryManager::GetInstance().adoptMapping(host_ptr, dev_ptr, bytes, device,
                                                                              HFK_MM_KIND_ADOPTED);
    if (rec == nullptr) return HostRegisteredMemoryManager::lastError();
    return HFK_MM_OK;
}

int hfk_mm_unregister(void* host_ptr) { return unregister_ptr(host_ptr); }

void hfk_mm_unregister_all(void) { HostRegisteredMemoryManager::GetInstance().unregisterAll(); }

void* hfk_mm_get_device_ptr(const void* host_ptr) {
    return HostRegisteredMemoryManager::GetInstance().getDevicePtr(host_ptr);
}

size_t hfk_mm_record_size(const void* host_ptr) {
    return HostRegisteredMemoryManager::GetInstance().getRecordSize(host_ptr);
}

size_t hfk_mm_record_count(void) { return HostRegisteredMemoryManager::GetInstance().recordCount(); }

int hfk_mm_device_numa_node(int device, int* node_out) {
    if (node_out == nullptr) return HFK_MM_ERR_BAD_ARGUMENT;
    *node_out = -1;
    char bdf[64] = {0};
    hipError_t e = hipDeviceGetPCIBusId(bdf, sizeof(bdf) - 1, device);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return static_cast<int>(e);
    }
    std::string id(bdf);
    for (char& c : id) c = static_cast<char>(std::tolower(static_cast<unsigned char>(c)));
    std::ifstream f("/sys/bus/pci/devices/" + id + "/numa_node");
    if (!f.is_open()) return HFK_MM_OK;  // sysfs hidden (containers): treat as "no NUMA information"
    int node = -1;
    f >> node;
    if (!f.fail()) *node_out = node;
    return HFK_MM_OK;
}

int hfk_mm_alloc_pinned(size_t bytes, int numa_node, unsigned flags, void** host_ptr_out) {
    if (bytes == 0 || host_ptr_out == nullptr) return HFK_MM_ERR_BAD_ARGUMENT;
    *host_ptr_out = nullptr;
    void* p = nullptr;
    hipError_t e;
    {
        ScopedNodeBinding bind(numa_node);
        unsigned hip_flags = hipHostMallocMapped | hipHostMallocPortable;
        if (bind.active()) hip_flags |= hipHostMallocNumaUser;
        if (flags & HFK_MM_ALLOC_NONCOHERENT) hip_flags |= hipHostMallocNonCoherent;
        e = hipHostMalloc(&p, bytes, hip_flags);
    }
    if (e != hipSuccess || p == nullptr) {
        (void)hipGetLastError();
        return e != hipSuccess ? static_cast<int>(e) : HFK_MM_ERR_OS;
    }
    zero_fill(p, bytes, numa_node);
    void* dev = nullptr;
    e = hipHostGetDevicePointer(&dev, p, 0);
    if (e != hipSuccess || dev == nullptr) {
        (void)hipGetLastError();
        (void)hipHostFree(p);
        return e != hipSuccess ? static_cast<int>(e) : HFK_MM_ERR_OS;
    }
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess) {
        (void)hipGetLastError();
        device = -1;
    }
    const auto* rec = HostRegisteredMemoryManager::GetInstance().adoptMapping(p, dev, bytes, device,
                                                                              HFK_MM_KIND_ALLOCATED);
    if (rec == nullptr) {
        (void)hipHostFree(p);
        return HostRegisteredMemoryManager::lastError();
    }
    *host_ptr_out = p;
    return HFK_MM_OK;
}

int hfk_mm_free_pinned(void* host_ptr) {
    if (host_ptr == nullptr) return HFK_MM_ERR_BAD_ARGUMENT;
    (void)HostRegisteredMemoryManager::GetInstance().unregisterHostPtr(host_ptr);
    hipError_t e = hipHostFree(host_ptr);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return static_cast<int>(e);
    }
    return HFK_MM_OK;
}

const char* hfk_mm_status_string(int status) {
    switch (status) {
        case HFK_MM_OK: return "ok";
        case HFK_MM_ERR_BAD_ARGUMENT: return "managed_memory: null pointer or zero size";
        case HFK_MM_ERR_OVERLAP: return "managed_memory: range overlaps a different registration";
        case HFK_MM_ERR_NOT_FOUND: return "managed_memory: pointer is not registered";
        case HFK_MM_ERR_OS: return "managed_memory: operating-system call failed";
        case HFK_MM_ERR_NOT_PINNED:
            return "managed_memory: the range is not pinned host memory (allocate it with hfk_mm_alloc_pinned / "
                   "alloc_numa_pinned_tensor, or pin it yourself before registering it)";
        default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "managed_memory: unknown status";
}

}  // extern "C"
