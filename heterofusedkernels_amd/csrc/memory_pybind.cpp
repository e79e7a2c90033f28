// heterofusedkernels.memory: the three Python callables of the reference's common
// package (common/csrc/pybind.cpp:7-11) on top of libmanaged_memory.so, plus two
// small additions (host_unregister, device_numa_node).
#include <hip/hip_runtime_api.h>
#include <torch/extension.h>

#include <cstdlib>
#include <string>

#include "hfk_managed_memory.h"
#include "managed_mem.h"

namespace {

// torch answers Tensor::is_pinned() through its device hooks, which report "not pinned"
// until torch itself has initialised the device; a tensor handed out here must say it is pinned.
// Without a usable GPU the initialisation throws; the callers' own checks then report the problem.
void ensure_torch_device_ready() {
    try {
        at::globalContext().lazyInitDevice(c10::DeviceType::CUDA);
    } catch (const c10::Error&) {
    }
}

int current_hip_device() {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    TORCH_CHECK(e == hipSuccess, "Unable to obtain device Id: ", hipGetErrorString(e));
    return dev;
}

// 1-D int8 CPU tensor over zero-filled pinned memory on the current device's NUMA
// node; the deleter drops the registry record and frees the pinning.
// Mirrors common/csrc/mem_alloc.cpp:17-64.
torch::Tensor alloc_numa_pinned_tensor(std::size_t size) {
    TORCH_CHECK(size > 0, "alloc_numa_pinned_tensor: size must be positive");
    ensure_torch_device_ready();
    const int dev = current_hip_device();
    int node = -1;
    int rc = hfk_mm_device_numa_node(dev, &node);
    TORCH_CHECK(rc == 0, "Unable to look up the NUMA node of device ", dev, ": ", hfk_mm_status_string(rc));
    unsigned flags = 0;
    const char* nc = std::getenv("HFK_PINNED_NONCOHERENT");
    if (nc != nullptr && nc[0] == '1') flags |= HFK_MM_ALLOC_NONCOHERENT;
    void* ptr = nullptr;
    rc = hfk_mm_alloc_pinned(size, node, flags, &ptr);
    TORCH_CHECK(rc == 0 && ptr != nullptr, "unable to allocate ", size,
                " bytes of pinned NUMA host memory: ", hfk_mm_status_string(rc));
    auto options = torch::TensorOptions().dtype(torch::kInt8).device(torch::kCPU).pinned_memory(true);
    auto deleter = [](void* p) {
        const int err = hfk_mm_free_pinned(p);
        if (err != 0) {  // never throw from a deleter
            std::fprintf(stderr, "heterofusedkernels.memory: freeing pinned memory failed: %s\n",
                         hfk_mm_status_string(err));
        }
    };
    return torch::from_blob(ptr, {static_cast<int64_t>(size)}, deleter, options);
}

// Registers an existing pinned CPU tensor, returns its device-visible address.
// Mirrors common/csrc/managed_memory/managed_mem.cpp:336-364 (`register_tensor`):
// a tensor that is not on the CPU or not pinned is rejected with the same message.
uintptr_t host_register(torch::Tensor& tensor) {
    if (tensor.device().is_cpu()) ensure_torch_device_ready();
    if (!tensor.device().is_cpu() || !tensor.is_pinned()) {
        TORCH_CHECK(false, "Invalid device. Device must be CPU and tensor must be pinned.");
    }
    void* host = tensor.data_ptr();
    void* dev = nullptr;
    const int rc = hfk_mm_register(host, tensor.nbytes(), &dev);
    TORCH_CHECK(rc == 0 && dev != nullptr, "Failed to register memory: ", hfk_mm_status_string(rc));
    return reinterpret_cast<uintptr_t>(dev);
}

// Mirrors managed_mem.cpp:366-370 (`unregister_tensor`, not bound in the reference).
void host_unregister(torch::Tensor& tensor) { (void)hfk_mm_unregister(tensor.data_ptr()); }

// Mirrors managed_mem.cpp:372-375: 0 for an address that was never registered.
uintptr_t get_device_ptr_py(uintptr_t host_ptr) { return get_device_ptr(host_ptr); }

int device_numa_node(int device) {
    int node = -1;
    const int rc = hfk_mm_device_numa_node(device, &node);
    TORCH_CHECK(rc == 0, "device_numa_node: ", hfk_mm_status_string(rc));
    return node;
}

}  // namespace

PYBIND11_MODULE(memory, m) {
    m.def("alloc_numa_pinned_tensor", &alloc_numa_pinned_tensor);
    m.def("host_register", &host_register);
    m.def("get_device_ptr", &get_device_ptr_py);
    m.def("host_unregister", &host_unregister);
    m.def("device_numa_node", &device_numa_node);
    m.def("record_count", []() { return hfk_mm_record_count(); });
}
