/*
 * hfk_managed_memory.h - C-ABI of libmanaged_memory.so: the process-wide registry
 * of device-visible host memory and the NUMA-aware pinned allocator.
 *
 * The registry maps a host address range to the address a GPU kernel uses for
 * the same bytes, so an op that receives a pinned CPU tensor can hand the kernel
 * a pointer it may dereference. Interior pointers resolve by range + offset.
 * All functions are thread-safe (readers share, writers exclude).
 *
 * Return convention: 0 = success, negative = hfk_mm_status, positive = hipError_t.
 */
#ifndef HFK_MANAGED_MEMORY_H
#define HFK_MANAGED_MEMORY_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HFK_MM_API __attribute__((visibility("default")))

enum hfk_mm_status {
    HFK_MM_OK = 0,
    HFK_MM_ERR_BAD_ARGUMENT = -1, /* null pointer or zero size                           */
    HFK_MM_ERR_OVERLAP = -2,      /* range overlaps a different existing registration   */
    HFK_MM_ERR_NOT_FOUND = -3,
    HFK_MM_ERR_OS = -4,           /* mmap / sysfs / policy failure, see errno           */
    HFK_MM_ERR_NOT_PINNED = -5    /* the range is pageable memory: this library adopts pinned
                                     memory and allocates its own, it never pins existing memory */
};

/* How a record came to exist; decides what unregistering undoes. */
enum hfk_mm_kind {
    HFK_MM_KIND_ALLOCATED = 0,  /* hfk_mm_alloc_pinned: freed with the allocation        */
    HFK_MM_KIND_REGISTERED = 1, /* unused (kept for numbering): this library pins nothing itself */
    HFK_MM_KIND_ADOPTED = 2     /* already pinned elsewhere / caller-supplied mapping    */
};

/* Flags for hfk_mm_alloc_pinned. */
#define HFK_MM_ALLOC_NONCOHERENT 1u /* coarse-grained (GPU-cacheable) host memory */

/*
 * Record [host_ptr, host_ptr + bytes) and the address kernels use for it.
 * The memory must be pinned already (hipHostMalloc, torch pin_memory, or a
 * hipHostRegister(Mapped) the caller made itself on a platform that allows it); it is
 * adopted via hipHostGetDevicePointer. Pageable memory is refused with
 * HFK_MM_ERR_NOT_PINNED and leaves no record: use hfk_mm_alloc_pinned instead.
 * Registering the same start address again returns the existing record.
 * Replaces common/csrc/managed_memory/managed_mem.cpp:45-66 (`registerHostPtr`)
 * and :305-323 (`register_ptr`).
 */
HFK_MM_API int hfk_mm_register(void* host_ptr, size_t bytes, void** dev_ptr_out);

/*
 * Record a mapping the caller established itself (no HIP call is made).
 * No counterpart in the reference; it is what lets the registry be exercised
 * without a device and lets callers bring their own pinning.
 */
HFK_MM_API int hfk_mm_adopt(void* host_ptr, void* dev_ptr, size_t bytes, int device);

/*
 * Drop the record that starts at host_ptr (the pinning stays with whoever made it).
 * Unknown pointers are not an error.
 * Replaces managed_mem.cpp:105-118 (`aclUnregisterHostPtr`), :325-334 (`unregister_ptr`).
 */
HFK_MM_API int hfk_mm_unregister(void* host_ptr);

/* Drop every record. Replaces managed_mem.cpp:23-37 (`unregisterAll`). */
HFK_MM_API void hfk_mm_unregister_all(void);

/*
 * Device-visible address for any host address inside a recorded range, NULL when
 * unknown. Replaces managed_mem.cpp:139-160 (`getDevicePtr`, a linear scan there;
 * an ordered-map range lookup here).
 */
HFK_MM_API void* hfk_mm_get_device_ptr(const void* host_ptr);

/* Size of the record containing host_ptr, 0 when unknown.
 * Replaces managed_mem.cpp:163-179 (`getRecordSize`). */
HFK_MM_API size_t hfk_mm_record_size(const void* host_ptr);

/* Number of live records. */
HFK_MM_API size_t hfk_mm_record_count(void);

/*
 * NUMA node the given HIP device hangs off (-1 = unknown / single node), read
 * from /sys/bus/pci/devices/<bdf>/numa_node with <bdf> from hipDeviceGetPCIBusId.
 * Replaces common/csrc/mem_alloc.cpp:18-38 and the vendor-library lookup in
 * common/csrc/dcmi_management.cpp:27-39.
 */
HFK_MM_API int hfk_mm_device_numa_node(int device, int* node_out);

/*
 * Allocate `bytes` of zero-filled pinned, device-mapped host memory, bound to
 * `numa_node` when >= 0, and record it. Pinning goes through hipHostMalloc under
 * a temporary MPOL_BIND policy (hipHostMallocNumaUser), not mmap + register. The zero fill is
 * the pages' first touch, which is where pinning spends its time, so ranges of 256 MiB and more
 * are filled by up to 8 threads, each under the same node binding (16 GiB: 1.5 s instead of 6.2 s).
 * Replaces common/csrc/mem_alloc.cpp:79-115 (`alloc_pinned_numa_ptr`).
 */
HFK_MM_API int hfk_mm_alloc_pinned(size_t bytes, int numa_node, unsigned flags, void** host_ptr_out);

/* Free memory from hfk_mm_alloc_pinned and drop its record.
 * Replaces common/csrc/mem_alloc.cpp:66-77 (`free_pinned_numa_ptr`). */
HFK_MM_API int hfk_mm_free_pinned(void* host_ptr);

HFK_MM_API const char* hfk_mm_status_string(int status);

#ifdef __cplusplus
}
#endif
#endif /* HFK_MANAGED_MEMORY_H */
