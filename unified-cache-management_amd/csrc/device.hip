// Transfer device of the store layer: the HIP twin of the reference's CudaDevice
// (ucm/store/device/cuda/cuda_device.cu:107-227) on top of its buffered base
// (ucm/store/device/ibuffered_device.h:32-66, interface ucm/store/device/idevice.h:33-58):
// a pool of equally sized pinned host buffers handed out by index, synchronous and
// stream-ordered copies in both directions, a completion callback, and batched
// copies between arrays of device and host addresses, which are one launch of the
// pointer-array copy kernel (the host buffers are mapped into the device's address
// space, so the kernel reads or writes them directly).
#include <mutex>
#include <new>
#include <utility>
#include <vector>

#include "common.h"

struct ucm_device {
    int device_id = 0;
    size_t buffer_size = 0, buffer_number = 0;
    unsigned char* pool = nullptr;          // buffer_number * buffer_size bytes of pinned host memory
    std::vector<size_t> free_slots;         // indices into the pool that are not handed out
    std::mutex lock;
    hipStream_t stream = nullptr;
    void** ptr_arrays = nullptr;            // device scratch for the two pointer arrays of a batch
    size_t ptr_capacity = 0;                // pointers per array
};

namespace {

struct Closure {
    ucm_device_callback_t cb;
    void* user;
};

void trampoline(hipStream_t, hipError_t status, void* data)
{
    Closure* c = static_cast<Closure*>(data);
    c->cb(status == hipSuccess ? 1 : 0, c->user);
    delete c;
}

// Can a kernel dereference this address?  The device's own pinned pool: yes.  Anything else is asked of the
// runtime: device memory (the answer covers its whole allocation, remembered in `known` so that the many blocks of
// one cache tensor cost one query), pinned or registered host memory and managed memory are mapped into the
// device's address space; pageable host memory is not, and a kernel touching it would fault.
bool kernel_can_touch(const ucm_device* dev, const void* p, size_t count, std::vector<std::pair<uintptr_t, uintptr_t>>& known)
{
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    if (dev && dev->pool) {
        const uintptr_t lo = reinterpret_cast<uintptr_t>(dev->pool), hi = lo + dev->buffer_size * dev->buffer_number;
        if (a >= lo && a + count <= hi) { return true; }
    }
    for (const auto& r : known) {
        if (a >= r.first && a + count <= r.second) { return true; }
    }
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();              // an unknown address is an answer, not a failure of this call
        return false;
    }
    if (attr.type == hipMemoryTypeDevice) {
        hipDeviceptr_t base = nullptr;
        size_t size = 0;
        if (hipMemGetAddressRange(&base, &size, const_cast<void*>(p)) == hipSuccess && size) {
            const uintptr_t lo = reinterpret_cast<uintptr_t>(base);
            known.emplace_back(lo, lo + size);
            return a + count <= lo + size;
        }
        (void)hipGetLastError();
        return true;
    }
    return attr.type == hipMemoryTypeHost || attr.type == hipMemoryTypeManaged;
}

int batch(ucm_device* dev, void* const* dst_host_array, const void* const* src_host_array, size_t number, size_t count,
          const char* what)
{
    UCM_REQUIRE(dev && (number == 0 || (dst_host_array && src_host_array)), "%s: null argument", what);
    if (number == 0 || count == 0) { return UCM_OK; }
    if (int rc = ucm::check_hip(hipSetDevice(dev->device_id), what)) { return rc; }
    bool vector_ok = count % 16 == 0;
    std::vector<std::pair<uintptr_t, uintptr_t>> known;
    for (size_t i = 0; vector_ok && i < number; ++i) {
        UCM_REQUIRE(dst_host_array[i] && src_host_array[i], "%s: null address in entry %zu", what, i);
        vector_ok = ucm::aligned16(dst_host_array[i]) && ucm::aligned16(src_host_array[i]) &&
                    kernel_can_touch(dev, dst_host_array[i], count, known) && kernel_can_touch(dev, src_host_array[i], count, known);
    }
    if (!vector_ok) {
        // sizes or addresses the 16-byte copy kernel cannot take (odd sizes, unaligned addresses, pageable host
        // memory, which no kernel may touch): one runtime copy per pair, same stream, same wait
        for (size_t i = 0; i < number; ++i) {
            if (int rc = ucm::check_hip(hipMemcpyAsync(dst_host_array[i], src_host_array[i], count, hipMemcpyDefault, dev->stream), what)) {
                return rc;
            }
        }
        return ucm::check_hip(hipStreamSynchronize(dev->stream), what);
    }
    std::lock_guard<std::mutex> guard(dev->lock);   // one batch at a time shares the pointer scratch
    if (number > dev->ptr_capacity) {
        if (dev->ptr_arrays) {
            if (int rc = ucm::check_hip(hipStreamSynchronize(dev->stream), what)) { return rc; }
            (void)hipFree(dev->ptr_arrays);
            dev->ptr_arrays = nullptr;
            dev->ptr_capacity = 0;
        }
        size_t cap = 256;
        while (cap < number) { cap *= 2; }
        if (int rc = ucm::check_hip(hipMalloc(reinterpret_cast<void**>(&dev->ptr_arrays), 2 * cap * sizeof(void*)), what)) { return rc; }
        dev->ptr_capacity = cap;
    }
    void** d_dst = dev->ptr_arrays;
    void** d_src = dev->ptr_arrays + dev->ptr_capacity;
    if (int rc = ucm::check_hip(hipMemcpyAsync(d_dst, dst_host_array, number * sizeof(void*), hipMemcpyHostToDevice, dev->stream), what)) { return rc; }
    if (int rc = ucm::check_hip(hipMemcpyAsync(d_src, src_host_array, number * sizeof(void*), hipMemcpyHostToDevice, dev->stream), what)) { return rc; }
    if (int rc = ucm_copy_batch(d_dst, const_cast<const void* const*>(d_src), number, count, reinterpret_cast<ucm_stream_t>(dev->stream))) { return rc; }
    return ucm::check_hip(hipStreamSynchronize(dev->stream), what);
}

}  // namespace

extern "C" int ucm_kernel_can_access(const void* address, size_t count)
{
    if (!address) { return 0; }
    std::vector<std::pair<uintptr_t, uintptr_t>> known;
    return kernel_can_touch(nullptr, address, count, known) ? 1 : 0;
}

extern "C" int ucm_device_create(int device_id, size_t buffer_size, size_t buffer_number, ucm_device_t** out)
{
    UCM_REQUIRE(out != nullptr && device_id >= 0, "ucm_device_create: bad argument");
    *out = nullptr;
    if (int rc = ucm::check_hip(hipSetDevice(device_id), "ucm_device_create (set device)")) { return rc; }
    ucm_device* dev = new (std::nothrow) ucm_device;
    if (!dev) { return ucm::fail(UCM_ENOMEM, "ucm_device_create: out of memory"); }
    dev->device_id = device_id;
    dev->buffer_size = buffer_size;
    dev->buffer_number = buffer_number;
    const size_t total = buffer_size * buffer_number;
    if (total) {
        if (hipHostMalloc(reinterpret_cast<void**>(&dev->pool), total, hipHostMallocDefault) != hipSuccess) {
            delete dev;
            return ucm::fail(UCM_ENOMEM, "ucm_device_create: %zu bytes of pinned host memory refused", total);
        }
        dev->free_slots.reserve(buffer_number);
        for (size_t i = buffer_number; i-- > 0;) { dev->free_slots.push_back(i); }   // slot 0 goes out first
    }
    if (int rc = ucm::check_hip(hipStreamCreate(&dev->stream), "ucm_device_create (stream)")) {   // default priority
        if (dev->pool) { (void)hipHostFree(dev->pool); }
        delete dev;
        return rc;
    }
    *out = dev;
    return UCM_OK;
}

extern "C" void ucm_device_destroy(ucm_device_t* dev)
{
    if (!dev) { return; }
    (void)hipSetDevice(dev->device_id);
    if (dev->stream) {
        (void)hipStreamSynchronize(dev->stream);
        (void)hipStreamDestroy(dev->stream);
    }
    if (dev->ptr_arrays) { (void)hipFree(dev->ptr_arrays); }
    if (dev->pool) { (void)hipHostFree(dev->pool); }
    delete dev;
}

extern "C" void* ucm_device_get_buffer(ucm_device_t* dev, size_t size)
{
    if (!dev || size == 0) { return nullptr; }
    if (dev->pool && size <= dev->buffer_size) {
        std::lock_guard<std::mutex> guard(dev->lock);
        if (!dev->free_slots.empty()) {
            const size_t idx = dev->free_slots.back();
            dev->free_slots.pop_back();
            return dev->pool + idx * dev->buffer_size;
        }
    }
    // pool exhausted or request too large: a buffer of its own, as the reference's MakeBuffer fallback
    void* p = nullptr;
    (void)hipSetDevice(dev->device_id);
    if (hipHostMalloc(&p, size, hipHostMallocDefault) != hipSuccess) { return nullptr; }
    return p;
}

extern "C" void ucm_device_release_buffer(ucm_device_t* dev, void* buffer)
{
    if (!dev || !buffer) { return; }
    unsigned char* p = static_cast<unsigned char*>(buffer);
    if (dev->pool && p >= dev->pool && p < dev->pool + dev->buffer_size * dev->buffer_number) {
        std::lock_guard<std::mutex> guard(dev->lock);
        dev->free_slots.push_back(static_cast<size_t>(p - dev->pool) / dev->buffer_size);
        return;
    }
    (void)hipHostFree(buffer);
}

extern "C" int ucm_device_h2d_sync(ucm_device_t* dev, void* dst, const void* src, size_t count)
{
    UCM_REQUIRE(dev && (count == 0 || (dst && src)), "ucm_device_h2d_sync: null argument");
    return ucm::check_hip(hipMemcpy(dst, src, count, hipMemcpyHostToDevice), "ucm_device_h2d_sync");
}

extern "C" int ucm_device_d2h_sync(ucm_device_t* dev, void* dst, const void* src, size_t count)
{
    UCM_REQUIRE(dev && (count == 0 || (dst && src)), "ucm_device_d2h_sync: null argument");
    return ucm::check_hip(hipMemcpy(dst, src, count, hipMemcpyDeviceToHost), "ucm_device_d2h_sync");
}

extern "C" int ucm_device_h2d_async(ucm_device_t* dev, void* dst, const void* src, size_t count)
{
    UCM_REQUIRE(dev && (count == 0 || (dst && src)), "ucm_device_h2d_async: null argument");
    return ucm::check_hip(hipMemcpyAsync(dst, src, count, hipMemcpyHostToDevice, dev->stream), "ucm_device_h2d_async");
}

extern "C" int ucm_device_d2h_async(ucm_device_t* dev, void* dst, const void* src, size_t count)
{
    UCM_REQUIRE(dev && (count == 0 || (dst && src)), "ucm_device_d2h_async: null argument");
    return ucm::check_hip(hipMemcpyAsync(dst, src, count, hipMemcpyDeviceToHost, dev->stream), "ucm_device_d2h_async");
}

extern "C" int ucm_device_append_callback(ucm_device_t* dev, ucm_device_callback_t cb, void* user)
{
    UCM_REQUIRE(dev && cb, "ucm_device_append_callback: null argument");
    Closure* c = new (std::nothrow) Closure{cb, user};
    if (!c) { return ucm::fail(UCM_ENOMEM, "ucm_device_append_callback: out of memory"); }
    const int rc = ucm::check_hip(hipStreamAddCallback(dev->stream, trampoline, c, 0), "ucm_device_append_callback");
    if (rc != UCM_OK) { delete c; }
    return rc;
}

extern "C" int ucm_device_synchronized(ucm_device_t* dev)
{
    UCM_REQUIRE(dev != nullptr, "ucm_device_synchronized: null device");
    return ucm::check_hip(hipStreamSynchronize(dev->stream), "ucm_device_synchronized");
}

extern "C" ucm_stream_t ucm_device_stream(ucm_device_t* dev) { return dev ? reinterpret_cast<ucm_stream_t>(dev->stream) : nullptr; }

extern "C" int ucm_device_h2d_batch_sync(ucm_device_t* dev, void* const* d_arr, const void* const* h_arr, size_t number,
                                         size_t count)
{
    return batch(dev, d_arr, h_arr, number, count, "ucm_device_h2d_batch_sync");
}

extern "C" int ucm_device_d2h_batch_sync(ucm_device_t* dev, void* const* h_arr, const void* const* d_arr, size_t number,
                                         size_t count)
{
    return batch(dev, h_arr, d_arr, number, count, "ucm_device_d2h_batch_sync");
}
