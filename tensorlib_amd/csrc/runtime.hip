// Runtime half of the C ABI: device selection, stream, memory, copies, error text.
// Counterpart of the allocation / memcpy / error-check plumbing in the reference's
// tensorLib/src/device/cuda/CUDA.cu:16-32,71-81 and tensorLib/include/device/cuda/CUDA.cuh:131-151.
#include <atomic>
#include <cstring>
#include <mutex>

#include "tl_internal.h"

namespace tl {

static thread_local char g_err[512] = {0};

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}
void clear_error() { g_err[0] = 0; }

static std::mutex g_mu;
static DeviceInfo g_info;
static std::atomic<bool> g_ready{false};
static hipStream_t g_stream = nullptr;

hipStream_t stream() { return g_stream; }
const DeviceInfo& device_info() { return g_info; }

static int init_locked(int ordinal) {
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0)
        return set_error(TL_EHIP, "no HIP device available (%s)", hipGetErrorString(e));
    if (ordinal < 0 || ordinal >= count)
        return set_error(TL_EINVAL, "device ordinal %d out of range [0,%d)", ordinal, count);
    TL_HIP_TRY(hipSetDevice(ordinal));
    hipDeviceProp_t p;
    TL_HIP_TRY(hipGetDeviceProperties(&p, ordinal));
    g_info.ordinal = ordinal;
    g_info.cu_count = p.multiProcessorCount;
    g_info.wave_size = p.warpSize;
    g_info.lds_per_block = p.sharedMemPerBlock;
    strncpy(g_info.arch, p.gcnArchName, sizeof(g_info.arch) - 1);
    if (strncmp(g_info.arch, "gfx950", 6) != 0)
        return set_error(TL_EHIP, "this library is built for gfx950 only, device %d is %s", ordinal,
                         g_info.arch);
    // resolve the static scratch of the entry point that allocates nothing now, with this device current,
    // so that entry point itself only reads a table
    int rc = attention_static_scratch(nullptr);
    if (rc != TL_OK) return rc;
    g_ready.store(true, std::memory_order_release);
    return TL_OK;
}

int ensure_init() {
    if (g_ready.load(std::memory_order_acquire)) return TL_OK;
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_ready.load(std::memory_order_relaxed)) return TL_OK;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    return init_locked(dev);
}

static std::atomic<bool> g_ws_in_use{false};
bool workspaces_in_use() { return g_ws_in_use.load(std::memory_order_acquire); }

int Workspace::acquire(size_t floats, size_t min_floats, const char* what, Lease* lease) {
    lease->lock = std::unique_lock<std::mutex>(mu_);
    hipStream_t st = stream();
    if (floats > floats_) {
        if (ptr_) {
            TL_HIP_TRY(hipStreamSynchronize(st));
            TL_HIP_TRY(hipFree(ptr_));
            ptr_ = nullptr;
            floats_ = 0;
        }
        const size_t want = floats < min_floats ? min_floats : floats;
        hipError_t e = hipMalloc((void**)&ptr_, want * sizeof(float));
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return set_error(TL_ENOMEM, "%s: hipMalloc(%zu bytes) failed: %s", what, want * sizeof(float),
                             hipGetErrorString(e));
        }
        floats_ = want;
        // users keep counters in the buffer that are zero between calls (tickets): start from zeros
        int rc = launch_fill_f16(ptr_, 0, want * 2);
        if (rc != TL_OK) return rc;
    }
    g_ws_in_use.store(true, std::memory_order_release);
    lease->ptr = ptr_;
    return TL_OK;
}

int Workspace::zero_head(size_t floats) {
    std::lock_guard<std::mutex> lk(mu_);
    if (!ptr_) return TL_OK;
    return launch_fill_f16(ptr_, 0, (floats < floats_ ? floats : floats_) * 2);
}

}  // namespace tl

extern "C" {

int tl_init(int device_ordinal) {
    std::lock_guard<std::mutex> lk(tl::g_mu);
    if (tl::g_ready.load(std::memory_order_acquire) && tl::g_info.ordinal == device_ordinal) return TL_OK;
    return tl::init_locked(device_ordinal);
}

const char* tl_last_error(void) { return tl::g_err; }

const char* tl_version(void) { return "tensorlib_amd 0.1 gfx950"; }

int tl_device_cu_count(void) { return tl::g_ready.load(std::memory_order_acquire) ? tl::g_info.cu_count : 0; }

int tl_set_stream(void* hip_stream) {
    hipStream_t next = static_cast<hipStream_t>(hip_stream);
    // Work queued on the stream being replaced may still use the library's scratch buffers, which the next call on
    // the new stream reuses: drain it here, while the caller's handle is certainly still valid.
    if (next != tl::g_stream && tl::g_ws_in_use.exchange(false)) TL_HIP_TRY(hipStreamSynchronize(tl::g_stream));
    tl::g_stream = next;
    return TL_OK;
}
void* tl_get_stream(void) { return tl::g_stream; }

int tl_malloc(void** dev_ptr, size_t bytes) {
    TL_ENSURE_INIT();
    TL_REQUIRE(dev_ptr != nullptr, "tl_malloc: dev_ptr is null");
    *dev_ptr = nullptr;
    if (bytes == 0) return TL_OK;
    hipError_t e = hipMalloc(dev_ptr, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return tl::set_error(TL_ENOMEM, "hipMalloc(%zu bytes) failed: %s", bytes, hipGetErrorString(e));
    }
    return TL_OK;
}

int tl_free(void* dev_ptr) {
    if (dev_ptr == nullptr) return TL_OK;
    TL_HIP_TRY(hipFree(dev_ptr));
    return TL_OK;
}

int tl_memcpy_h2d(void* dst, const void* host_src, size_t bytes) {
    TL_ENSURE_INIT();
    if (bytes == 0) return TL_OK;
    TL_REQUIRE(dst && host_src, "tl_memcpy_h2d: null pointer");
    TL_HIP_TRY(hipMemcpyAsync(dst, host_src, bytes, hipMemcpyHostToDevice, tl::stream()));
    TL_HIP_TRY(hipStreamSynchronize(tl::stream()));
    return TL_OK;
}

int tl_memcpy_d2h(void* host_dst, const void* src, size_t bytes) {
    TL_ENSURE_INIT();
    if (bytes == 0) return TL_OK;
    TL_REQUIRE(host_dst && src, "tl_memcpy_d2h: null pointer");
    TL_HIP_TRY(hipMemcpyAsync(host_dst, src, bytes, hipMemcpyDeviceToHost, tl::stream()));
    TL_HIP_TRY(hipStreamSynchronize(tl::stream()));
    return TL_OK;
}

int tl_memcpy_d2d(void* dst, const void* src, size_t bytes) {
    TL_ENSURE_INIT();
    if (bytes == 0) return TL_OK;
    TL_REQUIRE(dst && src, "tl_memcpy_d2d: null pointer");
    TL_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, tl::stream()));
    return TL_OK;
}

int tl_synchronize(void) {
    TL_ENSURE_INIT();
    TL_HIP_TRY(hipStreamSynchronize(tl::stream()));
    return TL_OK;
}

int tl_reset_scratch(void) {
    TL_ENSURE_INIT();
    int rc = tl::attention_reset_tickets();
    if (rc != TL_OK) return rc;
    return tl::splitk_reset_tickets();
}

}  // extern "C"
