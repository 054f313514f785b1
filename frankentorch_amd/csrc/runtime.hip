// Runtime half of the C ABI: availability probe, error slots, hipMalloc-backed buffers with
// explicit copies, streams and events. Nothing here computes.

#include <mutex>
#include <string>

#include "common.hpp"

namespace fth {

fth_error_info &last_error() {
    static thread_local fth_error_info info = {};
    return info;
}

int32_t set_error(int32_t code, const char *fmt, ...) {
    fth_error_info &e = last_error();
    std::memset(&e, 0, sizeof(e));
    e.code = code;
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(e.message, sizeof(e.message), fmt, ap);
    va_end(ap);
    return code;
}

int32_t hip_fail(hipError_t err, const char *what) {
    int32_t code = (err == hipErrorOutOfMemory) ? FTH_ERR_BUFFER_TOO_LARGE : FTH_ERR_KERNEL;
    return set_error(code, "%s: %s", what, hipGetErrorString(err));
}

namespace {
struct DeviceState {
    bool ok = false;
    int cus = 0;
    std::string arch;
    hipDeviceProp_t prop;
    hipStream_t stream = nullptr;
};
DeviceState &state() {
    static DeviceState st;
    static std::once_flag once;
    std::call_once(once, [] {
        int n = 0;
        if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            return;
        }
        if (hipGetDeviceProperties(&st.prop, 0) != hipSuccess) {
            (void)hipGetLastError();
            return;
        }
        st.arch = st.prop.gcnArchName;
        st.cus = st.prop.multiProcessorCount;
        // The code objects in this library are built for gfx950 only.
        if (st.arch.rfind("gfx950", 0) != 0) return;
        if (hipSetDevice(0) != hipSuccess) return;
        if (hipStreamCreate(&st.stream) != hipSuccess) return;
        st.ok = true;
    });
    return st;
}
}  // namespace

bool available() { return state().ok; }
int compute_units() { return state().cus; }
hipStream_t resolve_stream(fth_stream s) { return s ? static_cast<hipStream_t>(s) : state().stream; }

}  // namespace fth

extern "C" {

int32_t fth_last_error(fth_error_info *out) {
    if (out) *out = fth::last_error();
    return fth::last_error().code;
}

const char *fth_status_name(int32_t code) {
    switch (code) {
        case FTH_OK: return "Ok";
        case FTH_ERR_DTYPE_MISMATCH: return "Incompatible(DTypeMismatch)";
        case FTH_ERR_DEVICE_MISMATCH: return "Incompatible(DeviceMismatch)";
        case FTH_ERR_SHAPE_MISMATCH: return "ShapeMismatch";
        case FTH_ERR_UNSUPPORTED_LAYOUT: return "UnsupportedLayout";
        case FTH_ERR_STORAGE_SPAN_OVERFLOW: return "StorageSpanOverflow";
        case FTH_ERR_INSUFFICIENT_STORAGE: return "InsufficientStorage";
        case FTH_ERR_INVALID_DIMENSION: return "InvalidDimension";
        case FTH_ERR_SHAPE_OVERFLOW: return "ShapeOverflow";
        case FTH_ERR_EMPTY_REDUCTION_DIM: return "EmptyReductionDim";
        case FTH_ERR_UNAVAILABLE: return "Unavailable";
        case FTH_ERR_KERNEL: return "Kernel";
        case FTH_ERR_SIZE_OVERFLOW: return "SizeOverflow";
        case FTH_ERR_BUFFER_TOO_LARGE: return "BufferTooLarge";
        case FTH_ERR_STREAM: return "CommandBuffer";
        case FTH_ERR_INVALID_ARGUMENT: return "InvalidArgument";
        case FTH_ERR_OUTPUT_TOO_SMALL: return "OutputTooSmall";
        case FTH_ERR_CORRUPT: return "Corrupt";
        case FTH_ERR_IO: return "Io";
        case FTH_ERR_INVALID_MAGIC: return "InvalidMagic";
        case FTH_ERR_UNSUPPORTED_VERSION: return "UnsupportedVersion";
        default: return "Unknown";
    }
}

int32_t fth_is_available(void) { return fth::available() ? 1 : 0; }

int32_t fth_device_info(char *arch, size_t arch_cap, int32_t *compute_units, uint64_t *hbm_bytes,
                        int32_t *engine_clock_khz, int32_t *memory_clock_khz) {
    FTH_REQUIRE_DEVICE();
    hipDeviceProp_t prop;
    FTH_HIP(hipGetDeviceProperties(&prop, 0));
    if (arch && arch_cap) {
        std::snprintf(arch, arch_cap, "%s", prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (hbm_bytes) *hbm_bytes = prop.totalGlobalMem;
    if (engine_clock_khz) *engine_clock_khz = prop.clockRate;
    if (memory_clock_khz) *memory_clock_khz = prop.memoryClockRate;
    return FTH_OK;
}

int32_t fth_malloc(void **dptr, size_t bytes) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(dptr != nullptr, "fth_malloc: dptr is NULL");
    *dptr = nullptr;
    if (bytes == 0) return FTH_OK;
    FTH_HIP(hipMalloc(dptr, bytes));
    return FTH_OK;
}

int32_t fth_free(void *dptr) {
    if (!dptr) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    FTH_HIP(hipFree(dptr));
    return FTH_OK;
}

int32_t fth_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    FTH_REQUIRE_DEVICE();
    if (bytes == 0) return FTH_OK;
    FTH_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return FTH_OK;
}

int32_t fth_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    FTH_REQUIRE_DEVICE();
    if (bytes == 0) return FTH_OK;
    FTH_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return FTH_OK;
}

int32_t fth_memcpy_d2d(void *dst, const void *src, size_t bytes) {
    FTH_REQUIRE_DEVICE();
    if (bytes == 0) return FTH_OK;
    FTH_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice));
    return FTH_OK;
}

int32_t fth_memset_zero(void *dst, size_t bytes) {
    FTH_REQUIRE_DEVICE();
    if (bytes == 0) return FTH_OK;
    FTH_HIP(hipMemset(dst, 0, bytes));
    return FTH_OK;
}

int32_t fth_device_memory_info(uint64_t *free_bytes, uint64_t *total_bytes) {
    FTH_REQUIRE_DEVICE();
    size_t f = 0, tot = 0;
    FTH_HIP(hipMemGetInfo(&f, &tot));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = tot;
    return FTH_OK;
}

int32_t fth_host_malloc(void **hptr, size_t bytes) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(hptr != nullptr, "fth_host_malloc: hptr is NULL");
    *hptr = nullptr;
    if (bytes == 0) return FTH_OK;
    FTH_HIP(hipHostMalloc(hptr, bytes, hipHostMallocDefault));
    return FTH_OK;
}

int32_t fth_host_free(void *hptr) {
    if (!hptr) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    FTH_HIP(hipHostFree(hptr));
    return FTH_OK;
}

int32_t fth_memcpy_async(void *dst, const void *src, size_t bytes, int32_t kind, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(kind >= 1 && kind <= 3, "fth_memcpy_async: kind %d is not 1 (H2D), 2 (D2H) or 3 (D2D)", kind);
    if (bytes == 0) return FTH_OK;
    const hipMemcpyKind k = kind == 1 ? hipMemcpyHostToDevice : kind == 2 ? hipMemcpyDeviceToHost : hipMemcpyDeviceToDevice;
    FTH_HIP(hipMemcpyAsync(dst, src, bytes, k, fth::resolve_stream(s)));
    return FTH_OK;
}

int32_t fth_stream_create(fth_stream *s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(s != nullptr, "fth_stream_create: s is NULL");
    hipStream_t st;
    FTH_HIP(hipStreamCreate(&st));
    *s = st;
    return FTH_OK;
}

int32_t fth_stream_destroy(fth_stream s) {
    FTH_REQUIRE_DEVICE();
    if (!s) return FTH_OK;
    FTH_HIP(hipStreamDestroy(static_cast<hipStream_t>(s)));
    return FTH_OK;
}

int32_t fth_stream_synchronize(fth_stream s) {
    FTH_REQUIRE_DEVICE();
    hipError_t e = hipStreamSynchronize(fth::resolve_stream(s));
    if (e != hipSuccess) {
        fth::hip_fail(e, "hipStreamSynchronize");
        fth::last_error().code = FTH_ERR_STREAM;
        return FTH_ERR_STREAM;
    }
    return FTH_OK;
}

int32_t fth_device_synchronize(void) {
    FTH_REQUIRE_DEVICE();
    FTH_HIP(hipDeviceSynchronize());
    return FTH_OK;
}

int32_t fth_event_create(fth_event *e) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(e != nullptr, "fth_event_create: e is NULL");
    hipEvent_t ev;
    FTH_HIP(hipEventCreate(&ev));
    *e = ev;
    return FTH_OK;
}

int32_t fth_event_destroy(fth_event e) {
    FTH_REQUIRE_DEVICE();
    if (!e) return FTH_OK;
    FTH_HIP(hipEventDestroy(static_cast<hipEvent_t>(e)));
    return FTH_OK;
}

int32_t fth_event_record(fth_event e, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_HIP(hipEventRecord(static_cast<hipEvent_t>(e), fth::resolve_stream(s)));
    return FTH_OK;
}

int32_t fth_event_synchronize(fth_event e) {
    FTH_REQUIRE_DEVICE();
    FTH_HIP(hipEventSynchronize(static_cast<hipEvent_t>(e)));
    return FTH_OK;
}

int32_t fth_event_elapsed_ms(fth_event start, fth_event stop, float *ms) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(ms != nullptr, "fth_event_elapsed_ms: ms is NULL");
    FTH_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return FTH_OK;
}

}  // extern "C"
