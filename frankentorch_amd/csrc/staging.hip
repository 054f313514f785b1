// Pinned staging rings, copy threads and the upload / compute / download pipeline behind the
// host-slice entry points (see staging.hpp). Host code only: nothing here launches a kernel.

#include "staging.hpp"

#include <algorithm>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

#include "common.hpp"

namespace fth {
namespace {

constexpr int kRing = 4;  // pinned chunks per direction
constexpr int kLag = 2;   // a chunk's output is copied out to the caller this many chunks later

// A few threads that split one large memcpy between them. The copy between a pageable slice and
// a pinned chunk runs at about 10 GB/s on one core, a fifth of the host link.
class CopyPool {
   public:
    explicit CopyPool(int workers) {
        for (int i = 0; i < workers; ++i) {
            std::thread t([this, i] { run(i); });
            t.detach();  // the pool lives until the process ends
            ++workers_;
        }
    }
    void copy(void *dst, const void *src, size_t bytes) {
        if (workers_ == 0 || bytes < ((size_t)256 << 10)) {
            std::memcpy(dst, src, bytes);
            return;
        }
        const int parts = workers_ + 1;
        size_t slice = (bytes + parts - 1) / parts;
        slice = (slice + 4095) & ~(size_t)4095;
        {
            std::lock_guard<std::mutex> lk(mu_);
            dst_ = static_cast<char *>(dst);
            src_ = static_cast<const char *>(src);
            bytes_ = bytes;
            slice_ = slice;
            pending_ = workers_;
            ++gen_;
        }
        work_.notify_all();
        std::memcpy(dst, src, std::min(slice, bytes));  // the caller takes the first slice
        std::unique_lock<std::mutex> lk(mu_);
        done_.wait(lk, [this] { return pending_ == 0; });
    }

   private:
    void run(int idx) {
        uint64_t seen = 0;
        for (;;) {
            std::unique_lock<std::mutex> lk(mu_);
            work_.wait(lk, [&] { return gen_ != seen; });
            seen = gen_;
            const size_t begin = (size_t)(idx + 1) * slice_;
            const size_t end = std::min(begin + slice_, bytes_);
            char *d = dst_;
            const char *s = src_;
            lk.unlock();
            if (begin < end) std::memcpy(d + begin, s + begin, end - begin);
            lk.lock();
            if (--pending_ == 0) done_.notify_one();
        }
    }
    std::mutex mu_;
    std::condition_variable work_, done_;
    uint64_t gen_ = 0;
    int pending_ = 0, workers_ = 0;
    char *dst_ = nullptr;
    const char *src_ = nullptr;
    size_t bytes_ = 0, slice_ = 0;
};

struct Stager {
    std::mutex mu;  // one staged transfer at a time: the rings are shared by every caller
    bool ready = false;
    hipStream_t in_st = nullptr, out_st = nullptr;
    void *pin_in[kRing] = {}, *pin_out[kRing] = {};
    hipEvent_t in_done[kRing] = {}, k_done[kRing] = {}, out_done[kRing] = {};
    hipEvent_t fence = nullptr;
    CopyPool *copier = nullptr;

    int32_t init() {
        if (ready) return FTH_OK;
        FTH_HIP(hipStreamCreate(&in_st));
        FTH_HIP(hipStreamCreate(&out_st));
        for (int i = 0; i < kRing; ++i) {
            FTH_HIP(hipHostMalloc(&pin_in[i], kStageChunk, hipHostMallocDefault));
            FTH_HIP(hipHostMalloc(&pin_out[i], kStageChunk, hipHostMallocDefault));
            FTH_HIP(hipEventCreateWithFlags(&in_done[i], hipEventDisableTiming));
            FTH_HIP(hipEventCreateWithFlags(&k_done[i], hipEventDisableTiming));
            FTH_HIP(hipEventCreateWithFlags(&out_done[i], hipEventDisableTiming));
        }
        FTH_HIP(hipEventCreateWithFlags(&fence, hipEventDisableTiming));
        int workers = 7;
        if (const char *e = std::getenv("FT_HIP_STAGE_THREADS")) workers = std::atoi(e) - 1;  // tuning knob: threads per copy, the caller included
        const int hw = (int)std::thread::hardware_concurrency();
        if (hw > 0 && workers > hw - 1) workers = hw - 1;
        workers = std::max(0, std::min(workers, 31));
        copier = new CopyPool(workers);
        ready = true;
        return FTH_OK;
    }
    // Waits for all three streams; used before an error is returned so that no DMA is left
    // reading or writing a buffer the caller is about to release.
    void drain(hipStream_t compute) {
        (void)hipStreamSynchronize(in_st);
        (void)hipStreamSynchronize(compute);
        (void)hipStreamSynchronize(out_st);
    }
};

Stager &stager() {
    static Stager *s = new Stager();  // never destroyed: HIP may already be torn down at exit
    return *s;
}

// True when [p, p + bytes) is page-locked host memory the DMA engines can address (hipHostMalloc): both ends must be
// page-locked AND belong to one allocation (a slice that starts in one pinned block and ends in another, with pageable
// memory between them, must not be handed to the DMA engine whole).
bool is_pinned(const void *p, size_t bytes) {
    if (bytes == 0) return false;
    hipPointerAttribute_t a;
    if (hipPointerGetAttributes(&a, p) != hipSuccess) {
        (void)hipGetLastError();  // an ordinary pointer is reported as an error by some runtimes
        return false;
    }
    if (a.type != hipMemoryTypeHost) return false;
    hipPointerAttribute_t b;
    const char *last = static_cast<const char *>(p) + bytes - 1;
    if (hipPointerGetAttributes(&b, last) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    if (b.type != hipMemoryTypeHost) return false;
    // Same allocation: ask the runtime for the block that holds the first byte and require the last byte inside it.
    // (Where the runtime cannot answer for host memory the two page-locked ends are all there is to go by.)
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    if (hipMemGetAddressRange(&base, &size, const_cast<void *>(p)) != hipSuccess) {
        (void)hipGetLastError();
        return true;
    }
    return last < static_cast<const char *>(base) + size && static_cast<const char *>(p) >= static_cast<const char *>(base);
}

#define FTH_STAGE(expr)                                      \
    do {                                                     \
        hipError_t _e = (expr);                              \
        if (_e != hipSuccess) {                              \
            sg.drain(compute);                               \
            return fth::hip_fail(_e, #expr);                 \
        }                                                    \
    } while (0)

}  // namespace

int32_t staged_upload(void *dev, const void *host, size_t bytes, hipStream_t compute) {
    if (bytes == 0) return FTH_OK;
    Stager &sg = stager();
    std::lock_guard<std::mutex> lock(sg.mu);
    if (int32_t rc = sg.init()) return rc;
    // `dev` may have been handed out by the pool with its previous user's kernels still queued
    // on the compute stream: the first chunk must not land before they finish.
    FTH_STAGE(hipEventRecord(sg.fence, compute));
    FTH_STAGE(hipStreamWaitEvent(sg.in_st, sg.fence, 0));
    const char *src = static_cast<const char *>(host);
    char *dst = static_cast<char *>(dev);
    if (is_pinned(host, bytes)) {  // the caller's slice is page-locked: one DMA straight out of it
        FTH_STAGE(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, sg.in_st));
        FTH_STAGE(hipEventRecord(sg.in_done[0], sg.in_st));
        FTH_STAGE(hipStreamWaitEvent(compute, sg.in_done[0], 0));
        FTH_STAGE(hipEventSynchronize(sg.in_done[0]));
        return FTH_OK;
    }
    int last = 0;
    size_t off = 0;
    for (int64_t c = 0; off < bytes; ++c) {
        const int slot = (int)(c % kRing);
        const size_t n = std::min(kStageChunk, bytes - off);
        if (c >= kRing) FTH_STAGE(hipEventSynchronize(sg.in_done[slot]));  // the DMA that read this chunk last has finished
        sg.copier->copy(sg.pin_in[slot], src + off, n);
        FTH_STAGE(hipMemcpyAsync(dst + off, sg.pin_in[slot], n, hipMemcpyHostToDevice, sg.in_st));
        FTH_STAGE(hipEventRecord(sg.in_done[slot], sg.in_st));
        last = slot;
        off += n;
    }
    FTH_STAGE(hipStreamWaitEvent(compute, sg.in_done[last], 0));
    // The pinned chunks are reused by the next call: their DMAs must be over before it refills them.
    FTH_STAGE(hipEventSynchronize(sg.in_done[last]));
    return FTH_OK;
}

int32_t staged_download(void *host, const void *dev, size_t bytes, hipStream_t compute) {
    Stager &sg = stager();
    std::lock_guard<std::mutex> lock(sg.mu);
    if (int32_t rc = sg.init()) return rc;
    FTH_STAGE(hipEventRecord(sg.fence, compute));
    FTH_STAGE(hipStreamWaitEvent(sg.out_st, sg.fence, 0));
    const char *src = static_cast<const char *>(dev);
    char *dst = static_cast<char *>(host);
    if (is_pinned(host, bytes)) {
        FTH_STAGE(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, sg.out_st));
        FTH_STAGE(hipStreamSynchronize(sg.out_st));
        return FTH_OK;
    }
    const int64_t chunks = (int64_t)((bytes + kStageChunk - 1) / kStageChunk);
    auto span = [&](int64_t c) { return std::min(kStageChunk, bytes - (size_t)c * kStageChunk); };
    auto collect = [&](int64_t c) -> hipError_t {
        const int slot = (int)(c % kRing);
        hipError_t e = hipEventSynchronize(sg.out_done[slot]);
        if (e == hipSuccess) sg.copier->copy(dst + (size_t)c * kStageChunk, sg.pin_out[slot], span(c));
        return e;
    };
    for (int64_t c = 0; c < chunks; ++c) {
        const int slot = (int)(c % kRing);
        if (c >= kRing) FTH_STAGE(collect(c - kRing));
        FTH_STAGE(hipMemcpyAsync(sg.pin_out[slot], src + (size_t)c * kStageChunk, span(c), hipMemcpyDeviceToHost, sg.out_st));
        FTH_STAGE(hipEventRecord(sg.out_done[slot], sg.out_st));
    }
    for (int64_t c = std::max<int64_t>(0, chunks - kRing); c < chunks; ++c) FTH_STAGE(collect(c));
    if (chunks == 0) FTH_STAGE(hipStreamSynchronize(compute));
    return FTH_OK;
}

bool row_pipeline_applies(const RowOp &op) {
    size_t in_row = 0;
    for (int i = 0; i < op.n_in; ++i) in_row += op.in_row_bytes[i];
    if (op.rows <= 0 || in_row == 0 || op.out_row_bytes == 0) return false;
    if (in_row > kStageChunk || op.out_row_bytes > kStageChunk) return false;
    return (size_t)op.rows * std::max(in_row, op.out_row_bytes) >= kStagedMinBytes;
}

int32_t row_pipeline(const RowOp &op, const std::function<int32_t(int64_t, int64_t)> &launch, hipStream_t compute) {
    Stager &sg = stager();
    std::lock_guard<std::mutex> lock(sg.mu);
    if (int32_t rc = sg.init()) return rc;
    size_t in_row = 0;
    for (int i = 0; i < op.n_in; ++i) in_row += op.in_row_bytes[i];
    const int64_t rows_per_chunk = (int64_t)std::min(kStageChunk / in_row, kStageChunk / op.out_row_bytes);
    if (rows_per_chunk < 1) return fth::set_error(FTH_ERR_KERNEL, "row_pipeline: a row does not fit a staging chunk");
    const int64_t chunks = (op.rows + rows_per_chunk - 1) / rows_per_chunk;
    auto chunk_rows = [&](int64_t c) { return std::min(rows_per_chunk, op.rows - c * rows_per_chunk); };
    FTH_STAGE(hipEventRecord(sg.fence, compute));
    FTH_STAGE(hipStreamWaitEvent(sg.in_st, sg.fence, 0));
    // Operands in page-locked memory are read and written in place by the DMA engines.
    bool in_pinned[2] = {false, false};
    for (int i = 0; i < op.n_in; ++i) in_pinned[i] = is_pinned(op.host_in[i], (size_t)op.rows * op.in_row_bytes[i]);
    const bool out_pinned = is_pinned(op.host_out, (size_t)op.rows * op.out_row_bytes);
    auto collect = [&](int64_t c) -> hipError_t {
        const int slot = (int)(c % kRing);
        hipError_t e = hipEventSynchronize(sg.out_done[slot]);
        if (e == hipSuccess && !out_pinned)
            sg.copier->copy(static_cast<char *>(op.host_out) + (size_t)(c * rows_per_chunk) * op.out_row_bytes, sg.pin_out[slot],
                            (size_t)chunk_rows(c) * op.out_row_bytes);
        return e;
    };
    for (int64_t c = 0; c < chunks; ++c) {
        const int slot = (int)(c % kRing);
        const int64_t row0 = c * rows_per_chunk, nr = chunk_rows(c);
        // upload
        if (c >= kRing) FTH_STAGE(hipEventSynchronize(sg.in_done[slot]));
        size_t sub = 0;
        for (int i = 0; i < op.n_in; ++i) {
            const size_t n = (size_t)nr * op.in_row_bytes[i], at = (size_t)row0 * op.in_row_bytes[i];
            const char *from = static_cast<const char *>(op.host_in[i]) + at;
            if (!in_pinned[i]) {
                char *pin = static_cast<char *>(sg.pin_in[slot]) + sub;
                sg.copier->copy(pin, from, n);
                from = pin;
            }
            FTH_STAGE(hipMemcpyAsync(static_cast<char *>(op.dev_in[i]) + at, from, n, hipMemcpyHostToDevice, sg.in_st));
            sub += (size_t)rows_per_chunk * op.in_row_bytes[i];
        }
        FTH_STAGE(hipEventRecord(sg.in_done[slot], sg.in_st));
        // compute
        FTH_STAGE(hipStreamWaitEvent(compute, sg.in_done[slot], 0));
        if (int32_t rc = launch(row0, nr)) {
            sg.drain(compute);
            return rc;
        }
        FTH_STAGE(hipEventRecord(sg.k_done[slot], compute));
        // download: the pinned output chunk of slot was last filled by chunk c - kRing, which was
        // copied out to the caller kLag chunks after its own turn
        FTH_STAGE(hipStreamWaitEvent(sg.out_st, sg.k_done[slot], 0));
        void *to = out_pinned ? static_cast<void *>(static_cast<char *>(op.host_out) + (size_t)row0 * op.out_row_bytes) : sg.pin_out[slot];
        FTH_STAGE(hipMemcpyAsync(to, static_cast<const char *>(op.dev_out) + (size_t)row0 * op.out_row_bytes,
                                 (size_t)nr * op.out_row_bytes, hipMemcpyDeviceToHost, sg.out_st));
        FTH_STAGE(hipEventRecord(sg.out_done[slot], sg.out_st));
        if (c >= kLag) FTH_STAGE(collect(c - kLag));
    }
    for (int64_t c = std::max<int64_t>(0, chunks - kLag); c < chunks; ++c) FTH_STAGE(collect(c));
    // every upload DMA has been consumed by a kernel that has finished, so the rings are idle
    return FTH_OK;
}

}  // namespace fth
