// Host <-> device transfers for the host-slice entry points: pinned staging rings, a small pool of
// copy threads, and a three-stream pipeline (upload, compute, download) for ops whose rows are
// independent. The caller's slices are ordinary pageable memory (a Rust `&[f32]` / `Vec<f32>`,
// crates/ft-dispatch/src/lib.rs:5110-5231), which the DMA engines cannot read at link speed, so
// every byte goes through a pinned chunk; the copy threads keep that host-side copy from being
// the bottleneck and the rings keep it overlapped with the DMA.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <functional>

namespace fth {

// Transfers below this size use one plain asynchronous copy on the compute stream.
constexpr size_t kStagedMinBytes = (size_t)1 << 20;
// Size of one pinned chunk; the rings hold four chunks per direction.
constexpr size_t kStageChunk = (size_t)8 << 20;

// host -> dev. On return every chunk has been enqueued and `compute` waits for the last one.
// Work already queued on `compute` is ordered before the first chunk lands in `dev`.
int32_t staged_upload(void *dev, const void *host, size_t bytes, hipStream_t compute);

// dev -> host after everything queued on `compute`. Returns when `host` holds the data.
int32_t staged_download(void *host, const void *dev, size_t bytes, hipStream_t compute);

// An op over `rows` independent rows: up to two row-aligned inputs, one row-aligned output.
struct RowOp {
    int n_in = 0;
    const void *host_in[2] = {nullptr, nullptr};
    void *dev_in[2] = {nullptr, nullptr};
    size_t in_row_bytes[2] = {0, 0};
    void *host_out = nullptr;
    void *dev_out = nullptr;
    size_t out_row_bytes = 0;
    int64_t rows = 0;
};

// True when a row of every operand fits a pinned chunk and the op is large enough to pipeline.
bool row_pipeline_applies(const RowOp &op);

// Runs the op in chunks of rows: upload of chunk i, `launch(row0, nrows)` of chunk i - 1 (on
// `compute`) and download of chunk i - 2 proceed together. `launch` reads dev_in + row0 * row
// bytes and writes dev_out + row0 * row bytes. Returns when `host_out` holds every row.
int32_t row_pipeline(const RowOp &op, const std::function<int32_t(int64_t row0, int64_t nrows)> &launch, hipStream_t compute);

}  // namespace fth
