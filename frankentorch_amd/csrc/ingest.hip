// Weight ingestion: a safetensors reader whose tensors go straight into resident device buffers.
//
// replaces load_safetensors / load_safetensors_from_bytes / load_safetensors_metadata
// (crates/ft-serialize/src/lib.rs:2170-2241, 2274-2286) for the loading direction. The reference
// parses the container with the `safetensors` crate (0.8.0, Cargo.lock:2081-2084), which is not in
// the checkout; the container rules restated here are that crate's published ones:
//
//   bytes 0..8   N, little-endian u64, at most 100 000 000
//   bytes 8..8+N a UTF-8 JSON object that starts with '{':  name -> {"dtype", "shape", "data_offsets": [begin, end]},
//                plus an optional "__metadata__" object of string -> string
//   the rest     the data buffer; the tensors, ordered by offset, tile it with no hole and no overlap
//                starting at 0, each of exactly numel * width bytes, and the last one ends the file.
//
// Any violation is FTH_ERR_CORRUPT (TensorIOError::Corrupt); a file that cannot be read is
// FTH_ERR_IO. Like the reference's loader, only F64 / F32 / F16 / BF16 tensors can be read; a file
// holding any other dtype is refused at open, as load_safetensors_from_bytes refuses it as a whole.
//
// The file is memory-mapped. A device read moves the tensor's bytes through two pinned 16 MiB
// staging buffers with asynchronous copies (the CPU fills one while the DMA engine drains the
// other) and, when the stored type or layout differs from the one asked for, converts
// (F16 / BF16 / F64 <-> F32 / F64) and transposes on the GPU, so no converted host copy is made.

//
// The same handle also reads the reference's NATIVE state-dict format (fth_statedict_*), the loading direction of
// load_state_dict / load_state_dict_from_bytes (crates/ft-serialize/src/lib.rs:996-1160; layout written by
// write_state_dict_to_writer :786-860), all integers little-endian:
//
//   "FTSV" | version u32 (<= 1) | tensor count u64 | per tensor: key length u64, key (UTF-8), ndim u64, ndim x u64 dims,
//   dtype tag u8 (0 F64, 1 F32, 2 F16, 3 BF16), numel x width payload bytes | end of file.
//
// Its failures keep the reference's variants and reason strings: InvalidMagic, UnsupportedVersion{found, max},
// Corrupt{reason}.

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <map>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "common.hpp"
#include "pool.hpp"

namespace {

constexpr uint64_t kMaxHeader = 100000000ull;  // the crate's MAX_HEADER_SIZE
constexpr int kMaxDepth = 128;                  // serde_json's recursion limit

struct Entry {
    std::string name;
    int32_t dtype = -1;  // FTH_DTYPE_* for the four readable types, -1 for the rest
    std::string dtype_name;
    int bits = 0;
    std::vector<uint64_t> shape;
    uint64_t begin = 0, end = 0, numel = 0;
};

// ---- a JSON reader for the header grammar ------------------------------------------------------
struct Json {
    const uint8_t *p, *e;
    std::string err;
    int depth = 0;

    bool fail(const char *what) {
        if (err.empty()) err = what;
        return false;
    }
    void ws() {
        while (p < e && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) ++p;
    }
    bool lit(char c) {
        ws();
        if (p < e && *p == (uint8_t)c) {
            ++p;
            return true;
        }
        return false;
    }
    static void put_utf8(std::string &s, uint32_t c) {
        if (c < 0x80) s.push_back((char)c);
        else if (c < 0x800) {
            s.push_back((char)(0xC0 | (c >> 6)));
            s.push_back((char)(0x80 | (c & 0x3F)));
        } else if (c < 0x10000) {
            s.push_back((char)(0xE0 | (c >> 12)));
            s.push_back((char)(0x80 | ((c >> 6) & 0x3F)));
            s.push_back((char)(0x80 | (c & 0x3F)));
        } else {
            s.push_back((char)(0xF0 | (c >> 18)));
            s.push_back((char)(0x80 | ((c >> 12) & 0x3F)));
            s.push_back((char)(0x80 | ((c >> 6) & 0x3F)));
            s.push_back((char)(0x80 | (c & 0x3F)));
        }
    }
    bool hex4(uint32_t &v) {
        if (e - p < 4) return fail("truncated \\u escape");
        v = 0;
        for (int i = 0; i < 4; ++i) {
            const uint8_t c = *p++;
            v <<= 4;
            if (c >= '0' && c <= '9') v |= c - '0';
            else if (c >= 'a' && c <= 'f') v |= c - 'a' + 10;
            else if (c >= 'A' && c <= 'F') v |= c - 'A' + 10;
            else return fail("bad \\u escape");
        }
        return true;
    }
    bool string(std::string &out) {
        ws();
        if (p >= e || *p != '"') return fail("expected a string");
        ++p;
        out.clear();
        while (p < e) {
            const uint8_t c = *p++;
            if (c == '"') return true;
            if (c < 0x20) return fail("control character in a string");
            if (c != '\\') {
                out.push_back((char)c);
                continue;
            }
            if (p >= e) break;
            const uint8_t esc = *p++;
            switch (esc) {
                case '"': out.push_back('"'); break;
                case '\\': out.push_back('\\'); break;
                case '/': out.push_back('/'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'n': out.push_back('\n'); break;
                case 'r': out.push_back('\r'); break;
                case 't': out.push_back('\t'); break;
                case 'u': {
                    uint32_t c1;
                    if (!hex4(c1)) return false;
                    if (c1 >= 0xD800 && c1 <= 0xDBFF) {
                        uint32_t c2;
                        if (e - p < 2 || p[0] != '\\' || p[1] != 'u') return fail("lone surrogate");
                        p += 2;
                        if (!hex4(c2)) return false;
                        if (c2 < 0xDC00 || c2 > 0xDFFF) return fail("lone surrogate");
                        c1 = 0x10000 + ((c1 - 0xD800) << 10) + (c2 - 0xDC00);
                    } else if (c1 >= 0xDC00 && c1 <= 0xDFFF) {
                        return fail("lone surrogate");
                    }
                    put_utf8(out, c1);
                    break;
                }
                default: return fail("bad escape");
            }
        }
        return fail("unterminated string");
    }
    // A JSON number that is a non-negative integer below 2^64 with no fraction or exponent (what
    // serde accepts for u64 / usize).
    bool u64(uint64_t &v) {
        ws();
        if (p >= e || *p < '0' || *p > '9') return fail("expected a non-negative integer");
        if (*p == '0' && p + 1 < e && p[1] >= '0' && p[1] <= '9') return fail("leading zero");
        v = 0;
        while (p < e && *p >= '0' && *p <= '9') {
            const uint64_t d = *p++ - '0';
            if (v > (UINT64_MAX - d) / 10) return fail("integer out of range");
            v = v * 10 + d;
        }
        if (p < e && (*p == '.' || *p == 'e' || *p == 'E')) return fail("expected an integer");
        return true;
    }
    bool skip_number() {
        if (p < e && *p == '-') ++p;
        if (p >= e || *p < '0' || *p > '9') return fail("bad number");
        if (*p == '0') ++p;
        else
            while (p < e && *p >= '0' && *p <= '9') ++p;
        if (p < e && *p == '.') {
            ++p;
            if (p >= e || *p < '0' || *p > '9') return fail("bad number");
            while (p < e && *p >= '0' && *p <= '9') ++p;
        }
        if (p < e && (*p == 'e' || *p == 'E')) {
            ++p;
            if (p < e && (*p == '+' || *p == '-')) ++p;
            if (p >= e || *p < '0' || *p > '9') return fail("bad number");
            while (p < e && *p >= '0' && *p <= '9') ++p;
        }
        return true;
    }
    bool word(const char *w) {
        const size_t n = std::strlen(w);
        if ((size_t)(e - p) < n || std::memcmp(p, w, n) != 0) return fail("bad literal");
        p += n;
        return true;
    }
    // Any JSON value, discarded (fields the tensor record does not name).
    bool skip() {
        ws();
        if (p >= e) return fail("unexpected end");
        if (++depth > kMaxDepth) return fail("nesting too deep");
        bool ok = true;
        const uint8_t c = *p;
        if (c == '"') {
            std::string s;
            ok = string(s);
        } else if (c == '{') {
            ++p;
            if (!lit('}')) {
                do {
                    std::string k;
                    ok = string(k) && (lit(':') || fail("expected ':'")) && skip();
                } while (ok && lit(','));
                ok = ok && (lit('}') || fail("expected '}'"));
            }
        } else if (c == '[') {
            ++p;
            if (!lit(']')) {
                do ok = skip();
                while (ok && lit(','));
                ok = ok && (lit(']') || fail("expected ']'"));
            }
        } else if (c == 't') ok = word("true");
        else if (c == 'f') ok = word("false");
        else if (c == 'n') ok = word("null");
        else ok = skip_number();
        --depth;
        return ok;
    }
    bool u64_list(std::vector<uint64_t> &out) {
        out.clear();
        if (!lit('[')) return fail("expected '['");
        if (lit(']')) return true;
        do {
            uint64_t v;
            if (!u64(v)) return false;
            out.push_back(v);
        } while (lit(','));
        return lit(']') || fail("expected ']'");
    }
};

bool valid_utf8(const uint8_t *p, size_t n) {
    size_t i = 0;
    while (i < n) {
        const uint8_t c = p[i];
        if (c < 0x80) {
            ++i;
            continue;
        }
        int len;
        uint32_t cp;
        if ((c & 0xE0) == 0xC0) len = 2, cp = c & 0x1F;
        else if ((c & 0xF0) == 0xE0) len = 3, cp = c & 0x0F;
        else if ((c & 0xF8) == 0xF0) len = 4, cp = c & 0x07;
        else return false;
        if (i + len > n) return false;
        for (int k = 1; k < len; ++k) {
            if ((p[i + k] & 0xC0) != 0x80) return false;
            cp = (cp << 6) | (p[i + k] & 0x3F);
        }
        if ((len == 2 && cp < 0x80) || (len == 3 && cp < 0x800) || (len == 4 && (cp < 0x10000 || cp > 0x10FFFF))) return false;
        if (cp >= 0xD800 && cp <= 0xDFFF) return false;
        i += len;
    }
    return true;
}

// The crate's Dtype names and widths in bits.
int dtype_bits(const std::string &s) {
    static const std::pair<const char *, int> table[] = {
        {"BOOL", 8}, {"F4", 4},   {"F6_E2M3", 6}, {"F6_E3M2", 6}, {"U8", 8},   {"I8", 8},   {"F8_E5M2", 8}, {"F8_E4M3", 8},
        {"F8_E8M0", 8}, {"I16", 16}, {"U16", 16},   {"F16", 16},    {"BF16", 16}, {"I32", 32}, {"U32", 32},    {"F32", 32},
        {"C64", 64}, {"F64", 64}, {"I64", 64},    {"U64", 64}};
    for (const auto &t : table)
        if (s == t.first) return t.second;
    return 0;
}

int32_t corrupt(const char *fmt, const std::string &a = std::string(), const std::string &b = std::string()) {
    return fth::set_error(FTH_ERR_CORRUPT, fmt, a.c_str(), b.c_str());
}

}  // namespace

struct fth_safetensors {
    const uint8_t *base = nullptr;
    size_t len = 0;
    bool mapped = false;
    const uint8_t *data = nullptr;  // start of the data buffer
    std::vector<Entry> tensors;     // sorted by name (the order of the reference's BTreeMap)
    bool has_metadata = false;
    std::map<std::string, std::string> metadata;

    ~fth_safetensors() {
        if (mapped && base) munmap(const_cast<uint8_t *>(base), len);
    }
    const Entry *find(const char *name) const {
        if (!name) return nullptr;
        auto it = std::lower_bound(tensors.begin(), tensors.end(), name, [](const Entry &t, const char *n) { return t.name < n; });
        return (it != tensors.end() && it->name == name) ? &*it : nullptr;
    }
};

namespace {

// SafeTensors::read_metadata + Metadata::validate of the crate, then the reference's own dtype and
// payload-width checks (crates/ft-serialize/src/lib.rs:1964-1978, 2243-2271).
int32_t parse(fth_safetensors *f) {
    if (f->len < 8) return corrupt("safetensors deserialization failed: HeaderTooSmall");
    uint64_t n = 0;
    for (int i = 7; i >= 0; --i) n = (n << 8) | f->base[i];
    if (n > kMaxHeader) return corrupt("safetensors deserialization failed: HeaderTooLarge");
    if (n + 8 > f->len) return corrupt("safetensors deserialization failed: InvalidHeaderLength");
    const uint8_t *h = f->base + 8;
    if (!valid_utf8(h, (size_t)n)) return corrupt("safetensors deserialization failed: InvalidHeader");
    if (n == 0 || h[0] != '{') return corrupt("safetensors deserialization failed: InvalidHeaderStart");
    Json js{h, h + n};
    std::map<std::string, Entry> by_name;
    bool ok = js.lit('{');
    if (ok && !js.lit('}')) {
        do {
            std::string key;
            ok = js.string(key) && (js.lit(':') || js.fail("expected ':'"));
            if (!ok) break;
            if (key == "__metadata__") {
                // Option<HashMap<String, String>>: null or an object of strings
                js.ws();
                if (js.p < js.e && *js.p == 'n') {
                    ok = js.word("null");
                    f->has_metadata = false;
                    f->metadata.clear();
                    continue;
                }
                ok = js.lit('{') || js.fail("__metadata__ is not an object");
                f->has_metadata = true;
                f->metadata.clear();
                if (ok && !js.lit('}')) {
                    do {
                        std::string k, v;
                        ok = js.string(k) && (js.lit(':') || js.fail("expected ':'")) && js.string(v);
                        if (ok) f->metadata[k] = v;
                    } while (ok && js.lit(','));
                    ok = ok && (js.lit('}') || js.fail("expected '}'"));
                }
                continue;
            }
            Entry t;
            t.name = key;
            bool has_dtype = false, has_shape = false, has_off = false;
            ok = js.lit('{') || js.fail("tensor record is not an object");
            if (ok && !js.lit('}')) {
                do {
                    std::string field;
                    ok = js.string(field) && (js.lit(':') || js.fail("expected ':'"));
                    if (!ok) break;
                    // a derived serde struct refuses a field given twice
                    if ((field == "dtype" && has_dtype) || (field == "shape" && has_shape) || (field == "data_offsets" && has_off)) {
                        ok = js.fail("duplicate field");
                        break;
                    }
                    if (field == "dtype") {
                        ok = js.string(t.dtype_name);
                        if (ok) {
                            t.bits = dtype_bits(t.dtype_name);
                            if (t.bits == 0) ok = js.fail("unknown dtype");
                        }
                        has_dtype = true;
                    } else if (field == "shape") {
                        ok = js.u64_list(t.shape);
                        has_shape = true;
                    } else if (field == "data_offsets") {
                        std::vector<uint64_t> o;
                        ok = js.u64_list(o) && (o.size() == 2 || js.fail("data_offsets is not a pair"));
                        if (ok) t.begin = o[0], t.end = o[1];
                        has_off = true;
                    } else {
                        ok = js.skip();
                    }
                } while (ok && js.lit(','));
                ok = ok && (js.lit('}') || js.fail("expected '}'"));
            }
            ok = ok && ((has_dtype && has_shape && has_off) || js.fail("tensor record misses a field"));
            if (ok) by_name[key] = std::move(t);  // a repeated key keeps the last record, as a serde map does
        } while (ok && js.lit(','));
        ok = ok && (js.lit('}') || js.fail("expected '}'"));
    }
    if (ok) {
        js.ws();
        if (js.p != js.e) ok = js.fail("trailing characters");
    }
    if (!ok) return corrupt("safetensors deserialization failed: InvalidHeaderDeserialization (%s)", js.err);

    // Metadata::validate: in offset order the tensors tile the buffer from 0 without holes.
    std::vector<const Entry *> order;
    for (const auto &kv : by_name) order.push_back(&kv.second);
    std::stable_sort(order.begin(), order.end(), [](const Entry *a, const Entry *b) {
        return a->begin != b->begin ? a->begin < b->begin : a->end < b->end;
    });
    uint64_t start = 0;
    for (const Entry *t : order) {
        if (t->begin != start || t->end < t->begin) return corrupt("safetensors deserialization failed: InvalidOffset(%s)", t->name);
        start = t->end;
        uint64_t numel = 1;
        for (uint64_t dim : t->shape)
            if (__builtin_mul_overflow(numel, dim, &numel)) return corrupt("safetensors deserialization failed: ValidationOverflow (%s)", t->name);
        uint64_t nbits;
        if (__builtin_mul_overflow(numel, (uint64_t)t->bits, &nbits)) return corrupt("safetensors deserialization failed: ValidationOverflow (%s)", t->name);
        if (nbits % 8) return corrupt("safetensors deserialization failed: MisalignedSlice (%s)", t->name);
        if (t->end - t->begin != nbits / 8) return corrupt("safetensors deserialization failed: TensorInvalidInfo (%s)", t->name);
        const_cast<Entry *>(t)->numel = numel;
    }
    if (start + 8 + n != f->len) return corrupt("safetensors deserialization failed: MetadataIncompleteBuffer");
    f->data = f->base + 8 + n;

    // st_dtype_to_ft: the DenseTensor loader reads four dtypes and refuses the file otherwise.
    for (auto &kv : by_name) {
        Entry &t = kv.second;
        if (t.dtype_name == "F64") t.dtype = FTH_DTYPE_F64;
        else if (t.dtype_name == "F32") t.dtype = FTH_DTYPE_F32;
        else if (t.dtype_name == "F16") t.dtype = FTH_DTYPE_F16;
        else if (t.dtype_name == "BF16") t.dtype = FTH_DTYPE_BF16;
        else if (t.dtype_name == "I64" || t.dtype_name == "I32" || t.dtype_name == "BOOL")
            return corrupt("integer/bool SafeTensors dtype (%s) is unsupported by the DenseTensor loader (tensor '%s')", t.dtype_name, t.name);
        else
            return corrupt("unsupported SafeTensors dtype: %s (tensor '%s')", t.dtype_name, t.name);
        f->tensors.push_back(std::move(t));  // std::map iterates in name order
    }
    return FTH_OK;
}

// ---- device side: widen / narrow and transpose while copying --------------------------------------
__device__ __forceinline__ float load_as_float(const float *p, int64_t i) { return p[i]; }
__device__ __forceinline__ float load_as_float(const double *p, int64_t i) { return (float)p[i]; }
struct Half { uint16_t v; };
struct Bf16 { uint16_t v; };
__device__ __forceinline__ float load_as_float(const Half *p, int64_t i) {
    // IEEE binary16 -> binary32, exact (subnormals, infinities and NaN payloads included)
    const uint32_t h = p[i].v, sign = (h & 0x8000u) << 16, ex = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    uint32_t bits;
    if (ex == 0) {
        if (man == 0) bits = sign;
        else {
            const int shift = __builtin_clz(man) - 21;  // leading zeros inside the 10-bit field, plus one
            bits = sign | ((uint32_t)(113 - shift) << 23) | ((man << shift) & 0x3FFu) << 13;
        }
    } else if (ex == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((ex + 112) << 23) | (man << 13);
    }
    return __uint_as_float(bits);
}
__device__ __forceinline__ float load_as_float(const Bf16 *p, int64_t i) { return __uint_as_float((uint32_t)p[i].v << 16); }
__device__ __forceinline__ double load_as_double(const double *p, int64_t i) { return p[i]; }
template <typename S> __device__ __forceinline__ double load_as_double(const S *p, int64_t i) { return (double)load_as_float(p, i); }
template <typename D, typename S> __device__ __forceinline__ D load_as(const S *p, int64_t i) {
    if constexpr (sizeof(D) == 8) return load_as_double(p, i);
    else return load_as_float(p, i);
}

template <typename D, typename S> __global__ __launch_bounds__(256) void convert_kernel(const S *__restrict__ src, D *__restrict__ dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = load_as<D>(src, i);
}

// dst [cols, rows] = src [rows, cols]^T through a 32 x 33 LDS tile (both sides coalesced).
template <typename D, typename S>
__global__ __launch_bounds__(256) void convert_transpose_kernel(const S *__restrict__ src, D *__restrict__ dst, int64_t rows, int64_t cols) {
    __shared__ D tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    const int64_t c0 = (int64_t)blockIdx.x * 32, r0 = (int64_t)blockIdx.y * 32;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int64_t r = r0 + ty + 8 * k, c = c0 + tx;
        if (r < rows && c < cols) tile[ty + 8 * k][tx] = load_as<D>(src, r * cols + c);
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int64_t c = c0 + ty + 8 * k, r = r0 + tx;
        if (r < rows && c < cols) dst[c * rows + r] = tile[tx][ty + 8 * k];
    }
}

// Two pinned staging buffers shared by every reader in the process (allocated at the first device
// read and kept; calls are serialised by the mutex).
constexpr size_t kStage = 16u << 20;
struct Staging {
    std::mutex mu;
    void *buf[2] = {nullptr, nullptr};
    hipEvent_t done[2] = {nullptr, nullptr};
};
Staging &staging() {
    static Staging s;
    return s;
}

// Host bytes -> device, through the pinned pair. On return the copies have been enqueued on `st`
// and the last use of each staging buffer is marked by its event.
int32_t upload(const uint8_t *src, size_t bytes, void *dst, hipStream_t st) {
    Staging &sg = staging();
    for (int i = 0; i < 2; ++i) {
        if (!sg.buf[i]) {
            FTH_HIP(hipHostMalloc(&sg.buf[i], kStage, hipHostMallocDefault));
            FTH_HIP(hipEventCreateWithFlags(&sg.done[i], hipEventDisableTiming));
            FTH_HIP(hipEventRecord(sg.done[i], st));
        }
    }
    size_t off = 0;
    for (int turn = 0; off < bytes; turn ^= 1) {
        const size_t n = std::min(kStage, bytes - off);
        FTH_HIP(hipEventSynchronize(sg.done[turn]));  // the DMA that last read this buffer has finished
        std::memcpy(sg.buf[turn], src + off, n);
        FTH_HIP(hipMemcpyAsync(static_cast<uint8_t *>(dst) + off, sg.buf[turn], n, hipMemcpyHostToDevice, st));
        FTH_HIP(hipEventRecord(sg.done[turn], st));
        off += n;
    }
    return FTH_OK;
}

template <typename D, typename S>
int32_t convert_launch(const void *raw, D *dst, int64_t rows, int64_t cols, bool transpose, hipStream_t st) {
    const S *src = static_cast<const S *>(raw);
    if (transpose) {
        const int64_t gx = fth::ceil_div(cols, 32), gy = fth::ceil_div(rows, 32);
        FTH_ARG(gx <= 2147483647LL && gy <= 65535, "safetensors: matrix too large to transpose in one launch");
        convert_transpose_kernel<D, S><<<dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, st>>>(src, dst, rows, cols);
    } else {
        const int64_t n = rows * cols, grid = fth::ceil_div(n, 256);
        FTH_ARG(grid <= 2147483647LL, "safetensors: tensor too large for one launch");
        convert_kernel<D, S><<<dim3((unsigned)grid), dim3(256), 0, st>>>(src, dst, n);
    }
    FTH_CHECK_LAUNCH("safetensors_convert");
    return FTH_OK;
}

template <typename D>
int32_t read_dev(const fth_safetensors *f, const char *name, int32_t transpose_2d, D *dst, size_t dst_elems, fth_stream s) {
    FTH_ARG(f != nullptr && name != nullptr, "safetensors_read_dev: NULL argument");
    const Entry *t = f->find(name);
    FTH_ARG(t != nullptr, "safetensors: no tensor named '%s'", name);
    FTH_ARG(dst_elems >= t->numel, "safetensors: destination holds %zu elements, tensor '%s' has %llu", dst_elems, name,
            (unsigned long long)t->numel);
    FTH_ARG(!transpose_2d || t->shape.size() == 2, "safetensors: transpose asked for '%s', which is not a matrix", name);
    if (t->numel == 0) return FTH_OK;
    FTH_ARG(dst != nullptr, "safetensors_read_dev: NULL destination");
    FTH_REQUIRE_DEVICE();
    hipStream_t st = fth::resolve_stream(s);
    const uint8_t *src = f->data + t->begin;
    const size_t bytes = (size_t)(t->end - t->begin);
    const bool same_type = t->dtype == (sizeof(D) == 4 ? FTH_DTYPE_F32 : FTH_DTYPE_F64);
    std::lock_guard<std::mutex> lock(staging().mu);
    int32_t rc;
    if (same_type && !transpose_2d) {
        rc = upload(src, bytes, dst, st);
    } else {
        fth::Scratch sc;  // raw bytes on the device, released once the kernel has run
        void *raw = nullptr;
        if ((rc = sc.get(&raw, bytes))) return rc;
        rc = upload(src, bytes, raw, st);
        const int64_t rows = transpose_2d ? (int64_t)t->shape[0] : 1, cols = transpose_2d ? (int64_t)t->shape[1] : (int64_t)t->numel;
        if (!rc) {
            switch (t->dtype) {
                case FTH_DTYPE_F64: rc = convert_launch<D, double>(raw, dst, rows, cols, transpose_2d != 0, st); break;
                case FTH_DTYPE_F32: rc = convert_launch<D, float>(raw, dst, rows, cols, transpose_2d != 0, st); break;
                case FTH_DTYPE_F16: rc = convert_launch<D, Half>(raw, dst, rows, cols, transpose_2d != 0, st); break;
                default: rc = convert_launch<D, Bf16>(raw, dst, rows, cols, transpose_2d != 0, st); break;
            }
        }
        hipError_t e = hipStreamSynchronize(st);  // the temporary goes back to the pool only after its reader
        if (!rc && e != hipSuccess) rc = fth::hip_fail(e, "hipStreamSynchronize");
        return rc;
    }
    if (rc) return rc;
    FTH_HIP(hipStreamSynchronize(st));  // the mapping may be closed as soon as this returns
    return FTH_OK;
}

// ---- the reference's native state-dict container -------------------------------------------------
// load_state_dict_from_bytes (crates/ft-serialize/src/lib.rs:1005-1160), check for check and in its order. Tensors are
// not copied: an entry records where its payload sits in the mapped bytes.
constexpr uint32_t kNativeVersion = 1;        // FT_STATE_FORMAT_VERSION (:596)
constexpr uint64_t kNativeMinTensorBytes = 17;  // FT_MIN_NATIVE_TENSOR_HEADER_BYTES (:601): key length + ndim + dtype tag

bool native_u64(const uint8_t *base, size_t len, size_t &pos, uint64_t &v) {
    if (len - pos < 8) return false;  // pos <= len always
    v = 0;
    for (int i = 7; i >= 0; --i) v = (v << 8) | base[pos + (size_t)i];
    pos += 8;
    return true;
}

int32_t parse_native(fth_safetensors *f) {
    const uint8_t *d = f->base;
    const size_t len = f->len;
    size_t pos = 0;
    if (len < 4 || std::memcmp(d, "FTSV", 4) != 0)
        return fth::set_error(FTH_ERR_INVALID_MAGIC, "invalid magic bytes: not a FrankenTorch state file");
    pos = 4;
    if (len - pos < 4) return corrupt("truncated u32");
    const uint32_t version = (uint32_t)d[4] | ((uint32_t)d[5] << 8) | ((uint32_t)d[6] << 16) | ((uint32_t)d[7] << 24);
    pos = 8;
    if (version > kNativeVersion) {
        fth::set_error(FTH_ERR_UNSUPPORTED_VERSION, "unsupported format version %u (max supported: %u)", version, kNativeVersion);
        fth::last_error().a = version;
        fth::last_error().b = kNativeVersion;
        return FTH_ERR_UNSUPPORTED_VERSION;
    }
    uint64_t count = 0;
    if (!native_u64(d, len, pos, count)) return corrupt("truncated u64");
    const uint64_t remaining = len - pos;
    if (count > remaining / kNativeMinTensorBytes)
        return fth::set_error(FTH_ERR_CORRUPT, "claimed %llu tensors but only %llu bytes remain (min %llu per tensor)",
                              (unsigned long long)count, (unsigned long long)remaining, (unsigned long long)kNativeMinTensorBytes);
    std::map<std::string, Entry> seen;  // name order, as the reference's BTreeMap
    static const char *const kNames[4] = {"f64", "f32", "f16", "bf16"};
    static const int kWidth[4] = {8, 4, 2, 2};
    for (uint64_t i = 0; i < count; ++i) {
        uint64_t key_len = 0;
        if (!native_u64(d, len, pos, key_len)) return corrupt("truncated u64");
        if (key_len > UINT64_MAX - pos) return corrupt("key length overflow");
        if (key_len > len - pos) return corrupt("truncated key data");
        if (!valid_utf8(d + pos, (size_t)key_len)) return corrupt("invalid UTF-8 in key");
        std::string key(reinterpret_cast<const char *>(d + pos), (size_t)key_len);
        pos += (size_t)key_len;
        if (seen.count(key)) return corrupt("duplicate tensor key in native state dict: '%s'", key);
        // (The reference accepts any UTF-8 key. One with a NUL byte cannot be named through a C string, so this reader
        // refuses the container instead of listing a key that could not be looked up.)
        if (key.find('\0') != std::string::npos) return corrupt("tensor key contains a NUL byte, which this interface cannot address");
        uint64_t ndim = 0;
        if (!native_u64(d, len, pos, ndim)) return corrupt("truncated u64");
        if (ndim > (len - pos) / 8) return corrupt("truncated shape data for tensor '%s'", key);
        Entry e;
        e.name = key;
        e.shape.reserve((size_t)ndim);
        uint64_t numel = 1;
        bool overflow = false;
        for (uint64_t k = 0; k < ndim; ++k) {
            uint64_t dim = 0;
            if (!native_u64(d, len, pos, dim)) return corrupt("truncated u64");
            if (!overflow && __builtin_mul_overflow(numel, dim, &numel)) overflow = true;
            e.shape.push_back(dim);
        }
        if (pos >= len) return corrupt("truncated dtype");
        const uint8_t tag = d[pos];
        if (tag > 3) return fth::set_error(FTH_ERR_CORRUPT, "unknown dtype tag: %u", (unsigned)tag);
        pos += 1;
        if (overflow) return corrupt("shape overflow in native state dict tensor '%s'", key);
        uint64_t needed = 0, end = 0;
        if (__builtin_mul_overflow(numel, (uint64_t)kWidth[tag], &needed) || __builtin_add_overflow((uint64_t)pos, needed, &end))
            return corrupt("byte count overflow for %s tensor '%s'", kNames[tag], key);
        if (end > len) return corrupt("truncated %s data", kNames[tag]);
        e.dtype = tag;  // the tags are the FTH_DTYPE_* values (crates/ft-serialize/src/lib.rs:597-600)
        e.bits = 8 * kWidth[tag];
        e.begin = pos;
        e.end = end;
        e.numel = numel;
        pos = (size_t)end;
        seen.emplace(std::move(key), std::move(e));
    }
    if (pos != len)
        return fth::set_error(FTH_ERR_CORRUPT, "trailing bytes after state dict payload: remaining=%llu", (unsigned long long)(len - pos));
    f->data = f->base;  // payload positions are absolute
    f->tensors.reserve(seen.size());
    for (auto &kv : seen) f->tensors.push_back(std::move(kv.second));
    return FTH_OK;
}

int32_t finish_open(fth_safetensors *f, fth_safetensors **out, bool native = false) {
    if (int32_t rc = native ? parse_native(f) : parse(f)) {
        delete f;
        return rc;
    }
    *out = f;
    return FTH_OK;
}

int32_t open_path(const char *path, fth_safetensors **out, bool native) {
    FTH_ARG(path != nullptr && out != nullptr, "open: NULL argument");
    *out = nullptr;
    const int fd = ::open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return fth::set_error(FTH_ERR_IO, "cannot open '%s': %s", path, std::strerror(errno));
    struct stat sb;
    if (fstat(fd, &sb) != 0) {
        const int e = errno;
        ::close(fd);
        return fth::set_error(FTH_ERR_IO, "cannot stat '%s': %s", path, std::strerror(e));
    }
    if (!S_ISREG(sb.st_mode)) {
        ::close(fd);
        return fth::set_error(FTH_ERR_IO, "'%s' is not a regular file", path);
    }
    fth_safetensors *f = new (std::nothrow) fth_safetensors();
    if (!f) {
        ::close(fd);
        return fth::set_error(FTH_ERR_KERNEL, "open: host allocation failed");
    }
    f->len = (size_t)sb.st_size;
    if (f->len > 0) {
        void *m = mmap(nullptr, f->len, PROT_READ, MAP_PRIVATE, fd, 0);
        if (m == MAP_FAILED) {
            const int e = errno;
            ::close(fd);
            delete f;
            return fth::set_error(FTH_ERR_IO, "cannot map '%s': %s", path, std::strerror(e));
        }
        f->base = static_cast<const uint8_t *>(m);
        f->mapped = true;
        (void)madvise(m, f->len, MADV_SEQUENTIAL);
    }
    ::close(fd);
    return finish_open(f, out, native);
}


int32_t open_bytes(const void *data, size_t len, fth_safetensors **out, bool native) {
    FTH_ARG(out != nullptr && (data != nullptr || len == 0), "open_bytes: NULL argument");
    *out = nullptr;
    fth_safetensors *f = new (std::nothrow) fth_safetensors();
    if (!f) return fth::set_error(FTH_ERR_KERNEL, "open_bytes: host allocation failed");
    f->base = static_cast<const uint8_t *>(data);
    f->len = len;
    return finish_open(f, out, native);
}

}  // namespace

extern "C" {

int32_t fth_safetensors_open(const char *path, fth_safetensors **out) { return open_path(path, out, false); }

int32_t fth_safetensors_open_bytes(const void *data, size_t len, fth_safetensors **out) { return open_bytes(data, len, out, false); }

int32_t fth_safetensors_close(fth_safetensors *f) {
    delete f;
    return FTH_OK;
}

int64_t fth_safetensors_count(const fth_safetensors *f) { return f ? (int64_t)f->tensors.size() : 0; }

const char *fth_safetensors_name(const fth_safetensors *f, int64_t index) {
    return (f && index >= 0 && (size_t)index < f->tensors.size()) ? f->tensors[(size_t)index].name.c_str() : nullptr;
}

int32_t fth_safetensors_info(const fth_safetensors *f, const char *name, fth_safetensors_tensor *info) {
    FTH_ARG(f != nullptr && name != nullptr && info != nullptr, "safetensors_info: NULL argument");
    const Entry *t = f->find(name);
    FTH_ARG(t != nullptr, "safetensors: no tensor named '%s'", name);
    FTH_ARG(t->shape.size() <= FTH_MAX_DIMS, "safetensors: tensor '%s' has %zu dimensions, more than %d", name, t->shape.size(), FTH_MAX_DIMS);
    std::memset(info, 0, sizeof(*info));
    info->dtype = t->dtype;
    info->ndim = (int32_t)t->shape.size();
    for (size_t i = 0; i < t->shape.size(); ++i) info->shape[i] = t->shape[i];
    info->numel = t->numel;
    info->byte_len = t->end - t->begin;
    return FTH_OK;
}

int32_t fth_safetensors_read(const fth_safetensors *f, const char *name, void *dst, size_t dst_bytes) {
    FTH_ARG(f != nullptr && name != nullptr, "safetensors_read: NULL argument");
    const Entry *t = f->find(name);
    FTH_ARG(t != nullptr, "safetensors: no tensor named '%s'", name);
    const size_t bytes = (size_t)(t->end - t->begin);
    if (dst_bytes < bytes) return fth::set_error(FTH_ERR_OUTPUT_TOO_SMALL, "safetensors: tensor '%s' has %zu bytes, destination %zu", name, bytes, dst_bytes);
    if (bytes) {
        FTH_ARG(dst != nullptr, "safetensors_read: NULL destination");
        std::memcpy(dst, f->data + t->begin, bytes);
    }
    return FTH_OK;
}

int32_t fth_safetensors_read_f32_dev(const fth_safetensors *f, const char *name, int32_t transpose_2d, float *dst_dev, size_t dst_elems,
                                     fth_stream s) {
    return read_dev<float>(f, name, transpose_2d, dst_dev, dst_elems, s);
}

int32_t fth_safetensors_read_f64_dev(const fth_safetensors *f, const char *name, int32_t transpose_2d, double *dst_dev, size_t dst_elems,
                                     fth_stream s) {
    return read_dev<double>(f, name, transpose_2d, dst_dev, dst_elems, s);
}

int32_t fth_safetensors_metadata_count(const fth_safetensors *f) { return (f && f->has_metadata) ? (int32_t)f->metadata.size() : -1; }

const char *fth_safetensors_metadata(const fth_safetensors *f, const char *key) {
    if (!f || !key || !f->has_metadata) return nullptr;
    auto it = f->metadata.find(key);
    return it == f->metadata.end() ? nullptr : it->second.c_str();
}

// The native state-dict container through the same handle: listing, info and reads are the safetensors functions.
int32_t fth_statedict_open(const char *path, fth_statedict **out) { return open_path(path, out, true); }
int32_t fth_statedict_open_bytes(const void *data, size_t len, fth_statedict **out) { return open_bytes(data, len, out, true); }
int32_t fth_statedict_close(fth_statedict *f) { return fth_safetensors_close(f); }
int64_t fth_statedict_count(const fth_statedict *f) { return fth_safetensors_count(f); }
const char *fth_statedict_name(const fth_statedict *f, int64_t index) { return fth_safetensors_name(f, index); }
int32_t fth_statedict_info(const fth_statedict *f, const char *name, fth_safetensors_tensor *info) { return fth_safetensors_info(f, name, info); }
int32_t fth_statedict_read(const fth_statedict *f, const char *name, void *dst, size_t dst_bytes) { return fth_safetensors_read(f, name, dst, dst_bytes); }
int32_t fth_statedict_read_f32_dev(const fth_statedict *f, const char *name, int32_t transpose_2d, float *dst_dev, size_t dst_elems, fth_stream s) {
    return read_dev<float>(f, name, transpose_2d, dst_dev, dst_elems, s);
}
int32_t fth_statedict_read_f64_dev(const fth_statedict *f, const char *name, int32_t transpose_2d, double *dst_dev, size_t dst_elems, fth_stream s) {
    return read_dev<double>(f, name, transpose_2d, dst_dev, dst_elems, s);
}

}  // extern "C"
