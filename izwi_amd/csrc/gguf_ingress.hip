// GGUF ingress: container parse (host only), tensor lookup, upload into weight handles.
//
// Mirrors the reference's GgufLoader (crates/izwi-core/src/models/shared/weights/gguf.rs:36-203)
// over candle-core 0.10.2's gguf_file::Content, whose source is not shipped with the
// reference; the container layout followed here is the public GGUF specification
// (versions 1-3).  Everything is little-endian and this library only runs on
// little-endian hosts.
#include <fcntl.h>
#include <hip/hip_runtime.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <new>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "../../include/izwi_gguf.h"
#include "qmm_internal.h"

namespace {

struct TypeSize {
    int id, block, bytes;
};
// ggml tensor types whose storage size is known here (GgmlDType::{block_size, type_size})
constexpr TypeSize kTypes[] = {
    {0, 1, 4},      // F32
    {1, 1, 2},      // F16
    {2, 32, 18},    // Q4_0
    {3, 32, 20},    // Q4_1
    {6, 32, 22},    // Q5_0
    {7, 32, 24},    // Q5_1
    {8, 32, 34},    // Q8_0
    {9, 32, 36},    // Q8_1
    {10, 256, 84},  // Q2_K
    {11, 256, 110}, // Q3_K
    {12, 256, 144}, // Q4_K
    {13, 256, 176}, // Q5_K
    {14, 256, 210}, // Q6_K
    {15, 256, 292}, // Q8_K
    {30, 1, 2},     // BF16
};

const TypeSize* type_size(int id) {
    for (const TypeSize& t : kTypes)
        if (t.id == id) return &t;
    return nullptr;
}

int scalar_bytes(int type) {
    switch (type) {
    case IZWI_GGUF_U8:
    case IZWI_GGUF_I8:
    case IZWI_GGUF_BOOL: return 1;
    case IZWI_GGUF_U16:
    case IZWI_GGUF_I16: return 2;
    case IZWI_GGUF_U32:
    case IZWI_GGUF_I32:
    case IZWI_GGUF_F32: return 4;
    case IZWI_GGUF_U64:
    case IZWI_GGUF_I64:
    case IZWI_GGUF_F64: return 8;
    default: return 0;
    }
}

struct Value {
    int type = -1;
    uint8_t raw[8] = {0, 0, 0, 0, 0, 0, 0, 0};           // scalar value, little-endian
    std::string str;                                      // STRING
    int elem_type = -1;                                   // ARRAY
    uint64_t count = 0;                                   // ARRAY
    const uint8_t* data = nullptr;                        // ARRAY of fixed-size elements
    std::vector<std::pair<const char*, uint64_t>> strs;   // ARRAY of strings (in the mapping)
};

struct Tensor {
    std::string name;
    izwi_gguf_tensor_info info;
};

} // namespace

struct izwi_gguf {
    std::string path;
    const uint8_t* map = nullptr; // the file's bytes: a read-only mapping, or a heap copy read with read(2)
    size_t size = 0;
    bool mapped = false;
    uint32_t version = 0, alignment = 32;
    uint64_t data_offset = 0;
    std::vector<std::string> keys;
    std::vector<Value> values;
    std::unordered_map<std::string, size_t> key_index;
    std::vector<Tensor> tensors;
    std::unordered_map<std::string, size_t> tensor_index;
    ~izwi_gguf() {
        if (map && mapped) munmap(const_cast<uint8_t*>(map), size);
        else if (map) free(const_cast<uint8_t*>(map));
    }
};

namespace {

// Bounds-checked reader over the mapping.
struct Cursor {
    const uint8_t* base;
    size_t size, pos = 0;
    bool v1 = false; // version 1: 32-bit counts and lengths
    bool ok = true;
    bool need(uint64_t n) {
        if (!ok || n > size - pos) ok = false;
        return ok;
    }
    template <class T>
    T get() {
        T v{};
        if (need(sizeof(T))) {
            memcpy(&v, base + pos, sizeof(T));
            pos += sizeof(T);
        }
        return v;
    }
    uint64_t len() { return v1 ? (uint64_t)get<uint32_t>() : get<uint64_t>(); }
    // a gguf string: length, then bytes (no terminator)
    bool str(const char** p, uint64_t* n) {
        *n = len();
        if (!need(*n)) return false;
        *p = reinterpret_cast<const char*>(base + pos);
        pos += *n;
        return true;
    }
};

bool read_value(Cursor& c, int type, Value& v, int depth) {
    v.type = type;
    const int sb = scalar_bytes(type);
    if (sb) {
        if (!c.need(sb)) return false;
        memcpy(v.raw, c.base + c.pos, sb);
        c.pos += sb;
        return true;
    }
    if (type == IZWI_GGUF_STRING) {
        const char* p;
        uint64_t n;
        if (!c.str(&p, &n)) return false;
        v.str.assign(p, n);
        return true;
    }
    if (type == IZWI_GGUF_ARRAY && depth < 4) {
        v.elem_type = (int)c.get<uint32_t>();
        v.count = c.len();
        if (!c.ok) return false;
        const int eb = scalar_bytes(v.elem_type);
        if (eb) {
            if (v.count > (c.size - c.pos) / eb) return c.ok = false;
            v.data = c.base + c.pos;
            c.pos += v.count * eb;
            return true;
        }
        if (v.elem_type == IZWI_GGUF_STRING) {
            // every string takes at least its length field (8 bytes, 4 in version 1)
            if (v.count > (c.size - c.pos) / (c.v1 ? 4 : 8)) return c.ok = false;
            v.strs.reserve((size_t)std::min<uint64_t>(v.count, 1u << 16)); // grows as strings are really read
            for (uint64_t i = 0; i < v.count; i++) {
                const char* p;
                uint64_t n;
                if (!c.str(&p, &n)) return false;
                v.strs.emplace_back(p, n);
            }
            return true;
        }
        if (v.elem_type == IZWI_GGUF_ARRAY) { // nested arrays: walked, their elements are not kept
            for (uint64_t i = 0; i < v.count; i++) {
                Value inner;
                if (!read_value(c, IZWI_GGUF_ARRAY, inner, depth + 1)) return false;
            }
            return true;
        }
    }
    return c.ok = false;
}

const Value* find_value(const izwi_gguf* g, const char* key) {
    if (!g || !key) return nullptr;
    auto it = g->key_index.find(key);
    return it == g->key_index.end() ? nullptr : &g->values[it->second];
}

const Tensor* find_tensor(const izwi_gguf* g, const char* name) {
    if (!g || !name) return nullptr;
    auto it = g->tensor_index.find(name);
    return it == g->tensor_index.end() ? nullptr : &g->tensors[it->second];
}

template <class T>
T raw_as(const Value& v) {
    T t;
    memcpy(&t, v.raw, sizeof(T));
    return t;
}

int64_t elem_count(const izwi_gguf_tensor_info& t) {
    int64_t n = 1;
    for (int i = 0; i < t.n_dims; i++) n *= t.dims[i];
    return n;
}

__global__ void half_to_f32_kernel(const uint16_t* __restrict__ in, float* __restrict__ out, uint64_t count,
                                   int is_bf16) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    out[i] = is_bf16 ? qmm_bf16_bits_to_f32(in[i]) : qmm_f16_bits_to_f32(in[i]);
}

// Q6_K blocks in their file layout (ql[128], qh[64], int8 scales[16], f16 d: 210 B per 256
// elements) -> f32, as candle-core's `BlockQ6K::to_float`: y = d * scale * (q - 32), evaluated
// left to right (the library is built without floating-point contraction).  One thread per
// (block, half, l): the four elements l, l + 32, l + 64, l + 96 of a half of 128.
__global__ void dequant_q6k_kernel(const uint8_t* __restrict__ blocks, float* __restrict__ out, uint64_t n_blocks) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t blk = idx >> 6;
    if (blk >= n_blocks) return;
    const int half = (int)(idx >> 5) & 1, l = (int)idx & 31, is = l >> 4;
    const uint8_t* b = blocks + blk * 210;
    const uint8_t* ql = b + 64 * half;
    const uint8_t qh = b[128 + 32 * half + l];
    const int8_t* sc = reinterpret_cast<const int8_t*>(b + 192) + 8 * half;
    const float d = qmm_f16_bits_to_f32((uint16_t)(b[208] | (b[209] << 8)));
    const int q1 = (int)((ql[l] & 0xF) | ((qh & 3) << 4)) - 32;
    const int q2 = (int)((ql[l + 32] & 0xF) | (((qh >> 2) & 3) << 4)) - 32;
    const int q3 = (int)((ql[l] >> 4) | (((qh >> 4) & 3) << 4)) - 32;
    const int q4 = (int)((ql[l + 32] >> 4) | (((qh >> 6) & 3) << 4)) - 32;
    float* y = out + blk * 256 + 128 * half;
    y[l] = d * (float)sc[is] * (float)q1;
    y[l + 32] = d * (float)sc[is + 2] * (float)q2;
    y[l + 64] = d * (float)sc[is + 4] * (float)q3;
    y[l + 96] = d * (float)sc[is + 6] * (float)q4;
}

struct DeviceBuffer {
    void* p = nullptr;
    ~DeviceBuffer() {
        if (p) (void)hipFree(p);
    }
};

} // namespace

extern "C" {

int izwi_gguf_is_gguf_file(const char* path) {
    if (!path) return 0;
    const int fd = open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return 0;
    char magic[4];
    const ssize_t n = read(fd, magic, 4);
    close(fd);
    return n == 4 && memcmp(magic, "GGUF", 4) == 0;
}

// `GgufMmapMode::parse` (model_io.rs:26-35): -1 for the empty string and unknown words.
int izwi_gguf_parse_mmap_mode(const char* raw) {
    if (!raw) return -1;
    std::string s(raw);
    const size_t b = s.find_first_not_of(" \t\r\n"), e = s.find_last_not_of(" \t\r\n");
    s = b == std::string::npos ? std::string() : s.substr(b, e - b + 1);
    for (auto& ch : s) ch = (char)tolower((unsigned char)ch);
    if (s == "auto") return IZWI_GGUF_MMAP_AUTO;
    if (s == "on" || s == "true" || s == "1" || s == "yes") return IZWI_GGUF_MMAP_ON;
    if (s == "off" || s == "false" || s == "0" || s == "no") return IZWI_GGUF_MMAP_OFF;
    return -1;
}

// `resolve_gguf_mmap_mode` (model_io.rs:63-67): the configured mode, else IZWI_GGUF_MMAP, else auto.
int izwi_gguf_resolve_mmap_mode(int configured) {
    if (configured == IZWI_GGUF_MMAP_AUTO || configured == IZWI_GGUF_MMAP_ON || configured == IZWI_GGUF_MMAP_OFF)
        return configured;
    const int env = izwi_gguf_parse_mmap_mode(getenv("IZWI_GGUF_MMAP"));
    return env >= 0 ? env : IZWI_GGUF_MMAP_AUTO;
}

int izwi_gguf_reader_kind(const izwi_gguf* g) {
    if (!g) return -1;
    return g->mapped ? IZWI_GGUF_READER_MAPPED : IZWI_GGUF_READER_BUFFERED;
}

} // extern "C"

namespace {

// The whole file through read(2) into one heap block (the buffered reader of model_io.rs:160; the
// handle's tensor pointers must stay valid until close, so the bytes are kept rather than streamed).
// On failure returns NULL and leaves errno describing it: ENOMEM, the error of read(2), or 0 for a
// file that ended before `size` bytes (read returned 0: errno would otherwise be stale).
uint8_t* read_whole_file(int fd, size_t size) {
    uint8_t* buf = static_cast<uint8_t*>(malloc(size));
    if (!buf) {
        errno = ENOMEM;
        return nullptr;
    }
    size_t done = 0;
    while (done < size) {
        errno = 0;
        const ssize_t n = read(fd, buf + done, std::min<size_t>(size - done, (size_t)1 << 30));
        if (n < 0 && errno == EINTR) continue;
        if (n <= 0) {
            const int err = n == 0 ? 0 : errno;
            free(buf);
            errno = err;
            return nullptr;
        }
        done += (size_t)n;
    }
    return buf;
}

int open_impl(const char* path, int configured_mode, izwi_gguf** out) {
    if (!out) return qmm_fail(IZWI_QMM_ERR_INVALID, "out is NULL");
    *out = nullptr;
    if (!path) return qmm_fail(IZWI_QMM_ERR_INVALID, "path is NULL");
    if (configured_mode < -1 || configured_mode > IZWI_GGUF_MMAP_OFF)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "bad mmap mode %d", configured_mode);
    // `gguf_mmap_enabled` (model_io.rs:77-83): auto maps on every backend
    const bool mmap_enabled = izwi_gguf_resolve_mmap_mode(configured_mode) != IZWI_GGUF_MMAP_OFF;
    const int fd = open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return qmm_fail(IZWI_QMM_ERR_INVALID, "Failed to open GGUF file: %s: %s", path, strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) {
        close(fd);
        return qmm_fail(IZWI_QMM_ERR_INVALID, "Failed to parse GGUF file: %s is empty or not a regular file", path);
    }
    const uint8_t* bytes = nullptr;
    bool mapped = false;
    if (mmap_enabled) {
        // _IZWI_GGUF_PRIVATE_TEST_FAIL_MMAP=1 makes the mapping attempt fail: a private hook of this
        // library's own test of the fallback below (a mapping of a readable regular file does not fail
        // otherwise); not a setting, not part of the interface
        const char* inject = getenv("_IZWI_GGUF_PRIVATE_TEST_FAIL_MMAP");
        void* map = (inject && inject[0] == '1') ? MAP_FAILED
                                                 : mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
        if (map != MAP_FAILED) {
            bytes = static_cast<const uint8_t*>(map);
            mapped = true;
        } else if (getenv("IZWI_GGUF_VERBOSE")) {
            // the reference warns and falls back to buffered I/O (model_io.rs:146-157)
            fprintf(stderr, "Failed to memory-map GGUF file %s; falling back to buffered I/O\n", path);
        }
    }
    if (!bytes) {
        bytes = read_whole_file(fd, (size_t)st.st_size);
        if (!bytes) {
            const int err = errno;
            close(fd);
            return qmm_fail(IZWI_QMM_ERR_INVALID, "Failed to open GGUF file: reading %s: %s", path,
                            err ? strerror(err) : "unexpected end of file");
        }
    }
    close(fd);
    izwi_gguf* g = new (std::nothrow) izwi_gguf;
    if (!g) {
        if (mapped) munmap(const_cast<uint8_t*>(bytes), (size_t)st.st_size);
        else free(const_cast<uint8_t*>(bytes));
        return qmm_fail(IZWI_QMM_ERR_INVALID, "Failed to open GGUF file: out of memory");
    }
    g->map = bytes;
    g->size = (size_t)st.st_size;
    g->mapped = mapped;
    g->path = path;
    auto bad = [&](const char* what) {
        const int rc = qmm_fail(IZWI_QMM_ERR_INVALID, "Failed to parse GGUF file: %s (%s)", what, path);
        delete g;
        return rc;
    };

    Cursor c{g->map, g->size};
    const uint32_t magic = c.get<uint32_t>();
    if (!c.ok || magic != 0x46554747u) return bad("bad magic, not a GGUF file"); // "GGUF"
    g->version = c.get<uint32_t>();
    if (!c.ok || g->version < 1 || g->version > 3) return bad("unsupported GGUF version");
    c.v1 = g->version == 1;
    const uint64_t n_tensors = c.len();
    const uint64_t n_kv = c.len();
    if (!c.ok) return bad("truncated header");
    // every entry takes at least a length field and a type: cheap plausibility bound
    if (n_kv > g->size / 8 || n_tensors > g->size / 8) return bad("implausible tensor or metadata count");

    g->keys.reserve(n_kv);
    g->values.reserve(n_kv);
    for (uint64_t i = 0; i < n_kv; i++) {
        const char* kp;
        uint64_t kn;
        if (!c.str(&kp, &kn)) return bad("truncated metadata key");
        const int type = (int)c.get<uint32_t>();
        Value v;
        if (!c.ok || !read_value(c, type, v, 0)) return bad("truncated or malformed metadata value");
        std::string key(kp, kn);
        g->key_index[key] = g->values.size(); // a repeated key keeps its last value, as a map insert does
        g->keys.push_back(std::move(key));
        g->values.push_back(std::move(v));
    }
    if (const Value* a = find_value(g, "general.alignment")) {
        uint64_t al = 0;
        if (a->type == IZWI_GGUF_U32) al = raw_as<uint32_t>(*a);
        else if (a->type == IZWI_GGUF_U64) al = raw_as<uint64_t>(*a);
        else if (a->type == IZWI_GGUF_U16) al = raw_as<uint16_t>(*a);
        else if (a->type == IZWI_GGUF_U8) al = raw_as<uint8_t>(*a);
        else if (a->type == IZWI_GGUF_I32 && raw_as<int32_t>(*a) > 0) al = (uint64_t)raw_as<int32_t>(*a);
        else return bad("general.alignment has a non-integer type");
        if (al == 0 || al > (1u << 30)) return bad("general.alignment out of range");
        g->alignment = (uint32_t)al;
    }

    g->tensors.reserve(n_tensors);
    for (uint64_t i = 0; i < n_tensors; i++) {
        const char* np;
        uint64_t nn;
        if (!c.str(&np, &nn)) return bad("truncated tensor name");
        Tensor t;
        t.name.assign(np, nn);
        memset(&t.info, 0, sizeof t.info);
        const uint32_t n_dims = c.get<uint32_t>();
        if (!c.ok || n_dims > IZWI_GGUF_MAX_DIMS) return bad("tensor with too many dimensions");
        t.info.n_dims = (int32_t)n_dims;
        int64_t count = 1;
        for (uint32_t d = 0; d < n_dims; d++) {
            const uint64_t dim = c.len();
            if (!c.ok || dim > (uint64_t)INT64_MAX || (dim != 0 && count > INT64_MAX / (int64_t)dim))
                return bad("tensor dimension overflows");
            t.info.dims[n_dims - 1 - d] = (int64_t)dim; // the file lists the innermost dimension first
            count *= (int64_t)dim;
        }
        t.info.ggml_dtype = (int32_t)c.get<uint32_t>();
        t.info.offset = c.get<uint64_t>();
        if (!c.ok) return bad("truncated tensor info");
        if (const TypeSize* ts = type_size(t.info.ggml_dtype)) {
            if (count % ts->block != 0) return bad("tensor element count is not a multiple of its block size");
            t.info.nbytes = (uint64_t)(count / ts->block) * (uint64_t)ts->bytes;
        }
        g->tensor_index[t.name] = g->tensors.size();
        g->tensors.push_back(std::move(t));
    }
    g->data_offset = (c.pos + g->alignment - 1) / g->alignment * g->alignment;
    for (Tensor& t : g->tensors) {
        if (t.info.nbytes == 0) continue;
        if (g->data_offset > g->size || t.info.offset > g->size - g->data_offset ||
            t.info.nbytes > g->size - g->data_offset - t.info.offset)
            return bad("tensor data lies outside the file");
        t.info.data = g->map + g->data_offset + t.info.offset;
    }
    *out = g;
    return IZWI_QMM_OK;
}

// No C++ exception may cross the C boundary: a crafted file can make the parser ask for more
// memory than there is.
template <class F>
int guarded(const char* what, F&& f) {
    try {
        return f();
    } catch (const std::bad_alloc&) {
        return qmm_fail(IZWI_QMM_ERR_INVALID, "%s: out of memory", what);
    } catch (const std::exception& e) {
        return qmm_fail(IZWI_QMM_ERR_INVALID, "%s: %s", what, e.what());
    } catch (...) {
        return qmm_fail(IZWI_QMM_ERR_INVALID, "%s: unknown failure", what);
    }
}

} // namespace

extern "C" {

int izwi_gguf_open(const char* path, izwi_gguf** out) {
    return guarded("Failed to parse GGUF file", [&] { return open_impl(path, -1, out); });
}

int izwi_gguf_open_with_mode(const char* path, int mmap_mode, izwi_gguf** out) {
    return guarded("Failed to parse GGUF file", [&] { return open_impl(path, mmap_mode, out); });
}

void izwi_gguf_close(izwi_gguf* g) { delete g; }

int izwi_gguf_header(const izwi_gguf* g, uint32_t* version, uint32_t* alignment, uint64_t* data_offset) {
    if (!g) return qmm_fail(IZWI_QMM_ERR_INVALID, "NULL gguf handle");
    if (version) *version = g->version;
    if (alignment) *alignment = g->alignment;
    if (data_offset) *data_offset = g->data_offset;
    return IZWI_QMM_OK;
}

int64_t izwi_gguf_tensor_count(const izwi_gguf* g) { return g ? (int64_t)g->tensors.size() : 0; }

int izwi_gguf_tensor_name(const izwi_gguf* g, int64_t index, const char** name) {
    if (!g || !name) return qmm_fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    if (index < 0 || index >= (int64_t)g->tensors.size())
        return qmm_fail(IZWI_QMM_ERR_INVALID, "tensor index %lld out of range", (long long)index);
    *name = g->tensors[(size_t)index].name.c_str();
    return IZWI_QMM_OK;
}

int izwi_gguf_tensor_info_get(const izwi_gguf* g, const char* name, izwi_gguf_tensor_info* out) {
    if (!g || !name || !out) return qmm_fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    const Tensor* t = find_tensor(g, name);
    if (!t) return qmm_fail(IZWI_QMM_ERR_INVALID, "tensor not found: '%s'", name);
    *out = t->info;
    return IZWI_QMM_OK;
}

int64_t izwi_gguf_metadata_count(const izwi_gguf* g) { return g ? (int64_t)g->keys.size() : 0; }

int izwi_gguf_metadata_key(const izwi_gguf* g, int64_t index, const char** key) {
    if (!g || !key) return qmm_fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    if (index < 0 || index >= (int64_t)g->keys.size())
        return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata index %lld out of range", (long long)index);
    *key = g->keys[(size_t)index].c_str();
    return IZWI_QMM_OK;
}

int izwi_gguf_metadata_type(const izwi_gguf* g, const char* key) {
    const Value* v = find_value(g, key);
    return v ? v->type : -1;
}

int izwi_gguf_metadata_string(const izwi_gguf* g, const char* key, const char** str, uint64_t* len) {
    const Value* v = find_value(g, key);
    if (!v || !str) return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata key not found: '%s'", key ? key : "(null)");
    if (v->type != IZWI_GGUF_STRING) return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata '%s' is not a string", key);
    *str = v->str.c_str();
    if (len) *len = v->str.size();
    return IZWI_QMM_OK;
}

int izwi_gguf_metadata_u64(const izwi_gguf* g, const char* key, uint64_t* value) {
    const Value* v = find_value(g, key);
    if (!v || !value) return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata key not found: '%s'", key ? key : "(null)");
    switch (v->type) { // the three types get_metadata_u64 accepts (gguf.rs:172-181)
    case IZWI_GGUF_U64: *value = raw_as<uint64_t>(*v); return IZWI_QMM_OK;
    case IZWI_GGUF_I64: *value = (uint64_t)raw_as<int64_t>(*v); return IZWI_QMM_OK;
    case IZWI_GGUF_U32: *value = raw_as<uint32_t>(*v); return IZWI_QMM_OK;
    default: return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata '%s' is not a u64, i64 or u32", key);
    }
}

int izwi_gguf_metadata_f64(const izwi_gguf* g, const char* key, double* value) {
    const Value* v = find_value(g, key);
    if (!v || !value) return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata key not found: '%s'", key ? key : "(null)");
    switch (v->type) {
    case IZWI_GGUF_U8: *value = raw_as<uint8_t>(*v); break;
    case IZWI_GGUF_I8: *value = raw_as<int8_t>(*v); break;
    case IZWI_GGUF_U16: *value = raw_as<uint16_t>(*v); break;
    case IZWI_GGUF_I16: *value = raw_as<int16_t>(*v); break;
    case IZWI_GGUF_U32: *value = raw_as<uint32_t>(*v); break;
    case IZWI_GGUF_I32: *value = raw_as<int32_t>(*v); break;
    case IZWI_GGUF_F32: *value = raw_as<float>(*v); break;
    case IZWI_GGUF_BOOL: *value = raw_as<uint8_t>(*v) != 0; break;
    case IZWI_GGUF_U64: *value = (double)raw_as<uint64_t>(*v); break;
    case IZWI_GGUF_I64: *value = (double)raw_as<int64_t>(*v); break;
    case IZWI_GGUF_F64: *value = raw_as<double>(*v); break;
    default: return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata '%s' is not a scalar number", key);
    }
    return IZWI_QMM_OK;
}

int izwi_gguf_metadata_array(const izwi_gguf* g, const char* key, int32_t* elem_type, uint64_t* count,
                             const void** data) {
    const Value* v = find_value(g, key);
    if (!v) return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata key not found: '%s'", key ? key : "(null)");
    if (v->type != IZWI_GGUF_ARRAY) return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata '%s' is not an array", key);
    if (elem_type) *elem_type = v->elem_type;
    if (count) *count = v->count;
    if (data) *data = v->data;
    return IZWI_QMM_OK;
}

int izwi_gguf_metadata_array_string(const izwi_gguf* g, const char* key, uint64_t index, const char** str,
                                    uint64_t* len) {
    const Value* v = find_value(g, key);
    if (!v || !str || !len) return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata key not found: '%s'", key ? key : "(null)");
    if (v->type != IZWI_GGUF_ARRAY || v->elem_type != IZWI_GGUF_STRING)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "metadata '%s' is not an array of strings", key);
    if (index >= v->strs.size())
        return qmm_fail(IZWI_QMM_ERR_INVALID, "index %llu out of range for '%s'", (unsigned long long)index, key);
    *str = v->strs[index].first; // in the mapping: not terminated, *len bytes
    *len = v->strs[index].second;
    return IZWI_QMM_OK;
}

static int gguf_load_weight_impl(const izwi_gguf* g, const char* name, izwi_qmm_weight** out) {
    if (!g || !name || !out) return qmm_fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    const Tensor* t = find_tensor(g, name);
    if (!t) return qmm_fail(IZWI_QMM_ERR_INVALID, "Failed to load tensor '%s' from GGUF: tensor not found", name);
    const izwi_gguf_tensor_info& ti = t->info;
    if (ti.ggml_dtype != IZWI_QMM_Q8_0 && ti.ggml_dtype != IZWI_QMM_Q4_K && ti.ggml_dtype != IZWI_QMM_Q6_K)
        return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED,
                        "Failed to load tensor '%s' from GGUF: ggml dtype %d is not supported (Q8_0 = 8, Q4_K = 12, Q6_K = 14)",
                        name, ti.ggml_dtype);
    if (ti.n_dims != 2)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "Failed to load tensor '%s' from GGUF: %d dimensions, a projection has 2",
                        name, ti.n_dims);
    return izwi_qmm_weight_create(ti.ggml_dtype, ti.dims[0], ti.dims[1], ti.data, ti.nbytes, IZWI_QMM_HOST, out);
}

static int gguf_load_packed_impl(const izwi_gguf* g, const char* const* names, int32_t n_names,
                          izwi_qmm_weight** out) {
    if (!g || !names || !out) return qmm_fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    if (n_names < 1) return qmm_fail(IZWI_QMM_ERR_INVALID, "Cannot pack empty Qwen3 quantized projection group");
    std::vector<int64_t> rows((size_t)n_names);
    std::vector<const void*> blocks((size_t)n_names);
    std::vector<uint64_t> nbytes((size_t)n_names);
    int dtype = 0;
    int64_t k = 0;
    for (int32_t i = 0; i < n_names; i++) {
        const Tensor* t = find_tensor(g, names[i]);
        if (!t)
            return qmm_fail(IZWI_QMM_ERR_INVALID, "Failed to load tensor '%s' from GGUF: tensor not found",
                            names[i] ? names[i] : "(null)");
        const izwi_gguf_tensor_info& ti = t->info;
        if (ti.n_dims != 2)
            return qmm_fail(IZWI_QMM_ERR_INVALID, "Failed to load tensor '%s' from GGUF: %d dimensions, a projection has 2",
                            names[i], ti.n_dims);
        if (i == 0) dtype = ti.ggml_dtype, k = ti.dims[1];
        if (ti.dims[1] != k) // the input width is compared first, as packed_qmatmul_from_qtensors does
            return qmm_fail(IZWI_QMM_ERR_INVALID, "Qwen3 quantized projection group input mismatch: expected %lld, got %lld",
                            (long long)k, (long long)ti.dims[1]);
        if (ti.ggml_dtype != dtype)
            return qmm_fail(IZWI_QMM_ERR_INVALID,
                            "Qwen3 quantized projection group dtype mismatch: expected ggml dtype %d, got %d", dtype,
                            ti.ggml_dtype);
        rows[(size_t)i] = ti.dims[0];
        blocks[(size_t)i] = ti.data;
        nbytes[(size_t)i] = ti.nbytes;
    }
    return izwi_qmm_weight_create_packed(dtype, n_names, rows.data(), k, blocks.data(), nbytes.data(), IZWI_QMM_HOST, out);
}

static int gguf_load_tensor_f32_impl(const izwi_gguf* g, const char* name, float* out, uint64_t count,
                              int mem_space, void* stream_) {
    if (!g || !name) return qmm_fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    if (mem_space != IZWI_QMM_DEVICE && mem_space != IZWI_QMM_HOST)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "bad mem_space %d", mem_space);
    const Tensor* t = find_tensor(g, name);
    if (!t) return qmm_fail(IZWI_QMM_ERR_INVALID, "Failed to load tensor '%s' from GGUF: tensor not found", name);
    const izwi_gguf_tensor_info& ti = t->info;
    const int64_t elems = elem_count(ti);
    if ((uint64_t)elems != count)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "tensor '%s' has %lld elements, the output holds %llu", name,
                        (long long)elems, (unsigned long long)count);
    if (elems == 0) return IZWI_QMM_OK;
    if (!out) return qmm_fail(IZWI_QMM_ERR_INVALID, "out is NULL");
    hipStream_t stream = (hipStream_t)stream_;
    auto hip_fail = [&](hipError_t e, const char* what) {
        return qmm_fail(e == hipErrorNoDevice || e == hipErrorInvalidDevice ? IZWI_QMM_ERR_NO_DEVICE : IZWI_QMM_ERR_HIP,
                        "Failed to load tensor '%s': %s: %s", name, what, hipGetErrorString(e));
    };
    switch (ti.ggml_dtype) {
    case 0: { // F32
        if (mem_space == IZWI_QMM_HOST) {
            memcpy(out, ti.data, (size_t)ti.nbytes);
            return IZWI_QMM_OK;
        }
        const hipError_t e = hipMemcpy(out, ti.data, (size_t)ti.nbytes, hipMemcpyHostToDevice);
        return e == hipSuccess ? IZWI_QMM_OK : hip_fail(e, "copy to the device");
    }
    case 1:    // F16
    case 14:   // Q6_K straight from its file layout
    case 30: { // BF16
        DeviceBuffer raw, tmp;
        hipError_t e = hipMalloc(&raw.p, (size_t)ti.nbytes);
        if (e != hipSuccess) return hip_fail(e, "device allocation");
        e = hipMemcpy(raw.p, ti.data, (size_t)ti.nbytes, hipMemcpyHostToDevice);
        if (e != hipSuccess) return hip_fail(e, "copy to the device");
        float* dst = out;
        if (mem_space == IZWI_QMM_HOST) {
            e = hipMalloc(&tmp.p, (size_t)elems * sizeof(float));
            if (e != hipSuccess) return hip_fail(e, "device allocation");
            dst = static_cast<float*>(tmp.p);
        }
        const uint64_t grid = ((uint64_t)elems + 255) / 256;
        if (grid > 0x7fffffffu) return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED, "tensor '%s' is too large to convert", name);
        if (ti.ggml_dtype == 14) // 64 threads per block of 256 elements
            dequant_q6k_kernel<<<(unsigned)(((uint64_t)elems / 4 + 255) / 256), 256, 0, stream>>>(
                static_cast<const uint8_t*>(raw.p), dst, (uint64_t)elems / 256);
        else
            half_to_f32_kernel<<<(unsigned)grid, 256, 0, stream>>>(static_cast<const uint16_t*>(raw.p), dst,
                                                                  (uint64_t)elems, ti.ggml_dtype == 30);
        e = hipGetLastError();
        if (e == hipSuccess) e = hipStreamSynchronize(stream); // `raw` is freed on return
        if (e != hipSuccess) return hip_fail(e, "conversion kernel");
        if (mem_space == IZWI_QMM_HOST) {
            e = hipMemcpy(out, tmp.p, (size_t)elems * sizeof(float), hipMemcpyDeviceToHost);
            if (e != hipSuccess) return hip_fail(e, "copy to the host");
        }
        return IZWI_QMM_OK;
    }
    case IZWI_QMM_Q8_0:
    case IZWI_QMM_Q4_K: {
        if (ti.n_dims < 1) return qmm_fail(IZWI_QMM_ERR_INVALID, "tensor '%s' has no dimensions", name);
        const int64_t k = ti.dims[ti.n_dims - 1];
        izwi_qmm_weight* w = nullptr;
        int rc = izwi_qmm_weight_create(ti.ggml_dtype, k ? elems / k : 0, k, ti.data, ti.nbytes, IZWI_QMM_HOST, &w);
        if (rc) return rc;
        rc = izwi_qmm_dequantize_f32(w, out, mem_space, stream_);
        if (rc == IZWI_QMM_OK && mem_space == IZWI_QMM_DEVICE) {
            const hipError_t e = hipStreamSynchronize(stream); // the handle's memory is released below
            if (e != hipSuccess) rc = hip_fail(e, "dequantization");
        }
        izwi_qmm_weight_destroy(w);
        return rc;
    }
    default:
        return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED,
                        "Failed to dequantize tensor '%s': ggml dtype %d is not supported (F32, F16, BF16, Q8_0, Q4_K, Q6_K)",
                        name, ti.ggml_dtype);
    }
}

int izwi_gguf_load_weight(const izwi_gguf* g, const char* name, izwi_qmm_weight** out) {
    return guarded("Failed to load tensor from GGUF", [&] { return gguf_load_weight_impl(g, name, out); });
}

int izwi_gguf_load_packed(const izwi_gguf* g, const char* const* names, int32_t n_names, izwi_qmm_weight** out) {
    return guarded("Failed to load tensors from GGUF", [&] { return gguf_load_packed_impl(g, names, n_names, out); });
}

int izwi_gguf_load_tensor_f32(const izwi_gguf* g, const char* name, float* out, uint64_t count, int mem_space,
                              void* stream_) {
    return guarded("Failed to load tensor from GGUF",
                   [&] { return gguf_load_tensor_f32_impl(g, name, out, count, mem_space, stream_); });
}

} // extern "C"
