// C ABI of libizwi_qmm: argument checking, device memory staging and kernel
// dispatch.  No arithmetic of the path lives here and there is no CPU fallback.
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include <algorithm>

#include "izwi_decode_ops.h"
#include "izwi_qmm.h"
#include "qmm_internal.h"

struct izwi_qmm_weight {
    QmmLayout layout;
    uint64_t nbytes; // GGUF block bytes
    void* tiled;     // device, layout.n_stacked * layout.matrix_bytes
    int device;
    int n_cus;
    std::atomic<int> is_lm_head;
};

static_assert(QMM_ERR_HIP_CODE == IZWI_QMM_ERR_HIP, "qmm_guarded reports IZWI_QMM_ERR_HIP");

namespace {

thread_local std::string g_error;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

} // namespace

// the same thread-local message for the library's other translation units
int qmm_fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

namespace {

int fail_hip(hipError_t e, const char* what) {
    return fail(IZWI_QMM_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t _e = (expr);                         \
        if (_e != hipSuccess) return fail_hip(_e, #expr); \
    } while (0)

struct DeviceInfo {
    bool ok = false;
    int n_cus = 0;
};
std::mutex g_dev_mutex;
DeviceInfo g_devices[64];

int ensure_device(int device, int* n_cus) {
    if (device < 0 || device >= 64) return fail(IZWI_QMM_ERR_INVALID, "bad device ordinal %d", device);
    std::lock_guard<std::mutex> lock(g_dev_mutex);
    if (!g_devices[device].ok) {
        int count = 0;
        hipError_t e = hipGetDeviceCount(&count);
        if (e != hipSuccess || count == 0) {
            (void)hipGetLastError();
            return fail(IZWI_QMM_ERR_NO_DEVICE,
                        "no HIP device available (%s); libizwi_qmm has no CPU fallback",
                        e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
        }
        if (device >= count)
            return fail(IZWI_QMM_ERR_NO_DEVICE, "device %d requested but only %d present", device, count);
        hipDeviceProp_t prop;
        HIP_TRY(hipGetDeviceProperties(&prop, device));
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            return fail(IZWI_QMM_ERR_NO_DEVICE, "device %d is %s; this library is built for gfx950 only",
                        device, prop.gcnArchName);
        g_devices[device].ok = true;
        g_devices[device].n_cus = prop.multiProcessorCount;
    }
    if (n_cus) *n_cus = g_devices[device].n_cus;
    return IZWI_QMM_OK;
}

// Whether the expert MLP runs on 16-row matrix-core tiles instead of 4-row dot4 segments: from 3.5
// sorted pairs per expert on average (IZWI_QMM_MOE_MFMA_MIN_ROWS = a whole number of pairs instead).
// Measured at 128 experts, top-8, per layer, segments / tiles: 68.6 / 80.4 us at 32 tokens, 78.1 / 83.9
// at 40, 83.5 / 85.4 at 48 (3 pairs per expert), 91.0 / 86.1 at 56, 99 / 87.1 at 64 (4 pairs): the tile
// path reads every expert once and costs about the same from 16 to 128 tokens, the segment path
// grows with the pairs.
bool moe_on_tiles(int64_t pairs, int n_experts) {
    static const int forced = [] {
        const char* s = getenv("IZWI_QMM_MOE_MFMA_MIN_ROWS");
        const int n = s ? atoi(s) : 0;
        return n < 1 ? 0 : n;
    }();
    return forced ? pairs >= (int64_t)forced * n_experts : 2 * pairs >= (int64_t)7 * n_experts;
}

// Most (token, slot) pairs for which izwi_moe_layer_f32 runs as two launches (every pair streams its
// expert's weights on its own; measured at 128 experts, top-8: 13.7 / 15.7 / 24.8 / 40.2 us per layer at
// 1 / 2 / 4 / 8 tokens against 23.3 / 26.5 / 33.4 / 46.6 on the grouped path, which reads an expert
// once per segment and wins beyond).  IZWI_QMM_MOE_SMALL_MAX_PAIRS overrides; 0 turns it off.
int moe_small_max_pairs() {
    static const int v = [] {
        const char* s = getenv("IZWI_QMM_MOE_SMALL_MAX_PAIRS");
        return s ? atoi(s) : 64;
    }();
    return v;
}

// hipGetDevice with the missing-GPU case reported as such (not as a generic HIP error)
int current_device(int* device) {
    hipError_t e = hipGetDevice(device);
    if (e == hipSuccess) return IZWI_QMM_OK;
    (void)hipGetLastError();
    if (e == hipErrorNoDevice || e == hipErrorInsufficientDriver || e == hipErrorInvalidDevice)
        return fail(IZWI_QMM_ERR_NO_DEVICE, "no HIP device available (%s); libizwi_qmm has no CPU fallback",
                    hipGetErrorString(e));
    return fail_hip(e, "hipGetDevice");
}

int type_supported(int dtype) { return dtype == IZWI_QMM_Q8_0 || dtype == IZWI_QMM_Q4_K || dtype == IZWI_QMM_Q6_K; }

int storage_bytes(int dtype, int64_t rows, int64_t cols, uint64_t* out) {
    if (!type_supported(dtype))
        return fail(IZWI_QMM_ERR_UNSUPPORTED, "ggml dtype %d is not supported (Q8_0 = 8, Q4_K = 12, Q6_K = 14)", dtype);
    if (rows < 0 || cols < 0) return fail(IZWI_QMM_ERR_INVALID, "negative shape [%lld, %lld]", (long long)rows, (long long)cols);
    unsigned __int128 elems = (unsigned __int128)rows * (unsigned __int128)cols;
    if (elems > (unsigned __int128)1 << 62)
        return fail(IZWI_QMM_ERR_INVALID, "quantized projection shape overflows");
    uint64_t e = (uint64_t)elems;
    uint64_t bs = (uint64_t)qmm_block_elems(dtype);
    if (e % bs)
        return fail(IZWI_QMM_ERR_INVALID,
                    "quantized projection element count %llu is not divisible by block size %llu",
                    (unsigned long long)e, (unsigned long long)bs);
    *out = e / bs * (uint64_t)qmm_block_bytes(dtype);
    return IZWI_QMM_OK;
}

struct Part {
    const void* data;
    uint64_t nbytes;
};

// Uploads the parts back to back, re-tiles them and returns the handle.
int create_from_parts(int dtype, int64_t n_stacked, int64_t n, int64_t k, const Part* parts,
                      int n_parts, int mem_space, izwi_qmm_weight** out) {
    if (!out) return fail(IZWI_QMM_ERR_INVALID, "out is NULL");
    *out = nullptr;
    if (mem_space != IZWI_QMM_DEVICE && mem_space != IZWI_QMM_HOST)
        return fail(IZWI_QMM_ERR_INVALID, "bad mem_space %d", mem_space);
    if (k <= 0 || k % qmm_block_elems(dtype))
        return fail(IZWI_QMM_ERR_INVALID, "k = %lld is not a positive multiple of the block size %d",
                    (long long)k, qmm_block_elems(dtype));
    int device = 0;
    if (int rc = current_device(&device)) return rc;
    int n_cus = 0;
    int rc = ensure_device(device, &n_cus);
    if (rc) return rc;

    uint64_t total = 0;
    for (int i = 0; i < n_parts; i++) total += parts[i].nbytes;
    QmmLayout L = qmm_make_layout(dtype, n_stacked, n, k);
    // the kernels index panels, rows and k-units with 32-bit integers
    if (n > ((int64_t)1 << 24) || k > ((int64_t)1 << 22) || n_stacked > 65536 ||
        L.row_tiles * L.k_groups >= ((int64_t)1 << 31))
        return fail(IZWI_QMM_ERR_UNSUPPORTED,
                    "shape [%lld x %lld x %lld] exceeds the kernels' limits (n <= 2^24, k <= 2^22, "
                    "n*k/4096 < 2^31 panels, <= 65536 stacked matrices)",
                    (long long)n_stacked, (long long)n, (long long)k);
    izwi_qmm_weight* w = new izwi_qmm_weight();
    w->layout = L;
    w->nbytes = total;
    w->tiled = nullptr;
    w->device = device;
    w->n_cus = n_cus;
    w->is_lm_head = 0;
    const uint64_t tiled_bytes = (uint64_t)L.n_stacked * (uint64_t)L.matrix_bytes;
    if (tiled_bytes == 0) {
        *out = w;
        return IZWI_QMM_OK;
    }
    void* staging = nullptr;
    hipError_t e = hipMalloc(&w->tiled, tiled_bytes);
    if (e == hipSuccess) e = hipMalloc(&staging, total);
    uint64_t off = 0;
    for (int i = 0; i < n_parts && e == hipSuccess; i++) {
        if (parts[i].nbytes)
            e = hipMemcpy((uint8_t*)staging + off, parts[i].data, parts[i].nbytes,
                          mem_space == IZWI_QMM_HOST ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice);
        off += parts[i].nbytes;
    }
    if (e == hipSuccess) e = qmm_launch_repack(L, staging, w->tiled, nullptr);
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    if (staging) (void)hipFree(staging);
    if (e != hipSuccess) {
        if (w->tiled) (void)hipFree(w->tiled);
        delete w;
        return fail_hip(e, "weight upload");
    }
    *out = w;
    return IZWI_QMM_OK;
}

// Device view of a caller buffer: the pointer itself, or a staged copy.
// Host-pointer calls: inputs are copied to the device before the launches and outputs back behind
// them.  Up to kStageMaxBytes a copy goes through a pooled pair of buffers (pinned host memory +
// device memory, kept until the process ends and reused by the next call): no allocation, no free
// and no pageable transfer per call.  Inputs: memcpy into the pinned buffer, then a copy kernel
// into the device buffer (the launches read an input many times: once over the host link, then
// from device memory).  Outputs: the kernels store straight into the pinned buffer (posted writes
// over the host link, no transfer behind the last launch), memcpy to the caller after the wait.
// The pool hands a pair to one Staged object at a time; the object gives it back when it is
// destroyed, after the stream has been waited for (finish() of the call's outputs, or the
// destructor itself on a path that returns early).  Larger copies allocate for the call and use
// pageable transfers.
constexpr size_t kStageMaxBytes = (size_t)8 << 20;
struct StagePair {
    int device = -1;
    void* pinned = nullptr;
    void* dev = nullptr;
    size_t cap = 0;
};
std::mutex g_stage_mutex;
std::vector<StagePair*> g_stage_free;
thread_local uint64_t t_stage_syncs = 0; // stream waits done by finish() on this thread

hipError_t stage_acquire(size_t bytes, StagePair** out) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    StagePair* best = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_stage_mutex);
        size_t at = 0;
        for (size_t i = 0; i < g_stage_free.size(); i++) {
            StagePair* c = g_stage_free[i];
            if (c->device != device) continue;
            // the smallest pair that is large enough, else the largest one (it grows below)
            const bool better = !best || (best->cap >= bytes ? (c->cap >= bytes && c->cap < best->cap) : c->cap > best->cap);
            if (better) best = c, at = i;
        }
        if (best) g_stage_free.erase(g_stage_free.begin() + (ptrdiff_t)at);
    }
    if (!best) {
        best = new (std::nothrow) StagePair;
        if (!best) return hipErrorOutOfMemory;
        best->device = device;
    }
    if (best->cap < bytes) {
        // nobody uses this pair: its last user waited for its stream before giving it back
        if (best->pinned) (void)hipHostFree(best->pinned);
        if (best->dev) (void)hipFree(best->dev);
        best->pinned = best->dev = nullptr;
        size_t cap = best->cap * 2 > bytes ? best->cap * 2 : bytes;
        cap = (cap + 65535) & ~(size_t)65535;
        best->cap = 0;
        e = hipHostMalloc(&best->pinned, cap, hipHostMallocDefault);
        if (e == hipSuccess) e = hipMalloc(&best->dev, cap);
        if (e != hipSuccess) {
            if (best->pinned) (void)hipHostFree(best->pinned);
            delete best;
            return e;
        }
        best->cap = cap;
    }
    *out = best;
    return hipSuccess;
}
void stage_release(StagePair* p) {
    std::lock_guard<std::mutex> lock(g_stage_mutex);
    g_stage_free.push_back(p);
}

// pinned host memory -> device memory by a kernel (16 bytes per thread and step; n16 = bytes / 16
// rounded up, both buffers are sized in multiples of 64 KiB): a launch starts sooner than a copy
// engine transfer of a few KB
__global__ void stage_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

struct Staged {
    void* dev = nullptr;
    void* host = nullptr;
    size_t bytes = 0;
    bool owned = false; // dev was allocated for this call (copies beyond kStageMaxBytes)
    bool copy_back = false;
    StagePair* pair = nullptr;
    bool direct = false;
    hipStream_t pair_stream = nullptr;
    uint64_t syncs_at_start = 0;
    Staged() = default;
    Staged(const Staged&) = delete;
    Staged& operator=(const Staged&) = delete;
    ~Staged() {
        if (owned && dev) (void)hipFree(dev);
        if (pair) {
            // (a path that returned before any finish(): queued work may still touch the pair)
            if (t_stage_syncs == syncs_at_start) (void)hipStreamSynchronize(pair_stream);
            stage_release(pair);
        }
    }
    hipError_t in(const void* p, size_t n, int mem_space, hipStream_t stream) {
        bytes = n;
        if (mem_space == IZWI_QMM_DEVICE || n == 0) {
            dev = const_cast<void*>(p);
            return hipSuccess;
        }
        if (n <= kStageMaxBytes) {
            hipError_t e = stage_acquire(n, &pair);
            if (e != hipSuccess) return e;
            pair_stream = stream;
            syncs_at_start = t_stage_syncs;
            dev = pair->dev;
            memcpy(pair->pinned, p, n);
            {
                void* src = nullptr;
                hipError_t e2 = hipHostGetDevicePointer(&src, pair->pinned, 0);
                if (e2 != hipSuccess) return e2;
                const size_t n16 = (n + 15) / 16;
                const unsigned grid = (unsigned)((n16 + 255) / 256 < 1024 ? (n16 + 255) / 256 : 1024);
                stage_copy_kernel<<<grid, 256, 0, stream>>>((const uint4*)src, (uint4*)dev, n16);
                return hipGetLastError();
            }
        }
        owned = true;
        hipError_t e = hipMalloc(&dev, n);
        if (e != hipSuccess) return e;
        return hipMemcpy(dev, p, n, hipMemcpyHostToDevice);
    }
    // direct_ok: every byte of the output is written by kernel stores and read by no launch (false
    // for the target of a copy call, which wants device memory)
    hipError_t out(void* p, size_t n, int mem_space, hipStream_t stream, bool direct_ok = true) {
        bytes = n;
        if (mem_space == IZWI_QMM_DEVICE || n == 0) {
            dev = p;
            return hipSuccess;
        }
        copy_back = true;
        host = p;
        if (n <= kStageMaxBytes) {
            hipError_t e = stage_acquire(n, &pair);
            if (e != hipSuccess) return e;
            pair_stream = stream;
            syncs_at_start = t_stage_syncs;
            // the kernels store straight into the pinned buffer (posted writes over the host link):
            // no copy engine transfer behind the last launch
            direct = direct_ok;
            if (direct) return hipHostGetDevicePointer(&dev, pair->pinned, 0);
            dev = pair->dev;
            return hipSuccess;
        }
        owned = true;
        return hipMalloc(&dev, n);
    }
    hipError_t finish(hipStream_t stream) {
        if (!copy_back) return hipSuccess;
        if (pair) {
            hipError_t e = direct ? hipSuccess : hipMemcpyAsync(pair->pinned, dev, bytes, hipMemcpyDeviceToHost, stream);
            if (e == hipSuccess) e = hipStreamSynchronize(stream);
            if (e != hipSuccess) return e;
            t_stage_syncs++;
            memcpy(host, pair->pinned, bytes);
            return hipSuccess;
        }
        hipError_t e = hipStreamSynchronize(stream);
        if (e != hipSuccess) return e;
        t_stage_syncs++;
        return hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost);
    }
};

// Scratch for kernels that need device memory beyond inputs and outputs (the
// quantized activations of the batched decode kernels, the intermediates of the
// expert MLP, the counting sort's histograms, split-k partial tiles).  One buffer
// per (device, stream).
//
// Exclusive use: a library call that asks for scratch holds its stream's buffer
// from that request until the call returns (QmmCallScope, below), i.e. until
// every launch that reads or writes the buffer has been queued.  A second host
// thread calling on the same stream waits there, so its launches are queued
// behind the first call's and, work on a stream being ordered, run behind them:
// two calls never interleave on one buffer.  Calls on different streams use
// different buffers and do not wait for each other.
//
// Growth: a larger request allocates a new buffer; the old one is RETIRED, never
// freed before the process ends: launches already queued, and HIP graphs captured
// earlier, keep addresses into it.  Sizes grow geometrically, so the retired
// buffers of a stream add up to less than four times its largest.  A request
// that would have to grow while its stream is being captured fails
// (hipErrorStreamCaptureUnsupported): allocate beforehand with
// izwi_qmm_scratch_reserve or with one eager call of the same size.
struct Scratch {
    std::mutex in_use; // held by the call that uses the buffer, from its first request to its return
    void* ptr = nullptr;
    size_t bytes = 0;
    std::vector<void*> retired;
};
std::mutex g_scratch_mutex;                              // guards the map, not the buffers
std::unordered_map<uint64_t, std::unique_ptr<Scratch>> g_scratch;
std::atomic<uint64_t> g_scratch_retired_bytes{0};

thread_local int t_call_depth = 0;            // nested library calls of this thread
thread_local std::vector<Scratch*> t_leased;  // buffers this thread's outermost call holds
thread_local uint64_t t_thread_tag = 0;

uint64_t scratch_key(int device, hipStream_t stream) {
    uint64_t key = ((uint64_t)(uintptr_t)stream) ^ ((uint64_t)device << 56);
    if (stream == hipStreamPerThread) {
        // one handle value, a different stream in every host thread
        static std::atomic<uint64_t> next{1};
        if (!t_thread_tag) t_thread_tag = next.fetch_add(1);
        key ^= t_thread_tag << 24;
    }
    return key;
}

bool stream_is_capturing(hipStream_t stream) {
    if (!stream) return false; // the legacy default stream cannot be captured
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return st != hipStreamCaptureStatusNone;
}

hipError_t get_scratch(int device, hipStream_t stream, size_t bytes, void** out) {
    Scratch* s = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        auto& slot = g_scratch[scratch_key(device, stream)];
        if (!slot) slot.reset(new Scratch());
        s = slot.get();
    }
    const bool held = std::find(t_leased.begin(), t_leased.end(), s) != t_leased.end();
    if (!held) s->in_use.lock();
    hipError_t e = hipSuccess;
    if (s->bytes < bytes) {
        if (stream_is_capturing(stream)) {
            e = hipErrorStreamCaptureUnsupported;
        } else {
            size_t want = bytes < (1u << 20) ? (1u << 20) : bytes + bytes / 2;
            void* p = nullptr;
            e = hipMalloc(&p, want);
            if (e == hipSuccess) {
                if (s->ptr) {
                    s->retired.push_back(s->ptr);
                    g_scratch_retired_bytes.fetch_add(s->bytes, std::memory_order_relaxed);
                }
                s->ptr = p;
                s->bytes = want;
            }
        }
    }
    *out = s->ptr;
    if (!held) {
        // inside a library call: keep the buffer until the call returns; outside (a reservation):
        // nothing is launched on it, release at once
        if (t_call_depth > 0 && e == hipSuccess) t_leased.push_back(s);
        else s->in_use.unlock();
    }
    return e;
}

// Smallest m that takes the batched (MFMA) decode kernel for a weight of this k; below it the fused
// single-launch kernel runs.  Three, and five where k is short (up to 3072): a call of three or four
// rows on the batched kernels is two launches whose chains - quantizer, window copy, panel, k-split -
// take 9 us however small the matrix, the single-launch kernel with four rows per pass takes 6 (Q8_0 at
// the 0.6B shapes, per call: 5.9 against 9.2 us for o, 6.3 against 9.4 for down), while at k = 4096 and
// beyond it re-reads enough activations per workgroup to lose (8B shapes: o 8.2 against 8.3, down 15.0
// against 12.6).  The rule looks at k only, which the members of a projection group share: a group and
// its members' separate calls take the same kernel, so their results stay the same bits.
// IZWI_QMM_MFMA_MIN_M overrides it for every k (tuning knob).
constexpr int64_t kShortK = 3072;
int mfma_min_m(int64_t k) {
    static int forced = [] {
        const char* e = getenv("IZWI_QMM_MFMA_MIN_M");
        int n = e ? atoi(e) : 0;
        return n > 0 ? n : 0;
    }();
    if (forced) return forced;
    return k <= kShortK ? 5 : 3;
}

// Arithmetic of f32 / fused calls with more than 64 activation rows: 0 = activations rounded to
// bf16, weights dequantized to bf16, bf16 matrix cores (the prefill kernel); 1 = the reference's
// integer block dots on quantized activations, 64 rows at a time through the batched decode kernel.
// IZWI_QMM_LARGE_M=int8 selects 1 at start-up; izwi_qmm_set_large_m_arithmetic changes it later.
std::atomic<int> g_large_m_mode{-1};
int large_m_mode() {
    int v = g_large_m_mode.load(std::memory_order_relaxed);
    if (v < 0) {
        const char* e = getenv("IZWI_QMM_LARGE_M");
        v = (e && (!strcmp(e, "int8") || !strcmp(e, "1"))) ? IZWI_QMM_LARGE_M_INT8 : IZWI_QMM_LARGE_M_BF16;
        g_large_m_mode.store(v, std::memory_order_relaxed);
    }
    return v;
}

int check_space(int mem_space) {
    if (mem_space != IZWI_QMM_DEVICE && mem_space != IZWI_QMM_HOST)
        return fail(IZWI_QMM_ERR_INVALID, "bad mem_space %d", mem_space);
    return IZWI_QMM_OK;
}

// ---- profiling -----------------------------------------------------------
std::atomic<int> g_profile{-1}; // -1: read the environment on first use
std::atomic<uint64_t> g_calls{0}, g_ns{0}, g_in_casts{0}, g_in_cast_ns{0}, g_out_casts{0},
    g_out_cast_ns{0}, g_lm_calls{0}, g_lm_ns{0}, g_silu_fused{0}, g_silu_fallback{0}, g_argmax_calls{0}, g_argmax_ns{0};

bool parse_env_bool(const char* raw) {
    if (!raw) return false;
    std::string s(raw);
    for (auto& c : s) c = (char)tolower(c);
    return s == "1" || s == "true" || s == "yes" || s == "on";
}

bool profiling() {
    int v = g_profile.load(std::memory_order_relaxed);
    if (v < 0) {
        v = parse_env_bool(getenv("IZWI_QWEN3_PROFILE")) ? 1 : 0;
        g_profile.store(v, std::memory_order_relaxed);
    }
    return v != 0;
}

struct ProfileScope {
    bool on;
    hipStream_t stream;
    const izwi_qmm_weight* w;
    std::chrono::steady_clock::time_point t0;
    ProfileScope(const izwi_qmm_weight* w_, hipStream_t s) : on(profiling()), stream(s), w(w_) {
        if (on) t0 = std::chrono::steady_clock::now();
    }
    ~ProfileScope() {
        if (!on) return;
        if (stream_is_capturing(stream)) return; // nothing runs during a capture, and a wait would end it
        (void)hipStreamSynchronize(stream); // time the execution, not the launch
        uint64_t ns = (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(
                          std::chrono::steady_clock::now() - t0)
                          .count();
        g_calls.fetch_add(1, std::memory_order_relaxed);
        g_ns.fetch_add(ns, std::memory_order_relaxed);
        if (w && w->is_lm_head.load(std::memory_order_relaxed)) {
            g_lm_calls.fetch_add(1, std::memory_order_relaxed);
            g_lm_ns.fetch_add(ns, std::memory_order_relaxed);
        }
    }
};

} // namespace

// The current device, checked (a gfx950 device is present) and with its CU count; the library's
// per-(device, stream) scratch buffer.  For the other source files of the library.
int qmm_current_device(int* device, int* n_cus) {
    if (int rc = current_device(device)) return rc;
    return ensure_device(*device, n_cus);
}
hipError_t qmm_get_scratch(int device, hipStream_t stream, size_t bytes, void** out) {
    return get_scratch(device, stream, bytes, out);
}
std::atomic<int> g_moe_expert_form{-2}; // -2: read IZWI_QMM_MOE_EXPERT_FORM on first use; then -1 (by size), 0, 1, 2
int qmm_moe_expert_form() {
    int v = g_moe_expert_form.load(std::memory_order_relaxed);
    if (v < -1) {
        const char* e = getenv("IZWI_QMM_MOE_EXPERT_FORM");
        v = e && e[0] == '2' ? 2 : e && e[0] == '1' ? 1 : e && e[0] == '0' ? 0 : -1;
        g_moe_expert_form.store(v, std::memory_order_relaxed);
    }
    return v;
}
const QmmLayout* qmm_weight_layout(const izwi_qmm_weight* w) { return &w->layout; }
const void* qmm_weight_tiled(const izwi_qmm_weight* w) { return w->tiled; }
int qmm_weight_device(const izwi_qmm_weight* w) { return w->device; }
bool qmm_profiling() { return profiling(); }
bool qmm_stream_is_capturing(hipStream_t stream) { return stream_is_capturing(stream); }
void qmm_profile_count_argmax(uint64_t ns) {
    g_argmax_calls.fetch_add(1, std::memory_order_relaxed);
    g_argmax_ns.fetch_add(ns, std::memory_order_relaxed);
}
QmmCallScope::QmmCallScope() { t_call_depth++; }
QmmCallScope::~QmmCallScope() {
    if (--t_call_depth > 0) return;
    for (Scratch* s : t_leased) s->in_use.unlock();
    t_leased.clear();
}

namespace {
int batched_group_on_records(const izwi_qmm_weight* const* weights, int32_t n_weights, const float* x, int64_t m,
                             float* const* ys, void* records, hipStream_t stream);
} // namespace

// ---- the entry point that allocates nothing ---------------------------------
// Scratch of izwi_qmm_forward_f32_noalloc: the quantized activation records of the batched decode
// kernels (up to 64 rows), held in the library's image on every GPU it runs on instead of being
// allocated.  `noalloc_scratch` is the host-side name of the array, not a device address: the
// device address of each GPU's own copy is looked up once per device and only that pointer is
// handed to kernels.
static __device__ __align__(256) unsigned char noalloc_scratch[IZWI_QMM_NOALLOC_SCRATCH_BYTES];

namespace {
std::mutex g_noalloc_mutex;
void* g_noalloc_ptr[64] = {};

// Device address of `device`'s copy of the array; `device` must be the current device.
hipError_t noalloc_scratch_ptr(int device, void** out) {
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    if (!g_noalloc_ptr[device]) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(noalloc_scratch));
        if (e != hipSuccess) return e;
        g_noalloc_ptr[device] = p;
    }
    *out = g_noalloc_ptr[device];
    return hipSuccess;
}
} // namespace

extern "C" {

int izwi_qmm_abi_version(void) { return IZWI_QMM_ABI_VERSION; }

const char* izwi_qmm_last_error(void) { return g_error.c_str(); }

int izwi_qmm_init(int device) {
    return qmm_guarded("izwi_qmm_abi_version", [&]() -> int {
    int rc = ensure_device(device, nullptr);
    if (rc) return rc;
    HIP_TRY(hipSetDevice(device));
    void* p = nullptr;
    HIP_TRY(noalloc_scratch_ptr(device, &p)); // the static scratch of this device, looked up once
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_storage_bytes(int ggml_dtype, int64_t rows, int64_t cols, uint64_t* out_bytes) {
    return qmm_guarded("izwi_qmm_storage_bytes", [&]() -> int {
    if (!out_bytes) return fail(IZWI_QMM_ERR_INVALID, "out_bytes is NULL");
    return storage_bytes(ggml_dtype, rows, cols, out_bytes);
    });
}

int izwi_qmm_weight_create(int ggml_dtype, int64_t n, int64_t k, const void* blocks,
                           uint64_t nbytes, int mem_space, izwi_qmm_weight** out) {
    return qmm_guarded("izwi_qmm_weight_create", [&]() -> int {
    return izwi_qmm_weight_create_stacked(ggml_dtype, 1, n, k, blocks, nbytes, mem_space, out);
    });
}

int izwi_qmm_weight_create_stacked(int ggml_dtype, int32_t n_experts, int64_t n, int64_t k,
                                   const void* blocks, uint64_t nbytes, int mem_space,
                                   izwi_qmm_weight** out) {
    return qmm_guarded("izwi_qmm_weight_create_stacked", [&]() -> int {
    if (n_experts < 1) return fail(IZWI_QMM_ERR_INVALID, "n_experts must be >= 1");
    uint64_t expected = 0;
    int rc = storage_bytes(ggml_dtype, (int64_t)n_experts * n, k, &expected);
    if (rc) return rc;
    if (nbytes != expected)
        return fail(IZWI_QMM_ERR_INVALID, "quantized projection has %llu bytes, expected %llu",
                    (unsigned long long)nbytes, (unsigned long long)expected);
    if (expected && !blocks) return fail(IZWI_QMM_ERR_INVALID, "blocks is NULL");
    Part part{blocks, nbytes};
    return create_from_parts(ggml_dtype, n_experts, n, k, &part, 1, mem_space, out);
    });
}

int izwi_qmm_weight_create_packed(int ggml_dtype, int32_t n_parts, const int64_t* part_rows,
                                  int64_t k, const void* const* part_blocks,
                                  const uint64_t* part_nbytes, int mem_space,
                                  izwi_qmm_weight** out) {
    return qmm_guarded("izwi_qmm_weight_create_packed", [&]() -> int {
    if (n_parts <= 0 || !part_rows || !part_blocks || !part_nbytes)
        return fail(IZWI_QMM_ERR_INVALID, "Cannot pack empty Qwen3 quantized projection group");
    int64_t total_rows = 0;
    uint64_t total_bytes = 0;
    std::vector<Part> parts;
    for (int i = 0; i < n_parts; i++) {
        uint64_t expected = 0;
        int rc = storage_bytes(ggml_dtype, part_rows[i], k, &expected);
        if (rc) return rc;
        if (part_nbytes[i] != expected)
            return fail(IZWI_QMM_ERR_INVALID,
                        "Qwen3 quantized projection group input mismatch: part %d has %llu bytes, "
                        "expected %llu for [%lld, %lld]",
                        i, (unsigned long long)part_nbytes[i], (unsigned long long)expected,
                        (long long)part_rows[i], (long long)k);
        if (expected && !part_blocks[i]) return fail(IZWI_QMM_ERR_INVALID, "part %d is NULL", i);
        total_rows += part_rows[i];
        total_bytes += part_nbytes[i];
        parts.push_back(Part{part_blocks[i], part_nbytes[i]});
    }
    uint64_t expected_total = 0;
    int rc = storage_bytes(ggml_dtype, total_rows, k, &expected_total);
    if (rc) return rc;
    if (expected_total != total_bytes)
        return fail(IZWI_QMM_ERR_INVALID,
                    "Qwen3 packed quantized projection has %llu bytes, expected %llu",
                    (unsigned long long)total_bytes, (unsigned long long)expected_total);
    return create_from_parts(ggml_dtype, 1, total_rows, k, parts.data(), n_parts, mem_space, out);
    });
}

void izwi_qmm_weight_destroy(izwi_qmm_weight* w) {
    if (!w) return;
    if (w->tiled) (void)hipFree(w->tiled);
    delete w;
}

int izwi_qmm_weight_get_info(const izwi_qmm_weight* w, izwi_qmm_weight_info* out) {
    return qmm_guarded("izwi_qmm_weight_get_info", [&]() -> int {
    if (!w || !out) return fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    out->ggml_dtype = w->layout.dtype;
    out->n_stacked = (int32_t)w->layout.n_stacked;
    out->n = w->layout.n;
    out->k = w->layout.k;
    out->nbytes = w->nbytes;
    out->device = w->device;
    out->reserved = 0;
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_weight_set_lm_head(izwi_qmm_weight* w, int is_lm_head) {
    return qmm_guarded("izwi_qmm_weight_set_lm_head", [&]() -> int {
    if (!w) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    w->is_lm_head.store(is_lm_head ? 1 : 0, std::memory_order_relaxed);
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_weight_data(const izwi_qmm_weight* w, void* out_blocks, uint64_t nbytes,
                         int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_weight_data", [&]() -> int {
    if (!w) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    if (int rc = check_space(mem_space)) return rc;
    if (nbytes != w->nbytes)
        return fail(IZWI_QMM_ERR_INVALID, "buffer has %llu bytes, tensor data has %llu",
                    (unsigned long long)nbytes, (unsigned long long)w->nbytes);
    if (nbytes == 0) return IZWI_QMM_OK;
    if (!out_blocks) return fail(IZWI_QMM_ERR_INVALID, "out_blocks is NULL");
    hipStream_t stream = (hipStream_t)stream_;
    Staged o;
    HIP_TRY(o.out(out_blocks, nbytes, mem_space, stream));
    HIP_TRY(qmm_launch_unpack(w->layout, w->tiled, o.dev, stream));
    HIP_TRY(o.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_dequantize_f32(const izwi_qmm_weight* w, float* out, int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_dequantize_f32", [&]() -> int {
    if (!w) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    if (int rc = check_space(mem_space)) return rc;
    const QmmLayout& L = w->layout;
    size_t bytes = (size_t)L.n_stacked * L.n * L.k * sizeof(float);
    if (bytes == 0) return IZWI_QMM_OK;
    if (!out) return fail(IZWI_QMM_ERR_INVALID, "out is NULL");
    hipStream_t stream = (hipStream_t)stream_;
    Staged o;
    HIP_TRY(o.out(out, bytes, mem_space, stream));
    HIP_TRY(qmm_launch_dequant(L, w->tiled, (float*)o.dev, stream));
    HIP_TRY(o.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_dequantize_rows(const izwi_qmm_weight* w, const int32_t* row_ids, int64_t n_rows, int ids_mem_space,
                             void* out, int out_dtype, int out_mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_dequantize_rows", [&]() -> int {
    if (!w) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    if (int rc = check_space(ids_mem_space)) return rc;
    if (int rc = check_space(out_mem_space)) return rc;
    if (out_dtype != IZWI_QMM_OUT_F32 && out_dtype != IZWI_QMM_OUT_BF16)
        return fail(IZWI_QMM_ERR_INVALID, "out_dtype %d is neither f32 nor bf16", out_dtype);
    if (n_rows < 0 || n_rows > 0x7fffffff) return fail(IZWI_QMM_ERR_INVALID, "n_rows = %lld is out of range", (long long)n_rows);
    const QmmLayout& L = w->layout;
    if (n_rows == 0 || L.k == 0) return IZWI_QMM_OK;
    if (!row_ids || !out) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    if (ids_mem_space == IZWI_QMM_HOST) // the reference's index_select refuses such an id; ids in device memory are not read here
        for (int64_t i = 0; i < n_rows; i++)
            if (row_ids[i] < 0 || row_ids[i] >= L.n)
                return fail(IZWI_QMM_ERR_INVALID, "row id %d at position %lld is out of range for %lld rows", row_ids[i],
                            (long long)i, (long long)L.n);
    int device = 0;
    if (int rc = current_device(&device)) return rc;
    if (device != w->device) return fail(IZWI_QMM_ERR_INVALID, "weight lives on device %d, current device is %d", w->device, device);
    hipStream_t stream = (hipStream_t)stream_;
    Staged ids, o;
    HIP_TRY(ids.in(row_ids, (size_t)n_rows * sizeof(int32_t), ids_mem_space, stream));
    HIP_TRY(o.out(out, (size_t)n_rows * L.k * (out_dtype == IZWI_QMM_OUT_BF16 ? 2 : 4), out_mem_space, stream));
    HIP_TRY(qmm_launch_dequant_rows(L, w->tiled, (const int32_t*)ids.dev, n_rows, o.dev, out_dtype == IZWI_QMM_OUT_BF16, stream));
    HIP_TRY(o.finish(stream));
    if (ids.owned) HIP_TRY(hipStreamSynchronize(stream)); // the staged ids are freed on return
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_quantize_activations(int ggml_weight_dtype, const float* x, int64_t m, int64_t k,
                                  void* out_blocks, int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_quantize_activations", [&]() -> int {
    if (!type_supported(ggml_weight_dtype))
        return fail(IZWI_QMM_ERR_UNSUPPORTED, "ggml dtype %d is not supported", ggml_weight_dtype);
    if (int rc = check_space(mem_space)) return rc;
    if (m < 0 || k < 0) return fail(IZWI_QMM_ERR_INVALID, "negative shape");
    const int bs = ggml_weight_dtype == IZWI_QMM_Q8_0 ? 32 : 256;
    const int ts = ggml_weight_dtype == IZWI_QMM_Q8_0 ? 34 : 292;
    if (k % bs) return fail(IZWI_QMM_ERR_INVALID, "k = %lld is not a multiple of %d", (long long)k, bs);
    if (m == 0 || k == 0) return IZWI_QMM_OK;
    if (!x || !out_blocks) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    int device = 0;
    if (int rc = current_device(&device)) return rc;
    if (int rc = ensure_device(device, nullptr)) return rc;
    hipStream_t stream = (hipStream_t)stream_;
    Staged xi, o;
    HIP_TRY(xi.in(x, (size_t)m * k * sizeof(float), mem_space, stream));
    HIP_TRY(o.out(out_blocks, (size_t)m * (k / bs) * ts, mem_space, stream));
    HIP_TRY(qmm_launch_quantize_activations(ggml_weight_dtype, (const float*)xi.dev, m, k, o.dev, stream));
    HIP_TRY(o.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_quantize_weights_f32(int ggml_dtype, const float* w, int64_t n, int64_t k, void* out_blocks,
                                  int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_quantize_weights_f32", [&]() -> int {
    if (ggml_dtype != IZWI_QMM_Q8_0 && ggml_dtype != IZWI_QMM_Q4_K)
        return fail(IZWI_QMM_ERR_UNSUPPORTED, "quantize to ggml dtype %d (Q8_0 and Q4_K are built)", ggml_dtype);
    if (int rc = check_space(mem_space)) return rc;
    if (n < 0 || k < 0) return fail(IZWI_QMM_ERR_INVALID, "negative shape");
    const int bs = ggml_dtype == IZWI_QMM_Q8_0 ? 32 : 256;
    const int ts = ggml_dtype == IZWI_QMM_Q8_0 ? 34 : 144;
    if (k % bs) return fail(IZWI_QMM_ERR_INVALID, "k = %lld is not a multiple of the block size %d", (long long)k, bs);
    if (n == 0 || k == 0) return IZWI_QMM_OK;
    if (!w || !out_blocks) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    if (n > 0x7fffffffffffLL / k) return fail(IZWI_QMM_ERR_UNSUPPORTED, "tensor too large");
    int device = 0;
    if (int rc = current_device(&device)) return rc;
    if (int rc = ensure_device(device, nullptr)) return rc;
    hipStream_t stream = (hipStream_t)stream_;
    Staged wi, o;
    HIP_TRY(wi.in(w, (size_t)n * k * sizeof(float), mem_space, stream));
    HIP_TRY(o.out(out_blocks, (size_t)n * (k / bs) * ts, mem_space, stream));
    if (ggml_dtype == IZWI_QMM_Q8_0) // BlockQ8_0::from_float row by row: the activation quantizer's blocks
        HIP_TRY(qmm_launch_quantize_activations(IZWI_QMM_Q8_0, (const float*)wi.dev, n, k, o.dev, stream));
    else
        HIP_TRY(qmm_launch_quantize_q4k_weights((const float*)wi.dev, n * (k / 256), o.dev, stream));
    HIP_TRY(o.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_forward_f32(const izwi_qmm_weight* w, const float* x, int64_t m, float* y,
                         int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_forward_f32", [&]() -> int {
    QmmCallScope call;
    if (!w) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    if (int rc = check_space(mem_space)) return rc;
    const QmmLayout& L = w->layout;
    if (L.n_stacked != 1)
        return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack: use izwi_moe_forward_f32");
    if (m < 0) return fail(IZWI_QMM_ERR_INVALID, "negative m");
    if (m == 0 || L.n == 0) return IZWI_QMM_OK;
    if (!x) return fail(IZWI_QMM_ERR_INVALID, "x is NULL");
    if (!y) return fail(IZWI_QMM_ERR_INVALID, "y is NULL");
    hipStream_t stream = (hipStream_t)stream_;
    ProfileScope prof(w, stream);
    Staged xi, yo;
    HIP_TRY(xi.in(x, (size_t)m * L.k * sizeof(float), mem_space, stream));
    HIP_TRY(yo.out(y, (size_t)m * L.n * sizeof(float), mem_space, stream));
    if (m < mfma_min_m(L.k)) {
        HIP_TRY(qmm_launch_gemv(L, w->tiled, (const float*)xi.dev, m, (float*)yo.dev, w->n_cus, stream));
    } else if (m <= 64 || large_m_mode() == IZWI_QMM_LARGE_M_INT8) {
        // more than 64 rows in the integer arithmetic: 64 at a time, the records of one chunk
        // are overwritten by the next chunk's quantizer, which the stream runs behind its reader
        void* scratch = nullptr;
        HIP_TRY(get_scratch(w->device, stream, qmm_gemv_mfma_workspace_bytes(L, m < 64 ? m : 64), &scratch));
        for (int64_t r0 = 0; r0 < m; r0 += 64) {
            const int64_t rows = m - r0 < 64 ? m - r0 : 64;
            const float* xr = (const float*)xi.dev + r0 * L.k;
            float* yr = (float*)yo.dev + r0 * L.n;
            if (rows < mfma_min_m(L.k))
                HIP_TRY(qmm_launch_gemv(L, w->tiled, xr, rows, yr, w->n_cus, stream));
            else
                HIP_TRY(qmm_launch_gemv_mfma(L, w->tiled, xr, rows, yr, scratch, w->n_cus, stream));
        }
    } else {
        // prefill-sized m with f32 activations: convert once, then the MFMA kernel
        // scratch: [bf16 copy of x | split-k partial tiles]
        const size_t xb_bytes = (((size_t)m * L.k * sizeof(uint16_t)) + 255) & ~(size_t)255;
        const size_t ws_bytes = qmm_gemm_workspace_bytes(L, m, w->n_cus);
        void* xb = nullptr;
        HIP_TRY(get_scratch(w->device, stream, xb_bytes + ws_bytes, &xb));
        hipError_t e = qmm_launch_f32_to_bf16((const float*)xi.dev, (uint16_t*)xb, m * L.k, stream);
        if (e == hipSuccess)
            e = qmm_launch_gemm_bf16(L, w->tiled, (const uint16_t*)xb, m, yo.dev, 0,
                                     ws_bytes ? (uint8_t*)xb + xb_bytes : nullptr, w->n_cus, stream);
        if (e != hipSuccess) return fail_hip(e, "prefill kernel");
    }
    HIP_TRY(yo.finish(stream));
    return IZWI_QMM_OK;
    });
}

uint64_t izwi_qmm_records_bytes(int ggml_weight_dtype, int64_t m, int64_t k) {
    if (!type_supported(ggml_weight_dtype) || m < 0 || k < 0) return 0;
    return (uint64_t)qmm_records_bytes(ggml_weight_dtype, m, k);
}

namespace {
int records_args(int dtype, int64_t m, int64_t k, const void* a, const void* b) {
    if (!type_supported(dtype)) return fail(IZWI_QMM_ERR_UNSUPPORTED, "ggml dtype %d is not supported", dtype);
    const int bs = dtype == IZWI_QMM_Q8_0 ? 32 : 256;
    if (m < 0 || k <= 0 || k % bs) return fail(IZWI_QMM_ERR_INVALID, "bad shape [%lld, %lld] for block size %d", (long long)m, (long long)k, bs);
    if (m > 0 && (!a || !b)) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    int device = 0;
    if (int rc = current_device(&device)) return rc;
    return ensure_device(device, nullptr);
}
} // namespace

int izwi_qmm_quantize_records_f32(int ggml_weight_dtype, const float* x, int64_t m, int64_t k, void* records, void* stream) {
    return qmm_guarded("izwi_qmm_quantize_records_f32", [&]() -> int {
    if (int rc = records_args(ggml_weight_dtype, m, k, x, records)) return rc;
    if (m == 0) return IZWI_QMM_OK;
    HIP_TRY(qmm_launch_quantize_ws(ggml_weight_dtype, x, m, k, records, (hipStream_t)stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_silu_mul_quantize_records_f32(int ggml_weight_dtype, const float* gate, const float* up, int64_t m, int64_t k,
                                           void* records, void* stream) {
    return qmm_guarded("izwi_qmm_silu_mul_quantize_records_f32", [&]() -> int {
    if (int rc = records_args(ggml_weight_dtype, m, k, gate, records)) return rc;
    if (m == 0) return IZWI_QMM_OK;
    if (!up) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    if (profiling()) g_silu_fused.fetch_add(1, std::memory_order_relaxed);
    HIP_TRY(qmm_launch_quantize_silu_mul_ws(ggml_weight_dtype, gate, up, m, k, records, (hipStream_t)stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_forward_group_records_f32(const izwi_qmm_weight* const* weights, int32_t n_weights, const void* records,
                                       int64_t m, float* const* ys, void* stream_) {
    return qmm_guarded("izwi_qmm_forward_group_records_f32", [&]() -> int {
    if (!weights || !ys) return fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    if (n_weights < 1 || n_weights > QMM_MAX_GROUP)
        return fail(IZWI_QMM_ERR_INVALID, "projection group of %d weights (1..%d supported)", n_weights, QMM_MAX_GROUP);
    if (m < 3 || m > 64)
        return fail(IZWI_QMM_ERR_UNSUPPORTED, "records are the input of the batched decode kernels (3 <= m <= 64), got m = %lld",
                    (long long)m);
    if (!records) return fail(IZWI_QMM_ERR_INVALID, "records is NULL");
    const bool q8k = weights[0] && weights[0]->layout.dtype != IZWI_QMM_Q8_0;
    for (int i = 0; i < n_weights; i++) {
        if (!weights[i] || !ys[i]) return fail(IZWI_QMM_ERR_INVALID, "NULL weight or output");
        const QmmLayout& L = weights[i]->layout;
        if (L.n_stacked != 1 || L.n == 0) return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack or an empty weight");
        if (L.k != weights[0]->layout.k)
            return fail(IZWI_QMM_ERR_INVALID, "projection group input mismatch: expected %lld, got %lld",
                        (long long)weights[0]->layout.k, (long long)L.k);
        if ((L.dtype != IZWI_QMM_Q8_0) != q8k)
            return fail(IZWI_QMM_ERR_INVALID, "the group mixes weights that dot against Q8_0 and against Q8_K records");
        if (weights[i]->device != weights[0]->device) return fail(IZWI_QMM_ERR_INVALID, "weights on different devices");
    }
    int device = 0;
    if (int rc = current_device(&device)) return rc;
    if (device != weights[0]->device)
        return fail(IZWI_QMM_ERR_INVALID, "the weights live on device %d, the current device is %d", weights[0]->device, device);
    hipStream_t stream = (hipStream_t)stream_;
    // one launch per block type (Q4_K and Q6_K members read the same Q8_K records)
    bool done[QMM_MAX_GROUP] = {};
    for (int i = 0; i < n_weights; i++) {
        if (done[i]) continue;
        const izwi_qmm_weight* sub_w[QMM_MAX_GROUP];
        float* sub_y[QMM_MAX_GROUP];
        int n_sub = 0;
        for (int j = i; j < n_weights; j++)
            if (!done[j] && weights[j]->layout.dtype == weights[i]->layout.dtype)
                sub_w[n_sub] = weights[j], sub_y[n_sub] = ys[j], n_sub++, done[j] = true;
        if (int rc = batched_group_on_records(sub_w, n_sub, nullptr, m, sub_y, const_cast<void*>(records), stream)) return rc;
    }
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_forward_rows_f32(const izwi_qmm_weight* w, const uint32_t* row_ids, int64_t n_rows, const float* x,
                              int64_t m, float* y, int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_forward_rows_f32", [&]() -> int {
    QmmCallScope call;
    if (!w) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    if (int rc = check_space(mem_space)) return rc;
    const QmmLayout& L = w->layout;
    if (L.n_stacked != 1) return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack");
    if (m < 0 || n_rows < 0) return fail(IZWI_QMM_ERR_INVALID, "negative m or row count");
    if (m > 2)
        return fail(IZWI_QMM_ERR_UNSUPPORTED,
                    "Qwen3 selected-token logits expected one hidden state ([1,vocab] or [1,1,vocab] logits), "
                    "got %lld rows (at most 2 are supported)", (long long)m);
    if (m == 0 || n_rows == 0) return IZWI_QMM_OK; // `logits_for_tokens` of an empty id list is empty
    if (n_rows > (1 << 24)) return fail(IZWI_QMM_ERR_UNSUPPORTED, "too many selected rows (%lld)", (long long)n_rows);
    if (!row_ids || !x || !y) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    if (L.n == 0) return fail(IZWI_QMM_ERR_INVALID, "row index out of range: the weight has no rows");
    if (mem_space == IZWI_QMM_HOST) // `index_select` refuses an index beyond the dimension
        for (int64_t i = 0; i < n_rows; i++)
            if ((int64_t)row_ids[i] >= L.n)
                return fail(IZWI_QMM_ERR_INVALID, "row index %u out of range for a weight of %lld rows", row_ids[i],
                            (long long)L.n);
    hipStream_t stream = (hipStream_t)stream_;
    ProfileScope prof(w, stream);
    Staged xi, ii, yo;
    HIP_TRY(xi.in(x, (size_t)m * L.k * sizeof(float), mem_space, stream));
    HIP_TRY(ii.in(row_ids, (size_t)n_rows * sizeof(uint32_t), mem_space, stream));
    HIP_TRY(yo.out(y, (size_t)m * n_rows * sizeof(float), mem_space, stream));
    void* scratch = nullptr;
    HIP_TRY(get_scratch(w->device, stream, qmm_gemv_rows_workspace_bytes(m, n_rows), &scratch));
    HIP_TRY(qmm_launch_gemv_rows(L, w->tiled, (const float*)xi.dev, m, (const uint32_t*)ii.dev, n_rows, (float*)yo.dev,
                                 scratch, w->n_cus, stream));
    HIP_TRY(yo.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_forward_f32_noalloc(const izwi_qmm_weight* w, const float* x, int64_t m, float* y, void* stream_) {
    return qmm_guarded("izwi_qmm_forward_f32_noalloc", [&]() -> int {
    if (!w) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    const QmmLayout& L = w->layout;
    if (L.n_stacked != 1) return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack");
    if (m < 0) return fail(IZWI_QMM_ERR_INVALID, "negative m");
    if (m > 64)
        return fail(IZWI_QMM_ERR_UNSUPPORTED, "izwi_qmm_forward_f32_noalloc takes at most 64 rows, got %lld",
                    (long long)m);
    if (m == 0 || L.n == 0) return IZWI_QMM_OK;
    if (!x || !y) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    hipStream_t stream = (hipStream_t)stream_;
    int device = 0;
    if (int rc = current_device(&device)) return rc;
    if (device != w->device) // (before any launch: the one- and two-row kernel too runs on the weight's pointers)
        return fail(IZWI_QMM_ERR_INVALID, "the weight lives on device %d, the current device is %d", w->device, device);
    if (m < mfma_min_m(L.k)) { // a few rows: the single-launch kernel has no scratch at all
        HIP_TRY(qmm_launch_gemv(L, w->tiled, x, m, y, w->n_cus, stream));
        return IZWI_QMM_OK;
    }
    const size_t need = qmm_gemv_mfma_workspace_bytes(L, m);
    if (need > (size_t)IZWI_QMM_NOALLOC_SCRATCH_BYTES)
        return fail(IZWI_QMM_ERR_UNSUPPORTED,
                    "m = %lld rows of k = %lld need %zu bytes of activation records; the static scratch of "
                    "izwi_qmm_forward_f32_noalloc holds %d",
                    (long long)m, (long long)L.k, need, IZWI_QMM_NOALLOC_SCRATCH_BYTES);
    void* scratch = nullptr;
    HIP_TRY(noalloc_scratch_ptr(device, &scratch));
    // the quantizer writes every record the matmul reads (whole 16-row tiles, rows beyond m as
    // zeros), so nothing of an earlier call's contents is ever read
    HIP_TRY(qmm_launch_gemv_mfma(L, w->tiled, x, m, y, scratch, w->n_cus, stream));
    return IZWI_QMM_OK;
    });
}

} // extern "C"

namespace {

// Scratch a forward call on layout L with m rows may take from the start of the per-stream buffer
// (quantized activations, or the bf16 copy and the split-k partial tiles): callers that keep data
// of their own in the same buffer place it behind this many bytes.
size_t forward_scratch_need(const QmmLayout& L, int64_t m, int n_cus) {
    const size_t a = qmm_gemv_mfma_workspace_bytes(L, m);
    const size_t b = ((((size_t)m * L.k * sizeof(uint16_t)) + 255) & ~(size_t)255) + qmm_gemm_workspace_bytes(L, m, n_cus);
    return ((a > b ? a : b) + 255) & ~(size_t)255;
}

// rms_norm(x) * norm_weight into the per-stream scratch, behind `keep_free` bytes
int normed_copy(const izwi_qmm_weight* w, const float* x_dev, int64_t m, const float* norm_weight, float eps,
                size_t keep_free, size_t extra_behind, hipStream_t stream, float** out) {
    void* scratch = nullptr;
    const size_t bytes = (size_t)m * w->layout.k * sizeof(float);
    HIP_TRY(get_scratch(w->device, stream, keep_free + ((bytes + 255) & ~(size_t)255) + extra_behind, &scratch));
    float* normed = reinterpret_cast<float*>(static_cast<uint8_t*>(scratch) + keep_free);
    if (int rc = izwi_rms_norm_f32(x_dev, norm_weight, m, w->layout.k, eps, normed, IZWI_QMM_DEVICE, stream)) return rc;
    *out = normed;
    return IZWI_QMM_OK;
}

int forward_group_impl(const izwi_qmm_weight* const* weights, int32_t n_weights, const float* x, int64_t m,
                       float* const* ys, int mem_space, void* stream_, const float* norm_weight, float norm_eps);

} // namespace

extern "C" {

int izwi_qmm_forward_group_f32(const izwi_qmm_weight* const* weights, int32_t n_weights,
                               const float* x, int64_t m, float* const* ys, int mem_space,
                               void* stream_) {
    return qmm_guarded("izwi_qmm_forward_group_f32", [&]() -> int {
    return forward_group_impl(weights, n_weights, x, m, ys, mem_space, stream_, nullptr, 0.0f);
    });
}

int izwi_qmm_forward_group_normed_f32(const izwi_qmm_weight* const* weights, int32_t n_weights, const float* x,
                                      int64_t m, const float* norm_weight, float eps, float* const* ys,
                                      int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_forward_group_normed_f32", [&]() -> int {
    if (!norm_weight) return fail(IZWI_QMM_ERR_INVALID, "norm_weight is NULL");
    return forward_group_impl(weights, n_weights, x, m, ys, mem_space, stream_, norm_weight, eps);
    });
}

} // extern "C"

namespace {

int batched_group_on_records(const izwi_qmm_weight* const* weights, int32_t n_weights, const float* x, int64_t m,
                             float* const* ys, void* records, hipStream_t stream);

int forward_group_impl(const izwi_qmm_weight* const* weights, int32_t n_weights, const float* x, int64_t m,
                       float* const* ys, int mem_space, void* stream_, const float* norm_weight, float norm_eps) {
    QmmCallScope call;
    if (!weights || !ys) return fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    if (n_weights < 1 || n_weights > QMM_MAX_GROUP)
        return fail(IZWI_QMM_ERR_INVALID, "projection group of %d weights (1..%d supported)", n_weights, QMM_MAX_GROUP);
    if (int rc = check_space(mem_space)) return rc;
    bool uniform = true, splittable = true;
    for (int i = 0; i < n_weights; i++) {
        if (!weights[i]) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
        const QmmLayout& L = weights[i]->layout;
        if (L.n_stacked != 1) return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack");
        if (L.k != weights[0]->layout.k)
            return fail(IZWI_QMM_ERR_INVALID, "projection group input mismatch: expected %lld, got %lld",
                        (long long)weights[0]->layout.k, (long long)L.k);
        if (L.dtype != weights[0]->layout.dtype || L.n == 0 || weights[i]->device != weights[0]->device)
            uniform = false;
        if (L.n == 0 || weights[i]->device != weights[0]->device) splittable = false;
        if (m > 0 && L.n > 0 && !ys[i]) return fail(IZWI_QMM_ERR_INVALID, "y is NULL");
    }
    if (m < 0) return fail(IZWI_QMM_ERR_INVALID, "negative m");
    if (m == 0) return IZWI_QMM_OK;
    if (!x) return fail(IZWI_QMM_ERR_INVALID, "x is NULL");
    // Several block types in one group (a Q4_K_M file keeps attn_v of some layers in Q6_K beside Q4_K
    // attn_q / attn_k): one group call per type, in the order of each type's first member
    const bool by_type = mem_space == IZWI_QMM_DEVICE && !uniform && splittable && n_weights >= 2 && m <= 64;
    auto call_by_type = [&](const float* xin, const float* nw) -> int {
        bool done[QMM_MAX_GROUP] = {};
        // batched sizes: Q4_K and Q6_K weights dot against the same Q8_K records, quantized once
        bool q8k_records = !nw && m >= mfma_min_m(weights[0]->layout.k);
        for (int i = 0; i < n_weights; i++)
            if (weights[i]->layout.dtype != IZWI_QMM_Q4_K && weights[i]->layout.dtype != IZWI_QMM_Q6_K) q8k_records = false;
        void* records = nullptr;
        if (q8k_records) {
            hipStream_t stream = (hipStream_t)stream_;
            HIP_TRY(get_scratch(weights[0]->device, stream, qmm_gemv_mfma_workspace_bytes(weights[0]->layout, m), &records));
            HIP_TRY(qmm_launch_quantize_ws(IZWI_QMM_Q4_K, xin, m, weights[0]->layout.k, records, stream));
        }
        for (int i = 0; i < n_weights; i++) {
            if (done[i]) continue;
            const izwi_qmm_weight* sub_w[QMM_MAX_GROUP];
            float* sub_y[QMM_MAX_GROUP];
            int n_sub = 0;
            for (int j = i; j < n_weights; j++)
                if (!done[j] && weights[j]->layout.dtype == weights[i]->layout.dtype)
                    sub_w[n_sub] = weights[j], sub_y[n_sub] = ys[j], n_sub++, done[j] = true;
            if (records) {
                if (int rc = batched_group_on_records(sub_w, n_sub, xin, m, sub_y, records, (hipStream_t)stream_)) return rc;
            } else if (int rc = forward_group_impl(sub_w, n_sub, xin, m, sub_y, mem_space, stream_, nw, norm_eps)) {
                return rc;
            }
        }
        return IZWI_QMM_OK;
    };
    if (norm_weight) {
        hipStream_t stream = (hipStream_t)stream_;
        const izwi_qmm_weight* w0 = weights[0];
        // each type's launch normalizes for itself: x is read by every workgroup anyway
        if (by_type && m <= 2 && m < mfma_min_m(weights[0]->layout.k)) return call_by_type(x, norm_weight);
        // one launch: the decode kernel normalizes while it quantizes (device buffers, one block type, m <= 2)
        if (mem_space == IZWI_QMM_DEVICE && uniform && m <= 2 && m < mfma_min_m(w0->layout.k)) {
            const QmmLayout* layouts[QMM_MAX_GROUP];
            const void* tiled[QMM_MAX_GROUP];
            for (int i = 0; i < n_weights; i++) layouts[i] = &weights[i]->layout, tiled[i] = weights[i]->tiled;
            const QmmNorm norm{norm_weight, norm_eps};
            ProfileScope prof(w0, stream);
            hipError_t e = qmm_launch_gemv_multi(layouts, tiled, n_weights, x, m, ys, w0->n_cus, stream, &norm);
            if (e == hipSuccess) return IZWI_QMM_OK;
            if (e != hipErrorNotSupported) return fail_hip(e, "grouped decode kernel");
            (void)hipGetLastError();
        }
        // otherwise: the normalized activations into scratch (behind what the projections use of it),
        // then the plain group call
        Staged xi, wi, yo[QMM_MAX_GROUP];
        HIP_TRY(xi.in(x, (size_t)m * w0->layout.k * sizeof(float), mem_space, stream));
        HIP_TRY(wi.in(norm_weight, (size_t)w0->layout.k * sizeof(float), mem_space, stream));
        float* ydev[QMM_MAX_GROUP];
        size_t keep = 0;
        for (int i = 0; i < n_weights; i++) {
            HIP_TRY(yo[i].out(ys[i], (size_t)m * weights[i]->layout.n * sizeof(float), mem_space, stream));
            ydev[i] = (float*)yo[i].dev;
            keep = std::max(keep, forward_scratch_need(weights[i]->layout, m, weights[i]->n_cus));
        }
        float* normed = nullptr;
        if (int rc = normed_copy(w0, (const float*)xi.dev, m, (const float*)wi.dev, norm_eps, keep, 0, stream, &normed)) return rc;
        if (int rc = forward_group_impl(weights, n_weights, normed, m, ydev, IZWI_QMM_DEVICE, stream_, nullptr, 0.0f)) return rc;
        for (int i = 0; i < n_weights; i++) HIP_TRY(yo[i].finish(stream));
        return IZWI_QMM_OK;
    }
    if (by_type) return call_by_type(x, nullptr);
    // prefill sizes on the bf16 matrix cores: the activations are converted once and the members
    // share one launch (its grid is the members' column tiles one after the other)
    if (mem_space == IZWI_QMM_DEVICE && uniform && n_weights >= 2 && m > 128 && large_m_mode() == IZWI_QMM_LARGE_M_BF16) {
        hipStream_t stream = (hipStream_t)stream_;
        const izwi_qmm_weight* w0 = weights[0];
        const QmmLayout* layouts[QMM_MAX_GROUP];
        const void* tiled[QMM_MAX_GROUP];
        void* outs[QMM_MAX_GROUP];
        for (int i = 0; i < n_weights; i++) layouts[i] = &weights[i]->layout, tiled[i] = weights[i]->tiled, outs[i] = ys[i];
        const size_t xb_bytes = (((size_t)m * w0->layout.k * sizeof(uint16_t)) + 255) & ~(size_t)255;
        const size_t ws_bytes = qmm_gemm_group_workspace_bytes(layouts, n_weights, m, w0->n_cus);
        void* xb = nullptr;
        HIP_TRY(get_scratch(w0->device, stream, xb_bytes + ws_bytes, &xb));
        ProfileScope prof(w0, stream);
        HIP_TRY(qmm_launch_f32_to_bf16(x, (uint16_t*)xb, m * w0->layout.k, stream));
        hipError_t e = qmm_launch_gemm_bf16_multi(layouts, tiled, n_weights, (const uint16_t*)xb, m, outs, 0,
                                                  ws_bytes ? (uint8_t*)xb + xb_bytes : nullptr, w0->n_cus, stream);
        if (e == hipSuccess) return IZWI_QMM_OK;
        if (e != hipErrorNotSupported) return fail_hip(e, "grouped prefill kernel");
        (void)hipGetLastError();
    }
    // host buffers, mixed types, prefill sizes: one call per projection (same results)
    if (mem_space != IZWI_QMM_DEVICE || !uniform || n_weights == 1 || m > 64) {
        for (int i = 0; i < n_weights; i++)
            if (int rc = izwi_qmm_forward_f32(weights[i], x, m, ys[i], mem_space, stream_)) return rc;
        return IZWI_QMM_OK;
    }
    hipStream_t stream = (hipStream_t)stream_;
    const izwi_qmm_weight* w0 = weights[0];
    if (m < mfma_min_m(w0->layout.k)) {
        const QmmLayout* layouts[QMM_MAX_GROUP];
        const void* tiled[QMM_MAX_GROUP];
        for (int i = 0; i < n_weights; i++) layouts[i] = &weights[i]->layout, tiled[i] = weights[i]->tiled;
        // one launch for up to four rows (one pass of the kernel); more rows on this kernel (threshold
        // raised through the environment) go projection by projection
        if (m <= 4) {
            ProfileScope prof(w0, stream);
            hipError_t e = qmm_launch_gemv_multi(layouts, tiled, n_weights, x, m, ys, w0->n_cus, stream);
            if (e == hipSuccess) return IZWI_QMM_OK;
            if (e != hipErrorNotSupported) return fail_hip(e, "grouped decode kernel");
            (void)hipGetLastError();
        }
        for (int i = 0; i < n_weights; i++)
            if (int rc = izwi_qmm_forward_f32(weights[i], x, m, ys[i], mem_space, stream_)) return rc;
        return IZWI_QMM_OK;
    }
    // 3 <= m <= 64: the activations are quantized once, every projection reads the same records
    // (up to 16 rows in one launch for all of them)
    void* scratch = nullptr;
    HIP_TRY(get_scratch(w0->device, stream, qmm_gemv_mfma_workspace_bytes(w0->layout, m), &scratch));
    HIP_TRY(qmm_launch_quantize_ws(w0->layout.dtype, x, m, w0->layout.k, scratch, stream));
    return batched_group_on_records(weights, n_weights, x, m, ys, scratch, stream);
}

// The batched decode kernel for a group of one block type whose quantized activations are in `records`.
int batched_group_on_records(const izwi_qmm_weight* const* weights, int32_t n_weights, const float* x, int64_t m,
                             float* const* ys, void* records, hipStream_t stream) {
    const izwi_qmm_weight* w0 = weights[0];
    if (n_weights > 1) {
        const QmmLayout* layouts[QMM_MAX_GROUP];
        const void* tiled[QMM_MAX_GROUP];
        for (int i = 0; i < n_weights; i++) layouts[i] = &weights[i]->layout, tiled[i] = weights[i]->tiled;
        ProfileScope prof(w0, stream);
        hipError_t e = qmm_launch_gemv_mfma_multi(layouts, tiled, n_weights, m, ys, records, w0->n_cus, stream);
        if (e == hipSuccess) return IZWI_QMM_OK;
        if (e != hipErrorNotSupported) return fail_hip(e, "grouped batched decode kernel");
        (void)hipGetLastError();
    }
    for (int i = 0; i < n_weights; i++) {
        ProfileScope prof(weights[i], stream);
        HIP_TRY(qmm_launch_gemv_mfma(weights[i]->layout, weights[i]->tiled, x, m, ys[i], records,
                                     weights[i]->n_cus, stream, false));
    }
    return IZWI_QMM_OK;
}

int gate_up_silu_impl(const izwi_qmm_weight* gate, const izwi_qmm_weight* up, const float* x, int64_t m, float* h,
                      int mem_space, void* stream_, const float* norm_weight, float norm_eps);

} // namespace

extern "C" {

int izwi_qmm_forward_gate_up_silu_f32(const izwi_qmm_weight* gate, const izwi_qmm_weight* up,
                                      const float* x, int64_t m, float* h, int mem_space,
                                      void* stream_) {
    return qmm_guarded("izwi_qmm_forward_gate_up_silu_f32", [&]() -> int {
    return gate_up_silu_impl(gate, up, x, m, h, mem_space, stream_, nullptr, 0.0f);
    });
}

int izwi_qmm_forward_gate_up_silu_normed_f32(const izwi_qmm_weight* gate, const izwi_qmm_weight* up, const float* x,
                                             int64_t m, const float* norm_weight, float eps, float* h,
                                             int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_forward_gate_up_silu_normed_f32", [&]() -> int {
    if (!norm_weight) return fail(IZWI_QMM_ERR_INVALID, "norm_weight is NULL");
    return gate_up_silu_impl(gate, up, x, m, h, mem_space, stream_, norm_weight, eps);
    });
}

int izwi_qmm_mlp_forward_f32(const izwi_qmm_weight* gate, const izwi_qmm_weight* up, const izwi_qmm_weight* down,
                             const float* x, int64_t m, float* y, int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_mlp_forward_f32", [&]() -> int {
    QmmCallScope call;
    if (!gate || !up || !down) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    if (int rc = check_space(mem_space)) return rc;
    const QmmLayout& G = gate->layout;
    const QmmLayout& U = up->layout;
    const QmmLayout& D = down->layout;
    if (G.n_stacked != 1 || U.n_stacked != 1 || D.n_stacked != 1) return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack");
    if (G.n != U.n || G.k != U.k)
        return fail(IZWI_QMM_ERR_INVALID, "gate is [%lld, %lld], up is [%lld, %lld]", (long long)G.n, (long long)G.k,
                    (long long)U.n, (long long)U.k);
    if (D.k != G.n)
        return fail(IZWI_QMM_ERR_INVALID, "shape mismatch in qmatmul, lhs: [%lld, %lld], rhs: (%lld, %lld)", (long long)m,
                    (long long)G.n, (long long)D.n, (long long)D.k);
    if (gate->device != up->device || gate->device != down->device)
        return fail(IZWI_QMM_ERR_INVALID, "the weights live on different devices");
    if (m < 0) return fail(IZWI_QMM_ERR_INVALID, "negative m");
    if (m == 0 || D.n == 0) return IZWI_QMM_OK;
    if (!x) return fail(IZWI_QMM_ERR_INVALID, "x is NULL");
    if (!y) return fail(IZWI_QMM_ERR_INVALID, "y is NULL");
    hipStream_t stream = (hipStream_t)stream_;
    Staged xi, yo;
    HIP_TRY(xi.in(x, (size_t)m * G.k * sizeof(float), mem_space, stream));
    HIP_TRY(yo.out(y, (size_t)m * D.n * sizeof(float), mem_space, stream));
    auto align256 = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t part = align256((size_t)m * G.n * sizeof(float)); // one [m, intermediate] f32 matrix
    const bool records = m >= mfma_min_m(G.k) && m >= mfma_min_m(D.k) && m <= 64 && G.dtype == U.dtype;
    if (records) {
        // Rows for the matrix-core kernels: activation records all the way.  x is quantized once for
        // gate | up (one launch for both), silu(g) * u is quantized straight into the records that
        // down reads: four launches, the intermediate never exists as an f32 matrix of its own
        // beside g and u.  The arithmetic is that of the separate calls (same quantizers, same
        // kernels), so are the bits.
        const size_t rx = align256(qmm_records_bytes(G.dtype, m, G.k)), rh = align256(qmm_records_bytes(D.dtype, m, D.k));
        uint8_t* ws = nullptr;
        HIP_TRY(get_scratch(gate->device, stream, rx + 2 * part + rh, (void**)&ws));
        float* g = reinterpret_cast<float*>(ws + rx);
        float* u = reinterpret_cast<float*>(ws + rx + part);
        uint8_t* rec_h = ws + rx + 2 * part;
        if (profiling()) g_silu_fused.fetch_add(1, std::memory_order_relaxed);
        HIP_TRY(qmm_launch_quantize_ws(G.dtype, (const float*)xi.dev, m, G.k, ws, stream));
        const izwi_qmm_weight* gu[2] = {gate, up};
        float* gu_y[2] = {g, u};
        if (int rc = batched_group_on_records(gu, 2, nullptr, m, gu_y, ws, stream)) return rc;
        HIP_TRY(qmm_launch_quantize_silu_mul_ws(D.dtype, g, u, m, D.k, rec_h, stream));
        float* dy[1] = {(float*)yo.dev};
        if (int rc = batched_group_on_records(&down, 1, nullptr, m, dy, rec_h, stream)) return rc;
    } else {
        // One or two rows (the activation is applied inside the gate | up launch), prefill sizes and
        // a gate / up pair of two block types: the two calls, with the intermediate in the stream's
        // scratch behind everything those calls use of it themselves.
        const size_t gu_need = forward_scratch_need(G, m, gate->n_cus) + align256((size_t)m * G.k * sizeof(float)) + 2 * part + 1024;
        const size_t d_need = forward_scratch_need(D, m, down->n_cus);
        const size_t inner = align256(gu_need > d_need ? gu_need : d_need);
        uint8_t* ws = nullptr;
        HIP_TRY(get_scratch(gate->device, stream, inner + part, (void**)&ws));
        float* h = reinterpret_cast<float*>(ws + inner);
        if (int rc = gate_up_silu_impl(gate, up, (const float*)xi.dev, m, h, IZWI_QMM_DEVICE, stream_, nullptr, 0.0f)) return rc;
        if (int rc = izwi_qmm_forward_f32(down, h, m, (float*)yo.dev, IZWI_QMM_DEVICE, stream_)) return rc;
    }
    HIP_TRY(yo.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_forward_normed_f32(const izwi_qmm_weight* w, const float* x, int64_t m, const float* norm_weight,
                                float eps, float* y, int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_forward_normed_f32", [&]() -> int {
    QmmCallScope call;
    if (!w) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    if (!norm_weight) return fail(IZWI_QMM_ERR_INVALID, "norm_weight is NULL");
    if (int rc = check_space(mem_space)) return rc;
    const QmmLayout& L = w->layout;
    if (L.n_stacked != 1) return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack");
    if (m < 0) return fail(IZWI_QMM_ERR_INVALID, "negative m");
    if (m == 0 || L.n == 0) return IZWI_QMM_OK;
    if (!x || !y) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    hipStream_t stream = (hipStream_t)stream_;
    if (mem_space == IZWI_QMM_DEVICE && m <= 2 && m < mfma_min_m(L.k)) {
        const QmmNorm norm{norm_weight, eps};
        ProfileScope prof(w, stream);
        hipError_t e = qmm_launch_gemv(L, w->tiled, x, m, y, w->n_cus, stream, nullptr, &norm);
        if (e == hipSuccess) return IZWI_QMM_OK;
        if (e != hipErrorNotSupported) return fail_hip(e, "decode kernel");
        (void)hipGetLastError();
    }
    Staged xi, wi, yo;
    HIP_TRY(xi.in(x, (size_t)m * L.k * sizeof(float), mem_space, stream));
    HIP_TRY(wi.in(norm_weight, (size_t)L.k * sizeof(float), mem_space, stream));
    HIP_TRY(yo.out(y, (size_t)m * L.n * sizeof(float), mem_space, stream));
    float* normed = nullptr;
    if (int rc = normed_copy(w, (const float*)xi.dev, m, (const float*)wi.dev, eps, forward_scratch_need(L, m, w->n_cus), 0,
                             stream, &normed))
        return rc;
    if (int rc = izwi_qmm_forward_f32(w, normed, m, (float*)yo.dev, IZWI_QMM_DEVICE, stream_)) return rc;
    HIP_TRY(yo.finish(stream));
    return IZWI_QMM_OK;
    });
}

} // extern "C"

namespace {

int gate_up_silu_impl(const izwi_qmm_weight* gate, const izwi_qmm_weight* up, const float* x, int64_t m, float* h,
                      int mem_space, void* stream_, const float* norm_weight, float norm_eps) {
    QmmCallScope call;
    if (!gate || !up) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    if (int rc = check_space(mem_space)) return rc;
    const QmmLayout& L = gate->layout;
    const QmmLayout& U = up->layout;
    if (L.n_stacked != 1 || U.n_stacked != 1) return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack");
    if (L.n != U.n || L.k != U.k)
        return fail(IZWI_QMM_ERR_INVALID, "gate is [%lld, %lld], up is [%lld, %lld]", (long long)L.n, (long long)L.k,
                    (long long)U.n, (long long)U.k);
    if (L.dtype != U.dtype) return fail(IZWI_QMM_ERR_INVALID, "gate and up have different ggml dtypes (%d, %d)", L.dtype, U.dtype);
    if (gate->device != up->device) return fail(IZWI_QMM_ERR_INVALID, "gate and up live on different devices");
    if (m < 0) return fail(IZWI_QMM_ERR_INVALID, "negative m");
    if (m == 0 || L.n == 0) return IZWI_QMM_OK;
    if (!x) return fail(IZWI_QMM_ERR_INVALID, "x is NULL");
    if (!h) return fail(IZWI_QMM_ERR_INVALID, "h is NULL");
    hipStream_t stream = (hipStream_t)stream_;
    Staged xi, ho;
    HIP_TRY(xi.in(x, (size_t)m * L.k * sizeof(float), mem_space, stream));
    HIP_TRY(ho.out(h, (size_t)m * L.n * sizeof(float), mem_space, stream));
    if (profiling()) g_silu_fused.fetch_add(1, std::memory_order_relaxed);
    Staged wi;
    if (norm_weight) HIP_TRY(wi.in(norm_weight, (size_t)L.k * sizeof(float), mem_space, stream));
    const float* xin = (const float*)xi.dev;
    if (m < mfma_min_m(L.k) && m <= 2) {
        const QmmNorm norm{(const float*)wi.dev, norm_eps};
        ProfileScope prof(gate, stream);
        HIP_TRY(qmm_launch_gemv_gated(L, gate->tiled, up->tiled, xin, m, (float*)ho.dev, gate->n_cus, stream,
                                      norm_weight ? &norm : nullptr));
    } else {
        size_t behind = 0; // bytes of the scratch buffer's start that hold the normalized activations
        if (norm_weight) {
            // the normalized activations first (behind what the projections use), the two outputs behind them
            const size_t keep = forward_scratch_need(L, m, gate->n_cus);
            float* normed = nullptr;
            if (int rc = normed_copy(gate, xin, m, (const float*)wi.dev, norm_eps, keep, 2 * (size_t)m * L.n * sizeof(float) + 512,
                                     stream, &normed))
                return rc;
            xin = normed;
            behind = keep + (((size_t)m * L.k * sizeof(float) + 255) & ~(size_t)255);
        }
        // both projections into scratch (one projection-group call), then the elementwise product
        const size_t part = (size_t)m * L.n * sizeof(float);
        void* gu = nullptr;
        {
            // the group call below uses the start of the same per-stream scratch for the quantized
            // activations: its own need comes first, the two outputs behind it
            const size_t group_need =
                m <= 64 ? qmm_gemv_mfma_workspace_bytes(L, m)
                        : ((((size_t)m * L.k * sizeof(uint16_t)) + 255) & ~(size_t)255) + qmm_gemm_workspace_bytes(L, m, gate->n_cus);
            const size_t base = std::max((group_need + 255) & ~(size_t)255, behind);
            void* scratch = nullptr;
            HIP_TRY(get_scratch(gate->device, stream, base + 2 * part, &scratch));
            gu = static_cast<uint8_t*>(scratch) + base;
        }
        const izwi_qmm_weight* ws[2] = {gate, up};
        float* ys[2] = {static_cast<float*>(gu), reinterpret_cast<float*>(static_cast<uint8_t*>(gu) + part)};
        if (int rc = izwi_qmm_forward_group_f32(ws, 2, xin, m, ys, IZWI_QMM_DEVICE, stream_)) return rc;
        HIP_TRY(qmm_launch_silu_mul(ys[0], ys[1], (float*)ho.dev, (int64_t)m * L.n, stream));
    }
    HIP_TRY(ho.finish(stream));
    return IZWI_QMM_OK;
}

} // namespace

extern "C" {

int izwi_qmm_forward_bf16(const izwi_qmm_weight* w, const uint16_t* x_bf16, int64_t m, void* y,
                          int out_dtype, int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_forward_bf16", [&]() -> int {
    QmmCallScope call;
    if (!w) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    if (int rc = check_space(mem_space)) return rc;
    if (out_dtype != IZWI_QMM_OUT_F32 && out_dtype != IZWI_QMM_OUT_BF16)
        return fail(IZWI_QMM_ERR_INVALID, "bad out_dtype %d", out_dtype);
    const QmmLayout& L = w->layout;
    if (L.n_stacked != 1) return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack");
    if (m < 0) return fail(IZWI_QMM_ERR_INVALID, "negative m");
    if (m == 0 || L.n == 0) return IZWI_QMM_OK;
    if (!x_bf16) return fail(IZWI_QMM_ERR_INVALID, "x is NULL");
    if (!y) return fail(IZWI_QMM_ERR_INVALID, "y is NULL");
    hipStream_t stream = (hipStream_t)stream_;
    ProfileScope prof(w, stream);
    const size_t ybytes = (size_t)m * L.n * (out_dtype == IZWI_QMM_OUT_BF16 ? 2 : 4);
    Staged xi, yo;
    HIP_TRY(xi.in(x_bf16, (size_t)m * L.k * sizeof(uint16_t), mem_space, stream));
    HIP_TRY(yo.out(y, ybytes, mem_space, stream));
    void* workspace = nullptr; // split-k partial tiles, for products with few output tiles only
    if (const size_t ws_bytes = qmm_gemm_workspace_bytes(L, m, w->n_cus))
        HIP_TRY(get_scratch(w->device, stream, ws_bytes, &workspace));
    HIP_TRY(qmm_launch_gemm_bf16(L, w->tiled, (const uint16_t*)xi.dev, m, yo.dev,
                                 out_dtype == IZWI_QMM_OUT_BF16, workspace, w->n_cus, stream));
    HIP_TRY(yo.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_forward_group_bf16(const izwi_qmm_weight* const* weights, int32_t n_weights, const uint16_t* x_bf16,
                                int64_t m, void* const* ys, int out_dtype, int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_forward_group_bf16", [&]() -> int {
    QmmCallScope call;
    if (!weights || !ys) return fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    if (n_weights < 1 || n_weights > QMM_MAX_GROUP)
        return fail(IZWI_QMM_ERR_INVALID, "projection group of %d weights (1..%d supported)", n_weights, QMM_MAX_GROUP);
    if (int rc = check_space(mem_space)) return rc;
    if (out_dtype != IZWI_QMM_OUT_F32 && out_dtype != IZWI_QMM_OUT_BF16)
        return fail(IZWI_QMM_ERR_INVALID, "bad out_dtype %d", out_dtype);
    bool uniform = true;
    for (int i = 0; i < n_weights; i++) {
        if (!weights[i]) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
        const QmmLayout& L = weights[i]->layout;
        if (L.n_stacked != 1) return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack");
        if (L.k != weights[0]->layout.k)
            return fail(IZWI_QMM_ERR_INVALID, "projection group input mismatch: expected %lld, got %lld",
                        (long long)weights[0]->layout.k, (long long)L.k);
        if (L.dtype != weights[0]->layout.dtype || L.n == 0 || weights[i]->device != weights[0]->device) uniform = false;
        if (m > 0 && L.n > 0 && !ys[i]) return fail(IZWI_QMM_ERR_INVALID, "y is NULL");
    }
    if (m < 0) return fail(IZWI_QMM_ERR_INVALID, "negative m");
    if (m == 0) return IZWI_QMM_OK;
    if (!x_bf16) return fail(IZWI_QMM_ERR_INVALID, "x is NULL");
    if (mem_space == IZWI_QMM_DEVICE && uniform && n_weights >= 2 && m > 128) {
        hipStream_t stream = (hipStream_t)stream_;
        const izwi_qmm_weight* w0 = weights[0];
        const QmmLayout* layouts[QMM_MAX_GROUP];
        const void* tiled[QMM_MAX_GROUP];
        for (int i = 0; i < n_weights; i++) layouts[i] = &weights[i]->layout, tiled[i] = weights[i]->tiled;
        void* workspace = nullptr;
        if (const size_t ws_bytes = qmm_gemm_group_workspace_bytes(layouts, n_weights, m, w0->n_cus))
            HIP_TRY(get_scratch(w0->device, stream, ws_bytes, &workspace));
        ProfileScope prof(w0, stream);
        hipError_t e = qmm_launch_gemm_bf16_multi(layouts, tiled, n_weights, x_bf16, m, ys, out_dtype == IZWI_QMM_OUT_BF16,
                                                  workspace, w0->n_cus, stream);
        if (e == hipSuccess) return IZWI_QMM_OK;
        if (e != hipErrorNotSupported) return fail_hip(e, "grouped prefill kernel");
        (void)hipGetLastError();
    }
    for (int i = 0; i < n_weights; i++)
        if (int rc = izwi_qmm_forward_bf16(weights[i], x_bf16, m, ys[i], out_dtype, mem_space, stream_)) return rc;
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_forward_fused(const izwi_qmm_weight* w, const void* x, int x_dtype, int64_t m,
                           const void* residual, void* y, int y_dtype, int mem_space, void* stream_) {
    return qmm_guarded("izwi_qmm_forward_fused", [&]() -> int {
    QmmCallScope call;
    if (!w) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    if (int rc = check_space(mem_space)) return rc;
    if ((x_dtype != IZWI_QMM_OUT_F32 && x_dtype != IZWI_QMM_OUT_BF16) ||
        (y_dtype != IZWI_QMM_OUT_F32 && y_dtype != IZWI_QMM_OUT_BF16))
        return fail(IZWI_QMM_ERR_INVALID, "bad x_dtype %d / y_dtype %d (f32 = 0, bf16 = 1)", x_dtype, y_dtype);
    const QmmLayout& L = w->layout;
    if (L.n_stacked != 1) return fail(IZWI_QMM_ERR_INVALID, "forward on an expert stack");
    if (m < 0) return fail(IZWI_QMM_ERR_INVALID, "negative m");
    if (m == 0 || L.n == 0) return IZWI_QMM_OK;
    if (!x) return fail(IZWI_QMM_ERR_INVALID, "x is NULL");
    if (!y) return fail(IZWI_QMM_ERR_INVALID, "y is NULL");
    hipStream_t stream = (hipStream_t)stream_;
    const bool x_bf16 = x_dtype == IZWI_QMM_OUT_BF16, y_bf16 = y_dtype == IZWI_QMM_OUT_BF16;
    if (profiling()) {
        // the casts of Qwen3Projection::forward happen inside the kernels: counted, their time is
        // part of qmatmul_ns
        if (x_bf16) g_in_casts.fetch_add(1, std::memory_order_relaxed);
        if (y_bf16) g_out_casts.fetch_add(1, std::memory_order_relaxed);
    }
    ProfileScope prof(w, stream);
    const size_t xbytes = (size_t)m * L.k * (x_bf16 ? 2 : 4), ybytes = (size_t)m * L.n * (y_bf16 ? 2 : 4);
    Staged xi, ri, yo;
    HIP_TRY(xi.in(x, xbytes, mem_space, stream));
    if (residual) HIP_TRY(ri.in(residual, ybytes, mem_space, stream));
    HIP_TRY(yo.out(y, ybytes, mem_space, stream));
    QmmIo io{x_bf16 ? 1 : 0, residual ? ri.dev : nullptr, y_bf16 ? 1 : 0};
    if (m < mfma_min_m(L.k)) {
        const float* xf = (const float*)xi.dev;
        if (x_bf16 && m > 2) { // this kernel reads bf16 rows only in its one- and two-row forms
            void* wide = nullptr;
            HIP_TRY(get_scratch(w->device, stream, (size_t)m * L.k * sizeof(float), &wide));
            HIP_TRY(qmm_launch_bf16_to_f32((const uint16_t*)xi.dev, (float*)wide, m * L.k, stream));
            xf = (const float*)wide;
            io.x_bf16 = 0;
        }
        HIP_TRY(qmm_launch_gemv(L, w->tiled, xf, m, (float*)yo.dev, w->n_cus, stream, &io));
    } else if (m <= 64 || large_m_mode() == IZWI_QMM_LARGE_M_INT8) {
        const int64_t chunk = m < 64 ? m : 64;
        const size_t ws_bytes = (qmm_gemv_mfma_workspace_bytes(L, chunk) + 255) & ~(size_t)255;
        const size_t xe = x_bf16 ? 2 : 4, ye = y_bf16 ? 2 : 4;
        void* scratch = nullptr;
        HIP_TRY(get_scratch(w->device, stream, ws_bytes + (size_t)chunk * (L.n > L.k ? L.n : L.k) * sizeof(float), &scratch));
        float* spare = reinterpret_cast<float*>(static_cast<uint8_t*>(scratch) + ws_bytes);
        for (int64_t r0 = 0; r0 < m; r0 += 64) {
            const int64_t rows = m - r0 < 64 ? m - r0 : 64;
            const void* xr = static_cast<const uint8_t*>(xi.dev) + (size_t)r0 * L.k * xe;
            void* yr = static_cast<uint8_t*>(yo.dev) + (size_t)r0 * L.n * ye;
            QmmIo cio = io;
            if (io.residual) cio.residual = static_cast<const uint8_t*>(io.residual) + (size_t)r0 * L.n * ye;
            hipError_t e;
            if (rows < mfma_min_m(L.k)) { // a tail of a few rows: the single-launch kernel
                e = qmm_launch_gemv(L, w->tiled, (const float*)xr, rows, (float*)yr, w->n_cus, stream, &cio);
            } else {
                e = qmm_launch_gemv_mfma(L, w->tiled, (const float*)xr, rows, (float*)yr, scratch, w->n_cus, stream, true, &cio);
                if (e == hipErrorNotSupported) {
                    // (very tall matrix with k beyond one activation window) sums into scratch, then the epilogue
                    (void)hipGetLastError();
                    const QmmIo plain{cio.x_bf16, nullptr, 0};
                    e = qmm_launch_gemv_mfma(L, w->tiled, (const float*)xr, rows, spare, scratch, w->n_cus, stream, true, &plain);
                    if (e == hipSuccess) e = qmm_launch_epilogue(spare, cio.residual, yr, cio.y_bf16, rows * L.n, stream);
                }
            }
            if (e != hipSuccess) return fail_hip(e, "batched decode kernel");
        }
    } else {
        const size_t xb_bytes = x_bf16 ? 0 : ((((size_t)m * L.k * sizeof(uint16_t)) + 255) & ~(size_t)255);
        const size_t ws_bytes = qmm_gemm_workspace_bytes(L, m, w->n_cus);
        void* scratch = nullptr;
        if (xb_bytes + ws_bytes) HIP_TRY(get_scratch(w->device, stream, xb_bytes + ws_bytes, &scratch));
        const uint16_t* xb = (const uint16_t*)xi.dev;
        if (!x_bf16) {
            HIP_TRY(qmm_launch_f32_to_bf16((const float*)xi.dev, (uint16_t*)scratch, m * L.k, stream));
            xb = (const uint16_t*)scratch;
        }
        HIP_TRY(qmm_launch_gemm_bf16(L, w->tiled, xb, m, yo.dev, io.y_bf16,
                                     ws_bytes ? static_cast<uint8_t*>(scratch) + xb_bytes : nullptr, w->n_cus, stream,
                                     io.residual));
    }
    HIP_TRY(yo.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_moe_route(const float* logits, int64_t t, int32_t n_experts, int32_t top_k, int32_t* ids,
                   float* weights, int mem_space, void* stream_) {
    return qmm_guarded("izwi_moe_route", [&]() -> int {
    if (int rc = check_space(mem_space)) return rc;
    if (t < 0) return fail(IZWI_QMM_ERR_INVALID, "negative t");
    if (n_experts < 1 || n_experts > 1024)
        return fail(IZWI_QMM_ERR_UNSUPPORTED, "n_experts = %d outside 1..1024", n_experts);
    if (top_k < 1 || top_k > n_experts || top_k > 64)
        return fail(IZWI_QMM_ERR_INVALID, "top_k = %d outside 1..min(n_experts, 64)", top_k);
    if (t == 0) return IZWI_QMM_OK;
    if (!logits || !ids || !weights) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    int device = 0;
    if (int rc = current_device(&device)) return rc;
    if (int rc = ensure_device(device, nullptr)) return rc;
    hipStream_t stream = (hipStream_t)stream_;
    Staged li, io, wo;
    HIP_TRY(li.in(logits, (size_t)t * n_experts * sizeof(float), mem_space, stream));
    HIP_TRY(io.out(ids, (size_t)t * top_k * sizeof(int32_t), mem_space, stream));
    HIP_TRY(wo.out(weights, (size_t)t * top_k * sizeof(float), mem_space, stream));
    HIP_TRY(qmm_launch_moe_route((const float*)li.dev, t, n_experts, top_k, (int32_t*)io.dev,
                                 (float*)wo.dev, stream));
    HIP_TRY(io.finish(stream));
    HIP_TRY(wo.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_moe_sort(const int32_t* ids, int64_t t, int32_t top_k, int32_t n_experts, int32_t* perm,
                  int32_t* offsets, int mem_space, void* stream_) {
    return qmm_guarded("izwi_moe_sort", [&]() -> int {
    QmmCallScope call;
    if (int rc = check_space(mem_space)) return rc;
    if (t < 0 || top_k < 1 || n_experts < 1 || n_experts > 8192)
        return fail(IZWI_QMM_ERR_INVALID, "bad sort shape t=%lld top_k=%d n_experts=%d", (long long)t, top_k, n_experts);
    const int64_t pairs = t * top_k;
    if (pairs > 0x7fffffff) return fail(IZWI_QMM_ERR_UNSUPPORTED, "too many pairs");
    if (!offsets || (pairs && (!ids || !perm))) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    int device = 0;
    if (int rc = current_device(&device)) return rc;
    if (int rc = ensure_device(device, nullptr)) return rc;
    hipStream_t stream = (hipStream_t)stream_;
    Staged ii, po, oo;
    HIP_TRY(ii.in(ids, (size_t)pairs * sizeof(int32_t), mem_space, stream));
    // (the sort's later passes read what its earlier ones wrote: device memory)
    HIP_TRY(po.out(perm, (size_t)pairs * sizeof(int32_t), mem_space, stream, false));
    HIP_TRY(oo.out(offsets, (size_t)(n_experts + 1) * sizeof(int32_t), mem_space, stream, false));
    void* scratch = nullptr;
    HIP_TRY(get_scratch(device, stream, (size_t)qmm_moe_sort_scratch_ints(pairs, n_experts) * sizeof(int32_t), &scratch));
    hipError_t e = qmm_launch_moe_sort((const int32_t*)ii.dev, pairs, n_experts, (int32_t*)po.dev,
                                       (int32_t*)oo.dev, nullptr, (int32_t*)scratch, stream);
    if (e != hipSuccess) return fail_hip(e, "sort kernels");
    HIP_TRY(po.finish(stream));
    HIP_TRY(oo.finish(stream));
    return IZWI_QMM_OK;
    });
}

namespace {

int moe_check_stacks(const izwi_qmm_weight* gate, const izwi_qmm_weight* up, const izwi_qmm_weight* down) {
    if (!gate || !up || !down) return fail(IZWI_QMM_ERR_INVALID, "NULL weight");
    const QmmLayout& G = gate->layout;
    const QmmLayout& U = up->layout;
    const QmmLayout& D = down->layout;
    if (G.dtype != U.dtype || G.n != U.n || G.k != U.k || G.n_stacked != U.n_stacked)
        return fail(IZWI_QMM_ERR_INVALID, "gate and up stacks differ in shape or dtype");
    if (D.n_stacked != G.n_stacked || D.k != G.n || D.n != G.k)
        return fail(IZWI_QMM_ERR_INVALID, "down stack [%lld, %lld] does not match gate/up [%lld, %lld]",
                    (long long)D.n, (long long)D.k, (long long)G.n, (long long)G.k);
    return IZWI_QMM_OK;
}

// The expert MLP on device buffers.  With `logits` the routing is computed here too (ids,
// weights, perm, offsets are then ignored; ids_out / weights_out, if not NULL, receive it): for
// small batches routing, sort and segment tables are ONE launch.
int moe_core(const izwi_qmm_weight* gate, const izwi_qmm_weight* up, const izwi_qmm_weight* down,
             const float* x, int64_t t, int32_t top_k, const float* logits, const int32_t* ids,
             const float* weights, const int32_t* perm, const int32_t* offsets, int32_t* ids_out,
             float* weights_out, float* out, hipStream_t stream) {
    const QmmLayout& G = gate->layout;
    const QmmLayout& D = down->layout;
    const int64_t pairs = t * top_k;
    const int n_experts = (int)G.n_stacked;
    const int64_t hidden = G.k, inter = G.n;
    // every expert adds at most one partly filled segment
    const int64_t max_segments = pairs / QMM_MOE_SEG_ROWS + (pairs < n_experts ? pairs : n_experts);
    ProfileScope prof(nullptr, stream);

    // Many pairs per expert: 16-row tiles on the int8 matrix cores (the weights of an
    // expert are read once for all its pairs).  Few: 4-row segments on the dot4 kernel.
    const bool tiles = moe_on_tiles(pairs, n_experts) &&
                       qmm_gemv_mfma_grouped_supported(G) && qmm_gemv_mfma_grouped_supported(D);
    if (!tiles && max_segments > 65535)
        return fail(IZWI_QMM_ERR_UNSUPPORTED, "t * top_k = %lld is too large for one grouped launch", (long long)pairs);
    // workspace: h [pairs, inter] | y [pairs, hidden] | seg_offsets [E + 1]
    //            | tiles: u [pairs, inter], activation records; else: seg_expert [max_segments]
    //            | routing computed here: ids, weights, perm [pairs], offsets [E + 1], sort scratch
    auto align256 = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t h_bytes = align256((size_t)pairs * inter * sizeof(float));
    const size_t y_bytes = align256((size_t)pairs * hidden * sizeof(float));
    const size_t s_bytes = align256((size_t)(n_experts + 1) * sizeof(int32_t));
    const int64_t max_tiles = pairs / QMM_MOE_TILE_ROWS + (pairs < n_experts ? pairs : n_experts);
    // Where a stack runs in the expert form, its activations are quantized row by row (the token rows
    // inside the routing kernel, the rows of silu(gate) * up in pair order) and the kernel puts its tiles
    // together from the rows' records; otherwise tile by tile through the sort's tables.
    const bool g_rows = tiles && qmm_moe_row_records_apply(G, gate->n_cus, pairs, t, top_k);
    const bool d_rows = tiles && qmm_moe_row_records_apply(D, down->n_cus, pairs, pairs, 1);
    size_t r_bytes = 0;
    if (tiles) {
        const size_t r1 = g_rows ? qmm_row_records_bytes(t, hidden) : qmm_moe_records_bytes(G.dtype, max_tiles, hidden);
        const size_t r2 = d_rows ? qmm_row_records_bytes(pairs, inter) : qmm_moe_records_bytes(D.dtype, max_tiles, inter);
        r_bytes = align256(r1 > r2 ? r1 : r2);
    }
    const size_t te_bytes = tiles ? align256((size_t)max_tiles * 4) : 0; // tile -> expert
    const size_t mid_bytes = tiles ? h_bytes + r_bytes + te_bytes : align256((size_t)max_segments * 4);
    const size_t p_bytes = align256((size_t)pairs * 4);
    const size_t sort_bytes = align256((size_t)qmm_moe_sort_scratch_ints(pairs, n_experts) * sizeof(int32_t));
    // Segment path with the routing computed here, beyond the one-launch plan's sizes: the routing kernel
    // also quantizes the token rows (x blocks), which the gate / up launch then copies instead of
    // quantizing them in every workgroup of a segment.  Measured per layer at 128 experts, top-8,
    // without / with: 74 / 70 us at 24 tokens, 90 / 80 at 32, 103 / 90 at 40; up to 16 tokens, where most
    // segments hold one row and routing, sort and tables are one workgroup, it does not pay (60.4 / 62.6).
    const size_t xb_bytes = logits && !tiles && !qmm_moe_plan_small_supported(t, n_experts, top_k)
                                ? align256(qmm_x_blocks_bytes(t, hidden)) : 0;
    // (the one-workgroup sort, or the tile-table launch behind a caller's sort, also ranks the experts by
    // tile count for the expert kernels' work items)
    const bool order_ready = tiles && (logits ? qmm_moe_sort_ranks_experts(pairs, n_experts) : qmm_moe_segments_rank_experts(n_experts));
    const size_t order_bytes = order_ready ? align256((size_t)n_experts * 32) : 0;
    const size_t route_bytes = logits ? 3 * p_bytes + s_bytes + sort_bytes + xb_bytes : 0;
    uint8_t* ws = nullptr;
    HIP_TRY(get_scratch(gate->device, stream, h_bytes + y_bytes + s_bytes + mid_bytes + route_bytes + order_bytes, (void**)&ws));
    float* h = (float*)ws;
    float* y = (float*)(ws + h_bytes);
    int32_t* seg = (int32_t*)(ws + h_bytes + y_bytes);
    uint8_t* mid = ws + h_bytes + y_bytes + s_bytes;
    int32_t* seg_expert = (int32_t*)mid; // 4-row segment path only
    int32_t* tile_expert = (int32_t*)(mid + h_bytes + r_bytes); // tile path only
    bool segments_ready = false;
    void* x_blocks = nullptr; // written by the routing kernels below when set
    bool x_rows_ready = false; // the routing kernel has written the token rows' records
    int32_t* expert_order = order_ready ? (int32_t*)(mid + mid_bytes + route_bytes) : nullptr; // written by the sort / the tile-table launch
    hipError_t e = hipSuccess;
    if (logits) {
        uint8_t* r = mid + mid_bytes;
        int32_t* r_ids = (int32_t*)r;
        float* r_w = (float*)(r + p_bytes);
        int32_t* r_perm = (int32_t*)(r + 2 * p_bytes);
        int32_t* r_off = (int32_t*)(r + 3 * p_bytes);
        int32_t* r_sort = (int32_t*)(r + 3 * p_bytes + s_bytes);
        if (xb_bytes) x_blocks = r + 3 * p_bytes + s_bytes + sort_bytes;
        // a handful of pairs: the whole layer in two launches (routing inside gate / up, combine
        // inside down), same results
        if (!tiles && pairs <= moe_small_max_pairs() && qmm_moe_small_supported(G, D, t, n_experts, top_k)) {
            e = qmm_launch_moe_small(G, gate->tiled, up->tiled, D, down->tiled, logits, x, t, n_experts, top_k, h, r_ids,
                                     r_w, ids_out, weights_out, out, max_segments, gate->n_cus, stream);
            if (e == hipSuccess) {
                if (profiling()) g_silu_fused.fetch_add(1, std::memory_order_relaxed);
                return IZWI_QMM_OK;
            }
            if (e != hipErrorNotSupported) return fail_hip(e, "small-batch expert kernels");
            (void)hipGetLastError();
            e = hipSuccess;
        }
        if (!tiles && qmm_moe_plan_small_supported(t, n_experts, top_k)) {
            e = qmm_launch_moe_plan_small(logits, t, n_experts, top_k, QMM_MOE_SEG_ROWS, max_segments, r_ids, r_w,
                                          r_perm, r_off, seg, seg_expert, stream);
            segments_ready = true;
        } else {
            if (g_rows) {
                e = qmm_launch_moe_route_rows(logits, t, n_experts, top_k, r_ids, r_w, stream, x, hidden, G.dtype,
                                              mid + h_bytes);
                x_rows_ready = true;
            } else {
                e = qmm_launch_moe_route(logits, t, n_experts, top_k, r_ids, r_w, stream, x, hidden, G.dtype, x_blocks);
            }
            // the sort also leaves the table of the 16-row tiles the matrix-core path walks, or of the
            // 4-row segments of the decode kernel, with the expert of every tile / segment
            if (e == hipSuccess)
                e = qmm_launch_moe_sort(r_ids, pairs, n_experts, r_perm, r_off, seg, r_sort, stream,
                                        tiles ? QMM_MOE_TILE_ROWS : QMM_MOE_SEG_ROWS, tiles ? tile_expert : seg_expert,
                                        tiles ? max_tiles : max_segments, expert_order);
            segments_ready = true;
        }
        if (e != hipSuccess) return fail_hip(e, "routing kernels");
        if (ids_out) HIP_TRY(hipMemcpyAsync(ids_out, r_ids, (size_t)pairs * 4, hipMemcpyDeviceToDevice, stream));
        if (weights_out) HIP_TRY(hipMemcpyAsync(weights_out, r_w, (size_t)pairs * 4, hipMemcpyDeviceToDevice, stream));
        ids = r_ids, weights = r_w, perm = r_perm, offsets = r_off;
    }
    if (tiles) {
        float* u = (float*)mid;
        void* records = mid + h_bytes;
        if (!segments_ready)
            e = qmm_launch_moe_segments(offsets, n_experts, QMM_MOE_TILE_ROWS, seg, tile_expert, max_tiles, stream, expert_order);
        if (e == hipSuccess && !x_rows_ready)
            e = g_rows ? qmm_launch_quantize_rows(G.dtype, x, nullptr, t, hidden, records, stream)
                       : qmm_launch_quantize_grouped(G.dtype, x, nullptr, top_k, hidden, perm, offsets, seg, n_experts,
                                                     max_tiles, records, stream, tile_expert);
        if (e == hipSuccess)
            e = qmm_launch_gemv_mfma_grouped(G, gate->tiled, up->tiled, records, h, u, perm, offsets, seg, n_experts,
                                             pairs, stream, gate->n_cus, g_rows ? top_k : 0, expert_order);
        // silu(gate) * up is applied while the down projection's input is quantized
        if (e == hipSuccess)
            e = d_rows ? qmm_launch_quantize_rows(D.dtype, h, u, pairs, inter, records, stream)
                       : qmm_launch_quantize_grouped(D.dtype, h, u, 1, inter, perm, offsets, seg, n_experts, max_tiles,
                                                     records, stream, tile_expert);
        if (e == hipSuccess)
            e = qmm_launch_gemv_mfma_grouped(D, down->tiled, nullptr, records, y, nullptr, perm, offsets, seg,
                                             n_experts, pairs, stream, down->n_cus, d_rows ? 1 : 0, expert_order);
    } else {
        if (!segments_ready)
            e = qmm_launch_moe_segments(offsets, n_experts, QMM_MOE_SEG_ROWS, seg, seg_expert, max_segments, stream);
        if (e == hipSuccess)
            e = qmm_launch_gemv_grouped(G, gate->tiled, up->tiled, x, top_k, h, perm, offsets, seg, seg_expert,
                                        n_experts, max_segments, gate->n_cus, stream, x_blocks, t);
        if (e == hipSuccess)
            e = qmm_launch_gemv_grouped(D, down->tiled, nullptr, h, 1, y, perm, offsets, seg, seg_expert, n_experts,
                                        max_segments, gate->n_cus, stream);
    }
    if (e == hipSuccess) e = qmm_launch_moe_combine(y, weights, t, top_k, hidden, out, stream);
    if (e != hipSuccess) return fail_hip(e, "grouped expert kernels");
    if (profiling()) g_silu_fused.fetch_add(1, std::memory_order_relaxed);
    return IZWI_QMM_OK;
}

} // namespace

int izwi_moe_forward_f32(const izwi_qmm_weight* gate, const izwi_qmm_weight* up,
                         const izwi_qmm_weight* down, const float* x, int64_t t,
                         const int32_t* ids, const float* weights, int32_t top_k,
                         const int32_t* perm, const int32_t* offsets, float* out, int mem_space,
                         void* stream_) {
    return qmm_guarded("izwi_moe_forward_f32", [&]() -> int {
    QmmCallScope call;
    if (int rc = moe_check_stacks(gate, up, down)) return rc;
    if (int rc = check_space(mem_space)) return rc;
    if (t < 0) return fail(IZWI_QMM_ERR_INVALID, "negative t");
    if (top_k < 1 || top_k > 64 || top_k > (int)gate->layout.n_stacked)
        return fail(IZWI_QMM_ERR_INVALID, "top_k = %d outside 1..min(n_experts, 64)", top_k);
    if (t == 0) return IZWI_QMM_OK;
    if (t * (int64_t)top_k > 0x7fffffff) return fail(IZWI_QMM_ERR_UNSUPPORTED, "too many pairs");
    if (!x || !ids || !weights || !perm || !offsets || !out)
        return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    const int64_t pairs = t * top_k;
    const int n_experts = (int)gate->layout.n_stacked;
    const int64_t hidden = gate->layout.k;
    hipStream_t stream = (hipStream_t)stream_;
    Staged xi, ii, wi, pi, oi, oo;
    HIP_TRY(xi.in(x, (size_t)t * hidden * sizeof(float), mem_space, stream));
    HIP_TRY(ii.in(ids, (size_t)pairs * sizeof(int32_t), mem_space, stream));
    HIP_TRY(wi.in(weights, (size_t)pairs * sizeof(float), mem_space, stream));
    HIP_TRY(pi.in(perm, (size_t)pairs * sizeof(int32_t), mem_space, stream));
    HIP_TRY(oi.in(offsets, (size_t)(n_experts + 1) * sizeof(int32_t), mem_space, stream));
    HIP_TRY(oo.out(out, (size_t)t * hidden * sizeof(float), mem_space, stream));
    if (int rc = moe_core(gate, up, down, (const float*)xi.dev, t, top_k, nullptr, (const int32_t*)ii.dev,
                          (const float*)wi.dev, (const int32_t*)pi.dev, (const int32_t*)oi.dev, nullptr, nullptr,
                          (float*)oo.dev, stream))
        return rc;
    HIP_TRY(oo.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_moe_layer_f32(const izwi_qmm_weight* gate, const izwi_qmm_weight* up, const izwi_qmm_weight* down,
                       const float* logits, const float* x, int64_t t, int32_t top_k, float* out,
                       int32_t* ids_out, float* weights_out, int mem_space, void* stream_) {
    return qmm_guarded("izwi_moe_layer_f32", [&]() -> int {
    QmmCallScope call;
    if (int rc = moe_check_stacks(gate, up, down)) return rc;
    if (int rc = check_space(mem_space)) return rc;
    const int n_experts = (int)gate->layout.n_stacked;
    if (t < 0) return fail(IZWI_QMM_ERR_INVALID, "negative t");
    if (n_experts > 1024) return fail(IZWI_QMM_ERR_UNSUPPORTED, "n_experts = %d outside 1..1024", n_experts);
    if (top_k < 1 || top_k > n_experts || top_k > 64)
        return fail(IZWI_QMM_ERR_INVALID, "top_k = %d outside 1..min(n_experts, 64)", top_k);
    if (t == 0) return IZWI_QMM_OK;
    if (t * (int64_t)top_k > 0x7fffffff) return fail(IZWI_QMM_ERR_UNSUPPORTED, "too many pairs");
    if (!logits || !x || !out) return fail(IZWI_QMM_ERR_INVALID, "NULL buffer");
    const int64_t pairs = t * top_k, hidden = gate->layout.k;
    hipStream_t stream = (hipStream_t)stream_;
    Staged li, xi, oo, io, wo;
    HIP_TRY(li.in(logits, (size_t)t * n_experts * sizeof(float), mem_space, stream));
    HIP_TRY(xi.in(x, (size_t)t * hidden * sizeof(float), mem_space, stream));
    HIP_TRY(oo.out(out, (size_t)t * hidden * sizeof(float), mem_space, stream));
    // (ids and weights reach their outputs through device-to-device copy calls)
    if (ids_out) HIP_TRY(io.out(ids_out, (size_t)pairs * sizeof(int32_t), mem_space, stream, false));
    if (weights_out) HIP_TRY(wo.out(weights_out, (size_t)pairs * sizeof(float), mem_space, stream, false));
    if (int rc = moe_core(gate, up, down, (const float*)xi.dev, t, top_k, (const float*)li.dev, nullptr, nullptr,
                          nullptr, nullptr, (int32_t*)io.dev, (float*)wo.dev, (float*)oo.dev, stream))
        return rc;
    HIP_TRY(oo.finish(stream));
    if (ids_out) HIP_TRY(io.finish(stream));
    if (weights_out) HIP_TRY(wo.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_set_large_m_arithmetic(int mode) {
    return qmm_guarded("izwi_qmm_set_large_m_arithmetic", [&]() -> int {
    if (mode != IZWI_QMM_LARGE_M_BF16 && mode != IZWI_QMM_LARGE_M_INT8)
        return fail(IZWI_QMM_ERR_INVALID, "bad large-m arithmetic %d (bf16 = 0, int8 = 1)", mode);
    g_large_m_mode.store(mode, std::memory_order_relaxed);
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_get_large_m_arithmetic(void) { return large_m_mode(); }

int izwi_qmm_set_prefill_form(int form) {
    return qmm_guarded("izwi_qmm_get_large_m_arithmetic", [&]() -> int {
    if (form < IZWI_QMM_PREFILL_AUTO || form > IZWI_QMM_PREFILL_PLANE)
        return fail(IZWI_QMM_ERR_INVALID, "bad prefill form %d (auto = -1, lds = 0, plane = 1)", form);
    qmm_set_prefill_form(form);
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_get_prefill_form(void) { return qmm_get_prefill_form(); }

int izwi_qmm_set_moe_expert_form(int enabled) {
    return qmm_guarded("izwi_qmm_get_prefill_form", [&]() -> int {
    g_moe_expert_form.store(enabled < 0 ? -1 : enabled == 2 ? 2 : enabled ? 1 : 0, std::memory_order_relaxed);
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_scratch_reserve(uint64_t bytes, void* stream_) {
    return qmm_guarded("izwi_qmm_scratch_reserve", [&]() -> int {
    int device = 0;
    if (int rc = current_device(&device)) return rc;
    if (int rc = ensure_device(device, nullptr)) return rc;
    void* p = nullptr;
    HIP_TRY(get_scratch(device, (hipStream_t)stream_, (size_t)bytes, &p));
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_profile_enable(int enabled) {
    return qmm_guarded("izwi_qmm_profile_enable", [&]() -> int {
    g_profile.store(enabled ? 1 : 0, std::memory_order_relaxed);
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_profile_snapshot_get(izwi_qmm_profile_snapshot* out) {
    return qmm_guarded("izwi_qmm_profile_snapshot_get", [&]() -> int {
    if (!out) return fail(IZWI_QMM_ERR_INVALID, "out is NULL");
    out->qmatmul_calls = g_calls.load(std::memory_order_relaxed);
    out->qmatmul_ns = g_ns.load(std::memory_order_relaxed);
    out->qmatmul_input_casts = g_in_casts.load(std::memory_order_relaxed);
    out->qmatmul_input_cast_ns = g_in_cast_ns.load(std::memory_order_relaxed);
    out->qmatmul_output_casts = g_out_casts.load(std::memory_order_relaxed);
    out->qmatmul_output_cast_ns = g_out_cast_ns.load(std::memory_order_relaxed);
    out->lm_head_calls = g_lm_calls.load(std::memory_order_relaxed);
    out->lm_head_ns = g_lm_ns.load(std::memory_order_relaxed);
    out->silu_mul_fused_calls = g_silu_fused.load(std::memory_order_relaxed);
    out->silu_mul_fallback_calls = g_silu_fallback.load(std::memory_order_relaxed);
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_profile_enabled(void) { return profiling() ? 1 : 0; }

int izwi_qmm_profile_argmax_get(uint64_t* calls, uint64_t* ns) {
    return qmm_guarded("izwi_qmm_profile_enabled", [&]() -> int {
    if (!calls || !ns) return fail(IZWI_QMM_ERR_INVALID, "NULL argument");
    *calls = g_argmax_calls.load(std::memory_order_relaxed);
    *ns = g_argmax_ns.load(std::memory_order_relaxed);
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_profile_reset(void) {
    return qmm_guarded("izwi_qmm_profile_reset", [&]() -> int {
    for (auto* c : {&g_calls, &g_ns, &g_in_casts, &g_in_cast_ns, &g_out_casts, &g_out_cast_ns,
                    &g_lm_calls, &g_lm_ns, &g_silu_fused, &g_silu_fallback, &g_argmax_calls, &g_argmax_ns})
        c->store(0, std::memory_order_relaxed);
    return IZWI_QMM_OK;
    });
}

} // extern "C"
