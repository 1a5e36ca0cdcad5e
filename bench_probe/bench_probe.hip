// Measurement helpers of bench.py - NOT part of libizwi_qmm.so and of no use to a caller of the
// library.  Built by bench_probe/Makefile into bench_probe/libbench_probe.so, loaded by bench.py
// through ctypes.
//
//  * bench_probe_stream_read: one launch that only READS `bytes` of device memory (16-byte
//    non-temporal loads, several in flight per lane, nothing stored).  Timed over buffers of the
//    sizes of a model's weights, in the order and with the dependencies of its decode calls, it
//    shows what a plain read of the same bytes in the same launches reaches on this GPU.
//  * bench_probe_stream_copy: a plain copy kernel of the same shape (bytes read + bytes written).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Every lane keeps U 16-byte non-temporal loads in flight and folds what it read into a register
// that an empty volatile asm statement consumes: nothing is stored, and the loads cannot be
// dropped.  Two launch shapes, each the best of a sweep (unroll 4 / 8 / 9 / 16, 256 / 512 / 768
// threads, 1 - 16 workgroups per CU) for its sizes on an MI355X: from 40 MB one 768-thread
// workgroup per CU with nine loads per lane in flight (the decode kernel's own shape), below it
// 256-thread workgroups, up to sixteen per CU, four loads per lane.
template <int U, int T>
__global__ __launch_bounds__(T) void stream_read_kernel(const u32x4* __restrict__ src, int64_t n16) {
    const int64_t stride = (int64_t)gridDim.x * T;
    uint32_t fold = 0;
    int64_t i = (int64_t)blockIdx.x * T + threadIdx.x;
    for (; i + (U - 1) * stride < n16; i += U * stride) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < U; u++) fold |= v[u].x & v[u].y & v[u].z & v[u].w;
    }
    for (; i < n16; i += stride) {
        const u32x4 a = __builtin_nontemporal_load(src + i);
        fold |= a.x & a.y & a.z & a.w;
    }
    asm volatile("" ::"v"(fold));
}

template <int U, int T>
__global__ __launch_bounds__(T) void stream_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n16) {
    const int64_t stride = (int64_t)gridDim.x * T;
    int64_t i = (int64_t)blockIdx.x * T + threadIdx.x;
    for (; i + (U - 1) * stride < n16; i += U * stride) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < U; u++) __builtin_nontemporal_store(v[u], dst + i + u * stride);
    }
    for (; i < n16; i += stride) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

int cu_count() {
    int device = 0, n = 0;
    if (hipGetDevice(&device) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
    return n;
}
} // namespace

extern "C" {

// 0 on success, a hipError_t otherwise.  `src` 16-byte aligned; bytes beyond a multiple of 16 are not read.
int bench_probe_stream_read(const void* src, uint64_t bytes, void* stream) {
    if (!src || ((uintptr_t)src & 15) != 0) return (int)hipErrorInvalidValue;
    const int64_t n16 = (int64_t)(bytes / 16);
    if (n16 == 0) return 0;
    const int n_cus = cu_count();
    if (n_cus <= 0) return (int)hipErrorNoDevice;
    if (bytes >= ((uint64_t)40 << 20)) {
        stream_read_kernel<9, 768><<<(unsigned)n_cus, 768, 0, (hipStream_t)stream>>>((const u32x4*)src, n16);
    } else {
        int64_t wgs = (n16 + 4 * 256 - 1) / (4 * 256);
        if (wgs > (int64_t)n_cus * 16) wgs = (int64_t)n_cus * 16;
        stream_read_kernel<4, 256><<<(unsigned)wgs, 256, 0, (hipStream_t)stream>>>((const u32x4*)src, n16);
    }
    return (int)hipGetLastError();
}

// `wgs_per_cu` workgroups of 512 threads per CU, eight loads then eight stores per lane in flight.
int bench_probe_stream_copy(const void* src, void* dst, uint64_t bytes, int wgs_per_cu, void* stream) {
    if (!src || !dst || (((uintptr_t)src | (uintptr_t)dst) & 15) != 0) return (int)hipErrorInvalidValue;
    const int64_t n16 = (int64_t)(bytes / 16);
    if (n16 == 0) return 0;
    const int n_cus = cu_count();
    if (n_cus <= 0) return (int)hipErrorNoDevice;
    if (wgs_per_cu < 1) wgs_per_cu = 1;
    if (wgs_per_cu > 32) wgs_per_cu = 32;
    stream_copy_kernel<8, 512><<<(unsigned)(n_cus * wgs_per_cu), 512, 0, (hipStream_t)stream>>>((const u32x4*)src, (u32x4*)dst, n16);
    return (int)hipGetLastError();
}

} // extern "C"
