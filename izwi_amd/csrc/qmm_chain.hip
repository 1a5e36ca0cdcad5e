// Chained decode: a list of dependent single-row projection steps (each step's activations are
// written by an earlier step) as ONE kernel launch.
//
// Between two dependent launches of the per-call kernels about 1.4 us pass in which nothing runs,
// and every launch ramps up (first loads 0.4 us after its start, first data 0.7 us later) and
// drains (last multiply, k-split sum, store) on its own.  Here one resident grid (a workgroup of
// 12 waves per CU) walks through all steps:
//   * a wave requests the weight panel of its next piece of work BEFORE it waits for that work's
//     activations: weights do not depend on activations, so HBM keeps streaming the next step's
//     bytes while the current step's results travel;
//   * a step's results are written with device-scope (write-through) stores, its completion is
//     counted on per-step counters spread over 16 cache lines (256 increments of one line cost
//     4 us, of 16 lines 2.2 us), and consumers read the activations with device-scope loads:
//     no cache-wide write-back or invalidate is issued anywhere (one such fence per workgroup
//     costs 27 us per step);
//   * every wait is BOUNDED: after `spin_limit` polls a workgroup gives up, raises the error word
//     and runs on without waiting (results are then garbage, all workgroups still exit); the host
//     reports the error word as a failed call.
// The arithmetic is that of the per-call kernels (same quantizer, same panel products, same order
// of the sums): results are bit-identical to izwi_qmm_forward_group_f32 at m = 1.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

#include "izwi_qmm.h"
#include "qmm_gemv_blocks.h"
#include "qmm_internal.h"

namespace {

constexpr int kChainWaves = 12;
constexpr int kShards = 16;        // counter words of a step, one cache line (256 B) apart
constexpr int kShardStride = 64;   // in words
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct ChainWeight {
    const uint8_t* w; // tiled matrix
    float* y;         // [n]
    int n;
    int pad;
};

struct ChainPhase {
    const float* x; // [k] activations of the step
    int k, k_units, k_groups, slots;
    int s_units, panel_bytes;
    int nwk, nwr;   // waves along k, row-tiles side by side in a workgroup (nwk * nwr <= 12)
    int tiles;      // row tiles of all weights of the step
    int rounds;     // ceil(tiles / (grid * nwr))
    int n_weights;
    int participants; // workgroups that have work in this step: min(grid, tiles)
    int tile_end[QMM_MAX_GROUP]; // cumulative row tiles per weight
    ChainWeight wt[QMM_MAX_GROUP];
};

struct ChainParams {
    const ChainPhase* phases;
    int n_phases;
    unsigned* counters; // [n_phases][kShards * kShardStride]
    unsigned* err;      // != 0: a wait gave up
    unsigned spin_limit;
};

__device__ __forceinline__ unsigned load_dev(const unsigned* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Waits (wave 0) until step `p` has been completed by all its participants; bounded.
__device__ __forceinline__ void wait_step(const ChainParams& C, int p, int expected) {
    if (threadIdx.x < 64) {
        const unsigned* c = C.counters + (size_t)p * (kShards * kShardStride);
        unsigned spins = 0;
        while (true) {
            unsigned v = threadIdx.x < kShards ? load_dev(c + threadIdx.x * kShardStride) : 0u;
            // (the error word rides in lane 16: any workgroup that gave up releases all the others)
            if (threadIdx.x == kShards) v = load_dev(C.err) ? 0x40000000u : 0u;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o); // every lane of the wave holds the sum
            if (v >= (unsigned)expected) break;
            if (++spins > C.spin_limit) {
                if (threadIdx.x == 0) __hip_atomic_store(C.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
    }
    __syncthreads();
    asm volatile("" ::: "memory");
}

struct Item {
    const uint8_t* base; // panel of this wave
    bool ok;             // the wave has a panel in this (step, round)
};

// The panel of wave (slot, wk) in round r of a step, for workgroup b of a grid of G.
__device__ __forceinline__ Item item_of(const ChainPhase& ph, int b, int G, int r, int slot, int wk, int& tile_out,
                                        int& weight_out) {
    Item it;
    const int t = b + G * (r * ph.nwr + slot);
    const bool ok = slot < ph.nwr && t < ph.tiles && wk < ph.k_groups;
    int i = 0;
    while (i + 1 < ph.n_weights && t >= ph.tile_end[i]) i++;
    const int lt = t - (i ? ph.tile_end[i - 1] : 0);
    it.ok = ok;
    it.base = ok ? ph.wt[i].w + ((int64_t)lt * ph.k_groups + wk) * ph.panel_bytes : ph.wt[0].w;
    tile_out = lt;
    weight_out = i;
    return it;
}

template <int QT>
__global__ __launch_bounds__(64 * kChainWaves) void chain_kernel(ChainParams C) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int b = blockIdx.x, G = gridDim.x;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;

    Panel<QT> nxt;
    bool nxt_loaded = false; // uniform per wave: `nxt` holds (or is receiving) the panel of the next item

    for (int p = 0; p < C.n_phases; p++) {
        const ChainPhase& ph = C.phases[p];
        if (b >= ph.tiles) continue; // no row-tile of this step falls to this workgroup (uniform)
        const int slot = wave / ph.nwk, wk = wave - slot * ph.nwk;
        const int k_units = ph.k_units;
        const XLds<QT> l = carve<QT, 1>(smem, k_units);

        // the first panel of the step, unless the previous step already requested it
        int tile, wi;
        if (!nxt_loaded) {
            const Item it = item_of(ph, b, G, 0, slot, wk, tile, wi);
            load_panel<QT>(nxt, it.base, ph.slots, lane, it.ok && lane < ph.slots);
        }
        nxt_loaded = false;

        if (p > 0) wait_step(C, p - 1, C.phases[p - 1].participants);
        else __syncthreads();

        // activations: device-scope loads (another CU's write-through stores), quantized into LDS
        {
            const int group = threadIdx.x >> 4, j = threadIdx.x & 15;
            for (int item = group; item < k_units; item += 4 * kChainWaves) {
                const int k0 = item * 256 + 16 * j;
                const bool in_range = k0 + 16 <= ph.k;
                const float* src = ph.x + (in_range ? k0 : 0);
                // four 16-byte device-scope loads and the wait for them as one block: the compiler does
                // not count loads it has not issued itself
                f32x4 f0, f1, f2, f3;
                asm volatile("global_load_dwordx4 %0, %4, off sc1\n\t"
                             "global_load_dwordx4 %1, %4, off offset:16 sc1\n\t"
                             "global_load_dwordx4 %2, %4, off offset:32 sc1\n\t"
                             "global_load_dwordx4 %3, %4, off offset:48 sc1\n\t"
                             "s_waitcnt vmcnt(0)"
                             : "=&v"(f0), "=&v"(f1), "=&v"(f2), "=&v"(f3)
                             : "v"(src)
                             : "memory");
                const float4 f[4] = {make_float4(f0.x, f0.y, f0.z, f0.w), make_float4(f1.x, f1.y, f1.z, f1.w),
                                     make_float4(f2.x, f2.y, f2.z, f2.w), make_float4(f3.x, f3.y, f3.z, f3.w)};
                float v[16];
                x16_finish<false>(f, in_range, v);
                x_item_quantize<QT, 1>(l, k_units, item, v);
            }
        }
        lds_barrier();

        int red_buf = 0;
        for (int r = 0; r < ph.rounds; r++) {
            if (b + G * (r * ph.nwr) >= ph.tiles) break; // no tile of this round for the workgroup (uniform)
            Panel<QT> cur = nxt;
            const Item it = item_of(ph, b, G, r, slot, wk, tile, wi);
            // the next round's panel of this step is requested before this round's arithmetic
            const bool more = r + 1 < ph.rounds && b + G * ((r + 1) * ph.nwr) < ph.tiles;
            if (more) {
                int t2, w2;
                const Item n2 = item_of(ph, b, G, r + 1, slot, wk, t2, w2);
                load_panel<QT>(nxt, n2.base, ph.slots, lane, n2.ok && lane < ph.slots);
            }
            mask_panel<QT>(cur, it.ok && lane < ph.slots);
            float acc[1] = {0.0f};
            const int unit = min(wk * ph.s_units + (lane >> 4), k_units - 1);
            multiply_panel<QT, 1>(cur, l, unit, k_units, acc);
            acc[0] += __shfl_xor(acc[0], 16);
            acc[0] += __shfl_xor(acc[0], 32);
            float* red = l.red + red_buf * (kChainWaves * 16);
            if (lane < 16) red[wave * 16 + lane] = acc[0];
            __syncthreads();
            if (wk == 0 && it.ok && lane < 16) {
                float sum = 0.0f;
                for (int w2 = 0; w2 < ph.nwk; w2++) sum += red[(slot * ph.nwk + w2) * 16 + lane];
                const int row = tile * 16 + lane;
                if (row < ph.wt[wi].n)
                    __hip_atomic_store(ph.wt[wi].y + row, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            red_buf ^= 1;
        }

        // this step's results are complete (only stores are outstanding here), then counted
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0)
            __hip_atomic_fetch_add(C.counters + (size_t)p * (kShards * kShardStride) + (b % kShards) * kShardStride, 1u,
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // The step after this one in which the workgroup has work: its first panel is requested now,
        // before that step's activations are awaited, so that it travels while the results of this
        // step become visible and the other workgroups finish.
        int q = p + 1;
        while (q < C.n_phases && b >= C.phases[q].tiles) q++;
        if (q < C.n_phases) {
            const ChainPhase& nx = C.phases[q];
            const int s2 = wave / nx.nwk, k2 = wave - s2 * nx.nwk;
            int t2, w2;
            const Item n2 = item_of(nx, b, G, 0, s2, k2, t2, w2);
            load_panel<QT>(nxt, n2.base, nx.slots, lane, n2.ok && lane < nx.slots);
            nxt_loaded = true;
        }
    }

    // Workgroup 0 leaves the counters at zero for the next launch, once the last step is complete
    // (then no workgroup polls any counter any more).
    if (b == 0) {
        wait_step(C, C.n_phases - 1, C.phases[C.n_phases - 1].participants);
        for (int i = threadIdx.x; i < C.n_phases * kShards; i += blockDim.x)
            __hip_atomic_store(C.counters + (size_t)i * kShardStride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

} // namespace

struct izwi_qmm_chain {
    int dtype = 0, device = 0, n_phases = 0, grid = 0;
    size_t lds = 0;
    ChainPhase* d_phases = nullptr;
    unsigned* d_counters = nullptr;
    unsigned* d_err = nullptr;
    unsigned spin_limit = 1u << 21; // polls of about 0.5 us each before a wait gives up
    ~izwi_qmm_chain() {
        if (d_phases) (void)hipFree(d_phases);
        if (d_counters) (void)hipFree(d_counters);
        if (d_err) (void)hipFree(d_err);
    }
};

namespace {

template <int QT>
hipError_t launch_chain(const izwi_qmm_chain* c, hipStream_t stream) {
    ChainParams P{c->d_phases, c->n_phases, c->d_counters, c->d_err, c->spin_limit};
    if (c->lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&chain_kernel<QT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
    }
    chain_kernel<QT><<<dim3((unsigned)c->grid), dim3(64 * kChainWaves), c->lds, stream>>>(P);
    return hipGetLastError();
}

template <int QT>
hipError_t chain_occupancy(size_t lds, int* blocks) {
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&chain_kernel<QT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
    }
    return hipOccupancyMaxActiveBlocksPerMultiprocessor(blocks, chain_kernel<QT>, 64 * kChainWaves, lds);
}

int fail_hip(hipError_t e, const char* what) {
    (void)hipGetLastError();
    return qmm_fail(IZWI_QMM_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

} // namespace

extern "C" {

int izwi_qmm_chain_create(const izwi_qmm_chain_step* steps, int32_t n_steps, izwi_qmm_chain** out) {
    return qmm_guarded("izwi_qmm_chain_create", [&]() -> int {
    if (!out) return qmm_fail(IZWI_QMM_ERR_INVALID, "out is NULL");
    *out = nullptr;
    if (!steps || n_steps < 1 || n_steps > 65536)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "a chain has 1..65536 steps, got %d", n_steps);
    int device = 0, n_cus = 0;
    if (int rc = qmm_current_device(&device, &n_cus)) return rc;
    int dtype = 0;
    size_t lds = 0;
    std::vector<ChainPhase> phases((size_t)n_steps);
    const int grid = n_cus; // one 12-wave workgroup per CU: every workgroup is resident for the whole launch
    for (int32_t p = 0; p < n_steps; p++) {
        const izwi_qmm_chain_step& st = steps[p];
        if (st.n_weights < 1 || st.n_weights > QMM_MAX_GROUP)
            return qmm_fail(IZWI_QMM_ERR_INVALID, "step %d: projection group of %d weights (1..%d supported)", p,
                            st.n_weights, QMM_MAX_GROUP);
        if (!st.x) return qmm_fail(IZWI_QMM_ERR_INVALID, "step %d: x is NULL", p);
        ChainPhase& ph = phases[(size_t)p];
        memset(&ph, 0, sizeof ph);
        int64_t tiles = 0;
        for (int i = 0; i < st.n_weights; i++) {
            const izwi_qmm_weight* w = st.weights[i];
            if (!w || !st.ys[i]) return qmm_fail(IZWI_QMM_ERR_INVALID, "step %d: NULL weight or output", p);
            const QmmLayout& L = *qmm_weight_layout(w);
            if (L.n_stacked != 1) return qmm_fail(IZWI_QMM_ERR_INVALID, "step %d: forward on an expert stack", p);
            if (qmm_weight_device(w) != device)
                return qmm_fail(IZWI_QMM_ERR_INVALID, "step %d: the weight lives on device %d, the current device is %d", p,
                                qmm_weight_device(w), device);
            if (p == 0 && i == 0) dtype = L.dtype;
            if (L.dtype != dtype)
                return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED,
                                "step %d: ggml dtype %d in a chain of dtype %d (a chain holds one block type)", p, L.dtype,
                                dtype);
            const QmmLayout& L0 = *qmm_weight_layout(st.weights[0]);
            if (L.k != L0.k)
                return qmm_fail(IZWI_QMM_ERR_INVALID, "step %d: projection group input mismatch: expected %lld, got %lld", p,
                                (long long)L0.k, (long long)L.k);
            // (a very tall matrix runs with another split along k in the per-call kernel: its sums would
            // differ in the last bit; it is streamed at full rate by a launch of its own anyway)
            if (L.n == 0 || L.k_groups > kChainWaves || L.n > (1 << 24) || L.row_tiles >= 16 * (int64_t)n_cus)
                return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED,
                                "step %d: shape [%lld, %lld] has no chained form (1 <= n < %d, k <= %d)", p,
                                (long long)L.n, (long long)L.k, 16 * 16 * n_cus, kChainWaves * 256 * L.s);
            tiles += L.row_tiles;
            ph.tile_end[i] = (int)tiles;
            ph.wt[i] = ChainWeight{static_cast<const uint8_t*>(qmm_weight_tiled(w)), st.ys[i], (int)L.n, 0};
            if (i == 0) {
                ph.k = (int)L.k, ph.k_units = (int)L.k_units, ph.k_groups = (int)L.k_groups, ph.slots = L.slots;
                ph.s_units = L.s, ph.panel_bytes = (int)L.panel_bytes;
                ph.nwk = (int)L.k_groups;
                ph.nwr = kChainWaves / ph.nwk;
            }
        }
        if (tiles > 0x3fffffff) return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED, "step %d: too many rows", p);
        ph.x = st.x;
        ph.n_weights = st.n_weights;
        ph.tiles = (int)tiles;
        ph.rounds = (int)((tiles + (int64_t)grid * ph.nwr - 1) / ((int64_t)grid * ph.nwr));
        ph.participants = (int)std::min<int64_t>(grid, tiles);
        const size_t need = dtype == IZWI_QMM_Q4_K   ? lds_bytes<QMM_Q4_K, 1>(ph.k_units, kChainWaves)
                            : dtype == IZWI_QMM_Q6_K ? lds_bytes<QMM_Q6_K, 1>(ph.k_units, kChainWaves)
                                                     : lds_bytes<QMM_Q8_0, 1>(ph.k_units, kChainWaves);
        lds = std::max(lds, need);
    }
    if (lds > 160 * 1024) return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED, "activations too long for the chained kernel");
    int blocks = 0;
    hipError_t e = dtype == IZWI_QMM_Q4_K   ? chain_occupancy<QMM_Q4_K>(lds, &blocks)
                   : dtype == IZWI_QMM_Q6_K ? chain_occupancy<QMM_Q6_K>(lds, &blocks)
                                            : chain_occupancy<QMM_Q8_0>(lds, &blocks);
    if (e != hipSuccess) return fail_hip(e, "occupancy query of the chained kernel");
    if (blocks < 1) return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED, "the chained kernel does not fit a compute unit");
    izwi_qmm_chain* c = new (std::nothrow) izwi_qmm_chain;
    if (!c) return qmm_fail(IZWI_QMM_ERR_INVALID, "out of memory");
    c->dtype = dtype, c->device = device, c->n_phases = n_steps, c->grid = grid, c->lds = lds;
    if (const char* s = getenv("IZWI_QMM_CHAIN_SPIN_LIMIT")) c->spin_limit = (unsigned)strtoul(s, nullptr, 10);
    const size_t counter_bytes = (size_t)n_steps * kShards * kShardStride * sizeof(unsigned);
    e = hipMalloc(&c->d_phases, phases.size() * sizeof(ChainPhase));
    if (e == hipSuccess) e = hipMalloc(&c->d_counters, counter_bytes);
    if (e == hipSuccess) e = hipMalloc(&c->d_err, 256);
    if (e == hipSuccess) e = hipMemcpy(c->d_phases, phases.data(), phases.size() * sizeof(ChainPhase), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemset(c->d_counters, 0, counter_bytes);
    if (e == hipSuccess) e = hipMemset(c->d_err, 0, 256);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        delete c;
        return fail_hip(e, "chain set-up");
    }
    *out = c;
    return IZWI_QMM_OK;
    });
}

void izwi_qmm_chain_destroy(izwi_qmm_chain* c) { delete c; }

int izwi_qmm_chain_set_spin_limit(izwi_qmm_chain* c, uint32_t polls) {
    return qmm_guarded("izwi_qmm_chain_set_spin_limit", [&]() -> int {
    if (!c) return qmm_fail(IZWI_QMM_ERR_INVALID, "NULL chain");
    c->spin_limit = polls;
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_chain_run(izwi_qmm_chain* c, void* stream) {
    return qmm_guarded("izwi_qmm_chain_run", [&]() -> int {
    if (!c) return qmm_fail(IZWI_QMM_ERR_INVALID, "NULL chain");
    hipError_t e = c->dtype == IZWI_QMM_Q4_K   ? launch_chain<QMM_Q4_K>(c, (hipStream_t)stream)
                   : c->dtype == IZWI_QMM_Q6_K ? launch_chain<QMM_Q6_K>(c, (hipStream_t)stream)
                                               : launch_chain<QMM_Q8_0>(c, (hipStream_t)stream);
    if (e != hipSuccess) return fail_hip(e, "chained decode kernel");
    return IZWI_QMM_OK;
    });
}

int izwi_qmm_chain_status(izwi_qmm_chain* c, void* stream) {
    return qmm_guarded("izwi_qmm_chain_status", [&]() -> int {
    if (!c) return qmm_fail(IZWI_QMM_ERR_INVALID, "NULL chain");
    hipError_t e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return fail_hip(e, "hipStreamSynchronize");
    unsigned err = 0;
    e = hipMemcpy(&err, c->d_err, sizeof err, hipMemcpyDeviceToHost);
    if (e != hipSuccess) return fail_hip(e, "reading the chain's error word");
    if (!err) return IZWI_QMM_OK;
    // a wait gave up: the counters are left mid-count; clear everything for the next run
    const size_t counter_bytes = (size_t)c->n_phases * kShards * kShardStride * sizeof(unsigned);
    (void)hipMemset(c->d_counters, 0, counter_bytes);
    (void)hipMemset(c->d_err, 0, 256);
    (void)hipDeviceSynchronize();
    return qmm_fail(IZWI_QMM_ERR_HIP,
                    "chained decode: a wait for an earlier step gave up after %u polls (results of that run are invalid)",
                    c->spin_limit);
    });
}

} // extern "C"
