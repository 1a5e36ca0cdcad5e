// Prefill, plane form: the weights of a call are dequantized ONCE into a bf16 plane in scratch
// memory, and the product is a plain bf16 matrix-core loop whose two operands go from global
// memory to LDS with LDS-direct loads (no staging registers, no LDS write instructions, no
// dequantization arithmetic between the matrix instructions).
//
// The in-LDS form (qmm_gemm.hip) dequantizes every weight once per 256-row tile of activations -
// eight times at m = 2048 - between its matrix instructions; this form pays one HBM-bound pass
// over the weights per call instead.  Measured on the 8B shapes the matmul loop alone is about a
// tenth faster than the in-LDS kernel and the pass costs as much again, so the in-LDS form stays
// the default and this one is selected explicitly (izwi_qmm_set_prefill_form).
//
// Plane layout: the LDS image itself.  Block (t, s) = rows 256 t .. 256 t + 255 of the matrix,
// k elements 64 s .. 64 s + 63: 256 rows of 128 bytes; the 16-byte chunk c of row r sits at
// chunk position c ^ ((r >> 1) & 7), so that the 16 lanes of a quarter wave that read one chunk
// of 16 consecutive rows touch every LDS bank once.  Blocks are ordered [t][s]: a workgroup's
// weight tile of one k step is one contiguous run of 32 KiB (16 KiB for a 128-row tile).
// The activations stay row-major in global memory; their lanes pick the chunk that belongs to
// their LDS position.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "qmm_internal.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kRowBytes = 128;                  // 64 bf16: one tile row of one k step
constexpr int kBlockRows = 256;                 // rows of a plane block
constexpr int kBlockBytes = kBlockRows * kRowBytes;

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 v = {(__bf16)a, (__bf16)b}; // round to nearest even
    return __builtin_bit_cast(uint32_t, v);
}
template <int N>
__device__ __forceinline__ float ubyte_f32(uint32_t v) {
    return (float)((v >> (8 * N)) & 0xffu);
}

struct PlaneDequantParams {
    const uint8_t* w;
    uint16_t* plane;
    int64_t k_groups, panel_bytes, k_units;
    int s, slots, ksteps;
    int64_t waves; // row_tiles * k_groups * s * 2
};

// One wave = eight rows of one unit (256 k elements = four k steps); lane = (row, chunk position).
// Per k step a lane dequantizes the eight elements that belong at its chunk position and the
// wave's store is 1 KiB in one piece (eight whole plane rows).  The quants come as 8-byte loads
// (two lanes per nibble run read the same bytes; the panels are a fifth of the bytes moved and
// come through the caches).  The arithmetic is the in-LDS kernel's: fma(d * scale, q, -(dmin * min)),
// rounded to bf16 once.
template <int QT>
__global__ __launch_bounds__(256) void plane_dequant_kernel(PlaneDequantParams P) {
    const int64_t g = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (g >= P.waves) return;
    const int lane = threadIdx.x & 63, p = lane & 7, r8 = lane >> 3;
    const int half = (int)(g & 1);
    const int64_t gu = g >> 1;
    const int us = (int)(gu % P.s);
    const int64_t panel = gu / P.s;
    const int64_t rt = panel / P.k_groups;
    const int kg = (int)(panel - rt * P.k_groups);
    const int64_t unit = (int64_t)kg * P.s + us;
    if (unit >= P.k_units) return;
    const int slot = us * 16 + half * 8 + r8;
    const int64_t row = rt * 16 + half * 8 + r8;
    const int r = (int)(row & (kBlockRows - 1));
    const int c = p ^ ((r >> 1) & 7); // the logical chunk at this position: elements 8 c .. 8 c + 7 of a k step
    const uint8_t* base = P.w + panel * P.panel_bytes + (size_t)slot * 16;
    const size_t chunk_stride = (size_t)P.slots * 16;
    const u32x4 hdr = *reinterpret_cast<const u32x4*>(base);
    uint8_t* dst = reinterpret_cast<uint8_t*>(P.plane) + ((row >> 8) * P.ksteps + unit * 4) * (int64_t)kBlockBytes +
                   (int64_t)r * kRowBytes + p * 16;
    uint2 q[4];
    if (QT == QMM_Q4_K) {
        // k step j = sub-block pair j: nibble bytes 32 j .. 32 j + 31 (chunks 2 j, 2 j + 1); elements
        // 0..31 are the low nibbles, 32..63 the high ones
#pragma unroll
        for (int j = 0; j < 4; j++)
            q[j] = *reinterpret_cast<const uint2*>(base + (size_t)(1 + 2 * j + ((c & 3) >> 1)) * chunk_stride + (c & 1) * 8);
        const float d = qmm_f16_bits_to_f32((uint16_t)(hdr.x & 0xffffu));
        const float dmin = qmm_f16_bits_to_f32((uint16_t)(hdr.x >> 16));
        uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
        qmm_unpack_q4k_scales(hdr.y, hdr.z, hdr.w, sc_lo, sc_hi, mn_lo, mn_hi);
        const int hi = c >> 2;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (unit * 4 + j >= P.ksteps) break;
            const float ds = d * (float)qmm_byte_of(sc_lo, sc_hi, 2 * j + hi);
            const float ms = -(dmin * (float)qmm_byte_of(mn_lo, mn_hi, 2 * j + hi));
            const uint32_t v0 = (hi ? q[j].x >> 4 : q[j].x) & 0x0f0f0f0fu, v1 = (hi ? q[j].y >> 4 : q[j].y) & 0x0f0f0f0fu;
            uint4 o;
            o.x = pack_bf16(__builtin_fmaf(ds, ubyte_f32<0>(v0), ms), __builtin_fmaf(ds, ubyte_f32<1>(v0), ms));
            o.y = pack_bf16(__builtin_fmaf(ds, ubyte_f32<2>(v0), ms), __builtin_fmaf(ds, ubyte_f32<3>(v0), ms));
            o.z = pack_bf16(__builtin_fmaf(ds, ubyte_f32<0>(v1), ms), __builtin_fmaf(ds, ubyte_f32<1>(v1), ms));
            o.w = pack_bf16(__builtin_fmaf(ds, ubyte_f32<2>(v1), ms), __builtin_fmaf(ds, ubyte_f32<3>(v1), ms));
            *reinterpret_cast<uint4*>(dst + (size_t)j * kBlockBytes) = o;
        }
    } else {
        // Q8_0: k step j = blocks 2 j, 2 j + 1 of the unit (chunks 4 j .. 4 j + 3, 16 int8 each)
#pragma unroll
        for (int j = 0; j < 4; j++)
            q[j] = *reinterpret_cast<const uint2*>(base + (size_t)(1 + 4 * j + (c >> 1)) * chunk_stride + (c & 1) * 8);
        const uint32_t hw[4] = {hdr.x, hdr.y, hdr.z, hdr.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (unit * 4 + j >= P.ksteps) break;
            const float dd = qmm_f16_bits_to_f32((uint16_t)((c >> 2) ? hw[j] >> 16 : hw[j] & 0xffffu));
            const float bias = -128.0f * dd; // int8 q as unsigned byte u = q + 128
            const uint32_t v0 = q[j].x ^ 0x80808080u, v1 = q[j].y ^ 0x80808080u;
            uint4 o;
            o.x = pack_bf16(__builtin_fmaf(dd, ubyte_f32<0>(v0), bias), __builtin_fmaf(dd, ubyte_f32<1>(v0), bias));
            o.y = pack_bf16(__builtin_fmaf(dd, ubyte_f32<2>(v0), bias), __builtin_fmaf(dd, ubyte_f32<3>(v0), bias));
            o.z = pack_bf16(__builtin_fmaf(dd, ubyte_f32<0>(v1), bias), __builtin_fmaf(dd, ubyte_f32<1>(v1), bias));
            o.w = pack_bf16(__builtin_fmaf(dd, ubyte_f32<2>(v1), bias), __builtin_fmaf(dd, ubyte_f32<3>(v1), bias));
            *reinterpret_cast<uint4*>(dst + (size_t)j * kBlockBytes) = o;
        }
    }
}

template <int N, class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl<N>(f, std::make_integer_sequence<int, N>{});
}

struct PlaneGemmParams {
    const uint16_t* x; // bf16 [m, k]
    int64_t m, k;
    int ksteps;
    int tiles_m, tiles_n; // tiles_n: all members' column tiles
    int n_weights;        // >= 1
    int tn_end[QMM_MAX_GROUP];
    const uint16_t* plane_v[QMM_MAX_GROUP];
    void* y_v[QMM_MAX_GROUP];
    int64_t n_v[QMM_MAX_GROUP];
    int out_bf16;
    const void* residual; // single weight only
};

// 16 bytes per lane from global memory straight into LDS: lane l's bytes land at lds + 16 l.
__device__ __forceinline__ void load_to_lds(const uint8_t* base, uint32_t lane_off, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(lane_off), "s"(base) : "memory", "m0");
}

// BM x BN output tile, NW waves as an (NW / 2) x 2 grid, NS LDS stages of one 64-wide k step.
// The k loop has one barrier per step, at the three-quarter point: by then every fragment of the
// step is in registers, so the stage is free for the loads of step kt + NS, and the first
// fragments of step kt + 1 (landed: the wait in front of the barrier) are read behind the last
// quarter of the matrix instructions.
template <int BM, int BN, int NW, int NS, int ABL = 0>
__global__ __launch_bounds__(64 * NW) void gemm_plane_kernel(PlaneGemmParams P) {
    constexpr int WM = NW / 2;
    constexpr int MT = BM / WM / 32, NT = BN / 64;
    constexpr int kStage = (BM + BN) * kRowBytes;
    constexpr int XL = BM / 8 / NW, WL = BN / 8 / NW; // LDS-direct loads per wave and k step
    constexpr int LPT = XL + WL;
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0 && (4 * NW) % 8 == 0, "loads are spread evenly over the waves");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    // Workgroups go to the eight XCDs round-robin by their index, and every XCD has its own L2:
    // index = 8 * slot + xcd, and an XCD walks all row tiles of a column tile before the next
    // column tile, so a weight tile is fetched from memory by one XCD only and the activations
    // (small) by all of them.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int tm = slot % P.tiles_m;
    int tn = (slot / P.tiles_m) * 8 + xcd;
    if (tn >= P.tiles_n) return; // uniform
    int member = 0;
    while (member + 1 < P.n_weights && tn >= P.tn_end[member]) member++;
    tn -= member ? P.tn_end[member - 1] : 0;
    const int64_t n = P.n_v[member];
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- loads: instruction q of a tile covers rows 8 q .. 8 q + 7 (1 KiB of the stage)
    const uint8_t* x_tile = reinterpret_cast<const uint8_t*>(P.x) + m0 * P.k * 2;
    uint32_t x_off[XL];
    {
        const int r8 = lane >> 3, p = lane & 7;
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const int row = 8 * (wave + NW * i) + r8;
            const int c = p ^ ((row >> 1) & 7);
            x_off[i] = (uint32_t)((min(m0 + row, P.m - 1) - m0) * P.k * 2 + c * 16);
        }
    }
    const uint8_t* w_tile = reinterpret_cast<const uint8_t*>(P.plane_v[member]) +
                            (n0 >> 8) * (int64_t)P.ksteps * kBlockBytes + (n0 & 255) * kRowBytes;
    const uint32_t w_off = (uint32_t)(wave * 1024 + lane * 16);
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const int last = P.ksteps - 1;
    auto issue_tile = [&](int kt, int stage) {
        const int t = min(kt, last); // past the end: the last tile again, into a stage nobody reads
        const uint8_t* xs = x_tile + (size_t)t * kRowBytes;
        const uint8_t* ws = w_tile + (size_t)t * kBlockBytes;
        const uint32_t base = lds0 + stage * kStage + wave * 1024;
#pragma unroll
        for (int i = 0; i < XL; i++) load_to_lds(xs, x_off[i], base + i * NW * 1024);
#pragma unroll
        for (int i = 0; i < WL; i++) load_to_lds(ws, w_off + i * NW * 1024, base + BM * kRowBytes + i * NW * 1024);
    };

    f32x16 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // ---- fragments: lane l reads row (l & 31) of a 32-row block, chunk 2 kk + (l >> 5)
    const int sw = (lane >> 1) & 7;
    const int ch0 = ((lane >> 5) ^ sw) << 4; // chunk position of k16 step 0; step kk: ^ (kk << 5)
    const int frag_x = (wm * (BM / WM) + (lane & 31)) * kRowBytes + ch0;
    const int frag_w = (BM + wn * (BN / 2) + (lane & 31)) * kRowBytes + ch0;
    bf16x8 fa[2][MT], fb[2][NT];
    auto read_frags = [&](const uint8_t* stage, int kk, int set) {
#pragma unroll
        for (int j = 0; j < NT; j++)
            fb[set][j] = *reinterpret_cast<const bf16x8*>(stage + ((frag_w + j * 32 * kRowBytes) ^ (kk << 5)));
#pragma unroll
        for (int i = 0; i < MT; i++)
            fa[set][i] = *reinterpret_cast<const bf16x8*>(stage + ((frag_x + i * 32 * kRowBytes) ^ (kk << 5)));
    };

#pragma unroll
    for (int s = 0; s < NS; s++) issue_tile(s, s);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NS - 1) * LPT) : "memory");
    read_frags(smem, 0, 0);

    int cur = 0;
    for (int kt = 0; kt < P.ksteps; kt++) {
        const int nxt = cur + 1 == NS ? 0 : cur + 1;
        const uint8_t* cs = smem + cur * kStage;
        const uint8_t* ns = smem + nxt * kStage;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            if (kk == 3) {
                // every fragment of this step is in registers; step kt + 1 has landed for this wave
                if (ABL == 2 || ABL == 4) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((NS - 2) * LPT) : "memory");
                else asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((NS - 2) * LPT) : "memory");
                if (ABL == 0 || ABL == 3) issue_tile(kt + NS, cur);
            }
            if (ABL < 3) read_frags(kk < 3 ? cs : ns, (kk + 1) & 3, (kk + 1) & 1);
#pragma unroll
            for (int i = 0; i < MT; i++)
#pragma unroll
                for (int j = 0; j < NT; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[kk & 1][i], fb[kk & 1][j], acc[i][j], 0, 0, 0);
            // one matrix instruction, then one of the next step's fragment reads, while any remain
#pragma unroll
            for (int q = 0; q < MT * NT; q++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if (q < MT + NT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
        }
        cur = nxt;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the loads past the end

    // D[i][j]: lane holds column j = lane % 32 and rows 8 (r / 4) + 4 (lane / 32) + r % 4
    void* y = P.y_v[member];
    const QmmEpilogue ep{P.residual, P.out_bf16};
    const bool full = m0 + BM <= P.m && n0 + BN <= n; // uniform
    const int64_t gm_base = m0 + wm * (BM / WM) + 4 * (lane >> 5);
    const int64_t gn_base = n0 + wn * (BN / 2) + (lane & 31);
    static_for<MT>([&](auto I) {
        static_for<NT>([&](auto J) {
            constexpr int i = decltype(I)::value, j = decltype(J)::value;
            const int64_t gn = gn_base + j * 32;
            static_for<16>([&](auto R) {
                constexpr int r = decltype(R)::value;
                const int64_t gm = gm_base + i * 32 + 8 * (r >> 2) + (r & 3);
                float v = acc[i][j][r];
                // (with 256 accumulators they sit in the accumulation registers; read one by one here, or the
                // compiler moves all of them to ordinary registers at once behind the loop and spills)
                if constexpr (MT * NT == 16) asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(acc[i][j][r]));
                if (full || (gm < P.m && gn < n)) qmm_store(y, ep, gm * n + gn, v);
            });
            __builtin_amdgcn_sched_barrier(0); // tile by tile: the accumulators leave their registers as they are stored
        });
    });
}

template <int BM, int BN, int NW, int NS, int ABL = 0>
hipError_t launch_plane_tile(PlaneGemmParams P, hipStream_t stream) {
    P.tiles_m = (int)((P.m + BM - 1) / BM);
    int64_t t = 0;
    for (int i = 0; i < P.n_weights; i++) P.tn_end[i] = (int)(t += (P.n_v[i] + BN - 1) / BN);
    P.tiles_n = (int)t;
    const int64_t grid = (int64_t)P.tiles_m * ((P.tiles_n + 7) / 8) * 8;
    if (grid > 0x7fffffff) return hipErrorInvalidValue;
    constexpr size_t lds = (size_t)NS * (BM + BN) * kRowBytes;
    static_assert(lds <= 160 * 1024, "LDS of a CU");
    auto fn = &gemm_plane_kernel<BM, BN, NW, NS, ABL>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    fn<<<dim3((unsigned)grid), dim3(64 * NW), lds, stream>>>(P);
    return hipGetLastError();
}

// 0: in-LDS form always; 1: plane form wherever it can run (m > 128); -1: by size (today: in-LDS)
int plane_mode() {
    static const int mode = [] {
        const char* e = getenv("IZWI_QMM_PREFILL_FORM");
        if (e && (e[0] == 'l' || e[0] == 'L')) return 0; // "lds"
        if (e && (e[0] == 'p' || e[0] == 'P')) return 1; // "plane"
        return -1;
    }();
    return mode;
}
std::atomic<int> g_plane_override{-2};

int plane_tile_override() {
    static const int t = [] {
        const char* e = getenv("IZWI_QMM_PLANE_TILE"); // tuning aid: 0..3, see launch_plane
        return e && e[0] >= '0' && e[0] <= '9' ? atoi(e) : -1;
    }();
    return t;
}

int64_t plane_rows(int64_t n) { return (n + kBlockRows - 1) / kBlockRows * kBlockRows; }

hipError_t launch_plane(const PlaneGemmParams& P, int64_t n_total, int n_cus, hipStream_t stream) {
    // 256 x 256 tiles when they fill the chip, 256 x 128 otherwise
    const int64_t tm = (P.m + 255) / 256;
    int64_t t256 = 0;
    for (int i = 0; i < P.n_weights; i++) t256 += tm * ((P.n_v[i] + 255) / 256);
    int choice = t256 >= 2 * (int64_t)n_cus || (t256 % n_cus == 0 && t256 >= n_cus) ? 0 : 1;
    if (plane_tile_override() >= 0) choice = plane_tile_override();
    (void)n_total;
    switch (choice) {
        case 0: return launch_plane_tile<256, 256, 8, 2>(P, stream);
#ifdef QMM_PLANE_ABLATIONS
        case 5: return launch_plane_tile<256, 256, 8, 2, 1>(P, stream);
        case 6: return launch_plane_tile<256, 256, 8, 2, 2>(P, stream);
        case 7: return launch_plane_tile<256, 256, 8, 2, 3>(P, stream);
        case 8: return launch_plane_tile<256, 256, 8, 2, 4>(P, stream);
        case 9: return launch_plane_tile<256, 256, 4, 2, 1>(P, stream);
        case 10: return launch_plane_tile<256, 256, 4, 2, 3>(P, stream);
        case 11: return launch_plane_tile<256, 256, 4, 2, 4>(P, stream);
#endif
        case 1: return launch_plane_tile<256, 128, 8, 3>(P, stream);
        case 2: return launch_plane_tile<256, 256, 4, 2>(P, stream);
        default: return launch_plane_tile<256, 128, 4, 3>(P, stream);
    }
}

} // namespace

void qmm_set_prefill_form(int form) { g_plane_override.store(form, std::memory_order_relaxed); }
int qmm_get_prefill_form() {
    const int o = g_plane_override.load(std::memory_order_relaxed);
    return o != -2 ? o : plane_mode();
}

bool qmm_gemm_plane_applies(const QmmLayout& L, int64_t m) {
    if (L.dtype != QMM_Q4_K && L.dtype != QMM_Q8_0) return false;
    if (L.n_stacked != 1 || (L.k & 63) != 0 || m <= 128 || L.n == 0) return false;
    const int mode = qmm_get_prefill_form();
    if (mode == 0) return false;
    // by size: the in-LDS form (it is the faster one at every size measured, up to 4096 rows on the
    // 8B shapes: the pass that writes the plane costs more than the matmul loop gains)
    return mode == 1;
}

size_t qmm_gemm_plane_bytes(const QmmLayout& L) { return (size_t)plane_rows(L.n) * (size_t)L.k * sizeof(uint16_t); }

hipError_t qmm_launch_plane_dequant(const QmmLayout& L, const void* tiled, uint16_t* plane, hipStream_t stream) {
    PlaneDequantParams D;
    D.w = (const uint8_t*)tiled;
    D.plane = plane;
    D.k_groups = L.k_groups, D.panel_bytes = L.panel_bytes, D.k_units = L.k_units;
    D.s = L.s, D.slots = L.slots, D.ksteps = (int)(L.k / 64);
    D.waves = L.row_tiles * L.k_groups * L.s * 2;
    const int64_t blocks = (D.waves + 3) / 4;
    if (blocks > 0x7fffffff) return hipErrorInvalidValue;
    if (L.dtype == QMM_Q4_K) plane_dequant_kernel<QMM_Q4_K><<<(unsigned)blocks, 256, 0, stream>>>(D);
    else plane_dequant_kernel<QMM_Q8_0><<<(unsigned)blocks, 256, 0, stream>>>(D);
    return hipGetLastError();
}

hipError_t qmm_launch_gemm_plane(const QmmLayout* const* layouts, const void* const* tiled, int n_weights,
                                 const uint16_t* x_bf16, int64_t m, void* const* ys, int out_bf16, void* planes,
                                 int n_cus, hipStream_t stream, const void* residual) {
    if (n_weights < 1 || n_weights > QMM_MAX_GROUP) return hipErrorInvalidValue;
    PlaneGemmParams P;
    P.x = x_bf16;
    P.m = m;
    P.k = layouts[0]->k;
    P.ksteps = (int)(P.k / 64);
    P.tiles_m = P.tiles_n = 0;
    P.n_weights = n_weights;
    P.out_bf16 = out_bf16;
    P.residual = n_weights == 1 ? residual : nullptr;
    uint8_t* next = (uint8_t*)planes;
    int64_t n_total = 0;
    for (int i = 0; i < QMM_MAX_GROUP; i++) P.tn_end[i] = 0, P.plane_v[i] = nullptr, P.y_v[i] = nullptr, P.n_v[i] = 0;
    for (int i = 0; i < n_weights; i++) {
        const QmmLayout& L = *layouts[i];
        if (L.k != P.k || !qmm_gemm_plane_applies(L, m)) return hipErrorInvalidValue;
        hipError_t e = qmm_launch_plane_dequant(L, tiled[i], (uint16_t*)next, stream);
        if (e != hipSuccess) return e;
        P.plane_v[i] = (const uint16_t*)next;
        P.y_v[i] = ys[i];
        P.n_v[i] = L.n;
        n_total += L.n;
        next += qmm_gemm_plane_bytes(L);
    }
    return launch_plane(P, n_total, n_cus > 0 ? n_cus : 1, stream);
}
