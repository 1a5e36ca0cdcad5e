// Routing of one token by one wavefront (top-k of the logits, ties to the lower expert index,
// weights = softmax over the selected logits).  Shared by the routing kernels (qmm_moe.hip) and the
// small-batch expert kernels that route inside their own launch (qmm_gemv.hip); unnamed
// namespace, one copy per including file.
#ifndef IZWI_QMM_MOE_ROUTE_H
#define IZWI_QMM_MOE_ROUTE_H

#include <hip/hip_runtime.h>

namespace {
namespace moe_route {

constexpr int kRDppXor1 = 0xB1, kRDppXor2 = 0x4E, kRDppRor4 = 0x124, kRDppRor8 = 0x128;
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xf, 0xf, false);
}
// maximum over the 64 lanes, as a scalar: four DPP steps inside the 16-lane rows, then one
// lane of every row
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = max(v, dpp_u32<kRDppXor1>(v));
    v = max(v, dpp_u32<kRDppXor2>(v));
    v = max(v, dpp_u32<kRDppRor4>(v));
    v = max(v, dpp_u32<kRDppRor8>(v));
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return max(max(a, b), max(c, d));
}

// Order-preserving key of a logit: a larger logit has a larger key, equal logits (also -0 and
// +0) the same key, NaN the key 1 (below every number, so that the selection stays a total
// order), and 0 is left for "already taken / no such expert".
__device__ __forceinline__ uint32_t route_key(float v) {
    if (v != v) return 1u;
    uint32_t u = __float_as_uint(v);
    if (u == 0x80000000u) u = 0u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Routing of one token by one wavefront.  Lane l holds logits l, l+64, ...; top_k rounds of a
// wave-wide arg-max (larger logit first, lower expert index on ties): the maximum key by DPP,
// then the first lane (lowest index) that holds it by ballot.  Lane s < top_k returns slot s
// in (id, weight): weights = exp(l - lmax) over the selected slots, summed in slot order.
// `rounds` < top_k (uniform): only the slots below `rounds` are selected and no weight is worked out -
// for a caller that needs the expert of one slot (lane `rounds - 1` then holds its id).
template <int PER_LANE>
__device__ __forceinline__ void route_token(const float* __restrict__ row, int n_experts, int top_k, int lane,
                                            int& id, float& weight, int rounds = -1) {
    const bool ids_only = rounds >= 0 && rounds < top_k;
    const int n_rounds = ids_only ? rounds : top_k;
    float v[PER_LANE];
    uint32_t key[PER_LANE];
#pragma unroll
    for (int i = 0; i < PER_LANE; i++) {
        const int e = lane + 64 * i;
        v[i] = e < n_experts ? row[e] : 0.0f;
        key[i] = e < n_experts ? route_key(v[i]) : 0u;
    }
    float my_logit = 0.0f; // lane s keeps the logit of slot s
    int my_id = 0;
    float lmax = 0.0f;
    for (int s = 0; s < n_rounds; s++) {
        uint32_t kbest = 0;
#pragma unroll
        for (int i = 0; i < PER_LANE; i++) kbest = max(kbest, key[i]);
        const uint32_t wmax = wave_max_u32(kbest);
        int win = -1; // uniform
        float bv = 0.0f;
#pragma unroll
        for (int i = 0; i < PER_LANE; i++) {
            const unsigned long long holders = __ballot(key[i] == wmax);
            if (win < 0 && holders != 0) {
                const int l = __ffsll((long long)holders) - 1;
                win = l + 64 * i;
                bv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v[i]), l));
                if (lane == l) key[i] = 0u; // taken
            }
        }
        if (s == 0) lmax = bv;
        if (lane == s) {
            my_logit = bv;
            my_id = win;
        }
    }
    if (ids_only) {
        id = my_id;
        weight = 0.0f;
        return;
    }
    const float p = lane < top_k ? expf(my_logit - lmax) : 0.0f;
    float denom = 0.0f; // (slot s from lane s, a scalar read: a shuffle goes through the LDS crossbar)
    for (int s = 0; s < top_k; s++) denom += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), s));
    id = my_id;
    weight = p / denom;
}

} // namespace moe_route
} // namespace

#endif // IZWI_QMM_MOE_ROUTE_H
