// A feed-forward made of many small ones ("experts") of which a router picks a few per row, and the two gate units of feed-forwards
// whose activation is more than one function of one number.
//
// The routed experts run as ONE up product over all experts' matrices laid behind each other and ONE down product over their down
// matrices laid side by side: between the two, `expert_unit` multiplies every expert's hidden units by the row's weight for that
// expert, which is zero for the experts the router did not pick, so the down product's sum over all hidden units is the weighted sum
// over the picked experts. Nothing is planned on the host and no row's result depends on the other rows of the batch.
#include "common.h"

#include <math.h>

namespace {

constexpr int ROUTE_MAX_EXPERTS = 1024;

// (value, index) a is picked before b: the larger value, among equals the smaller index.
__device__ __forceinline__ bool picked_before(float a, int ia, float b, int ib) { return a > b || (a == b && ia < ib); }

// One wave a row. logits: the router's 32-bit sums [row, n_experts] (rows `stride` apart). Scores s = softmax over all n_experts;
// choice c = s + correction (null: none). The experts form n_groups equal groups of neighbours; a group's rank goes by the largest c
// in it, and only experts of the best `keep` groups can be picked (the others count as minus infinity). The `top` experts of largest
// c are picked; weights[row, e] = s_e / (sum of the picked experts' s + floor) for them and 0 for all others.
__global__ __launch_bounds__(WAVE) void route_kernel(const float* __restrict__ logits, int stride, const float* __restrict__ correction,
                                                     float* __restrict__ weights, int weights_stride, int n_experts, int top, int n_groups, int keep,
                                                     float floor) {
    __shared__ float score[ROUTE_MAX_EXPERTS], choice[ROUTE_MAX_EXPERTS], group_best[ROUTE_MAX_EXPERTS];
    const int lane = threadIdx.x, row = blockIdx.x;
    const float* z = logits + (size_t)row * stride;
    float largest = -INFINITY;
    for (int e = lane; e < n_experts; e += WAVE) largest = fmaxf(largest, z[e]);
    largest = wave_max(largest);
    float total = 0.0f;
    for (int e = lane; e < n_experts; e += WAVE) {
        const float p = expf(z[e] - largest);
        score[e] = p;
        total += p;
    }
    total = wave_sum(total);
    for (int e = lane; e < n_experts; e += WAVE) {
        const float s = score[e] / total;
        score[e] = s;
        choice[e] = s + (correction ? correction[e] : 0.0f);
    }
    __syncthreads();
    const int size = n_experts / n_groups;
    for (int g = lane; g < n_groups; g += WAVE) {
        float best = -INFINITY;
        for (int e = g * size; e < (g + 1) * size; e++) best = fmaxf(best, choice[e]);
        group_best[g] = best;
    }
    __syncthreads();
    for (int g = lane; g < n_groups; g += WAVE) {   // a group is kept if fewer than `keep` groups come before it
        const float mine = group_best[g];
        int before = 0;
        for (int o = 0; o < n_groups; o++) before += picked_before(group_best[o], o, mine, g) ? 1 : 0;
        if (before >= keep)
            for (int e = g * size; e < (g + 1) * size; e++) choice[e] = -INFINITY;
    }
    __syncthreads();
    float picked_sum = 0.0f;
    for (int e = lane; e < n_experts; e += WAVE) {
        const float mine = choice[e];
        int before = 0;
        for (int o = 0; o < n_experts; o++) before += picked_before(choice[o], o, mine, e) ? 1 : 0;
        const bool picked = before < top && mine > -INFINITY;
        picked_sum += picked ? score[e] : 0.0f;
        group_best[e] = picked ? 1.0f : 0.0f;   // every lane reads and writes its own experts' entries only from here on
    }
    picked_sum = wave_sum(picked_sum) + floor;
    for (int e = lane; e < n_experts; e += WAVE) weights[(size_t)row * weights_stride + e] = group_best[e] != 0.0f ? score[e] / picked_sum : 0.0f;
}

// up: [rows, n_routed * ff + shared] hidden units before their activation, expert by expert, then `shared` units of an expert that
// every row uses. out = relu(up)^2 * weights[row, expert] (shared units: relu(up)^2). Behind the `unit_blocks` blocks of the hidden units
// the grid goes on over `width` columns of `carried` (null: none): carried[row, :] = h[row, :] * (the sum of weights[row, n_routed ..
// n_routed + n_identity)), the share of the experts that hand their input on as it is. PIECES: a thread takes 16 bytes of units (ff and
// shared are multiples of that many units, so a piece lies in one expert).
template <typename T, bool PIECES>
__global__ __launch_bounds__(256) void expert_unit_kernel(const T* __restrict__ up, T* __restrict__ out, const float* __restrict__ weights, int weights_stride,
                                                          int n_routed, int ff, int shared, const T* __restrict__ h, float* __restrict__ carried,
                                                          int n_identity, int width, int unit_blocks) {
    constexpr int VEC = PIECES ? 16 / (int)sizeof(T) : 1;
    const int inner = n_routed * ff + shared;
    const size_t row = blockIdx.y;
    const float* w = weights + row * weights_stride;
    if ((int)blockIdx.x >= unit_blocks) {
        const int j = ((int)blockIdx.x - unit_blocks) * blockDim.x + threadIdx.x;
        if (carried == nullptr || j >= width) return;
        float share = 0.0f;
        for (int e = 0; e < n_identity; e++) share += w[n_routed + e];
        carried[row * width + j] = to_float(h[row * width + j]) * share;
        return;
    }
    const int j = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (j >= inner) return;
    const float weight = j < n_routed * ff ? w[j / ff] : 1.0f;
    if constexpr (PIECES) {
        const Vec16 in = *reinterpret_cast<const Vec16*>(up + row * inner + j);
        Vec16 result;
        const T* ie = reinterpret_cast<const T*>(&in);
        T* re = reinterpret_cast<T*>(&result);
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            const float u = fmaxf(to_float(ie[e]), 0.0f);
            re[e] = from_float<T>(u * u * weight);
        }
        *reinterpret_cast<Vec16*>(out + row * inner + j) = result;
    } else {
        const float u = fmaxf(to_float(up[row * inner + j]), 0.0f);
        out[row * inner + j] = from_float<T>(u * u * weight);
    }
}

// both: [rows, 2 * inner], a gate half and an up half. out = g * sigmoid(alpha * g) * (u + shift) with g = min(gate, limit) and u =
// clamp(up, -limit, limit) (limit infinite: unclamped). PIECES: a thread takes 16 bytes of each half.
template <typename T, bool PIECES>
__global__ __launch_bounds__(256) void gate_unit_kernel(const T* __restrict__ both, T* __restrict__ out, int inner, float limit, float alpha, float shift) {
    constexpr int VEC = PIECES ? 16 / (int)sizeof(T) : 1;
    const int j = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (j >= inner) return;
    const size_t row = blockIdx.y;
    const T* g_at = both + row * 2 * inner + j;
    const T* u_at = g_at + inner;
    T* out_at = out + row * inner + j;
    if constexpr (PIECES) {
        const Vec16 gs = *reinterpret_cast<const Vec16*>(g_at), us = *reinterpret_cast<const Vec16*>(u_at);
        Vec16 result;
        const T* ge = reinterpret_cast<const T*>(&gs);
        const T* ue = reinterpret_cast<const T*>(&us);
        T* re = reinterpret_cast<T*>(&result);
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            const float g = fminf(to_float(ge[e]), limit);
            const float u = fminf(fmaxf(to_float(ue[e]), -limit), limit);
            re[e] = from_float<T>(g / (1.0f + expf(-alpha * g)) * (u + shift));
        }
        *reinterpret_cast<Vec16*>(out_at) = result;
    } else {
        const float g = fminf(to_float(*g_at), limit);
        const float u = fminf(fmaxf(to_float(*u_at), -limit), limit);
        *out_at = from_float<T>(g / (1.0f + expf(-alpha * g)) * (u + shift));
    }
}

template <typename T>
void launch_expert_unit(const void* up, void* out, const float* weights, int weights_stride, int rows, int n_routed, int ff, int shared, const void* h,
                        float* carried, int n_identity, int width, hipStream_t stream) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const int inner = n_routed * ff + shared;
    const bool pieces = ff % VEC == 0 && shared % VEC == 0 && ((uintptr_t)up & 15) == 0 && ((uintptr_t)out & 15) == 0;
    const int unit_blocks = ceil_div(pieces ? inner / VEC : inner, 256);
    dim3 grid(unit_blocks + (carried != nullptr ? ceil_div(width, 256) : 0), rows);
    if (pieces)
        expert_unit_kernel<T, true><<<grid, 256, 0, stream>>>((const T*)up, (T*)out, weights, weights_stride, n_routed, ff, shared, (const T*)h, carried, n_identity,
                                                              width, unit_blocks);
    else
        expert_unit_kernel<T, false><<<grid, 256, 0, stream>>>((const T*)up, (T*)out, weights, weights_stride, n_routed, ff, shared, (const T*)h, carried, n_identity,
                                                               width, unit_blocks);
}

template <typename T>
void launch_gate_unit(const void* both, void* out, int rows, int inner, float limit, float alpha, float shift, hipStream_t stream) {
    constexpr int VEC = 16 / (int)sizeof(T);
    if (inner % VEC == 0 && ((uintptr_t)both & 15) == 0 && ((uintptr_t)out & 15) == 0) {
        dim3 grid(ceil_div(inner / VEC, 256), rows);
        gate_unit_kernel<T, true><<<grid, 256, 0, stream>>>((const T*)both, (T*)out, inner, limit, alpha, shift);
    } else {
        dim3 grid(ceil_div(inner, 256), rows);
        gate_unit_kernel<T, false><<<grid, 256, 0, stream>>>((const T*)both, (T*)out, inner, limit, alpha, shift);
    }
}

}  // namespace

MLLM_API int mllm_route(const float* logits, int stride, const float* correction, float* weights, int weights_stride, int n_rows, int n_experts, int top,
                        int n_groups, int keep, float floor, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_experts > 0 && n_experts <= ROUTE_MAX_EXPERTS, "route: %d experts (the kernel takes up to %d)", n_experts, ROUTE_MAX_EXPERTS);
    MLLM_REQUIRE(n_groups >= 1 && n_experts % n_groups == 0 && keep >= 1 && keep <= n_groups, "route: %d experts in %d groups of which %d are kept", n_experts, n_groups, keep);
    MLLM_REQUIRE(top >= 1 && top <= keep * (n_experts / n_groups), "route: %d experts to pick among %d groups of %d", top, keep, n_experts / n_groups);
    MLLM_REQUIRE(stride >= n_experts && weights_stride >= n_experts && logits != nullptr && weights != nullptr, "route: rows are too short or missing");
    if (n_rows == 0) return 0;
    mllm_count_kernel(MLLM_K_ROUTE);
    route_kernel<<<n_rows, WAVE, 0, stream>>>(logits, stride, correction, weights, weights_stride, n_experts, top, n_groups, keep, floor);
    return mllm_check_launch("route");
}

MLLM_API int mllm_expert_unit(const void* up, void* out, const float* weights, int weights_stride, int n_rows, int n_routed, int ff, int shared, const void* h,
                              float* carried, int n_identity, int width, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_routed >= 0 && ff > 0 && shared >= 0 && n_identity >= 0, "expert_unit: bad sizes");
    MLLM_REQUIRE(weights_stride >= n_routed + n_identity && up != nullptr && out != nullptr && weights != nullptr, "expert_unit: a missing operand or short weights");
    MLLM_REQUIRE(carried == nullptr || (h != nullptr && width > 0), "expert_unit: the rows that are handed on need the input rows");
    MLLM_REQUIRE(dtype == MLLM_F32 || dtype == MLLM_BF16, "expert_unit: unknown dtype %d", dtype);
    if (n_rows == 0) return 0;
    mllm_count_kernel(MLLM_K_EXPERT_UNIT);
    const long long inner = (long long)n_routed * ff + shared;
    const size_t element = dtype == MLLM_F32 ? 4 : 2;
    for (int row0 = 0; row0 < n_rows; row0 += 65535) {   // the grid's second dimension holds 65,535 rows
        const int rows = n_rows - row0 < 65535 ? n_rows - row0 : 65535;
        const char* up_at = (const char*)up + (size_t)row0 * inner * element;
        char* out_at = (char*)out + (size_t)row0 * inner * element;
        const char* h_at = h == nullptr ? nullptr : (const char*)h + (size_t)row0 * width * element;
        float* carried_at = carried == nullptr ? nullptr : carried + (size_t)row0 * width;
        const float* weights_at = weights + (size_t)row0 * weights_stride;
        if (dtype == MLLM_F32) launch_expert_unit<float>(up_at, out_at, weights_at, weights_stride, rows, n_routed, ff, shared, h_at, carried_at, n_identity, width, stream);
        else launch_expert_unit<bf16_t>(up_at, out_at, weights_at, weights_stride, rows, n_routed, ff, shared, h_at, carried_at, n_identity, width, stream);
    }
    return mllm_check_launch("expert_unit");
}

MLLM_API int mllm_gate_unit(const void* both, void* out, int n_rows, int inner, float limit, float alpha, float shift, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && inner > 0, "gate_unit: bad sizes");
    MLLM_REQUIRE(limit > 0.0f, "gate_unit: the limit must be positive (infinite: none)");
    MLLM_REQUIRE(dtype == MLLM_F32 || dtype == MLLM_BF16, "gate_unit: unknown dtype %d", dtype);
    if (n_rows == 0) return 0;
    mllm_count_kernel(MLLM_K_GATE_UNIT);
    const size_t element = dtype == MLLM_F32 ? 4 : 2;
    for (int row0 = 0; row0 < n_rows; row0 += 65535) {
        const int rows = n_rows - row0 < 65535 ? n_rows - row0 : 65535;
        const char* in_at = (const char*)both + (size_t)row0 * 2 * inner * element;
        char* out_at = (char*)out + (size_t)row0 * inner * element;
        if (dtype == MLLM_F32) launch_gate_unit<float>(in_at, out_at, rows, inner, limit, alpha, shift, stream);
        else launch_gate_unit<bf16_t>(in_at, out_at, rows, inner, limit, alpha, shift, stream);
    }
    return mllm_check_launch("gate_unit");
}
