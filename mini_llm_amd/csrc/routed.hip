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
// every row uses. out = relu(up)^2 * weights[row, expert] (shared units: relu(up)^2). Behind the hidden units the grid goes on over
// `width` columns of `carried` (null: none): carried[row, :] = h[row, :] * (the sum of weights[row, n_routed .. n_routed + n_identity)),
// the share of the experts that hand their input on as it is.
template <typename T>
__global__ __launch_bounds__(256) void expert_unit_kernel(const T* __restrict__ up, T* __restrict__ out, const float* __restrict__ weights, int weights_stride,
                                                          int n_routed, int ff, int shared, const T* __restrict__ h, float* __restrict__ carried,
                                                          int n_identity, int width) {
    const int inner = n_routed * ff + shared;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    const size_t row = blockIdx.y;
    const float* w = weights + row * weights_stride;
    if (j < inner) {
        const float u = fmaxf(to_float(up[row * inner + j]), 0.0f);
        const float weight = j < n_routed * ff ? w[j / ff] : 1.0f;
        out[row * inner + j] = from_float<T>(u * u * weight);
    } else if (carried != nullptr && j - inner < width) {
        float share = 0.0f;
        for (int e = 0; e < n_identity; e++) share += w[n_routed + e];
        carried[row * width + (j - inner)] = to_float(h[row * width + (j - inner)]) * share;
    }
}

// both: [rows, 2 * inner], a gate half and an up half. out = g * sigmoid(alpha * g) * (u + shift) with g = min(gate, limit) and u =
// clamp(up, -limit, limit) (limit infinite: unclamped).
template <typename T>
__global__ __launch_bounds__(256) void gate_unit_kernel(const T* __restrict__ both, T* __restrict__ out, int inner, float limit, float alpha, float shift) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= inner) return;
    const size_t row = blockIdx.y;
    const float g = fminf(to_float(both[row * 2 * inner + j]), limit);
    const float u = fminf(fmaxf(to_float(both[row * 2 * inner + inner + j]), -limit), limit);
    out[row * inner + j] = from_float<T>(g / (1.0f + expf(-alpha * g)) * (u + shift));
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
    const int columns = (int)inner + (carried != nullptr ? width : 0);
    const size_t element = dtype == MLLM_F32 ? 4 : 2;
    for (int row0 = 0; row0 < n_rows; row0 += 65535) {   // the grid's second dimension holds 65,535 rows
        const int rows = n_rows - row0 < 65535 ? n_rows - row0 : 65535;
        dim3 grid(ceil_div(columns, 256), rows);
        const char* up_at = (const char*)up + (size_t)row0 * inner * element;
        char* out_at = (char*)out + (size_t)row0 * inner * element;
        const char* h_at = h == nullptr ? nullptr : (const char*)h + (size_t)row0 * width * element;
        float* carried_at = carried == nullptr ? nullptr : carried + (size_t)row0 * width;
        const float* weights_at = weights + (size_t)row0 * weights_stride;
        if (dtype == MLLM_F32)
            expert_unit_kernel<float><<<grid, 256, 0, stream>>>((const float*)up_at, (float*)out_at, weights_at, weights_stride, n_routed, ff, shared,
                                                                (const float*)h_at, carried_at, n_identity, width);
        else
            expert_unit_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)up_at, (bf16_t*)out_at, weights_at, weights_stride, n_routed, ff, shared,
                                                                 (const bf16_t*)h_at, carried_at, n_identity, width);
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
        dim3 grid(ceil_div(inner, 256), rows);
        const char* in_at = (const char*)both + (size_t)row0 * 2 * inner * element;
        char* out_at = (char*)out + (size_t)row0 * inner * element;
        if (dtype == MLLM_F32) gate_unit_kernel<float><<<grid, 256, 0, stream>>>((const float*)in_at, (float*)out_at, inner, limit, alpha, shift);
        else gate_unit_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)in_at, (bf16_t*)out_at, inner, limit, alpha, shift);
    }
    return mllm_check_launch("gate_unit");
}
