// The sum of a layer whose two branches run side by side on one normed input: out = x + mult * (scale_a * sigmoid(gate_a) * a + scale_b *
// sigmoid(gate_b) * b), element by element in 32-bit, and, from the same launch, what the next layer's norm makes of that sum.
#include "common.h"

#include <math.h>

namespace {

constexpr int JOIN_WAVES = 4;   // rows a block

// A wave a row. x: the stream, float32 [rows, width]. a, b (b null: the layer has one branch): float32 [n, rows, width], the n partial
// products of a branch's last product (n = 1: the branch itself), matrices `*_stride` elements apart; `*_bias` (null: none) joins their
// sum. scale_a, scale_b: float32 [width] (null: 1). gates: float32 rows (null: no gates) with a's gate at column gate_a_at and b's at
// gate_b_at, before their sigmoid. stream_out = x + mult * (...). next_weight (null: none): rows_out = stream_out / sqrt(mean(stream_out^2)
// + eps) * (next_weight or, with one_plus, 1 + next_weight), in T. Rows of any width: the second pass reads the sums the lane itself has
// just stored.
template <typename T>
__global__ __launch_bounds__(64 * JOIN_WAVES) void branch_join_kernel(
    const float* __restrict__ x, const float* __restrict__ a, int n_a, long long a_stride, const float* __restrict__ a_bias, const float* __restrict__ b,
    int n_b, long long b_stride, const float* __restrict__ b_bias, const float* __restrict__ scale_a, const float* __restrict__ scale_b,
    const float* __restrict__ gates, int gates_stride, int gate_a_at, int gate_b_at, float mult, float* __restrict__ stream_out,
    const float* __restrict__ next_weight, int one_plus, float eps, T* __restrict__ rows_out, int n_rows, int width) {
    const int lane = threadIdx.x % WAVE;
    const int row = blockIdx.x * JOIN_WAVES + threadIdx.x / WAVE;
    if (row >= n_rows) return;
    const size_t at = (size_t)row * width;
    const float* gate_row = gates ? gates + (size_t)row * gates_stride : nullptr;
    float squares = 0.0f;
    for (int d = lane; d < width; d += WAVE) {
        float first = a_bias ? a_bias[d] : 0.0f;
        for (int p = 0; p < n_a; p++) first += a[(size_t)p * a_stride + at + d];
        if (scale_a) first *= scale_a[d];
        if (gate_row) first *= 1.0f / (1.0f + expf(-gate_row[gate_a_at + d]));
        float second = 0.0f;
        if (b) {
            second = b_bias ? b_bias[d] : 0.0f;
            for (int p = 0; p < n_b; p++) second += b[(size_t)p * b_stride + at + d];
            if (scale_b) second *= scale_b[d];
            if (gate_row) second *= 1.0f / (1.0f + expf(-gate_row[gate_b_at + d]));
        }
        const float sum = x[at + d] + mult * (first + second);
        stream_out[at + d] = sum;
        squares += sum * sum;
    }
    if (next_weight == nullptr) return;
    const float factor = 1.0f / sqrtf(wave_sum(squares) / (float)width + eps);
    for (int d = lane; d < width; d += WAVE)
        rows_out[at + d] = from_float<T>(stream_out[at + d] * factor * (one_plus ? 1.0f + next_weight[d] : next_weight[d]));
}

}  // namespace

MLLM_API int mllm_branch_join(const float* x, const float* a, int n_a, long long a_stride, const float* a_bias, const float* b, int n_b, long long b_stride,
                              const float* b_bias, const float* scale_a, const float* scale_b, const float* gates, int gates_stride, int gate_a_at,
                              int gate_b_at, float mult, float* stream_out, const float* next_weight, int one_plus, float eps, void* rows_out,
                              int rows_dtype, int n_rows, int width, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && width > 0, "branch_join: bad sizes rows=%d width=%d", n_rows, width);
    MLLM_REQUIRE(x != nullptr && a != nullptr && stream_out != nullptr && n_a >= 1 && (b == nullptr || n_b >= 1), "branch_join: a missing operand");
    MLLM_REQUIRE(stream_out != x, "branch_join: the sum is not written over the stream it reads");
    MLLM_REQUIRE((n_a == 1 || a_stride >= (long long)n_rows * width) && (b == nullptr || n_b == 1 || b_stride >= (long long)n_rows * width),
                 "branch_join: partial products lie a whole matrix apart");
    MLLM_REQUIRE(gates == nullptr || (gate_a_at >= 0 && gate_a_at + width <= gates_stride && (b == nullptr || (gate_b_at >= 0 && gate_b_at + width <= gates_stride))),
                 "branch_join: the gates lie beyond their rows");
    MLLM_REQUIRE(next_weight == nullptr || (rows_out != nullptr && (rows_dtype == MLLM_F32 || rows_dtype == MLLM_BF16) && eps > 0.0f),
                 "branch_join: a norm behind the sum writes rows of a known type");
    if (n_rows == 0) return 0;
    const int blocks = ceil_div(n_rows, JOIN_WAVES);
    mllm_count_kernel(MLLM_K_BRANCH_JOIN);
#define BRANCH_JOIN_ARGS(T) x, a, n_a, a_stride, a_bias, b, n_b, b_stride, b_bias, scale_a, scale_b, gates, gates_stride, gate_a_at, gate_b_at, mult, \
                            stream_out, next_weight, one_plus, eps, (T*)rows_out, n_rows, width
    if (next_weight == nullptr || rows_dtype == MLLM_F32) branch_join_kernel<float><<<blocks, 64 * JOIN_WAVES, 0, stream>>>(BRANCH_JOIN_ARGS(float));
    else branch_join_kernel<bf16_t><<<blocks, 64 * JOIN_WAVES, 0, stream>>>(BRANCH_JOIN_ARGS(bf16_t));
#undef BRANCH_JOIN_ARGS
    return mllm_check_launch("branch_join");
}
