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

// The same sum for rows of up to 64 * VEC * CHUNKS elements, every operand asked for at once: a lane owns VEC neighbouring elements in each
// of CHUNKS pieces of the row, loads them from clamped places whatever the row's width (what lies beyond it is masked when stored), and
// keeps its sums in registers for the norm. No operand is optional in here: the caller names a valid place for each (a branch that is
// missing reads the other's rows and counts 0 times, `*_on` are 0 or 1), so that no load waits behind a branch. VEC 4: 16-byte pieces
// (widths, strides and columns that are multiples of four elements); VEC 1: any.
template <typename T, int VEC, int CHUNKS>
__global__ __launch_bounds__(64 * JOIN_WAVES) void branch_join_rows_kernel(
    const float* __restrict__ x, const float* __restrict__ a, int n_a, long long a_stride, const float* __restrict__ a_bias, float a_bias_on,
    const float* __restrict__ b, int n_b, long long b_stride, const float* __restrict__ b_bias, float b_bias_on, float b_on,
    const float* __restrict__ scale_a, float scale_a_on, const float* __restrict__ scale_b, float scale_b_on, const float* __restrict__ gates,
    int gates_stride, int gate_a_at, int gate_b_at, float gates_on, float mult, float* __restrict__ stream_out, const float* __restrict__ next_weight,
    int has_next, int one_plus, float eps, T* __restrict__ rows_out, int n_rows, int width) {
    struct Piece {
        float v[VEC];
    };
    const int lane = threadIdx.x % WAVE;
    const int row = blockIdx.x * JOIN_WAVES + threadIdx.x / WAVE;
    if (row >= n_rows) return;
    const size_t at = (size_t)row * width;
    const float* gate_row = gates + (size_t)row * gates_stride;
    const int last = width - VEC;
    auto piece = [](const float* from) {
        Piece out;
        if constexpr (VEC == 4) {
            const f32x4 loaded = *reinterpret_cast<const f32x4*>(from);
#pragma unroll
            for (int e = 0; e < 4; e++) out.v[e] = loaded[e];
        } else {
            out.v[0] = *from;
        }
        return out;
    };
    Piece sums[CHUNKS], gains[CHUNKS];
    float squares = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
        const int d_real = (c * WAVE + lane) * VEC;
        const int d = d_real <= last ? d_real : last;
        const Piece xs = piece(x + at + d), ga = piece(gate_row + gate_a_at + d), gb = piece(gate_row + gate_b_at + d);
        const Piece sa = piece(scale_a + d), sb = piece(scale_b + d), ba = piece(a_bias + d), bb = piece(b_bias + d);
        Piece first = piece(a + at + d), second = piece(b + at + d);
        gains[c] = piece(next_weight + d);   // asked for with everything else: the norm behind the sum then waits for no trip of its own
        for (int p = 1; p < n_a; p++) {
            const Piece more = piece(a + (size_t)p * a_stride + at + d);
#pragma unroll
            for (int e = 0; e < VEC; e++) first.v[e] += more.v[e];
        }
        for (int p = 1; p < n_b; p++) {
            const Piece more = piece(b + (size_t)p * b_stride + at + d);
#pragma unroll
            for (int e = 0; e < VEC; e++) second.v[e] += more.v[e];
        }
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            float one = first.v[e] + (a_bias_on != 0.0f ? ba.v[e] : 0.0f);
            one *= scale_a_on != 0.0f ? sa.v[e] : 1.0f;
            one *= gates_on != 0.0f ? 1.0f / (1.0f + expf(-ga.v[e])) : 1.0f;
            float two = second.v[e] + (b_bias_on != 0.0f ? bb.v[e] : 0.0f);
            two *= scale_b_on != 0.0f ? sb.v[e] : 1.0f;
            two *= gates_on != 0.0f ? 1.0f / (1.0f + expf(-gb.v[e])) : 1.0f;
            const float sum = xs.v[e] + mult * (one + (b_on != 0.0f ? two : 0.0f));
            sums[c].v[e] = sum;
            squares += d_real <= last ? sum * sum : 0.0f;
        }
        if (d_real <= last) {
            if constexpr (VEC == 4) *reinterpret_cast<f32x4*>(stream_out + at + d) = f32x4{sums[c].v[0], sums[c].v[1], sums[c].v[2], sums[c].v[3]};
            else stream_out[at + d] = sums[c].v[0];
        }
    }
    if (!has_next) return;
    const float factor = 1.0f / sqrtf(wave_sum(squares) / (float)width + eps);
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
        const int d = (c * WAVE + lane) * VEC;
        if (d > last) continue;
#pragma unroll
        for (int e = 0; e < VEC; e++) rows_out[at + d + e] = from_float<T>(sums[c].v[e] * factor * (one_plus ? 1.0f + gains[c].v[e] : gains[c].v[e]));
    }
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
    // rows of up to 2,048 elements: every operand asked for at once, the sums kept in registers for the norm
    auto whole_pieces = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    const bool pieces = width % 4 == 0 && gates_stride % 4 == 0 && gate_a_at % 4 == 0 && gate_b_at % 4 == 0 && a_stride % 4 == 0 && b_stride % 4 == 0 &&
                        whole_pieces(x) && whole_pieces(a) && whole_pieces(b) && whole_pieces(a_bias) && whole_pieces(b_bias) && whole_pieces(scale_a) &&
                        whole_pieces(scale_b) && whole_pieces(gates) && whole_pieces(stream_out) && whole_pieces(next_weight);
    const int vec = pieces ? 4 : 1;
    const int chunks = ceil_div(width, 64 * vec);
    if (chunks <= 8) {
        const bool has_b = b != nullptr, has_gates = gates != nullptr;
        const float* any = x;   // a valid row-shaped place for operands that are absent (their shares count 0 times)
#define BRANCH_JOIN_ROWS_ARGS(T) x, a, n_a, a_stride, a_bias ? a_bias : any, a_bias ? 1.0f : 0.0f, has_b ? b : a, has_b ? n_b : 1, b_stride, \
                                 b_bias ? b_bias : any, b_bias ? 1.0f : 0.0f, has_b ? 1.0f : 0.0f, scale_a ? scale_a : any, scale_a ? 1.0f : 0.0f, \
                                 scale_b ? scale_b : any, scale_b ? 1.0f : 0.0f, has_gates ? gates : x, has_gates ? gates_stride : width, \
                                 has_gates ? gate_a_at : 0, has_gates && has_b ? gate_b_at : 0, has_gates ? 1.0f : 0.0f, mult, stream_out, \
                                 next_weight ? next_weight : any, next_weight ? 1 : 0, one_plus, eps, (T*)rows_out, n_rows, width
#define BRANCH_JOIN_ROWS(T, VEC, CHUNKS) branch_join_rows_kernel<T, VEC, CHUNKS><<<blocks, 64 * JOIN_WAVES, 0, stream>>>(BRANCH_JOIN_ROWS_ARGS(T))
#define BRANCH_JOIN_ROWS_OF(T)                                                  \
    do {                                                                        \
        if (pieces && chunks <= 1) BRANCH_JOIN_ROWS(T, 4, 1);                   \
        else if (pieces && chunks <= 2) BRANCH_JOIN_ROWS(T, 4, 2);              \
        else if (pieces && chunks <= 4) BRANCH_JOIN_ROWS(T, 4, 4);              \
        else if (pieces) BRANCH_JOIN_ROWS(T, 4, 8);                             \
        else if (chunks <= 2) BRANCH_JOIN_ROWS(T, 1, 2);                        \
        else BRANCH_JOIN_ROWS(T, 1, 8);                                         \
    } while (0)
        if (next_weight == nullptr || rows_dtype == MLLM_F32) BRANCH_JOIN_ROWS_OF(float);
        else BRANCH_JOIN_ROWS_OF(bf16_t);
#undef BRANCH_JOIN_ROWS_OF
#undef BRANCH_JOIN_ROWS
#undef BRANCH_JOIN_ROWS_ARGS
        return mllm_check_launch("branch_join");
    }
#define BRANCH_JOIN_ARGS(T) x, a, n_a, a_stride, a_bias, b, n_b, b_stride, b_bias, scale_a, scale_b, gates, gates_stride, gate_a_at, gate_b_at, mult, \
                            stream_out, next_weight, one_plus, eps, (T*)rows_out, n_rows, width
    if (next_weight == nullptr || rows_dtype == MLLM_F32) branch_join_kernel<float><<<blocks, 64 * JOIN_WAVES, 0, stream>>>(BRANCH_JOIN_ARGS(float));
    else branch_join_kernel<bf16_t><<<blocks, 64 * JOIN_WAVES, 0, stream>>>(BRANCH_JOIN_ARGS(bf16_t));
#undef BRANCH_JOIN_ARGS
    return mllm_check_launch("branch_join");
}
