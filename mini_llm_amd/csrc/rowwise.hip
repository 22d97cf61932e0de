// Row-wise kernels of layers that norm after the sum, norm their heads, rotate parts of their heads and gate their
// feed-forward: RMS norm (with the scaled residual sum on its way in), the per-head norm of queries and keys with the
// cache write, the rotation of a latent layer's queries and shared key part with its cache write, and silu(a) * b.
// Everything here is computed in 32-bit whatever the element type of what is read and written.
#include "common.h"

namespace {

__device__ __forceinline__ float load_as_float(const void* base, size_t index, int code) {
    return code == MLLM_F32 ? reinterpret_cast<const float*>(base)[index] : to_float(reinterpret_cast<const bf16_t*>(base)[index]);
}
__device__ __forceinline__ void store_from_float(void* base, size_t index, int code, float value) {
    if (code == MLLM_F32) reinterpret_cast<float*>(base)[index] = value;
    else reinterpret_cast<bf16_t*>(base)[index] = static_cast<bf16_t>(value);
}

// out = h / sqrt(mean(h^2) + eps) * g with h = alpha * x (+ y) and g = weight or 1 + weight. y may be n_partials partial
// products of a product cut along K ([n_partials, rows, width], 32-bit): their sum is taken here, in a fixed order.
// A wave per output row; a row
// of up to 64 * REGS elements stays in registers between the two passes, a longer one is read again. row_index, if
// given, names the input row of each output row. The result goes to `stream` (32-bit, what the residual stream goes on
// with) and / or `rows` (the element type the next product reads); either may be null. `residual` (32-bit, the output's
// shape), if given, is added to the normed rows: out = residual + norm(h) g, the sum of a layer whose norm sits on its
// branch's output. `next_weight`, if given (rows of up to 64 * REGS elements): `rows` are not the result itself but the result normed
// once more, out / sqrt(mean(out^2) + eps) * next_weight (or 1 + next_weight): what the norm in front of the next branch would
// make of the new stream, so that a layer with a norm behind one branch and another in front of the next runs one kernel for both.
template <int REGS>
__global__ __launch_bounds__(256) void rms_norm_kernel(const float* __restrict__ x, const void* __restrict__ y, int y_code, float alpha,
                                                       const int* __restrict__ row_index, const float* __restrict__ weight, int one_plus,
                                                       float eps, float* __restrict__ stream, void* __restrict__ rows, int rows_code,
                                                       int n_rows, int width, int n_partials, long long partial_stride,
                                                       const float* __restrict__ residual, const float* __restrict__ next_weight) {
    const int lane = threadIdx.x % WAVE;
    const int row = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (row >= n_rows) return;
    const int source = row_index ? row_index[row] : row;
    const size_t in_at = (size_t)source * width, out_at = (size_t)row * width;
    const float plus = one_plus ? 1.0f : 0.0f;
    if constexpr (REGS > 0) {
        // everything is asked for at once, from clamped places, so that the wave waits for memory once
        float kept[REGS], added[REGS], gains[REGS], base[REGS], next_gains[REGS];
#pragma unroll
        for (int r = 0; r < REGS; r++) {
            const int i = min(lane + r * WAVE, width - 1);
            kept[r] = x[in_at + i];
            gains[r] = weight[i];
            base[r] = residual ? residual[out_at + i] : 0.0f;
            next_gains[r] = next_weight ? next_weight[i] : 0.0f;
        }
        if (y) {
            if (y_code == MLLM_F32) {
#pragma unroll
                for (int r = 0; r < REGS; r++) added[r] = reinterpret_cast<const float*>(y)[in_at + min(lane + r * WAVE, width - 1)];
                // further partial products, a few asked for at a time (beyond the last one: the last once more, not added)
                constexpr int AHEAD = REGS <= 16 ? 4 : 2;
                for (int p0 = 1; p0 < n_partials; p0 += AHEAD) {
                    float more[AHEAD][REGS];
#pragma unroll
                    for (int u = 0; u < AHEAD; u++)
#pragma unroll
                        for (int r = 0; r < REGS; r++)
                            more[u][r] = reinterpret_cast<const float*>(y)[min(p0 + u, n_partials - 1) * partial_stride + in_at + min(lane + r * WAVE, width - 1)];
#pragma unroll
                    for (int u = 0; u < AHEAD; u++)
#pragma unroll
                        for (int r = 0; r < REGS; r++) added[r] += p0 + u < n_partials ? more[u][r] : 0.0f;
                }
            } else {
#pragma unroll
                for (int r = 0; r < REGS; r++) added[r] = to_float(reinterpret_cast<const bf16_t*>(y)[in_at + min(lane + r * WAVE, width - 1)]);
            }
        } else {
#pragma unroll
            for (int r = 0; r < REGS; r++) added[r] = 0.0f;
        }
        float squares = 0.0f;
#pragma unroll
        for (int r = 0; r < REGS; r++) {
            const float h = lane + r * WAVE < width ? alpha * kept[r] + added[r] : 0.0f;
            kept[r] = h;
            squares += h * h;
        }
        const float inverse = 1.0f / sqrtf(wave_total(squares) / (float)width + eps);
        if (next_weight) {   // (the same for all waves of the launch)
            float again = 0.0f;
#pragma unroll
            for (int r = 0; r < REGS; r++) {
                const float value = lane + r * WAVE < width ? base[r] + kept[r] * inverse * (plus + gains[r]) : 0.0f;
                kept[r] = value;
                again += value * value;
            }
            const float next_inverse = 1.0f / sqrtf(wave_total(again) / (float)width + eps);
#pragma unroll
            for (int r = 0; r < REGS; r++) {
                const int i = lane + r * WAVE;
                if (i < width) {
                    if (stream) stream[out_at + i] = kept[r];
                    if (rows) store_from_float(rows, out_at + i, rows_code, kept[r] * next_inverse * (plus + next_gains[r]));
                }
            }
            return;
        }
#pragma unroll
        for (int r = 0; r < REGS; r++) {
            const int i = lane + r * WAVE;
            if (i < width) {
                const float value = base[r] + kept[r] * inverse * (plus + gains[r]);
                if (stream) stream[out_at + i] = value;
                if (rows) store_from_float(rows, out_at + i, rows_code, value);
            }
        }
    } else {
        float squares = 0.0f;
        for (int i = lane; i < width; i += WAVE) {
            float h = alpha * x[in_at + i];
            for (int p = 0; y && p < n_partials; p++) h += load_as_float(y, p * partial_stride + in_at + i, y_code);
            squares += h * h;
        }
        const float inverse = 1.0f / sqrtf(wave_total(squares) / (float)width + eps);
        for (int i = lane; i < width; i += WAVE) {
            float h = alpha * x[in_at + i];
            for (int p = 0; y && p < n_partials; p++) h += load_as_float(y, p * partial_stride + in_at + i, y_code);
            const float value = (residual ? residual[out_at + i] : 0.0f) + h * inverse * (plus + weight[i]);
            if (stream) stream[out_at + i] = value;
            if (rows) store_from_float(rows, out_at + i, rows_code, value);
        }
    }
}

// The heads of a fused q/k/v product, a wave per (row, head): query heads are RMS-normed over their `dim` elements with one
// gain vector, multiplied by the row's temperature 1 + coef * ln(floor((p + 1) / every) + 1) and stored as q [rows,
// n_heads * head_size]; key heads are normed with their gain vector and stored in the key pages; value heads go to the
// value pages as they are. Pages hold heads of `head_size` >= dim, vdim: what lies beyond a head's own elements is zero.
// gains null: no norm; coef 0: no temperature. A negative slot (a padding row) stores no key and no value.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_kernel(const T* __restrict__ qkv, int qkv_stride, const float* __restrict__ q_gain,
                                                        const float* __restrict__ k_gain, float eps, float temp_coef, int temp_every,
                                                        const int* __restrict__ positions, const int* __restrict__ slots,
                                                        T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                                        int n_rows, int n_heads, int n_kv_heads, int dim, int vdim, int head_size,
                                                        int page_size, int write_cache) {
    const int lane = threadIdx.x % WAVE;
    const int per_row = n_heads + 2 * n_kv_heads;
    const long long item = (long long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (item >= (long long)n_rows * per_row) return;
    const int row = (int)(item / per_row), head = (int)(item % per_row);
    const T* in_row = qkv + (size_t)row * qkv_stride;
    if (head < n_heads) {
        const T* in = in_row + head * dim;
        float squares = 0.0f;
        for (int d = lane; d < dim; d += WAVE) {
            float v = to_float(in[d]);
            squares += v * v;
        }
        float factor = q_gain ? 1.0f / sqrtf(wave_sum(squares) / (float)dim + eps) : 1.0f;
        if (temp_coef != 0.0f) factor *= 1.0f + temp_coef * logf((float)((positions[row] + 1) / temp_every) + 1.0f);
        T* out = q_out + ((size_t)row * n_heads + head) * head_size;
        for (int d = lane; d < head_size; d += WAVE)
            out[d] = from_float<T>(d < dim ? to_float(in[d]) * factor * (q_gain ? q_gain[d] : 1.0f) : 0.0f);
        return;
    }
    if (!write_cache) return;
    const int slot = slots[row];
    if (slot < 0) return;
    const int page = slot / page_size, offset = slot % page_size;
    if (head < n_heads + n_kv_heads) {
        const int g = head - n_heads;
        const T* in = in_row + n_heads * dim + g * dim;
        float squares = 0.0f;
        for (int d = lane; d < dim; d += WAVE) {
            float v = to_float(in[d]);
            squares += v * v;
        }
        const float factor = k_gain ? 1.0f / sqrtf(wave_sum(squares) / (float)dim + eps) : 1.0f;
        T* out = k_pages + (((size_t)page * n_kv_heads + g) * page_size + offset) * head_size;
        for (int d = lane; d < head_size; d += WAVE)
            out[d] = from_float<T>(d < dim ? to_float(in[d]) * factor * (k_gain ? k_gain[d] : 1.0f) : 0.0f);
    } else {
        const int g = head - n_heads - n_kv_heads;
        const T* in = in_row + (n_heads + n_kv_heads) * dim + g * vdim;
        T* out = v_pages + (((size_t)page * n_kv_heads + g) * page_size + offset) * head_size;
        for (int d = lane; d < head_size; d += WAVE) out[d] = d < vdim ? in[d] : from_float<T>(0.0f);
    }
}

// The same for heads whose sizes are whole 16-byte pieces: LPH lanes take a head, a piece each (LPH a power of two, LPH pieces
// hold head_size elements), so a wave takes 64 / LPH heads and every lane moves 16 bytes in and 16 bytes out.
template <typename T, int LPH>
__global__ __launch_bounds__(256) void head_norm_pieces_kernel(const T* __restrict__ qkv, int qkv_stride, const float* __restrict__ q_gain,
                                                               const float* __restrict__ k_gain, float eps, float temp_coef, int temp_every,
                                                               const int* __restrict__ positions, const int* __restrict__ slots,
                                                               T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                                               int n_rows, int n_heads, int n_kv_heads, int dim, int vdim, int head_size,
                                                               int page_size, int write_cache) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const int per_row = n_heads + 2 * n_kv_heads;
    const long long item = ((long long)blockIdx.x * blockDim.x + threadIdx.x) / LPH;
    const int at = (threadIdx.x % LPH) * VEC;   // the lane's first element of the head
    const bool live = item < (long long)n_rows * per_row;
    const int row = live ? (int)(item / per_row) : 0, head = live ? (int)(item % per_row) : 0;
    const bool is_q = head < n_heads, is_k = !is_q && head < n_heads + n_kv_heads;
    const int own = is_q || is_k ? dim : vdim;   // the head's own elements
    const int g = is_q ? head : (is_k ? head - n_heads : head - n_heads - n_kv_heads);
    const T* in = qkv + (size_t)row * qkv_stride + (is_q ? 0 : (is_k ? n_heads * dim : (n_heads + n_kv_heads) * dim)) + (size_t)g * own;
    const bool has = live && at < own;
    Vec16 piece = {};
    if (has) piece = *reinterpret_cast<const Vec16*>(in + at);
    const T* e = reinterpret_cast<const T*>(&piece);
    float values[VEC], squares = 0.0f;
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        values[j] = to_float(e[j]);
        squares += values[j] * values[j];
    }
#pragma unroll
    for (int step = 1; step < LPH; step *= 2) squares += __shfl_xor(squares, step, WAVE);
    if (!live || at >= head_size) return;
    const float* gain = is_q ? q_gain : (is_k ? k_gain : nullptr);
    float factor = gain ? 1.0f / sqrtf(squares / (float)dim + eps) : 1.0f;
    if (is_q && temp_coef != 0.0f) factor *= 1.0f + temp_coef * logf((float)((positions[row] + 1) / temp_every) + 1.0f);
    T* out;
    if (is_q) {
        out = q_out + ((size_t)row * n_heads + head) * head_size;
    } else {
        if (!write_cache) return;
        const int slot = slots[row];
        if (slot < 0) return;
        out = (is_k ? k_pages : v_pages) + (((size_t)(slot / page_size) * n_kv_heads + g) * page_size + slot % page_size) * head_size;
    }
    Vec16 result;
    T* r = reinterpret_cast<T*>(&result);
    if (is_q || is_k) {
#pragma unroll
        for (int j = 0; j < VEC; j++) r[j] = from_float<T>(has ? values[j] * factor * (gain ? gain[at + j] : 1.0f) : 0.0f);
    } else {
        result = piece;   // a value head as it is (zeros beyond its own elements)
    }
    *reinterpret_cast<Vec16*>(out + at) = result;
}

// Rotation of `dims` elements in the "rotate half" pairing: element i pairs with i + dims / 2, and the pair (u, v) at
// position p becomes (u c - v s, v c + u s) with c = cos(p f_i) m, s = sin(p f_i) m. The angle is a 32-bit product.
__device__ __forceinline__ void rotated_pair(float u, float v, int position, float frequency, float magnitude, float& a, float& b) {
    const float angle = (float)position * frequency;
    const float c = cosf(angle) * magnitude, s = sinf(angle) * magnitude;
    a = u * c - v * s;
    b = v * c + u * s;
}

// A latent-attention layer's row-wise work, a wave per (row, head) and one more per row for what the layer keeps:
//  - query head h of q [rows, n_heads * (dim + rot)]: its last `rot` elements, rotated, go to q_full[row, h, rank ..
//    rank + rot) (32-bit; its first `rank` elements are filled by the product that folds the key expansion into the
//    query, what lies beyond rank + rot up to `row_size` is zero);
//  - the row of dkv [rows, rank + rot]: its first `rank` elements RMS-normed with `gain`, its last `rot` rotated, stored as
//    the row's cache line [rank | rot | zeros up to row_size] in pages [num_pages, page_size, row_size].
// The first `rot_dims` of the rot elements are rotated, the rest pass unchanged.
template <typename T>
__global__ __launch_bounds__(256) void latent_rows_kernel(const T* __restrict__ q, int q_stride, const T* __restrict__ dkv, int dkv_stride,
                                                          const float* __restrict__ gain, float eps, const float* __restrict__ frequencies,
                                                          float magnitude, int rot_dims, const int* __restrict__ positions,
                                                          const int* __restrict__ slots, float* __restrict__ q_full, T* __restrict__ pages,
                                                          int n_rows, int n_heads, int dim, int rot, int rank, int row_size, int page_size) {
    const int lane = threadIdx.x % WAVE;
    const int per_row = n_heads + 1;
    const long long item = (long long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (item >= (long long)n_rows * per_row) return;
    const int row = (int)(item / per_row), head = (int)(item % per_row);
    const int position = positions[row];
    const int half = rot_dims / 2;
    if (head < n_heads) {
        const T* in = q + (size_t)row * q_stride + (size_t)head * (dim + rot) + dim;
        float* out = q_full + ((size_t)row * n_heads + head) * row_size + rank;
        for (int i = lane; i < half; i += WAVE) {
            float a, b;
            rotated_pair(to_float(in[i]), to_float(in[i + half]), position, frequencies[i], magnitude, a, b);
            out[i] = a;
            out[i + half] = b;
        }
        for (int i = 2 * half + lane; i < row_size - rank; i += WAVE) out[i] = i < rot ? to_float(in[i]) : 0.0f;
        return;
    }
    if (dkv == nullptr) return;
    const int slot = slots[row];
    if (slot < 0) return;
    const T* in = dkv + (size_t)row * dkv_stride;
    T* out = pages + (size_t)slot * row_size;
    float squares = 0.0f;
    for (int d = lane; d < rank; d += WAVE) {
        float v = to_float(in[d]);
        squares += v * v;
    }
    const float inverse = 1.0f / sqrtf(wave_sum(squares) / (float)rank + eps);
    for (int d = lane; d < rank; d += WAVE) out[d] = from_float<T>(to_float(in[d]) * inverse * gain[d]);
    for (int i = lane; i < half; i += WAVE) {
        float a, b;
        rotated_pair(to_float(in[rank + i]), to_float(in[rank + i + half]), position, frequencies[i], magnitude, a, b);
        out[rank + i] = from_float<T>(a);
        out[rank + i + half] = from_float<T>(b);
    }
    for (int i = 2 * half + lane; i < row_size - rank; i += WAVE) out[rank + i] = i < rot ? in[rank + i] : from_float<T>(0.0f);
}

// out[row, j] = silu(both[row, j]) * both[row, inner + j]: the two halves of a fused gate / up product. A thread takes a
// 16-byte piece of each half where the rows are whole pieces (PIECES), else an element.
template <typename T, bool PIECES>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ both, T* __restrict__ out, int inner) {
    constexpr int VEC = PIECES ? 16 / (int)sizeof(T) : 1;
    const int j = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (j >= inner) return;
    const size_t row = blockIdx.y;
    const T* a_at = both + row * 2 * inner + j;
    const T* b_at = a_at + inner;
    T* out_at = out + row * inner + j;
    if constexpr (PIECES) {
        const Vec16 a = *reinterpret_cast<const Vec16*>(a_at), b = *reinterpret_cast<const Vec16*>(b_at);
        Vec16 result;
        const T* ae = reinterpret_cast<const T*>(&a);
        const T* be = reinterpret_cast<const T*>(&b);
        T* re = reinterpret_cast<T*>(&result);
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            const float av = to_float(ae[e]);
            re[e] = from_float<T>(av / (1.0f + expf(-av)) * to_float(be[e]));
        }
        *reinterpret_cast<Vec16*>(out_at) = result;
    } else {
        const float av = to_float(*a_at);
        *out_at = from_float<T>(av / (1.0f + expf(-av)) * to_float(*b_at));
    }
}

}  // namespace

MLLM_API int mllm_rms_norm(const float* x, const void* y, int y_dtype, float alpha, const int* row_index, const float* weight, int one_plus,
                           float eps, float* stream_out, void* rows_out, int rows_dtype, int n_rows, int width, int n_partials,
                           long long partial_stride, const float* residual, const float* next_weight, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && width > 0, "rms_norm: bad sizes rows=%d width=%d", n_rows, width);
    MLLM_REQUIRE(x != nullptr && weight != nullptr && (stream_out != nullptr || rows_out != nullptr), "rms_norm: a missing operand");
    MLLM_REQUIRE(y == nullptr || y_dtype == MLLM_F32 || y_dtype == MLLM_BF16, "rms_norm: unknown element type of the addend");
    MLLM_REQUIRE(rows_out == nullptr || rows_dtype == MLLM_F32 || rows_dtype == MLLM_BF16, "rms_norm: unknown element type of the rows");
    MLLM_REQUIRE(y == nullptr || row_index == nullptr, "rms_norm: gathered rows take no addend");
    MLLM_REQUIRE(n_partials >= 1 && (n_partials == 1 || (y != nullptr && y_dtype == MLLM_F32 && partial_stride >= (long long)n_rows * width)),
                 "rms_norm: partial products are 32-bit and lie a whole matrix apart");
    MLLM_REQUIRE(next_weight == nullptr || (width <= 2048 && rows_out != nullptr), "rms_norm: a second norm takes rows of up to 2048 elements and writes `rows`");
    if (n_rows == 0) return 0;
    const int waves = 4, blocks = ceil_div(n_rows, waves);
    mllm_count_kernel(MLLM_K_RMS_NORM);
#define LAUNCH(REGS) rms_norm_kernel<REGS><<<blocks, 64 * waves, 0, stream>>>(x, y, y_dtype, alpha, row_index, weight, one_plus, eps, stream_out, rows_out, rows_dtype, n_rows, width, n_partials, partial_stride, residual, next_weight)
    if (width <= 256) LAUNCH(4);
    else if (width <= 512) LAUNCH(8);
    else if (width <= 1024) LAUNCH(16);
    else if (width <= 2048) LAUNCH(32);
    else LAUNCH(0);
#undef LAUNCH
    return mllm_check_launch("rms_norm");
}

MLLM_API int mllm_head_norm(const void* qkv, int qkv_stride, const float* q_gain, const float* k_gain, float eps, float temp_coef, int temp_every,
                            const int* positions, const int* slots, void* q_out, void* k_pages, void* v_pages, int n_rows, int n_heads,
                            int n_kv_heads, int dim, int vdim, int head_size, int page_size, int write_cache, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_heads > 0 && n_kv_heads > 0 && dim > 0 && vdim > 0 && page_size > 0, "head_norm: bad sizes");
    MLLM_REQUIRE(head_size >= dim && head_size >= vdim, "head_norm: heads of %d do not hold %d / %d elements", head_size, dim, vdim);
    MLLM_REQUIRE(qkv_stride >= (n_heads + n_kv_heads) * dim + n_kv_heads * vdim, "head_norm: rows are too short for the heads");
    MLLM_REQUIRE(temp_coef == 0.0f || (temp_every > 0 && positions != nullptr), "head_norm: a temperature needs positions and a period");
    MLLM_REQUIRE(!write_cache || (slots != nullptr && k_pages != nullptr && v_pages != nullptr), "head_norm: a cache write needs slots and pages");
    if (n_rows == 0) return 0;
    const long long items = (long long)n_rows * (n_heads + 2 * n_kv_heads);
    mllm_count_kernel(MLLM_K_HEAD_NORM);
    const int vec = dtype == MLLM_F32 ? 4 : 2 * 4;
    const bool pieces = dim % vec == 0 && vdim % vec == 0 && head_size % vec == 0 && head_size / vec <= 64 && qkv_stride % vec == 0 &&
                        (size_t)qkv % 16 == 0 && (size_t)q_out % 16 == 0 && (size_t)k_pages % 16 == 0 && (size_t)v_pages % 16 == 0;
#define HEAD_NORM_ARGS(T) (const T*)qkv, qkv_stride, q_gain, k_gain, eps, temp_coef, temp_every, positions, slots, (T*)q_out, (T*)k_pages, (T*)v_pages, \
                          n_rows, n_heads, n_kv_heads, dim, vdim, head_size, page_size, write_cache
    if (pieces && (dtype == MLLM_F32 || dtype == MLLM_BF16)) {
        int lanes = 1;
        while (lanes * vec < head_size) lanes *= 2;
        const int blocks = (int)((items * lanes + 255) / 256);
#define HEAD_NORM_PIECES(LPH)                                                                                                   \
    case LPH:                                                                                                                   \
        if (dtype == MLLM_F32) head_norm_pieces_kernel<float, LPH><<<blocks, 256, 0, stream>>>(HEAD_NORM_ARGS(float));        \
        else head_norm_pieces_kernel<bf16_t, LPH><<<blocks, 256, 0, stream>>>(HEAD_NORM_ARGS(bf16_t));                        \
        break;
        switch (lanes) {
            HEAD_NORM_PIECES(1) HEAD_NORM_PIECES(2) HEAD_NORM_PIECES(4) HEAD_NORM_PIECES(8) HEAD_NORM_PIECES(16) HEAD_NORM_PIECES(32)
            HEAD_NORM_PIECES(64)
        }
#undef HEAD_NORM_PIECES
        return mllm_check_launch("head_norm");
    }
    const int blocks = (int)((items + 3) / 4);
    if (dtype == MLLM_F32)
        head_norm_kernel<float><<<blocks, 256, 0, stream>>>(HEAD_NORM_ARGS(float));
    else if (dtype == MLLM_BF16)
        head_norm_kernel<bf16_t><<<blocks, 256, 0, stream>>>(HEAD_NORM_ARGS(bf16_t));
    else
        MLLM_REQUIRE(false, "head_norm: unknown dtype %d", dtype);
#undef HEAD_NORM_ARGS
    return mllm_check_launch("head_norm");
}

MLLM_API int mllm_latent_rows(const void* q, int q_stride, const void* dkv, int dkv_stride, const float* gain, float eps, const float* frequencies,
                              float magnitude, int rot_dims, const int* positions, const int* slots, float* q_full, void* pages, int n_rows,
                              int n_heads, int dim, int rot, int rank, int row_size, int page_size, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_heads > 0 && dim > 0 && rot >= 0 && rank > 0 && page_size > 0, "latent_rows: bad sizes");
    MLLM_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= rot, "latent_rows: %d rotated elements of %d", rot_dims, rot);
    MLLM_REQUIRE(row_size >= rank + rot, "latent_rows: a row of %d does not hold %d + %d", row_size, rank, rot);
    MLLM_REQUIRE(q_stride >= n_heads * (dim + rot), "latent_rows: query rows are too short");
    MLLM_REQUIRE(dkv == nullptr || (dkv_stride >= rank + rot && gain != nullptr && slots != nullptr && pages != nullptr),
                 "latent_rows: the rows to keep need a gain vector, slots and pages");
    MLLM_REQUIRE(positions != nullptr && (rot_dims == 0 || frequencies != nullptr), "latent_rows: a rotation needs positions and frequencies");
    if (n_rows == 0) return 0;
    const long long items = (long long)n_rows * (n_heads + 1);
    const int blocks = (int)((items + 3) / 4);
    mllm_count_kernel(MLLM_K_LATENT_ROWS);
    if (dtype == MLLM_F32)
        latent_rows_kernel<float><<<blocks, 256, 0, stream>>>((const float*)q, q_stride, (const float*)dkv, dkv_stride, gain, eps, frequencies, magnitude,
                                                              rot_dims, positions, slots, q_full, (float*)pages, n_rows, n_heads, dim, rot, rank,
                                                              row_size, page_size);
    else if (dtype == MLLM_BF16)
        latent_rows_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)dkv, dkv_stride, gain, eps, frequencies,
                                                               magnitude, rot_dims, positions, slots, q_full, (bf16_t*)pages, n_rows, n_heads, dim, rot,
                                                               rank, row_size, page_size);
    else
        MLLM_REQUIRE(false, "latent_rows: unknown dtype %d", dtype);
    return mllm_check_launch("latent_rows");
}

template <typename T>
void launch_silu_mul(const void* both, void* out, int n_rows, int inner, hipStream_t stream) {
    constexpr int VEC = 16 / (int)sizeof(T);
    if (inner % VEC == 0) {
        dim3 grid(ceil_div(inner / VEC, 256), n_rows);
        silu_mul_kernel<T, true><<<grid, 256, 0, stream>>>((const T*)both, (T*)out, inner);
    } else {
        dim3 grid(ceil_div(inner, 256), n_rows);
        silu_mul_kernel<T, false><<<grid, 256, 0, stream>>>((const T*)both, (T*)out, inner);
    }
}

MLLM_API int mllm_silu_mul(const void* both, void* out, int n_rows, int inner, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_rows <= 65535 * 64 && inner > 0, "silu_mul: bad sizes");
    MLLM_REQUIRE(dtype == MLLM_F32 || dtype == MLLM_BF16, "silu_mul: unknown dtype %d", dtype);
    if (n_rows == 0) return 0;
    mllm_count_kernel(MLLM_K_SILU_MUL);
    for (int row0 = 0; row0 < n_rows; row0 += 65535) {   // the grid's second dimension holds 65,535 rows
        const int rows = n_rows - row0 < 65535 ? n_rows - row0 : 65535;
        const size_t element = dtype == MLLM_F32 ? 4 : 2;
        const char* in_at = (const char*)both + (size_t)row0 * 2 * inner * element;
        char* out_at = (char*)out + (size_t)row0 * inner * element;
        if (dtype == MLLM_F32) launch_silu_mul<float>(in_at, out_at, rows, inner, stream);
        else launch_silu_mul<bf16_t>(in_at, out_at, rows, inner, stream);
    }
    return mllm_check_launch("silu_mul");
}
