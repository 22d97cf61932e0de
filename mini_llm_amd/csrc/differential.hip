// The row-wise work of attention whose heads hold several maps: each (head, map) has a query and a key of its own, all maps of a
// head attend over the head's one value, and the maps' results are combined afterwards (differential attention subtracts the
// second map from the first).
//
// The paged attention kernels know nothing of maps: they see n_heads * maps query heads over n_kv_heads * maps key/value heads.
// With R = n_heads / n_kv_heads query heads to a key/value head, query head h = g R + r and map m are laid out as attention head
// (g * maps + m) * R + r, so that the kernels' grouping (attention head a reads key/value head a / R) hands every query its own
// map's keys, g * maps + m; the value head of g is stored under each of its maps' key heads.
#include "common.h"

namespace {

constexpr int MAP_WAVES = 4;   // waves (items) a block

// u, v -> the pair turned by position x frequency: the angle a 64-bit product brought into -pi .. pi (a 32-bit product of a position
// in the thousands is good to 1e-4 only), its sine and cosine taken in 32-bit.
__device__ __forceinline__ void turned(float u, float v, int position, double frequency, float& a, float& b) {
    const double angle = (double)position * frequency;
    const double turns = rint(angle * 0.15915494309189535);
    float s, c;
    sincosf((float)(angle - turns * 6.283185307179586), &s, &c);
    a = u * c - v * s;
    b = v * c + u * s;
}

// Element d (< rot_dims) of a head `in` after its pair has turned by sign x position x frequencies[pair]: pairs are (m, m + rot_dims / 2)
// or, with `neighbours`, (2m, 2m + 1).
__device__ __forceinline__ float turned_element(const float* in, int d, int rot_dims, int neighbours, int position, const double* frequencies, float sign) {
    const int half = rot_dims / 2;
    const bool first = neighbours ? (d & 1) == 0 : d < half;
    const int pair = neighbours ? d / 2 : (first ? d : d - half);
    const int other = neighbours ? d ^ 1 : (first ? d + half : d - half);
    float a, b;
    if (first) turned(in[d], in[other], position, sign * frequencies[pair], a, b);
    else turned(in[other], in[d], position, sign * frequencies[pair], b, a);
    return a;
}

// A wave per (row, head): the first rot_dims elements of the head turned by sign x position x frequencies[pair] (sign -1 turns back what
// turned_element with sign 1 turned), the elements behind them up to out_size copied. `in` heads lie in_size apart (float32 rows), `out`
// heads out_size apart, so that heads kept wider than their values leave at the values' own size.
template <typename T>
__global__ __launch_bounds__(64 * MAP_WAVES) void turn_heads_kernel(const float* __restrict__ in, int in_stride, T* __restrict__ out, int out_stride,
                                                                   const double* __restrict__ frequencies, int rot_dims, int neighbours, float sign,
                                                                   const int* __restrict__ positions, int n_rows, int n_heads, int in_size, int out_size) {
    const int lane = threadIdx.x % WAVE;
    const long long item = (long long)blockIdx.x * MAP_WAVES + threadIdx.x / WAVE;
    if (item >= (long long)n_rows * n_heads) return;
    const int row = (int)(item / n_heads), head = (int)(item % n_heads);
    const float* from = in + (size_t)row * in_stride + (size_t)head * in_size;
    T* to = out + (size_t)row * out_stride + (size_t)head * out_size;
    const int position = positions[row];
    for (int d = lane; d < out_size; d += WAVE)
        to[d] = from_float<T>(d < rot_dims ? turned_element(from, d, rot_dims, neighbours, position, frequencies, sign) : from[d]);
}

// Four neighbouring elements out, in 32-bit or rounded to bfloat16.
template <typename T>
__device__ __forceinline__ void store_four(T* to, f32x4 made) {
    if constexpr (sizeof(T) == 4) {
        *reinterpret_cast<f32x4*>(to) = made;
    } else {
        bf16x4 narrow;
#pragma unroll
        for (int e = 0; e < 4; e++) narrow[e] = from_float<T>(made[e]);
        *reinterpret_cast<bf16x4*>(to) = narrow;
    }
}

// Four pairs (from[d + e], from[d + half + e]) turned by sign x position x frequencies[d + e] and stored at to + d and to + d + half: the
// sine and cosine of a pair are taken once for both its elements.
template <typename T>
__device__ __forceinline__ void turn_four_pairs(const float* from, T* to, int d, int half, int position, const double* frequencies, float sign) {
    const f32x4 firsts = *reinterpret_cast<const f32x4*>(from + d), seconds = *reinterpret_cast<const f32x4*>(from + d + half);
    f32x4 a, b;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        float x, y;
        turned(firsts[e], seconds[e], position, sign * frequencies[d + e], x, y);
        a[e] = x, b[e] = y;
    }
    store_four(to + d, a);
    store_four(to + d + half, b);
}

// turn_heads_kernel four neighbouring elements a thread (pairing of halves; turned elements, heads and strides in whole fours, rows on 16 bytes).
template <typename T>
__global__ __launch_bounds__(256) void turn_heads_pieces_kernel(const float* __restrict__ in, int in_stride, T* __restrict__ out, int out_stride,
                                                                const double* __restrict__ frequencies, int rot_dims, float sign,
                                                                const int* __restrict__ positions, int n_rows, int n_heads, int in_size, int out_size) {
    const int quads = out_size / 4;
    const long long index = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= (long long)n_rows * n_heads * quads) return;
    const int row = (int)(index / (n_heads * quads)), within = (int)(index % (n_heads * quads));
    const int head = within / quads, d = (within % quads) * 4;
    const float* from = in + (size_t)row * in_stride + (size_t)head * in_size;
    T* to = out + (size_t)row * out_stride + (size_t)head * out_size;
    if (d < rot_dims) {   // the thread of a pair's first element makes both; the thread of the second has nothing to do
        if (d < rot_dims / 2) turn_four_pairs(from, to, d, rot_dims / 2, positions[row], frequencies, sign);
        return;
    }
    store_four(to + d, *reinterpret_cast<const f32x4*>(from + d));
}

// A wave per (row, item); a row's items are its n_heads * maps queries, then (where the layer keeps keys and values of its own: k_at
// >= 0) its n_kv_heads * maps keys and its n_kv_heads values. `rows` are the 32-bit sums of the product that made them, [.. | q | k |
// v | ..] at columns q_at, k_at, v_at: q as [n_heads, maps, dim], k as [n_kv_heads, maps, dim], v as [n_kv_heads, vdim].
// A query or key: RMS norm over its dim elements (gain [dim], shared by all heads and maps; null: no norm), then of its first
// rot_dims elements i and i + rot_dims / 2 turned as a pair by position x frequencies[i]. Queries go to q_out [row, n_kv_heads, maps, R,
// head_size], keys to head g * maps + m of the row's slot in k_pages, a value to heads g * maps + 0 .. maps - 1 of v_pages, zeros
// beyond dim / vdim up to head_size. Padding rows (slot < 0) store nothing.
// v_frequencies (null: values are kept as they are): of a value's first v_rot_dims elements every pair turns by position x
// v_frequencies[pair] before it is stored; v_neighbours 0 pairs element m with m + v_rot_dims / 2, 1 pairs 2m with 2m + 1.
template <typename T>
__global__ __launch_bounds__(64 * MAP_WAVES) void map_rows_kernel(
    const float* __restrict__ rows, int stride, int q_at, int k_at, int v_at, const float* __restrict__ q_gain, const float* __restrict__ k_gain,
    float eps, const double* __restrict__ frequencies, int rot_dims, const int* __restrict__ positions, const int* __restrict__ slots,
    T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages, int n_rows, int n_heads, int n_kv_heads, int maps, int dim,
    int vdim, int head_size, int page_size, const double* __restrict__ v_frequencies, int v_rot_dims, int v_neighbours) {
    const int lane = threadIdx.x % WAVE;
    const int n_q = n_heads * maps, n_k = k_at >= 0 ? n_kv_heads * maps : 0, n_v = k_at >= 0 ? n_kv_heads : 0;
    const int per_row = n_q + n_k + n_v;
    const long long item = (long long)blockIdx.x * MAP_WAVES + threadIdx.x / WAVE;
    if (item >= (long long)n_rows * per_row) return;
    const int row = (int)(item / per_row), which = (int)(item % per_row);
    const float* in_row = rows + (size_t)row * stride;
    const int per_group = n_heads / n_kv_heads;
    if (which >= n_q + n_k) {   // a value head, as it is, under each of its maps
        const int slot = slots[row];
        if (slot < 0) return;
        const int g = which - n_q - n_k;
        const float* in = in_row + v_at + (size_t)g * vdim;
        const int position = v_frequencies ? positions[row] : 0;
        for (int m = 0; m < maps; m++) {
            T* out = v_pages + (((size_t)(slot / page_size) * (n_kv_heads * maps) + g * maps + m) * page_size + slot % page_size) * head_size;
            for (int d = lane; d < head_size; d += WAVE) {
                float value = d < vdim ? in[d] : 0.0f;
                if (v_frequencies && d < v_rot_dims) value = turned_element(in, d, v_rot_dims, v_neighbours, position, v_frequencies, 1.0f);
                out[d] = from_float<T>(value);
            }
        }
        return;
    }
    const bool is_q = which < n_q;
    const int index = is_q ? which : which - n_q;          // (head, map) as stored: head * maps + map
    const int head = index / maps, map = index % maps;
    const float* in = in_row + (is_q ? q_at : k_at) + (size_t)index * dim;
    const float* gain = is_q ? q_gain : k_gain;
    T* out;
    if (is_q) {
        const int g = head / per_group, r = head % per_group;
        out = q_out + ((size_t)row * n_q + (size_t)(g * maps + map) * per_group + r) * head_size;
    } else {
        const int slot = slots[row];
        if (slot < 0) return;
        out = k_pages + (((size_t)(slot / page_size) * n_k + head * maps + map) * page_size + slot % page_size) * head_size;
    }
    float factor = 1.0f;
    if (gain) {
        float squares = 0.0f;
        for (int d = lane; d < dim; d += WAVE) squares += in[d] * in[d];
        factor = 1.0f / sqrtf(wave_sum(squares) / (float)dim + eps);
    }
    const int position = positions[row];
    const int half = rot_dims / 2;
    for (int d = lane; d < head_size; d += WAVE) {
        float value = 0.0f;
        if (d < dim) {
            value = in[d] * factor * (gain ? gain[d] : 1.0f);
            if (d < rot_dims) {
                const int other = d < half ? d + half : d - half;
                const float partner = in[other] * factor * (gain ? gain[other] : 1.0f);
                float a, b;
                if (d < half) turned(value, partner, position, frequencies[d], a, b);
                else turned(partner, value, position, frequencies[other], b, a);
                value = a;
            }
        }
        out[d] = from_float<T>(value);
    }
}

// The same work as map_rows_kernel for heads of one map without a norm, four neighbouring elements a thread: a thread makes elements d ..
// d + 3 of one query, key or value head from 16 bytes of the head and, where they turn, 16 bytes of their partners (pairing of halves; the
// turned elements, the elements behind them and the heads themselves come in whole fours, and the rows start on 16 bytes). A wave so makes
// 256 elements, not 64, and a row's heads need an eighth of the waves.
template <typename T>
__global__ __launch_bounds__(256) void rotate_rows_pieces_kernel(
    const float* __restrict__ rows, int stride, int q_at, int k_at, int v_at, const double* __restrict__ frequencies, int rot_dims,
    const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
    int n_rows, int n_heads, int n_kv_heads, int dim, int vdim, int head_size, int page_size, const double* __restrict__ v_frequencies, int v_rot_dims) {
    const int quads = head_size / 4;
    const int n_kept = k_at >= 0 ? n_kv_heads : 0;
    const int per_row = (n_heads + 2 * n_kept) * quads;
    const long long index = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= (long long)n_rows * per_row) return;
    const int row = (int)(index / per_row), within = (int)(index % per_row);
    const int item = within / quads, d = (within % quads) * 4;
    const float* in_row = rows + (size_t)row * stride;
    const float* in;
    T* out;
    int size = dim, turned_dims = rot_dims;
    const double* f = frequencies;
    if (item < n_heads) {
        in = in_row + q_at + (size_t)item * dim;
        out = q_out + ((size_t)row * n_heads + item) * head_size;
    } else {
        const int slot = slots[row];
        if (slot < 0) return;
        const bool is_key = item < n_heads + n_kept;
        const int g = item - n_heads - (is_key ? 0 : n_kept);
        const size_t place = (((size_t)(slot / page_size) * n_kept + g) * page_size + slot % page_size) * head_size;
        if (is_key) {
            in = in_row + k_at + (size_t)g * dim;
            out = k_pages + place;
        } else {
            in = in_row + v_at + (size_t)g * vdim;
            out = v_pages + place;
            size = vdim, turned_dims = v_frequencies ? v_rot_dims : 0, f = v_frequencies;
        }
    }
    if (d < turned_dims) {   // the thread of a pair's first element makes both; the thread of the second has nothing to do
        if (d < turned_dims / 2) turn_four_pairs(in, out, d, turned_dims / 2, positions[row], f, 1.0f);
        return;
    }
    f32x4 made = {0.0f, 0.0f, 0.0f, 0.0f};
    if (d < size) made = *reinterpret_cast<const f32x4*>(in + d);
    store_four(out + d, made);
}

// A wave per (row, head): with a1 and a2 the results of the head's two maps (attention heads (g * 2 + 0) * R + r and (g * 2 + 1) * R + r
// of `maps_out`, heads of head_size of which the first vdim count), x = a1 - lambda a2, out = x / sqrt(mean(x^2) + eps) * scale *
// sigmoid(gate) -> out [row, head * vdim ..]. gate: 32-bit rows (null: no gate), the head's vdim elements at column head * vdim. The
// maps' results may be of another type than out (32-bit results of the attention, out in the type the output product reads).
template <typename TIN, typename T>
__global__ __launch_bounds__(64 * MAP_WAVES) void map_difference_kernel(
    const TIN* __restrict__ maps_out, int maps_stride, const float* __restrict__ gate, int gate_stride, T* __restrict__ out, int out_stride,
    float lambda, float eps, float scale, int n_rows, int n_heads, int n_kv_heads, int vdim, int head_size) {
    constexpr int REGS = 4;   // heads up to 256 elements
    const int lane = threadIdx.x % WAVE;
    const long long item = (long long)blockIdx.x * MAP_WAVES + threadIdx.x / WAVE;
    if (item >= (long long)n_rows * n_heads) return;
    const int row = (int)(item / n_heads), head = (int)(item % n_heads);
    const int per_group = n_heads / n_kv_heads;
    const int g = head / per_group, r = head % per_group;
    const TIN* first = maps_out + (size_t)row * maps_stride + (size_t)((g * 2) * per_group + r) * head_size;
    const TIN* second = first + (size_t)per_group * head_size;
    float x[REGS], gates[REGS], squares = 0.0f;
#pragma unroll
    for (int e = 0; e < REGS; e++) {
        const int d = lane + e * WAVE;
        const bool has = d < vdim;
        x[e] = has ? to_float(first[d]) - lambda * to_float(second[d]) : 0.0f;
        gates[e] = has && gate ? gate[(size_t)row * gate_stride + head * vdim + d] : 0.0f;
        squares += x[e] * x[e];
    }
    const float factor = scale / sqrtf(wave_sum(squares) / (float)vdim + eps);
#pragma unroll
    for (int e = 0; e < REGS; e++) {
        const int d = lane + e * WAVE;
        if (d < vdim) out[(size_t)row * out_stride + head * vdim + d] = from_float<T>(x[e] * factor * (gate ? 1.0f / (1.0f + expf(-gates[e])) : 1.0f));
    }
}

}  // namespace

MLLM_API int mllm_map_rows(const float* rows, int stride, int q_at, int k_at, int v_at, const float* q_gain, const float* k_gain, float eps,
                           const double* frequencies, int rot_dims, const int* positions, const int* slots, void* q_out, void* k_pages,
                           void* v_pages, int n_rows, int n_heads, int n_kv_heads, int maps, int dim, int vdim, int head_size, int page_size,
                           int dtype, const double* v_frequencies, int v_rot_dims, int v_neighbours, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_heads > 0 && n_kv_heads > 0 && maps > 0 && dim > 0 && vdim > 0 && page_size > 0, "map_rows: bad sizes");
    MLLM_REQUIRE(n_heads % n_kv_heads == 0, "map_rows: %d heads do not divide into %d key/value heads", n_heads, n_kv_heads);
    MLLM_REQUIRE(head_size >= dim && head_size >= vdim, "map_rows: heads of %d do not hold %d / %d elements", head_size, dim, vdim);
    MLLM_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dim, "map_rows: %d rotated elements of %d", rot_dims, dim);
    MLLM_REQUIRE(rows != nullptr && q_out != nullptr && positions != nullptr && (rot_dims == 0 || frequencies != nullptr), "map_rows: a missing operand");
    MLLM_REQUIRE(q_at >= 0 && q_at + n_heads * maps * dim <= stride, "map_rows: the queries lie beyond the rows");
    MLLM_REQUIRE(k_at < 0 || (v_at >= 0 && k_at + n_kv_heads * maps * dim <= stride && v_at + n_kv_heads * vdim <= stride && slots != nullptr &&
                              k_pages != nullptr && v_pages != nullptr),
                 "map_rows: keys and values to keep need their columns, slots and pages");
    MLLM_REQUIRE(v_frequencies == nullptr || (v_rot_dims >= 0 && v_rot_dims % 2 == 0 && v_rot_dims <= vdim), "map_rows: %d turned elements of a value of %d", v_rot_dims, vdim);
    if (n_rows == 0) return 0;
    const long long items = (long long)n_rows * (n_heads * maps + (k_at >= 0 ? n_kv_heads * (maps + 1) : 0));
    const int blocks = (int)((items + MAP_WAVES - 1) / MAP_WAVES);
    mllm_count_kernel(MLLM_K_MAP_ROWS);
    // one map a head and no norm, everything in whole fours: four elements a thread
    const bool values_fit = v_frequencies == nullptr || v_rot_dims == 0 || (v_neighbours == 0 && v_rot_dims % 8 == 0);
    if (maps == 1 && q_gain == nullptr && k_gain == nullptr && rot_dims % 8 == 0 && dim % 4 == 0 && vdim % 4 == 0 && head_size % 4 == 0 && stride % 4 == 0 &&
        q_at % 4 == 0 && (k_at < 0 || (k_at % 4 == 0 && v_at % 4 == 0)) && ((uintptr_t)rows & 15) == 0 && ((uintptr_t)q_out & 15) == 0 &&
        (k_at < 0 || (((uintptr_t)k_pages & 15) == 0 && ((uintptr_t)v_pages & 15) == 0)) && values_fit) {
        const long long threads = (long long)n_rows * (n_heads + (k_at >= 0 ? 2 * n_kv_heads : 0)) * (head_size / 4);
        const int piece_blocks = (int)((threads + 255) / 256);
        const double* vf = v_rot_dims > 0 ? v_frequencies : nullptr;
#define ROTATE_ROWS_ARGS(T) rows, stride, q_at, k_at, v_at, frequencies, rot_dims, positions, slots, (T*)q_out, (T*)k_pages, (T*)v_pages, n_rows, n_heads, \
                            n_kv_heads, dim, vdim, head_size, page_size, vf, v_rot_dims
        if (dtype == MLLM_F32) rotate_rows_pieces_kernel<float><<<piece_blocks, 256, 0, stream>>>(ROTATE_ROWS_ARGS(float));
        else if (dtype == MLLM_BF16) rotate_rows_pieces_kernel<bf16_t><<<piece_blocks, 256, 0, stream>>>(ROTATE_ROWS_ARGS(bf16_t));
        else MLLM_REQUIRE(false, "map_rows: unknown dtype %d", dtype);
#undef ROTATE_ROWS_ARGS
        return mllm_check_launch("map_rows");
    }
#define MAP_ROWS_ARGS(T) rows, stride, q_at, k_at, v_at, q_gain, k_gain, eps, frequencies, rot_dims, positions, slots, (T*)q_out, (T*)k_pages, \
                         (T*)v_pages, n_rows, n_heads, n_kv_heads, maps, dim, vdim, head_size, page_size, v_frequencies, v_rot_dims, v_neighbours
    if (dtype == MLLM_F32) map_rows_kernel<float><<<blocks, 64 * MAP_WAVES, 0, stream>>>(MAP_ROWS_ARGS(float));
    else if (dtype == MLLM_BF16) map_rows_kernel<bf16_t><<<blocks, 64 * MAP_WAVES, 0, stream>>>(MAP_ROWS_ARGS(bf16_t));
    else MLLM_REQUIRE(false, "map_rows: unknown dtype %d", dtype);
#undef MAP_ROWS_ARGS
    return mllm_check_launch("map_rows");
}

MLLM_API int mllm_map_difference(const void* maps_out, int maps_stride, const float* gate, int gate_stride, void* out, int out_stride, float lambda,
                                 float eps, float scale, int n_rows, int n_heads, int n_kv_heads, int vdim, int head_size, int in_dtype, int dtype,
                                 hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_heads > 0 && n_kv_heads > 0 && vdim > 0, "map_difference: bad sizes");
    MLLM_REQUIRE(n_heads % n_kv_heads == 0, "map_difference: %d heads do not divide into %d key/value heads", n_heads, n_kv_heads);
    MLLM_REQUIRE(vdim <= head_size && vdim <= 256, "map_difference: heads of %d values (the kernel takes 256, the maps hold %d)", vdim, head_size);
    MLLM_REQUIRE(maps_stride >= 2 * n_heads * head_size && out_stride >= n_heads * vdim && (gate == nullptr || gate_stride >= n_heads * vdim),
                 "map_difference: rows are too short for the heads");
    MLLM_REQUIRE(maps_out != nullptr && out != nullptr, "map_difference: a missing operand");
    if (n_rows == 0) return 0;
    const long long items = (long long)n_rows * n_heads;
    const int blocks = (int)((items + MAP_WAVES - 1) / MAP_WAVES);
    mllm_count_kernel(MLLM_K_MAP_DIFFERENCE);
#define MAP_DIFFERENCE_ARGS(TIN, T) (const TIN*)maps_out, maps_stride, gate, gate_stride, (T*)out, out_stride, lambda, eps, scale, n_rows, n_heads, \
                                    n_kv_heads, vdim, head_size
    if (in_dtype == MLLM_F32 && dtype == MLLM_F32) map_difference_kernel<float, float><<<blocks, 64 * MAP_WAVES, 0, stream>>>(MAP_DIFFERENCE_ARGS(float, float));
    else if (in_dtype == MLLM_F32 && dtype == MLLM_BF16) map_difference_kernel<float, bf16_t><<<blocks, 64 * MAP_WAVES, 0, stream>>>(MAP_DIFFERENCE_ARGS(float, bf16_t));
    else if (in_dtype == MLLM_BF16 && dtype == MLLM_BF16) map_difference_kernel<bf16_t, bf16_t><<<blocks, 64 * MAP_WAVES, 0, stream>>>(MAP_DIFFERENCE_ARGS(bf16_t, bf16_t));
    else MLLM_REQUIRE(false, "map_difference: maps of dtype %d into rows of dtype %d", in_dtype, dtype);
#undef MAP_DIFFERENCE_ARGS
    return mllm_check_launch("map_difference");
}

MLLM_API int mllm_turn_heads(const float* in, int in_stride, void* out, int out_stride, const double* frequencies, int rot_dims, int neighbours, float sign,
                             const int* positions, int n_rows, int n_heads, int in_size, int out_size, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_heads > 0 && in_size > 0 && out_size > 0 && out_size <= in_size, "turn_heads: bad sizes");
    MLLM_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= out_size, "turn_heads: %d turned elements of %d", rot_dims, out_size);
    MLLM_REQUIRE(in_stride >= n_heads * in_size && out_stride >= n_heads * out_size, "turn_heads: rows are too short for the heads");
    MLLM_REQUIRE(in != nullptr && out != nullptr && positions != nullptr && (rot_dims == 0 || frequencies != nullptr), "turn_heads: a missing operand");
    if (n_rows == 0) return 0;
    const long long items = (long long)n_rows * n_heads;
    const int blocks = (int)((items + MAP_WAVES - 1) / MAP_WAVES);
    mllm_count_kernel(MLLM_K_TURN_HEADS);
    if (neighbours == 0 && rot_dims % 8 == 0 && in_size % 4 == 0 && out_size % 4 == 0 && in_stride % 4 == 0 && out_stride % 4 == 0 && ((uintptr_t)in & 15) == 0 &&
        ((uintptr_t)out & 15) == 0) {
        const long long threads = items * (out_size / 4);
        const int piece_blocks = (int)((threads + 255) / 256);
        if (dtype == MLLM_F32)
            turn_heads_pieces_kernel<float><<<piece_blocks, 256, 0, stream>>>(in, in_stride, (float*)out, out_stride, frequencies, rot_dims, sign, positions, n_rows, n_heads, in_size, out_size);
        else if (dtype == MLLM_BF16)
            turn_heads_pieces_kernel<bf16_t><<<piece_blocks, 256, 0, stream>>>(in, in_stride, (bf16_t*)out, out_stride, frequencies, rot_dims, sign, positions, n_rows, n_heads, in_size, out_size);
        else MLLM_REQUIRE(false, "turn_heads: unknown dtype %d", dtype);
        return mllm_check_launch("turn_heads");
    }
#define TURN_HEADS_ARGS(T) in, in_stride, (T*)out, out_stride, frequencies, rot_dims, neighbours, sign, positions, n_rows, n_heads, in_size, out_size
    if (dtype == MLLM_F32) turn_heads_kernel<float><<<blocks, 64 * MAP_WAVES, 0, stream>>>(TURN_HEADS_ARGS(float));
    else if (dtype == MLLM_BF16) turn_heads_kernel<bf16_t><<<blocks, 64 * MAP_WAVES, 0, stream>>>(TURN_HEADS_ARGS(bf16_t));
    else MLLM_REQUIRE(false, "turn_heads: unknown dtype %d", dtype);
#undef TURN_HEADS_ARGS
    return mllm_check_launch("turn_heads");
}
