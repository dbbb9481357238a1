// What stands before and behind the attention with biases whose values may be its keys.
//
// keyed_prepare, for every row and head, in float32:
//   q = proj q + bias,  k = proj k + bias      (the bias vector covers the row of projections; null: none)
//   v = k as it is here, before it is turned (values_at < 0), or proj[values_at ..] + bias
//   q, k:  (x_i, x_{i+rd/2}) <- (x_i cos - x_{i+rd/2} sin, x_{i+rd/2} cos + x_i sin), i < rd/2; the rest as it is
//   q -> q_out [rows, heads, head_dim]
//   k -> keys[page = table[seq][pos / page_size]][kv head][pos % page_size][:]
//   v -> values[page][kv head][:][pos % page_size]      (values are kept transposed)
// One wave a (row, head); the rotation's partner comes through the wave's piece of LDS.
//
// add_bias: y[row, :] += bias, in place.
#include "common.h"

#define KP_WAVES 4
#define KP_MAX_HEAD_DIM 1024

template <typename T>
__global__ void keyed_prepare_kernel(
    const T* __restrict__ proj, int ld, const float* __restrict__ bias, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const int* __restrict__ positions, const int* __restrict__ seq_of_row,
    const int* __restrict__ tables, int table_width, int page_size, int num_pages, int heads, int kv_heads, int head_dim,
    int values_at, const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rotary_dim,
    int table_positions) {
    extern __shared__ float kp_stage[];
    const int row = blockIdx.x;
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE;
    const int unit = blockIdx.y * KP_WAVES + wave;                      // q heads, then k heads
    if (unit >= heads + kv_heads) return;
    float* x = kp_stage + (size_t)wave * head_dim;
    const int pos = positions[row];
    const T* src_row = proj + (size_t)row * ld;
    const size_t at = (size_t)unit * head_dim;                          // q heads and k heads lie side by side
    for (int i = lane; i < head_dim; i += TLI_WAVE) x[i] = to_f32(src_row[at + i]) + (bias ? bias[at + i] : 0.f);
    wave_lds_sync();
    const int half = rotary_dim / 2;
    const bool turn = cos_table && pos >= 0 && pos < table_positions;
    const float* cos_row = turn ? cos_table + (size_t)pos * half : nullptr;
    const float* sin_row = turn ? sin_table + (size_t)pos * half : nullptr;
    auto turned = [&](int i) {
        if (!turn || i >= rotary_dim) return x[i];
        if (i < half) return x[i] * cos_row[i] - x[i + half] * sin_row[i];
        return x[i] * cos_row[i - half] + x[i - half] * sin_row[i - half];
    };
    if (unit < heads) {
        T* dst = q_out + ((size_t)row * heads + unit) * head_dim;
        for (int i = lane; i < head_dim; i += TLI_WAVE) from_f32(dst + i, turned(i));
        return;
    }
    const int g = unit - heads;
    const int page = tables[(size_t)seq_of_row[row] * table_width + pos / page_size];
    if (page < 0 || page >= num_pages) return;
    const int slot = pos % page_size;
    T* k_dst = k_cache + (((size_t)page * kv_heads + g) * page_size + slot) * head_dim;
    T* v_dst = v_cache + ((size_t)page * kv_heads + g) * head_dim * page_size + slot;
    const size_t v_src = values_at >= 0 ? (size_t)values_at + (size_t)g * head_dim : 0;
    for (int i = lane; i < head_dim; i += TLI_WAVE) {
        T k, v;
        from_f32(&k, turned(i));
        from_f32(&v, values_at >= 0 ? to_f32(src_row[v_src + i]) + (bias ? bias[v_src + i] : 0.f) : x[i]);
        k_dst[i] = cache_value(k);
        v_dst[(size_t)i * page_size] = cache_value(v);
    }
}

// proj: [rows, ld], q (heads * head_dim) then k (kv_heads * head_dim) first; bias: float32 [ld] or null;
// values_at: the column where the values' projection starts, or -1: the values are the keys before they are turned;
// cos, sin: float32 [table_positions, rotary_dim / 2] or null
extern "C" int tli_keyed_prepare(const void* proj, int ld, const float* bias, void* q_out, void* k_cache, void* v_cache,
                                 const int* positions, const int* seq_of_row, const int* tables, int table_width,
                                 int page_size, int num_pages, int rows, int heads, int kv_heads, int head_dim,
                                 int values_at, const float* cos_table, const float* sin_table, int rotary_dim,
                                 int table_positions, int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (head_dim <= 0 || head_dim > KP_MAX_HEAD_DIM) return tli_fail("keyed_prepare: head_dim %d is outside 1..%d", head_dim, KP_MAX_HEAD_DIM);
    if (heads <= 0 || kv_heads <= 0) return tli_fail("keyed_prepare: bad head counts");
    const int need = (heads + kv_heads) * head_dim;
    if (ld < need || (values_at >= 0 && (values_at < need || values_at + kv_heads * head_dim > ld)))
        return tli_fail("keyed_prepare: rows of %d do not hold the projections", ld);
    if (cos_table && (rotary_dim <= 0 || rotary_dim % 2 || rotary_dim > head_dim))
        return tli_fail("keyed_prepare: rotary_dim %d must be even and at most head_dim %d", rotary_dim, head_dim);
    if (page_size <= 0 || table_width <= 0 || num_pages <= 0) return tli_fail("keyed_prepare: bad cache geometry");
    const int units = heads + kv_heads;
    if ((units + KP_WAVES - 1) / KP_WAVES > 65535) return tli_fail("keyed_prepare: too many heads");
    const dim3 grid(rows, (units + KP_WAVES - 1) / KP_WAVES);
    const size_t lds = (size_t)KP_WAVES * head_dim * sizeof(float);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TLI_F32)
        hipLaunchKernelGGL((keyed_prepare_kernel<float>), grid, dim3(KP_WAVES * TLI_WAVE), lds, s, (const float*)proj, ld, bias,
                           (float*)q_out, (float*)k_cache, (float*)v_cache, positions, seq_of_row, tables, table_width,
                           page_size, num_pages, heads, kv_heads, head_dim, values_at, cos_table, sin_table, rotary_dim,
                           table_positions);
    else if (dtype == TLI_BF16)
        hipLaunchKernelGGL((keyed_prepare_kernel<bf16_t>), grid, dim3(KP_WAVES * TLI_WAVE), lds, s, (const bf16_t*)proj, ld, bias,
                           (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, positions, seq_of_row, tables, table_width,
                           page_size, num_pages, heads, kv_heads, head_dim, values_at, cos_table, sin_table, rotary_dim,
                           table_positions);
    else
        return tli_fail("keyed_prepare: unknown dtype %d", dtype);
    return tli_check_launch("keyed_prepare");
}

template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, const float* __restrict__ bias, int n, size_t total) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    from_f32(y + idx, to_f32(y[idx]) + bias[idx % n]);
}

// eight elements a thread, 16-byte accesses: n % 8 == 0
__global__ void add_bias_vec_kernel(bf16_t* __restrict__ y, const float* __restrict__ bias, int n, size_t groups) {
    const size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= groups) return;
    const int col = (int)(g % (n / 8)) * 8;
    uint4* at = reinterpret_cast<uint4*>(y) + g;
    const uint4 v = *at;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    const float4 b0 = *reinterpret_cast<const float4*>(bias + col), b1 = *reinterpret_cast<const float4*>(bias + col + 4);
    const float b[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        o[i] = pack_bf16x2(bf16_to_f32((bf16_t)(w[i] & 0xffffu)) + b[2 * i], bf16_to_f32((bf16_t)(w[i] >> 16)) + b[2 * i + 1]);
    *at = make_uint4(o[0], o[1], o[2], o[3]);
}

// y: [rows, n] in place; bias: float32 [n]
extern "C" int tli_add_bias(void* y, const float* bias, int rows, int n, int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (n <= 0) return tli_fail("add_bias: bad size %d", n);
    const size_t total = (size_t)rows * n;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TLI_F32) hipLaunchKernelGGL((add_bias_kernel<float>), dim3(blocks), dim3(256), 0, s, (float*)y, bias, n, total);
    else if (dtype == TLI_BF16 && n % 8 == 0 && !(((uintptr_t)y | (uintptr_t)bias) & 15))
        hipLaunchKernelGGL(add_bias_vec_kernel, dim3((unsigned)((total / 8 + 255) / 256)), dim3(256), 0, s, (bf16_t*)y, bias, n, total / 8);
    else if (dtype == TLI_BF16) hipLaunchKernelGGL((add_bias_kernel<bf16_t>), dim3(blocks), dim3(256), 0, s, (bf16_t*)y, bias, n, total);
    else return tli_fail("add_bias: unknown dtype %d", dtype);
    return tli_check_launch("add_bias");
}
