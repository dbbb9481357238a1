// Attention with two softmax maps a head: what stands before and behind the attention itself.
//
// prepare:  from the raw projections of a row (q of heads * 2 maps, k of kv_heads * 2 maps, v of kv_heads, then one
//           gate logit a head) the normed queries (RMS norm over a head's map with one weight vector for all),
//           the normed keys into the cache ([page][kv head * 2 + map][slot][dim]) and the values into theirs
//           ([page][kv head][vdim][slot]).  One wave a (row, unit); float32 arithmetic.
// combine:  o = a1 - lambda a2 from the two maps' float32 outputs, o / sqrt(mean(o^2) + eps) over the head's
//           values, times `after` (a constant) and sigmoid(gate logit of the head).  One wave a (row, head).
#include "common.h"

template <typename T>
__global__ __launch_bounds__(64) void diff_prepare_kernel(
    const T* __restrict__ proj, int ld, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ seq_of_row, const int* __restrict__ tables,
    int table_width, int page_size, int num_pages, int q_units, int k_units, int v_units, int dim, int vdim,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps) {
    const int row = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const T* src = proj + (size_t)row * ld;
    const int pos = positions[row];
    int page = -1;
    if (unit >= q_units) {
        page = tables[(size_t)seq_of_row[row] * table_width + pos / page_size];
        if (page < 0 || page >= num_pages) return;                  // (a row of no request without a page: nothing to keep)
    }
    const int slot = pos % page_size;
    if (unit < q_units + k_units) {
        const bool is_q = unit < q_units;
        const T* x = src + (size_t)unit * dim;                      // keys follow the queries, unit by unit
        const float* w = is_q ? q_weight : k_weight;
        float ssq = 0.f;
        for (int d = lane; d < dim; d += 64) {
            const float a = to_f32(x[d]);
            ssq = fmaf(a, a, ssq);
        }
        const float factor = 1.0f / sqrtf(wave_sum(ssq) / (float)dim + eps);
        T* dst = is_q ? q_out + ((size_t)row * q_units + unit) * dim
                      : k_cache + (((size_t)page * k_units + (unit - q_units)) * page_size + slot) * dim;
        for (int d = lane; d < dim; d += 64) {
            T r;
            from_f32(&r, to_f32(x[d]) * factor * w[d]);
            dst[d] = is_q ? r : cache_value(r);
        }
    } else {
        const int vh = unit - q_units - k_units;
        const T* x = src + (size_t)(q_units + k_units) * dim + (size_t)vh * vdim;
        T* dst = v_cache + ((size_t)page * v_units + vh) * vdim * page_size + slot;
        for (int d = lane; d < vdim; d += 64) dst[(size_t)d * page_size] = cache_value(x[d]);
    }
}

template <typename T>
__global__ __launch_bounds__(64) void diff_combine_kernel(const float* __restrict__ maps, const T* __restrict__ proj, int ld,
                                                          int gate_at, T* __restrict__ out, int heads, int vdim, float lambda,
                                                          float after, float eps) {
    const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const float* a1 = maps + ((size_t)row * heads + head) * 2 * vdim;
    const float* a2 = a1 + vdim;
    float ssq = 0.f;
    for (int d = lane; d < vdim; d += 64) {
        const float o = a1[d] - lambda * a2[d];
        ssq = fmaf(o, o, ssq);
    }
    const float z = to_f32(proj[(size_t)row * ld + gate_at + head]);
    const float gate = 1.0f / (1.0f + expf(-z));
    const float factor = after * gate / sqrtf(wave_sum(ssq) / (float)vdim + eps);
    T* dst = out + ((size_t)row * heads + head) * vdim;
    for (int d = lane; d < vdim; d += 64) from_f32(dst + d, (a1[d] - lambda * a2[d]) * factor);
}

// proj [rows, ld]: q (heads * 2 * dim) | k (kv_heads * 2 * dim) | v (kv_heads * vdim) | ...
extern "C" int tli_diff_prepare(const void* proj, int ld, void* q_out, void* k_cache, void* v_cache, const int* positions,
                                const int* seq_of_row, const int* tables, int table_width, int page_size, int num_pages,
                                int rows, int heads, int kv_heads, int dim, int vdim, const float* q_weight,
                                const float* k_weight, float eps, int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (heads <= 0 || kv_heads <= 0 || dim <= 0 || vdim <= 0 || ld < (heads + kv_heads) * 2 * dim + kv_heads * vdim)
        return tli_fail("diff_prepare: bad sizes");
    if (page_size <= 0 || table_width <= 0 || num_pages <= 0) return tli_fail("diff_prepare: bad cache geometry");
    const int units = (heads + kv_heads) * 2 + kv_heads;
    if (units > 65535) return tli_fail("diff_prepare: too many heads for one launch");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(rows, units);
    if (dtype == TLI_F32)
        diff_prepare_kernel<float><<<grid, 64, 0, s>>>((const float*)proj, ld, (float*)q_out, (float*)k_cache, (float*)v_cache,
                                                       positions, seq_of_row, tables, table_width, page_size, num_pages,
                                                       heads * 2, kv_heads * 2, kv_heads, dim, vdim, q_weight, k_weight, eps);
    else if (dtype == TLI_BF16)
        diff_prepare_kernel<bf16_t><<<grid, 64, 0, s>>>((const bf16_t*)proj, ld, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache,
                                                        positions, seq_of_row, tables, table_width, page_size, num_pages,
                                                        heads * 2, kv_heads * 2, kv_heads, dim, vdim, q_weight, k_weight, eps);
    else
        return tli_fail("diff_prepare: unknown dtype %d", dtype);
    return tli_check_launch("diff_prepare");
}

// maps [rows, heads, 2, vdim] float32; the gate logit of head h is proj[row, gate_at + h]; out [rows, heads * vdim]
extern "C" int tli_diff_combine(const float* maps, const void* proj, int ld, int gate_at, void* out, int rows, int heads,
                                int vdim, float lambda, float after, float eps, int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (heads <= 0 || heads > 65535 || vdim <= 0 || gate_at < 0 || ld < gate_at + heads) return tli_fail("diff_combine: bad sizes");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(rows, heads);
    if (dtype == TLI_F32)
        diff_combine_kernel<float><<<grid, 64, 0, s>>>(maps, (const float*)proj, ld, gate_at, (float*)out, heads, vdim, lambda, after, eps);
    else if (dtype == TLI_BF16)
        diff_combine_kernel<bf16_t><<<grid, 64, 0, s>>>(maps, (const bf16_t*)proj, ld, gate_at, (bf16_t*)out, heads, vdim, lambda, after, eps);
    else
        return tli_fail("diff_combine: unknown dtype %d", dtype);
    return tli_check_launch("diff_combine");
}
