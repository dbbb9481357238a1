// Plain attention over the paged cache for heads whose keys and values have sizes of their own: one
// workgroup per (row, query head, map), any sizes, float32 or bfloat16 storage, float32 arithmetic.  The
// float32 path, and the reference beside the matrix-core kernel.
//
// A query head may have several softmax maps over the same values (`maps`): map m of query head h reads
// key head g * maps + m with g = h / (heads / kv_heads), and the values of head g.  The values come from a
// cache of their own ([page][kv head][value_dim][slot]) or, without one, are the first value_dim elements
// of the key itself (keys that carry the vector their values are made from).
//
// With `sinks` (float32, one a (head, map)) the softmax's denominator also holds exp(sink): a logit without key or value.
//
// Row at position p sees key t <= p if p - t < window or t < keep_first (window 0: every t <= p).  The seen
// keys are walked in one fixed order (the kept first ones, then the window's), 256 at a time with a running
// maximum and sum; the order of additions depends on (p, window, keep_first) alone, never on the batch.
#include "common.h"

#define AS_THREADS 256
#define AS_MAX_DIM 1024

template <typename T, typename TO>
__global__ __launch_bounds__(AS_THREADS) void attention_sized_plain_kernel(
    const T* __restrict__ q, TO* __restrict__ out, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ seq_of_row, const int* __restrict__ tables,
    int table_width, int page_size, int num_pages, int heads, int kv_heads, int maps, int key_dim, int value_dim,
    float scale, int window, int keep_first, const float* __restrict__ sinks) {
    __shared__ float q_s[AS_MAX_DIM];
    __shared__ float p_s[AS_THREADS];
    __shared__ float red[16];
    const int row = blockIdx.x, unit = blockIdx.y;                      // unit = head * maps + map
    const int head = unit / maps, map = unit % maps;
    const int tid = threadIdx.x;
    const int g = head / (heads / kv_heads);
    const int kh = g * maps + map;
    const int pos = positions[row];
    const int* table = tables + (size_t)seq_of_row[row] * table_width;
    const int lo = (window > 0) ? max(0, pos - window + 1) : 0;
    const int kept = (window > 0) ? min(keep_first, lo) : 0;            // kept first keys that lie before the window
    const int seen = kept + (pos - lo + 1);
    const size_t k_page = (size_t)kv_heads * maps * page_size * key_dim;
    const size_t v_page = (size_t)kv_heads * page_size * value_dim;

    const T* q_row = q + ((size_t)row * heads * maps + unit) * key_dim;
    for (int d = tid; d < key_dim; d += AS_THREADS) q_s[d] = to_f32(q_row[d]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[AS_MAX_DIM / AS_THREADS];
#pragma unroll
    for (int i = 0; i < AS_MAX_DIM / AS_THREADS; ++i) acc[i] = 0.f;
    for (int base = 0; base < seen; base += AS_THREADS) {
        const int i = base + tid;
        float s = -INFINITY;
        if (i < seen) {
            const int t = i < kept ? i : lo + (i - kept);
            const int page = table[t / page_size];
            if (page >= 0 && page < num_pages) {
                const T* kp = k_cache + (size_t)page * k_page + ((size_t)kh * page_size + (t % page_size)) * key_dim;
                float dot = 0.f;
                for (int d = 0; d < key_dim; ++d) dot = fmaf(q_s[d], to_f32(kp[d]), dot);
                s = dot * scale;
            }
        }
        const float m_new = fmaxf(m, block_max(s, red));
        const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
        const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
        l = l * corr + block_sum(p, red);
        p_s[tid] = p;
        __syncthreads();
        const int count = min(AS_THREADS, seen - base);
#pragma unroll
        for (int part = 0; part < AS_MAX_DIM / AS_THREADS; ++part) {
            const int d = tid + part * AS_THREADS;
            if (d >= value_dim) break;
            float a = acc[part] * corr;
            for (int j = 0; j < count; ++j) {
                const int ii = base + j;
                const int t = ii < kept ? ii : lo + (ii - kept);
                const int page = table[t / page_size];
                if (page < 0 || page >= num_pages) continue;
                float v;
                if (v_cache)
                    v = to_f32(v_cache[(size_t)page * v_page + ((size_t)g * value_dim + d) * page_size + (t % page_size)]);
                else
                    v = to_f32(k_cache[(size_t)page * k_page + ((size_t)kh * page_size + (t % page_size)) * key_dim + d]);
                a = fmaf(p_s[j], v, a);
            }
            acc[part] = a;
        }
        m = m_new;
        __syncthreads();
    }
    TO* o_row = out + ((size_t)row * heads * maps + unit) * value_dim;
    float inv = (l > 0.f) ? 1.0f / l : 0.f;
    if (sinks) {                                                        // the denominator also holds exp(sink)
        const float top = fmaxf(m, sinks[unit]);
        const float keys = (m == -INFINITY) ? 0.f : expf(m - top);
        inv = keys / (l * keys + expf(sinks[unit] - top));
    }
#pragma unroll
    for (int part = 0; part < AS_MAX_DIM / AS_THREADS; ++part) {
        const int d = tid + part * AS_THREADS;
        if (d < value_dim) from_f32(o_row + d, acc[part] * inv);
    }
}

// q [rows, heads * maps, key_dim]; out [rows, heads * maps, value_dim] (float32 with out_f32, else the type of q);
// k_cache [pages][kv_heads * maps][slot][key_dim]; v_cache [pages][kv_heads][value_dim][slot] or null
extern "C" int tli_attention_sized_plain(
    const void* q, void* out, const void* k_cache, const void* v_cache, const int* positions, const int* seq_of_row,
    const int* tables, int table_width, int page_size, int num_pages, int rows, int heads, int kv_heads, int maps,
    int key_dim, int value_dim, float scale, int window, int keep_first, int dtype, int out_f32, const float* sinks,
    void* stream) {
    if (rows <= 0) return 0;
    if (key_dim <= 0 || key_dim > AS_MAX_DIM || value_dim <= 0 || value_dim > AS_MAX_DIM)
        return tli_fail("attention: heads of %d and %d elements are outside 1..%d", key_dim, value_dim, AS_MAX_DIM);
    if (!v_cache && value_dim > key_dim) return tli_fail("attention: values of %d elements cannot be the start of keys of %d", value_dim, key_dim);
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || maps <= 0)
        return tli_fail("attention: heads %d must be a multiple of kv heads %d", heads, kv_heads);
    if ((long long)heads * maps > 65535) return tli_fail("attention: %d heads exceed the grid limit 65535", heads * maps);
    if (page_size <= 0 || table_width <= 0 || num_pages <= 0) return tli_fail("attention: bad cache geometry");
    if (window < 0 || keep_first < 0) return tli_fail("attention: bad window %d with %d kept", window, keep_first);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(rows, heads * maps);
#define AS_ARGS positions, seq_of_row, tables, table_width, page_size, num_pages, heads, kv_heads, maps, key_dim, value_dim, scale, window, keep_first, sinks
    if (dtype == TLI_F32)
        attention_sized_plain_kernel<float, float><<<grid, AS_THREADS, 0, s>>>((const float*)q, (float*)out, (const float*)k_cache,
                                                                               (const float*)v_cache, AS_ARGS);
    else if (dtype == TLI_BF16 && out_f32)
        attention_sized_plain_kernel<bf16_t, float><<<grid, AS_THREADS, 0, s>>>((const bf16_t*)q, (float*)out, (const bf16_t*)k_cache,
                                                                                (const bf16_t*)v_cache, AS_ARGS);
    else if (dtype == TLI_BF16)
        attention_sized_plain_kernel<bf16_t, bf16_t><<<grid, AS_THREADS, 0, s>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)k_cache,
                                                                                 (const bf16_t*)v_cache, AS_ARGS);
    else
        return tli_fail("attention: unknown dtype %d", dtype);
#undef AS_ARGS
    return tli_check_launch("attention_sized_plain");
}
