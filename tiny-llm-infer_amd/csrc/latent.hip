// Attention over a latent vector a position: what stands before and behind the attention itself.
//
// prepare:        from the raw projections of a row (q of `heads` heads of dim + rot elements, then the latent
//                 vector of `rank` elements and one key part of `rot` elements) the cache entry of the position,
//                 [RMS norm of the latent vector with its weight | the key part, turned], and the queries' own
//                 turned parts, written behind the place where their `rank` elements in the latent space go.
//                 The first rot_dims elements of a part are turned in pairs (i, i + rot_dims / 2).  One workgroup
//                 a row; float32 arithmetic.
// head_products:  y[t, h, :] = W[h] x[t, h, :] for a matrix a head (float32 sums), with strides so that inputs
//                 and outputs may lie inside wider rows.  Plain: any sizes and both types.
#include "common.h"

#define LP_THREADS 256

template <typename T>
__global__ __launch_bounds__(LP_THREADS) void latent_prepare_kernel(
    const T* __restrict__ proj, int ld, T* __restrict__ q_out, T* __restrict__ cache, const int* __restrict__ positions,
    const int* __restrict__ seq_of_row, const int* __restrict__ tables, int table_width, int page_size, int num_pages,
    int heads, int dim, int rot, int rank, int rot_dims, const float* __restrict__ norm_weight, float eps,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t) {
    __shared__ float red[16];
    const int row = blockIdx.x, tid = threadIdx.x;
    const T* src = proj + (size_t)row * ld;
    const int pos = positions[row];
    const int half = rot_dims / 2;
    const float* cs = cos_t + (size_t)pos * half;
    const float* sn = sin_t + (size_t)pos * half;
    const int key = rank + rot;
    // the queries' turned parts
    for (int i = tid; i < heads * rot; i += LP_THREADS) {
        const int h = i / rot, d = i % rot;
        const T* part = src + (size_t)h * (dim + rot) + dim;
        float v = to_f32(part[d]);
        if (d < half) v = rotate_first_half(v, to_f32(part[d + half]), cs[d], sn[d]);
        else if (d < rot_dims) v = rotate_second_half(v, to_f32(part[d - half]), cs[d - half], sn[d - half]);
        from_f32(q_out + ((size_t)row * heads + h) * key + rank + d, v);
    }
    const int page = tables[(size_t)seq_of_row[row] * table_width + pos / page_size];
    const T* down = src + (size_t)heads * (dim + rot);
    float ssq = 0.f;
    for (int d = tid; d < rank; d += LP_THREADS) {
        const float a = to_f32(down[d]);
        ssq = fmaf(a, a, ssq);
    }
    const float factor = 1.0f / sqrtf(block_sum(ssq, red) / (float)rank + eps);
    if (page < 0 || page >= num_pages) return;
    T* dst = cache + ((size_t)page * page_size + pos % page_size) * key;
    for (int d = tid; d < rank; d += LP_THREADS) {
        T r;
        from_f32(&r, to_f32(down[d]) * factor * norm_weight[d]);
        dst[d] = cache_value(r);
    }
    const T* part = down + rank;
    for (int d = tid; d < rot; d += LP_THREADS) {
        float v = to_f32(part[d]);
        if (d < half) v = rotate_first_half(v, to_f32(part[d + half]), cs[d], sn[d]);
        else if (d < rot_dims) v = rotate_second_half(v, to_f32(part[d - half]), cs[d - half], sn[d - half]);
        T r;
        from_f32(&r, v);
        dst[rank + d] = cache_value(r);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void head_products_plain_kernel(const T* __restrict__ x, long long x_row, long long x_head,
                                                                  const T* __restrict__ w, T* __restrict__ y, long long y_row,
                                                                  long long y_head, int N, int K) {
    extern __shared__ float xs[];
    const int t = blockIdx.x, h = blockIdx.y;
    const T* xr = x + (size_t)t * x_row + (size_t)h * x_head;
    for (int k = threadIdx.x; k < K; k += blockDim.x) xs[k] = to_f32(xr[k]);
    __syncthreads();
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE, waves = blockDim.x / TLI_WAVE;
    for (int n = wave; n < N; n += waves) {
        const T* wr = w + ((size_t)h * N + n) * K;
        float a = 0.f;
        for (int k = lane; k < K; k += TLI_WAVE) a = fmaf(xs[k], to_f32(wr[k]), a);
        a = wave_sum(a);
        if (lane == 0) from_f32(y + (size_t)t * y_row + (size_t)h * y_head + n, a);
    }
}

// proj [rows, ld]: q (heads * (dim + rot)) | latent (rank) | key part (rot);  q_out [rows, heads, rank + rot] (only
// the last rot of every head are written);  cache [pages][slot][rank + rot];  cos_t, sin_t [positions, rot_dims / 2]
extern "C" int tli_latent_prepare(const void* proj, int ld, void* q_out, void* cache, const int* positions,
                                  const int* seq_of_row, const int* tables, int table_width, int page_size, int num_pages,
                                  int rows, int heads, int dim, int rot, int rank, int rot_dims, const float* norm_weight,
                                  float eps, const float* cos_t, const float* sin_t, int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (heads <= 0 || dim <= 0 || rot <= 0 || rank <= 0 || rot_dims <= 0 || rot_dims % 2 || rot_dims > rot ||
        ld < heads * (dim + rot) + rank + rot)
        return tli_fail("latent_prepare: bad sizes");
    if (page_size <= 0 || table_width <= 0 || num_pages <= 0) return tli_fail("latent_prepare: bad cache geometry");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TLI_F32)
        latent_prepare_kernel<float><<<rows, LP_THREADS, 0, s>>>((const float*)proj, ld, (float*)q_out, (float*)cache, positions,
                                                                 seq_of_row, tables, table_width, page_size, num_pages, heads, dim,
                                                                 rot, rank, rot_dims, norm_weight, eps, cos_t, sin_t);
    else if (dtype == TLI_BF16)
        latent_prepare_kernel<bf16_t><<<rows, LP_THREADS, 0, s>>>((const bf16_t*)proj, ld, (bf16_t*)q_out, (bf16_t*)cache, positions,
                                                                  seq_of_row, tables, table_width, page_size, num_pages, heads, dim,
                                                                  rot, rank, rot_dims, norm_weight, eps, cos_t, sin_t);
    else
        return tli_fail("latent_prepare: unknown dtype %d", dtype);
    return tli_check_launch("latent_prepare");
}

// y[t, h, n] = sum_k x[t, h, k] w[h, n, k];  x at x + t * x_row + h * x_head (elements), y likewise;  w [heads, N, K]
extern "C" int tli_head_products_plain(const void* x, long long x_row, long long x_head, const void* w, void* y, long long y_row,
                                       long long y_head, int rows, int heads, int N, int K, int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (heads <= 0 || heads > 65535 || N <= 0 || K <= 0 || K > 12288) return tli_fail("head_products: bad sizes");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(rows, heads);
    if (dtype == TLI_F32)
        head_products_plain_kernel<float><<<grid, 256, (size_t)K * 4, s>>>((const float*)x, x_row, x_head, (const float*)w, (float*)y,
                                                                           y_row, y_head, N, K);
    else if (dtype == TLI_BF16)
        head_products_plain_kernel<bf16_t><<<grid, 256, (size_t)K * 4, s>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)y,
                                                                            y_row, y_head, N, K);
    else
        return tli_fail("head_products: unknown dtype %d", dtype);
    return tli_check_launch("head_products_plain");
}
