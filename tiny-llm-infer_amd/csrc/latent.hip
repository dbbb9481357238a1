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

// ---------------------------------------------------------------------------------------------------------------
// head_products on the matrix cores (bfloat16, N and K in sixteens): a workgroup of four waves takes 16 rows and one
// head; its waves share out the head's blocks of 16 outputs.  A is a block of W (16 outputs x 16 of k), B the rows'
// fragments, which a wave holds in registers for all its blocks (k up to 640), so a lane ends with four consecutive
// outputs of one row.  v_mfma_f32_16x16x16_bf16.
// ---------------------------------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(4))) short hp_bf16x4;
typedef __attribute__((ext_vector_type(4))) float hp_f32x4;
union HpFrag {
    uint2 u;
    hp_bf16x4 v;
};

// A wave takes RT tiles of 16 rows and walks all blocks of 16 outputs, two at a time with a sum each, so that a
// matrix instruction does not wait for the one before it; a block of W that it has fetched serves all its row tiles.
// (A workgroup's four waves fetch the same blocks of W one after the other: three of them find it in the cache.)
// EXACT: K is 16 KM (no condition left in the loop over k).
template <int KM, bool EXACT, int RT>
__global__ __launch_bounds__(256) void head_products_mfma_kernel(const bf16_t* __restrict__ x, long long x_row, long long x_head,
                                                                 const bf16_t* __restrict__ w, bf16_t* __restrict__ y,
                                                                 long long y_row, long long y_head, int T, int N, int K) {
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int col = lane % 16, grp = lane / 16;
    const int t0 = (blockIdx.x * 4 + wave) * 16 * RT, h = blockIdx.y;
    if (t0 >= T) return;                                                // (the whole wave; no barriers in this kernel)
    const int nk = EXACT ? KM : K / 16;
    HpFrag xf[RT][KM];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const int t = min(t0 + r * 16 + col, T - 1);                    // (rows past the end repeat the last; never stored)
        const bf16_t* xr = x + (size_t)t * x_row + (size_t)h * x_head;
#pragma unroll
        for (int j = 0; j < KM; ++j) {
            xf[r][j].u = make_uint2(0, 0);
            if (j < nk) xf[r][j].u = *reinterpret_cast<const uint2*>(xr + j * 16 + grp * 4);
        }
    }
    // (few rows: the blocks of outputs are shared out over blockIdx.z, an even number each)
    const int per_z = (((N / 16 + gridDim.z - 1) / gridDim.z) + 1) & ~1;
    const int nblocks = min(N / 16, (int)(blockIdx.z + 1) * per_z);
    for (int nb = blockIdx.z * per_z; nb < nblocks; nb += 2) {
        const bool two = nb + 1 < nblocks;
        const bf16_t* wr0 = w + ((size_t)h * N + nb * 16 + col) * K + grp * 4;
        const bf16_t* wr1 = two ? wr0 + (size_t)16 * K : wr0;
        hp_f32x4 acc0[RT], acc1[RT];
#pragma unroll
        for (int r = 0; r < RT; ++r) acc0[r] = acc1[r] = (hp_f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KM; ++j) {
            if (j < nk) {
                HpFrag a0, a1;
                a0.u = *reinterpret_cast<const uint2*>(wr0 + j * 16);
                a1.u = *reinterpret_cast<const uint2*>(wr1 + j * 16);
#pragma unroll
                for (int r = 0; r < RT; ++r) {
                    acc0[r] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a0.v, xf[r][j].v, acc0[r], 0, 0, 0);
                    acc1[r] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a1.v, xf[r][j].v, acc1[r], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const int t = t0 + r * 16 + col;
            if (t < T) {
                bf16_t* yr = y + (size_t)t * y_row + (size_t)h * y_head + grp * 4 + nb * 16;
                uint2 st;
                st.x = pack_bf16x2(acc0[r][0], acc0[r][1]);
                st.y = pack_bf16x2(acc0[r][2], acc0[r][3]);
                *reinterpret_cast<uint2*>(yr) = st;
                if (two) {
                    st.x = pack_bf16x2(acc1[r][0], acc1[r][1]);
                    st.y = pack_bf16x2(acc1[r][2], acc1[r][3]);
                    *reinterpret_cast<uint2*>(yr + 16) = st;
                }
            }
        }
    }
}

// Many rows, k of 64, 128, 256 or 512: the head's matrix comes through LDS.  A workgroup takes one head and 64 RT rows
// (a wave RT tiles of 16, their fragments in registers) and walks the outputs in chunks of 8192 elements of W (NB
// blocks of 16 outputs), which its 256 threads bring into one of two LDS buffers with 16-byte loads while the chunk
// before is multiplied; the waves read the blocks' fragments from there (rows of k + 8 elements: 8-byte reads without
// bank conflicts), each fragment serving the wave's RT row tiles, with two sums a row tile taking turns.
template <int KM, int RT>
__global__ __launch_bounds__(256) void head_products_lds_kernel(const bf16_t* __restrict__ x, long long x_row, long long x_head,
                                                                const bf16_t* __restrict__ w, bf16_t* __restrict__ y,
                                                                long long y_row, long long y_head, int T, int N) {
    constexpr int K = KM * 16, LDW = K + 8, NB = 32 / KM, ROWS = NB * 16, PIECES = K / 8;
    __shared__ __align__(16) bf16_t wt[2][ROWS * LDW];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int col = lane % 16, grp = lane / 16;
    const int t0 = (blockIdx.x * 4 + wave) * 16 * RT, h = blockIdx.y;
    HpFrag xf[RT][KM];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const int t = min(t0 + r * 16 + col, T - 1);                    // (rows past the end repeat the last; never stored)
        const bf16_t* xr = x + (size_t)t * x_row + (size_t)h * x_head;
#pragma unroll
        for (int j = 0; j < KM; ++j) xf[r][j].u = *reinterpret_cast<const uint2*>(xr + j * 16 + grp * 4);
    }
    const bf16_t* wh = w + (size_t)h * N * K;
    const int chunks = (N + ROWS - 1) / ROWS;
    uint4 next[4];                                                      // ROWS * PIECES = 1024 pieces of 16 bytes a chunk
    auto fetch = [&](int c) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = i * 256 + tid;
            const int n = c * ROWS + idx / PIECES;
            next[i] = make_uint4(0, 0, 0, 0);
            if (n < N) next[i] = *reinterpret_cast<const uint4*>(wh + (size_t)n * K + (idx % PIECES) * 8);
        }
    };
    auto store = [&](bf16_t* buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = i * 256 + tid;
            *reinterpret_cast<uint4*>(buf + (idx / PIECES) * LDW + (idx % PIECES) * 8) = next[i];
        }
    };
    fetch(0);
    store(wt[0]);
    __syncthreads();
    for (int c = 0; c < chunks; ++c) {
        const bool more = c + 1 < chunks;
        if (more) fetch(c + 1);
        const bf16_t* buf = wt[c & 1];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            hp_f32x4 even[RT], odd[RT];
#pragma unroll
            for (int r = 0; r < RT; ++r) even[r] = odd[r] = (hp_f32x4){0.f, 0.f, 0.f, 0.f};
            const bf16_t* wr = buf + (nb * 16 + col) * LDW + grp * 4;
#pragma unroll
            for (int j = 0; j < KM; ++j) {
                HpFrag a;
                a.u = *reinterpret_cast<const uint2*>(wr + j * 16);
#pragma unroll
                for (int r = 0; r < RT; ++r) {
                    if (j % 2)
                        odd[r] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, xf[r][j].v, odd[r], 0, 0, 0);
                    else
                        even[r] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, xf[r][j].v, even[r], 0, 0, 0);
                }
            }
            const int n0 = (c * NB + nb) * 16;
            if (n0 < N) {
#pragma unroll
                for (int r = 0; r < RT; ++r) {
                    const int t = t0 + r * 16 + col;
                    if (t < T) {
                        uint2 st;
                        st.x = pack_bf16x2(even[r][0] + odd[r][0], even[r][1] + odd[r][1]);
                        st.y = pack_bf16x2(even[r][2] + odd[r][2], even[r][3] + odd[r][3]);
                        *reinterpret_cast<uint2*>(y + (size_t)t * y_row + (size_t)h * y_head + n0 + grp * 4) = st;
                    }
                }
            }
        }
        if (more) store(wt[(c + 1) & 1]);
        __syncthreads();                                // the next chunk is written; this one is read by all
    }
}

extern "C" int tli_head_products_mfma_takes(int N, int K, long long x_row, long long x_head, long long y_row, long long y_head) {
    return (N % 16 == 0 && K % 16 == 0 && N >= 16 && K >= 16 && K <= 640 && x_row % 4 == 0 && x_head % 4 == 0 &&
            y_row % 4 == 0 && y_head % 4 == 0) ? 1 : 0;
}

extern "C" int tli_head_products_mfma_bf16(const void* x, long long x_row, long long x_head, const void* w, void* y,
                                           long long y_row, long long y_head, int rows, int heads, int N, int K, void* stream) {
    if (rows <= 0) return 0;
    if (heads <= 0 || heads > 65535 || !tli_head_products_mfma_takes(N, K, x_row, x_head, y_row, y_head))
        return tli_fail("head_products: the matrix-core kernel takes sizes in sixteens (k up to 640), not %d x %d", N, K);
    if ((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 7)) return tli_fail("head_products: operands must be 8-byte aligned");
    if (rows >= 1024 && (K == 64 || K == 128 || K == 256 || K == 512)) {
        const dim3 lgrid((rows + 127) / 128, heads);
        hipStream_t ls = (hipStream_t)stream;
#define HP_LDS(KM)                                                                                                       \
    head_products_lds_kernel<KM, 2><<<lgrid, 256, 0, ls>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)y, \
                                                           y_row, y_head, rows, N)
        if (K == 64) HP_LDS(4);
        else if (K == 128) HP_LDS(8);
        else if (K == 256) HP_LDS(16);
        else HP_LDS(32);
#undef HP_LDS
        return tli_check_launch("head_products_lds");
    }
    // (many rows: a wave keeps 4 tiles of 16 rows, 2 where k is large, so that a block of W serves them all)
    const int rt = rows < 1024 ? 1 : (K <= 128 ? 4 : (K <= 512 ? 2 : 1));
    const int row_groups = (rows + 64 * rt - 1) / (64 * rt);
    int shares = 512 / (row_groups * heads);                           // enough workgroups for the chip
    shares = shares < 1 ? 1 : (shares > N / 32 ? (N / 32 < 1 ? 1 : N / 32) : shares);
    const dim3 grid(row_groups, heads, shares);
    hipStream_t s = (hipStream_t)stream;
#define HP_ONE(KM, EXACT, RT)                                                                                              \
    head_products_mfma_kernel<KM, EXACT, RT><<<grid, 256, 0, s>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, (bf16_t*)y, \
                                                                  y_row, y_head, rows, N, K)
    if (K == 64) { if (rt == 4) HP_ONE(4, true, 4); else HP_ONE(4, true, 1); }
    else if (K == 128) { if (rt == 4) HP_ONE(8, true, 4); else HP_ONE(8, true, 1); }
    else if (K == 256) { if (rt == 2) HP_ONE(16, true, 2); else HP_ONE(16, true, 1); }
    else if (K == 512) { if (rt == 2) HP_ONE(32, true, 2); else HP_ONE(32, true, 1); }
    else if (K <= 128) { if (rt == 4) HP_ONE(8, false, 4); else HP_ONE(8, false, 1); }
    else if (K <= 512) { if (rt == 2) HP_ONE(32, false, 2); else HP_ONE(32, false, 1); }
    else HP_ONE(40, false, 1);
#undef HP_ONE
    return tli_check_launch("head_products_mfma");
}
