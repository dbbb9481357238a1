// The residual of a block that norms what a sublayer gives:  x <- x + w * y / sqrt(mean(y^2) + eps).
//
// norm_add:       one workgroup a row: the sublayer's output y (the run's type) is read once into registers,
//                 its mean square summed in float32, the normed row added to the float32 residual, and the
//                 new residual written in the run's type for the next sublayer to read.
// residual_rows:  the residual's rows in the run's type (what the first block reads).
#include "common.h"

#define PN_THREADS 256
#define PN_MAX_PER_THREAD 32          // rows of up to 8192 elements stay in registers

template <typename T>
__global__ __launch_bounds__(PN_THREADS) void norm_add_kernel(float* __restrict__ resid, const T* __restrict__ y,
                                                                const float* __restrict__ weight, T* __restrict__ rows_out,
                                                                int n, float eps) {
    __shared__ float red[16];
    const size_t row = blockIdx.x;
    const T* yr = y + row * n;
    float v[PN_MAX_PER_THREAD];
    float ssq = 0.f;
#pragma unroll
    for (int i = 0; i < PN_MAX_PER_THREAD; ++i) {
        const int c = i * PN_THREADS + threadIdx.x;
        v[i] = c < n ? to_f32(yr[c]) : 0.f;
        ssq = fmaf(v[i], v[i], ssq);
    }
    // (beyond what the registers hold: read again below)
    for (int c = PN_MAX_PER_THREAD * PN_THREADS + threadIdx.x; c < n; c += PN_THREADS) {
        const float a = to_f32(yr[c]);
        ssq = fmaf(a, a, ssq);
    }
    const float factor = 1.0f / sqrtf(block_sum(ssq, red) / (float)n + eps);
    float* xr = resid + row * n;
#pragma unroll
    for (int i = 0; i < PN_MAX_PER_THREAD; ++i) {
        const int c = i * PN_THREADS + threadIdx.x;
        if (c < n) {
            const float x = xr[c] + v[i] * factor * weight[c];
            xr[c] = x;
            if (rows_out) from_f32(rows_out + row * n + c, x);
        }
    }
    for (int c = PN_MAX_PER_THREAD * PN_THREADS + threadIdx.x; c < n; c += PN_THREADS) {
        const float x = xr[c] + to_f32(yr[c]) * factor * weight[c];
        xr[c] = x;
        if (rows_out) from_f32(rows_out + row * n + c, x);
    }
}

// The same for bfloat16 rows whose length is a multiple of 8, up to 8192: 16-byte accesses, eight elements a
// thread and round.
#define PN_VEC_ROUNDS 4
__global__ __launch_bounds__(PN_THREADS) void norm_add_vec_kernel(float* __restrict__ resid, const bf16_t* __restrict__ y,
                                                                   const float* __restrict__ weight, bf16_t* __restrict__ rows_out,
                                                                   int n, float eps) {
    __shared__ float red[16];
    const size_t row = blockIdx.x;
    const bf16_t* yr = y + row * n;
    uint4 v[PN_VEC_ROUNDS];
    float ssq = 0.f;
#pragma unroll
    for (int i = 0; i < PN_VEC_ROUNDS; ++i) {
        const int c = (i * PN_THREADS + threadIdx.x) * 8;
        v[i] = make_uint4(0, 0, 0, 0);
        if (c < n) v[i] = *reinterpret_cast<const uint4*>(yr + c);
        const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float a = __uint_as_float(w[e] << 16), b = __uint_as_float(w[e] & 0xFFFF0000u);
            ssq = fmaf(a, a, ssq);
            ssq = fmaf(b, b, ssq);
        }
    }
    const float factor = 1.0f / sqrtf(block_sum(ssq, red) / (float)n + eps);
    float* xr = resid + row * n;
#pragma unroll
    for (int i = 0; i < PN_VEC_ROUNDS; ++i) {
        const int c = (i * PN_THREADS + threadIdx.x) * 8;
        if (c < n) {
            const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
            float x[8];
            *reinterpret_cast<float4*>(x) = *reinterpret_cast<const float4*>(xr + c);
            *reinterpret_cast<float4*>(x + 4) = *reinterpret_cast<const float4*>(xr + c + 4);
            float g[8];
            *reinterpret_cast<float4*>(g) = *reinterpret_cast<const float4*>(weight + c);
            *reinterpret_cast<float4*>(g + 4) = *reinterpret_cast<const float4*>(weight + c + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                x[2 * e] += __uint_as_float(w[e] << 16) * factor * g[2 * e];
                x[2 * e + 1] += __uint_as_float(w[e] & 0xFFFF0000u) * factor * g[2 * e + 1];
            }
            *reinterpret_cast<float4*>(xr + c) = *reinterpret_cast<const float4*>(x);
            *reinterpret_cast<float4*>(xr + c + 4) = *reinterpret_cast<const float4*>(x + 4);
            if (rows_out) {
                uint4 st;
                st.x = pack_bf16x2(x[0], x[1]);
                st.y = pack_bf16x2(x[2], x[3]);
                st.z = pack_bf16x2(x[4], x[5]);
                st.w = pack_bf16x2(x[6], x[7]);
                *reinterpret_cast<uint4*>(rows_out + row * n + c) = st;
            }
        }
    }
}

__global__ void residual_rows_kernel(const float* __restrict__ resid, bf16_t* __restrict__ out, long long count) {
    const long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i + 3 < count) {
        const float4 v = *reinterpret_cast<const float4*>(resid + i);
        uint2 st;
        st.x = pack_bf16x2(v.x, v.y);
        st.y = pack_bf16x2(v.z, v.w);
        *reinterpret_cast<uint2*>(out + i) = st;
    } else {
        for (long long j = i; j < count; ++j) out[j] = f32_to_bf16(resid[j]);
    }
}

// resid [rows, n] float32 += weight * y / rms(y);  rows_out [rows, n] in the type of y (may be null for float32, where
// the residual itself is what the next sublayer reads)
extern "C" int tli_norm_add(float* resid, const void* y, const float* weight, void* rows_out, int rows, int n, float eps,
                            int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (n <= 0) return tli_fail("norm_add: bad row length %d", n);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TLI_F32)
        norm_add_kernel<float><<<rows, PN_THREADS, 0, s>>>(resid, (const float*)y, weight, (float*)rows_out, n, eps);
    else if (dtype == TLI_BF16 && n % 8 == 0 && n <= 8 * PN_THREADS * PN_VEC_ROUNDS &&
             !(((uintptr_t)resid | (uintptr_t)y | (uintptr_t)weight | (uintptr_t)rows_out) & 15))
        norm_add_vec_kernel<<<rows, PN_THREADS, 0, s>>>(resid, (const bf16_t*)y, weight, (bf16_t*)rows_out, n, eps);
    else if (dtype == TLI_BF16)
        norm_add_kernel<bf16_t><<<rows, PN_THREADS, 0, s>>>(resid, (const bf16_t*)y, weight, (bf16_t*)rows_out, n, eps);
    else
        return tli_fail("norm_add: unknown dtype %d", dtype);
    return tli_check_launch("norm_add");
}

extern "C" int tli_residual_rows(const float* resid, void* out, long long count, void* stream) {
    if (count <= 0) return 0;
    if (((uintptr_t)resid & 15) || ((uintptr_t)out & 7)) return tli_fail("residual_rows: operands must be 16-byte aligned");
    const long long threads = (count + 3) / 4;
    residual_rows_kernel<<<(unsigned)((threads + 255) / 256), 256, 0, (hipStream_t)stream>>>(resid, (bf16_t*)out, count);
    return tli_check_launch("residual_rows");
}
