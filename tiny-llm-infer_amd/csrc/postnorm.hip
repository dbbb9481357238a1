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
