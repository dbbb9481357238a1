// Routed experts: the router's choice, and the chosen experts applied row by row.
//
// route:   s_e = sigmoid(z_e) for the E router logits of a row (float32), or softmax(z)_e.  The choice
//          looks at c_e = s_e + correction_e (a vector, if given); the weights use s.  The experts form
//          `groups` equal groups of neighbours; a group's score is the sum of its two largest c
//          (of its one, if it has one expert) or its largest c; only experts of the `keep` best groups can
//          be chosen (the others are out, whatever the sign of the scores).  The `top` largest c among
//          those are chosen, ties to the lower index; weight_j = s_j / (sum of the chosen s + 1e-20) * scale,
//          or s_j * scale without that division.  One more logit behind the E, if present, is the gate of
//          a shared expert: sigmoid of it.  Ids from `experts` on (see the kernels below) are experts that
//          hand their input on: they have no matrices.
// hidden:  for the pair (row, chosen expert e): a_f = silu(x . Wg_e[f]) * (x . Wu_e[f]), or the limited form of
//          common.h's gated_unit (limit > 0)
// down:    y_c = sum_j weight_j (a_j . Wd_e(j)[c])  (+ shared gate * shared_c), summed in the order of
//          the choice, so that a row's result does not depend on what else is in the step.
//
// These kernels walk the pairs one by one, each reading its expert's matrices: what a decode step
// needs anyway, and the float32 path.  Steps of many rows in bfloat16 sort the pairs by expert and
// multiply tile by tile (moe_grouped.hip).
#include "common.h"

#define MOE_MAX_TOP 32

__global__ void moe_route_kernel(const float* __restrict__ z, long long z_row, long long z_col, int* __restrict__ ids,
                                 float* __restrict__ weights, float* __restrict__ shared_gate, int T, int E,
                                 int top, int groups, int keep, float scale, int has_shared, int softmax_scores,
                                 int group_by_max, int normalize, const float* __restrict__ correction) {
    extern __shared__ float sig[];                 // [threads][2 E + 1]: a row's scores, then its choice scores (odd stride: no bank conflicts)
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= T) return;
    float* s = sig + (size_t)threadIdx.x * (2 * E + 1);
    float* c = s + E;
    const float* zr = z + (size_t)t * z_row;              // logit e of row t lies at t * z_row + e * z_col
    if (softmax_scores) {
        float top_z = -INFINITY, sum = 0.f;
        for (int e = 0; e < E; ++e) top_z = fmaxf(top_z, zr[(size_t)e * z_col]);
        for (int e = 0; e < E; ++e) {
            s[e] = expf(zr[(size_t)e * z_col] - top_z);
            sum += s[e];
        }
        for (int e = 0; e < E; ++e) s[e] /= sum;
    } else {
        for (int e = 0; e < E; ++e) s[e] = 1.0f / (1.0f + expf(-zr[(size_t)e * z_col]));
    }
    for (int e = 0; e < E; ++e) c[e] = correction ? s[e] + correction[e] : s[e];
    if (has_shared) shared_gate[t] = 1.0f / (1.0f + expf(-zr[(size_t)E * z_col]));
    const int per = E / groups;
    // the `keep` best groups, as a bit a group (groups <= 64)
    unsigned long long open = 0ull;
    if (keep >= groups) {
        open = ~0ull;
    } else {
        for (int n = 0; n < keep; ++n) {
            int best = -1;
            float best_score = 0.f;
            for (int g = 0; g < groups; ++g) {
                if ((open >> g) & 1ull) continue;
                float a = -INFINITY, b = -INFINITY;   // the two largest of the group
                for (int e = g * per; e < (g + 1) * per; ++e) {
                    const float v = c[e];
                    if (v > a) { b = a; a = v; }
                    else if (v > b) b = v;
                }
                const float score = (b > -INFINITY && !group_by_max) ? a + b : a;
                if (best < 0 || score > best_score) { best = g; best_score = score; }
            }
            open |= 1ull << best;
        }
    }
    int chosen[MOE_MAX_TOP];
    float total = 0.f;
    for (int n = 0; n < top; ++n) {
        int best = -1;
        float best_s = 0.f;
        for (int e = 0; e < E; ++e) {
            if (!((open >> (e / per)) & 1ull)) continue;
            bool taken = false;
            for (int m = 0; m < n; ++m) taken |= chosen[m] == e;
            if (taken) continue;
            if (best < 0 || c[e] > best_s) { best = e; best_s = c[e]; }
        }
        chosen[n] = best;
        total += s[best];
    }
    const float norm = normalize ? scale / (total + 1e-20f) : scale;
    for (int n = 0; n < top; ++n) {
        ids[(size_t)t * top + n] = chosen[n];
        weights[(size_t)t * top + n] = s[chosen[n]] * norm;
    }
}

// one workgroup a pair; a wave takes every (waves)th hidden unit, its lanes share out k
template <typename T>
__global__ void moe_hidden_kernel(const T* __restrict__ x, const int* __restrict__ ids, const T* __restrict__ w_gu,
                                  T* __restrict__ hid, int top, int D, int ff, int E, float limit, float slope) {
    extern __shared__ float xs[];                  // the pair's input row
    const int pair = blockIdx.x;
    const int t = pair / top;
    const int e = ids[pair];
    if (e < 0 || e >= E) return;                   // (an expert that hands its input on: no hidden units)
    for (int i = threadIdx.x; i < D; i += blockDim.x) xs[i] = to_f32(x[(size_t)t * D + i]);
    __syncthreads();
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE, waves = blockDim.x / TLI_WAVE;
    const T* wg = w_gu + (size_t)e * 2 * ff * D;
    const T* wu = wg + (size_t)ff * D;
    for (int f = wave; f < ff; f += waves) {
        const T* g = wg + (size_t)f * D;
        const T* u = wu + (size_t)f * D;
        float a = 0.f, b = 0.f;
        for (int i = lane; i < D; i += TLI_WAVE) {
            a = fmaf(xs[i], to_f32(g[i]), a);
            b = fmaf(xs[i], to_f32(u[i]), b);
        }
        a = wave_sum(a);
        b = wave_sum(b);
        if (lane == 0) from_f32(hid + (size_t)pair * ff + f, gated_unit(a, b, limit, slope));
    }
}

// one workgroup a row and block of columns; a wave takes a column at a time
template <typename T>
__global__ void moe_down_kernel(const T* __restrict__ hid, const int* __restrict__ ids, const float* __restrict__ weights,
                                const T* __restrict__ w_down, const T* __restrict__ shared,
                                const float* __restrict__ shared_gate, T* __restrict__ out, int top, int D, int ff,
                                int cols_a_block, int E, const T* __restrict__ x) {
    extern __shared__ float hs[];                  // [top][ff]: the row's hidden units of its chosen experts
    const int t = blockIdx.y;
    for (int i = threadIdx.x; i < top * ff; i += blockDim.x) hs[i] = to_f32(hid[(size_t)t * top * ff + i]);
    __syncthreads();
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE, waves = blockDim.x / TLI_WAVE;
    const int c0 = blockIdx.x * cols_a_block;
    const int c1 = min(D, c0 + cols_a_block);
    for (int c = c0 + wave; c < c1; c += waves) {
        float y = 0.f;
        for (int j = 0; j < top; ++j) {
            const int e = ids[(size_t)t * top + j];
            if (e < 0 || e >= E) {                 // hands its input on
                y = fmaf(weights[(size_t)t * top + j], to_f32(x[(size_t)t * D + c]), y);
                continue;
            }
            const T* w = w_down + ((size_t)e * D + c) * ff;
            float a = 0.f;
            for (int i = lane; i < ff; i += TLI_WAVE) a = fmaf(hs[(size_t)j * ff + i], to_f32(w[i]), a);
            y = fmaf(weights[(size_t)t * top + j], wave_sum(a), y);
        }
        if (shared) y = fmaf(shared_gate ? shared_gate[t] : 1.0f, to_f32(shared[(size_t)t * D + c]), y);
        if (lane == 0) from_f32(out + (size_t)t * D + c, y);
    }
}

extern "C" int tli_moe_route(const float* z, long long z_row, long long z_col, int* ids, float* weights,
                             float* shared_gate, int T, int E, int top, int groups, int keep, float scale, int has_shared,
                             int softmax_scores, int group_by_max, int normalize, const float* correction, void* stream) {
    if (T <= 0) return 0;
    if (E <= 0 || top <= 0 || top > E || top > MOE_MAX_TOP || groups <= 0 || groups > 64 || E % groups || keep <= 0 ||
        keep > groups || (long long)keep * (E / groups) < top || z_row <= 0 || z_col <= 0)
        return tli_fail("moe_route: bad sizes (experts %d, top %d (at most %d), groups %d (at most 64), keep %d)", E,
                        top, MOE_MAX_TOP, groups, keep);
    if (E > 2048) return tli_fail("moe_route: at most 2048 experts, got %d", E);
    int threads = 64;
    while (threads > 1 && (size_t)threads * (2 * E + 1) * sizeof(float) > 48 * 1024) threads /= 2;
    hipLaunchKernelGGL(moe_route_kernel, dim3((T + threads - 1) / threads), dim3(threads),
                       (size_t)threads * (2 * E + 1) * sizeof(float), (hipStream_t)stream, z, z_row, z_col, ids, weights, shared_gate,
                       T, E, top, groups, keep, scale, has_shared, softmax_scores, group_by_max, normalize, correction);
    return tli_check_launch("moe_route");
}

// x [T, D]; ids, weights [T, top]; w_gu [E, 2 ff, D] (an expert's gate rows, then its up rows);
// w_down [E, D, ff]; hid [T * top, ff] is scratch; shared [T, D] or null (shared_gate null: added as it is); out [T, D];
// an id outside 0..E-1 is an expert that hands its input on; limit, slope: the activation (gated_unit)
extern "C" int tli_moe_experts(const void* x, const int* ids, const float* weights, const void* w_gu,
                               const void* w_down, void* hid, const void* shared, const float* shared_gate, void* out,
                               int T, int top, int D, int ff, int E, int dtype, float limit, float slope, void* stream) {
    if (T <= 0) return 0;
    if (top <= 0 || D <= 0 || ff <= 0) return tli_fail("moe_experts: bad sizes");
    if ((size_t)D * 4 > 64 * 1024 || (size_t)top * ff * 4 > 64 * 1024)
        return tli_fail("moe_experts: a row of %d or %d x %d hidden units does not fit the workgroup's memory", D, top, ff);
    if (T > 65535) return tli_fail("moe_experts: at most 65535 rows a launch, got %d", T);
    hipStream_t s = (hipStream_t)stream;
    const int cols = 64;
    const dim3 dgrid((D + cols - 1) / cols, T);
    if (dtype == TLI_F32) {
        hipLaunchKernelGGL((moe_hidden_kernel<float>), dim3(T * top), dim3(256), (size_t)D * 4, s, (const float*)x, ids,
                           (const float*)w_gu, (float*)hid, top, D, ff, E, limit, slope);
        hipLaunchKernelGGL((moe_down_kernel<float>), dgrid, dim3(256), (size_t)top * ff * 4, s, (const float*)hid, ids,
                           weights, (const float*)w_down, (const float*)shared, shared_gate, (float*)out, top, D, ff, cols, E, (const float*)x);
    } else if (dtype == TLI_BF16) {
        hipLaunchKernelGGL((moe_hidden_kernel<bf16_t>), dim3(T * top), dim3(256), (size_t)D * 4, s, (const bf16_t*)x, ids,
                           (const bf16_t*)w_gu, (bf16_t*)hid, top, D, ff, E, limit, slope);
        hipLaunchKernelGGL((moe_down_kernel<bf16_t>), dgrid, dim3(256), (size_t)top * ff * 4, s, (const bf16_t*)hid, ids,
                           weights, (const bf16_t*)w_down, (const bf16_t*)shared, shared_gate, (bf16_t*)out, top, D, ff,
                           cols, E, (const bf16_t*)x);
    } else {
        return tli_fail("moe_experts: unknown dtype %d", dtype);
    }
    return tli_check_launch("moe_experts");
}
