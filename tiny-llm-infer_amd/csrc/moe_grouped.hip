// Routed experts on the matrix cores (bfloat16): the (row, chosen expert) pairs of a step are sorted
// by expert, and every expert multiplies its pairs tile by tile, reading its matrices once a tile.
//
//   sort:     pairs of one expert get consecutive slots, an expert's run of slots filled up to whole
//             tiles of RT slots (`order`: slot -> pair or -1, `pos`: pair -> slot, `tile_expert`: tile ->
//             expert).  How many tiles there are is known on the device only: the products are launched
//             for the most there can be (pairs / RT + experts) and a workgroup without a tile leaves.
//   gate/up:  hid[slot, f] = silu(x[row] . Wg_e[f]) * (x[row] . Wu_e[f])          (bfloat16; or the limited form of
//             common.h's gated_unit)
//   down:     part[slot, c] = hid[slot] . Wd_e[c]                                 (float32)
//   combine:  y[row] = sum_j weight[row, j] part[pos[row, j]]  (+ shared gate * shared), in the order of
//             the choice: a row's result does not depend on which other rows share its tiles, because the
//             rows of a tile never meet in a sum.
//
// The matrices are read in the tiled layout of the other products (blocks of 16 rows x 128 columns, 4
// KiB, in the order the operands of v_mfma_f32_16x16x32_bf16 want: a load instruction of a wave takes 1 KiB
// in a row); rows and columns that do not exist are zeros there.  A is a tile of W (16 outputs), B the
// rows of x, so a lane ends with 4 consecutive outputs of one row.  A wave takes 16 or 32 outputs and all
// RT rows of its tile; the four waves of a workgroup share the rows of x through LDS.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4g;
union Frag {
    uint4 u;
    u32x4g w;
    bf16x8 v;
};

__device__ __forceinline__ Frag frag_load(const bf16_t* p) {
    Frag f;
    f.u = *reinterpret_cast<const uint4*>(p);
    return f;
}

// ---------------------------------------------------------------------------------------------
// sort: one workgroup
// ---------------------------------------------------------------------------------------------
#define SORT_MAX_EXPERTS 2048

__global__ void __launch_bounds__(1024) moe_sort_kernel(const int* __restrict__ ids, int P, int E, int RT,
                                                         int tiles_max, int* __restrict__ order,
                                                         int* __restrict__ pos, int* __restrict__ tile_expert,
                                                         int* __restrict__ num_tiles) {
    __shared__ int count[SORT_MAX_EXPERTS], start[SORT_MAX_EXPERTS], fill[SORT_MAX_EXPERTS];
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = fill[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        const int e = ids[p];
        if (e >= 0 && e < E) atomicAdd(&count[e], 1);   // (any other id: an expert that hands its input on, no slot)
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int before = 0;                               // tiles of the experts before e
        for (int i = 0; i < e; ++i) before += (count[i] + RT - 1) / RT;
        start[e] = before * RT;
        const int mine = (count[e] + RT - 1) / RT;
        for (int i = 0; i < mine; ++i) tile_expert[before + i] = e;
        if (e == E - 1) {
            *num_tiles = before + mine;
            for (int i = before + mine; i < tiles_max; ++i) tile_expert[i] = -1;
        }
    }
    for (int s = threadIdx.x; s < tiles_max * RT; s += blockDim.x) order[s] = -1;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        const int e = ids[p];
        if (e < 0 || e >= E) {
            pos[p] = -1;
            continue;
        }
        const int slot = start[e] + atomicAdd(&fill[e], 1);
        order[slot] = p;
        pos[p] = slot;
    }
}

// ---------------------------------------------------------------------------------------------
// one tile's product: 16 RB rows of B against the wave's 16 rows of A (and of A2, if GATED)
// ---------------------------------------------------------------------------------------------
#define XT_STRIDE 136          // bfloat16 elements between two rows of the staged block of B: 128 and 8 more, so that
                               // the 16 rows a quarter of a wave reads lie in different banks

// The four waves of a workgroup read the same rows of B: a block of 128 columns of them is staged in
// LDS by all threads together (rows without a pair, and columns past the end, as zeros), then every
// wave takes its fragments from there.  `src_off`: for each of the tile's rows the offset of its
// source row, or a negative number.
// NB: blocks of 16 outputs a wave takes; a fragment of B from LDS serves that many products (of each of the two
// matrices, if GATED).  Two, but one where gate and up over 128 slots would leave no registers for running ahead.

template <int RB, int NB, bool GATED>
__device__ __forceinline__ void tile_product(const bf16_t* __restrict__ a1, const bf16_t* __restrict__ a2, size_t a_step,
                                             const bf16_t* __restrict__ src, const long long* src_off, int K, bool active,
                                             bf16_t* xt, f32x4 (&acc1)[NB][RB], f32x4 (&acc2)[NB][RB]) {
    const int lane = threadIdx.x % 64, r = lane % 16, c = lane / 16;
    const int kblocks = (K + 127) / 128;
    // Small tiles (decode steps) are few workgroups that stream whole matrices: the fragments of A of the block
    // of k after the current one are asked for before the current one's products run.  Large tiles have their
    // registers full of sums and many workgroups in flight instead.
    constexpr bool AHEAD = RB <= 2;
    Frag n1[4][NB], n2[4][NB];
    auto fetch_a = [&](int kb) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                n1[j][i] = frag_load(a1 + i * a_step + (size_t)kb * 2048 + j * 512);
                if (GATED) n2[j][i] = frag_load(a2 + i * a_step + (size_t)kb * 2048 + j * 512);
            }
    };
    if (AHEAD) {
        // no LDS and no barrier in the loop: a wave reads its fragments of the few rows of B itself (the four waves
        // of the workgroup read the same ones, from the cache), a block ahead like those of A
        __syncthreads();                                 // (src_off is written)
        if (!active) return;
        long long off[RB];
#pragma unroll
        for (int b = 0; b < RB; ++b) off[b] = src_off[b * 16 + r];
        Frag xn[4][RB];
        auto fetch_b = [&](int kb) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int b = 0; b < RB; ++b) {
                    const int k = kb * 128 + c * 32 + j * 8;
                    xn[j][b].u = make_uint4(0, 0, 0, 0);
                    if (off[b] >= 0 && k + 8 <= K) xn[j][b].u = *reinterpret_cast<const uint4*>(src + off[b] + k);
                }
        };
        fetch_a(0);
        fetch_b(0);
        for (int kb = 0; kb < kblocks; ++kb) {
            Frag f1[4][NB], f2[4][NB], fx[4][RB];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    f1[j][i] = n1[j][i];
                    if (GATED) f2[j][i] = n2[j][i];
                }
#pragma unroll
                for (int b = 0; b < RB; ++b) fx[j][b] = xn[j][b];
            }
            fetch_a(min(kb + 1, kblocks - 1));           // (the last block once more rather than a branch around loads)
            fetch_b(min(kb + 1, kblocks - 1));
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int b = 0; b < RB; ++b)
#pragma unroll
                    for (int i = 0; i < NB; ++i) {
                        acc1[i][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f1[j][i].v, fx[j][b].v, acc1[i][b], 0, 0, 0);
                        if (GATED) acc2[i][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f2[j][i].v, fx[j][b].v, acc2[i][b], 0, 0, 0);
                    }
        }
        return;
    }
    // Large tiles: the rows of B of the block of k after the current one wait in registers while the current one is
    // multiplied, and the fragments of A run one quarter block (32 columns of k) ahead of the products.
    uint4 xr[RB];
    auto fetch_x = [&](int kb) {
#pragma unroll
        for (int n = 0; n < RB; ++n) {
            const int id = threadIdx.x + n * 256, row = id / 16, kc = id % 16;
            const long long off = src_off[row];
            const int k = kb * 128 + kc * 8;
            xr[n] = make_uint4(0, 0, 0, 0);
            if (off >= 0 && k + 8 <= K) xr[n] = *reinterpret_cast<const uint4*>(src + off + k);
        }
    };
    Frag g1[NB], g2[NB];
    auto fetch_quarter = [&](int q) {                    // quarter q of all: block q / 4, step q % 4 (the last one again past the end)
        const int at = min(q, 4 * kblocks - 1);
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            g1[i] = frag_load(a1 + i * a_step + (size_t)(at / 4) * 2048 + (at % 4) * 512);
            if (GATED) g2[i] = frag_load(a2 + i * a_step + (size_t)(at / 4) * 2048 + (at % 4) * 512);
        }
    };
    __syncthreads();                                     // (src_off is written)
    fetch_x(0);
    if (active) fetch_quarter(0);
    for (int kb = 0; kb < kblocks; ++kb) {
        __syncthreads();
#pragma unroll
        for (int n = 0; n < RB; ++n) {
            const int id = threadIdx.x + n * 256, row = id / 16, kc = id % 16;
            *reinterpret_cast<uint4*>(xt + row * XT_STRIDE + kc * 8) = xr[n];
        }
        __syncthreads();
        if (kb + 1 < kblocks) fetch_x(kb + 1);
        if (!active) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            Frag f1[NB], f2[NB];
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                f1[i] = g1[i];
                if (GATED) f2[i] = g2[i];
            }
            fetch_quarter(kb * 4 + j + 1);
#pragma unroll
            for (int b = 0; b < RB; ++b) {
                Frag fx;
                fx.u = *reinterpret_cast<const uint4*>(xt + (b * 16 + r) * XT_STRIDE + c * 32 + j * 8);
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    acc1[i][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f1[i].v, fx.v, acc1[i][b], 0, 0, 0);
                    if (GATED) acc2[i][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f2[i].v, fx.v, acc2[i][b], 0, 0, 0);
                }
            }
        }
    }
}

// gate and up products with the activation: hid[slot, f] (a tile has 16 RB slots)
template <int RB, int NB>
__global__ void __launch_bounds__(256) moe_gate_up_kernel(const bf16_t* __restrict__ x, const int* __restrict__ order,
                                                           const int* __restrict__ tile_expert,
                                                           const int* __restrict__ num_tiles,
                                                           const bf16_t* __restrict__ gate_t,
                                                           const bf16_t* __restrict__ up_t, bf16_t* __restrict__ hid,
                                                           int top, int D, int ff, float limit, float slope) {
    __shared__ __attribute__((aligned(16))) bf16_t xt[16 * RB * XT_STRIDE];
    __shared__ long long src_off[16 * RB];
    const int tile = blockIdx.y;
    if (tile >= *num_tiles) return;                   // (the whole workgroup)
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int r = lane % 16, c = lane / 16;
    const int nb = (blockIdx.x * 4 + wave) * NB;      // the wave's first block of 16 hidden units
    const int nblocks = (ff + 15) / 16, kblocks = (D + 127) / 128;
    const bool active = nb < nblocks;
    const int e = tile_expert[tile];
    for (int i = threadIdx.x; i < 16 * RB; i += 256) {
        const int p = order[tile * 16 * RB + i];
        src_off[i] = p >= 0 ? (long long)(p / top) * D : -1;
    }
    // (a block past the last reads the one before it again and stores nothing)
    const size_t a_step = nb + 1 < nblocks ? (size_t)kblocks * 2048 : 0;
    const size_t block0 = ((size_t)e * nblocks + (active ? nb : 0)) * kblocks * 2048 + lane * 8;
    f32x4 ag[NB][RB], au[NB][RB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int b = 0; b < RB; ++b) ag[i][b] = au[i][b] = (f32x4){0.f, 0.f, 0.f, 0.f};
    tile_product<RB, NB, true>(gate_t + block0, up_t + block0, a_step, x, src_off, D, active, xt, ag, au);
    if (!active) return;
    // the lane holds hidden units (nb + i) * 16 + 4 c .. + 4 of the slots 16 b + r
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int n0 = (nb + i) * 16 + c * 4;
        if (nb + i >= nblocks) continue;
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            if (src_off[b * 16 + r] < 0) continue;
            float h[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) h[v] = gated_unit(ag[i][b][v], au[i][b][v], limit, slope);
            store4(hid + (size_t)((tile * RB + b) * 16 + r) * ff + n0, h, ff - n0, ff % 4 == 0);
        }
    }
}

// down product: float32 rows in the order of the slots
template <int RB, int NB>
__global__ void __launch_bounds__(256) moe_down_grouped_kernel(const bf16_t* __restrict__ hid, const int* __restrict__ order,
                                                                const int* __restrict__ tile_expert,
                                                                const int* __restrict__ num_tiles,
                                                                const bf16_t* __restrict__ down_t, float* __restrict__ part,
                                                                int D, int ff) {
    __shared__ __attribute__((aligned(16))) bf16_t xt[16 * RB * XT_STRIDE];
    __shared__ long long src_off[16 * RB];
    const int tile = blockIdx.y;
    if (tile >= *num_tiles) return;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int r = lane % 16, c = lane / 16;
    const int nb = (blockIdx.x * 4 + wave) * NB;      // the wave's first block of 16 output columns
    const int nblocks = (D + 15) / 16, kblocks = (ff + 127) / 128;
    const bool active = nb < nblocks;
    const int e = tile_expert[tile];
    for (int i = threadIdx.x; i < 16 * RB; i += 256) {
        const int slot = tile * 16 * RB + i;
        src_off[i] = order[slot] >= 0 ? (long long)slot * ff : -1;
    }
    const size_t a_step = nb + 1 < nblocks ? (size_t)kblocks * 2048 : 0;
    const bf16_t* wd = down_t + ((size_t)e * nblocks + (active ? nb : 0)) * kblocks * 2048 + lane * 8;
    f32x4 acc[NB][RB], unused[NB][RB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int b = 0; b < RB; ++b) acc[i][b] = (f32x4){0.f, 0.f, 0.f, 0.f};
    tile_product<RB, NB, false>(wd, nullptr, a_step, hid, src_off, ff, active, xt, acc, unused);
    if (!active) return;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int n0 = (nb + i) * 16 + c * 4;
        if (nb + i >= nblocks) continue;
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            if (src_off[b * 16 + r] < 0) continue;
            const float v[4] = {acc[i][b][0], acc[i][b][1], acc[i][b][2], acc[i][b][3]};
            store4(part + (size_t)((tile * RB + b) * 16 + r) * D + n0, v, D - n0, D % 4 == 0);
        }
    }
}

// y[row] = sum_j weight[row, j] part[pos[row, j]] (+ gate[row] * shared[row])
__global__ void moe_combine_kernel(const float* __restrict__ part, const int* __restrict__ pos,
                                   const float* __restrict__ weights, const bf16_t* __restrict__ shared,
                                   const float* __restrict__ shared_gate, bf16_t* __restrict__ out, int top, int D,
                                   const bf16_t* __restrict__ x) {
    const int t = blockIdx.x;
    for (int cidx = threadIdx.x; cidx < D; cidx += blockDim.x) {
        float y = 0.f;
        for (int j = 0; j < top; ++j) {
            const int slot = pos[(size_t)t * top + j];           // negative: the expert hands its input on
            const float v = slot >= 0 ? part[(size_t)slot * D + cidx] : bf16_to_f32(x[(size_t)t * D + cidx]);
            y = fmaf(weights[(size_t)t * top + j], v, y);
        }
        if (shared) y = fmaf(shared_gate ? shared_gate[t] : 1.0f, bf16_to_f32(shared[(size_t)t * D + cidx]), y);
        out[(size_t)t * D + cidx] = f32_to_bf16(y);
    }
}

// ---------------------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------------------
// How many slots a tile has for `pairs` pairs over `experts` experts: 16, 32, 64 or 128 (more rows a tile
// read an expert's matrices fewer times; fewer waste less on experts with few pairs).
extern "C" int tli_moe_grouped_tile(int pairs, int experts) {
    const int average = pairs / (experts > 0 ? experts : 1);
    return average >= 96 ? 128 : average >= 48 ? 64 : average >= 24 ? 32 : 16;
}

// scratch, all given by the caller: order [tiles_max * RT], pos [pairs], tile_expert [tiles_max],
// num_tiles [1] (int32); hid [tiles_max * RT, ff] (bfloat16); part [tiles_max * RT, D] (float32);
// with tiles_max = pairs / RT + experts.  gate_t, up_t: [E] tiled [ff, D]; down_t: [E] tiled [D, ff].
extern "C" int tli_moe_grouped_bf16(const void* x, const int* ids, const float* weights, const void* gate_t,
                                    const void* up_t, const void* down_t, int* order, int* pos, int* tile_expert,
                                    int* num_tiles, void* hid, float* part, const void* shared,
                                    const float* shared_gate, void* out, int T, int top, int E, int D, int ff, int RT,
                                    float limit, float slope, void* stream) {
    if (T <= 0) return 0;
    if (top <= 0 || E <= 0 || E > SORT_MAX_EXPERTS || D <= 0 || ff <= 0 || D % 8 || ff % 8)
        return tli_fail("moe_grouped: bad sizes (experts %d (at most %d), width %d and hidden units %d in eights)", E,
                        SORT_MAX_EXPERTS, D, ff);
    if (RT != 16 && RT != 32 && RT != 64 && RT != 128)
        return tli_fail("moe_grouped: tiles of 16, 32, 64 or 128 slots, not %d", RT);
    const long long pairs = (long long)T * top;
    const long long tiles_max = pairs / RT + E;
    if (tiles_max > 65535 || pairs > (1 << 28)) return tli_fail("moe_grouped: too many pairs for one launch (%lld)", pairs);
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, s, ids, (int)pairs, E, RT, (int)tiles_max, order, pos,
                       tile_expert, num_tiles);
#define TLI_GROUPED(RB, NBG)                                                                                          \
    hipLaunchKernelGGL((moe_gate_up_kernel<RB, NBG>), dim3((ff + 64 * NBG - 1) / (64 * NBG), (unsigned)tiles_max),      \
                       dim3(256), 0, s, (const bf16_t*)x, order, tile_expert, num_tiles, (const bf16_t*)gate_t,        \
                       (const bf16_t*)up_t, (bf16_t*)hid, top, D, ff, limit, slope);                                   \
    hipLaunchKernelGGL((moe_down_grouped_kernel<RB, 2>), dim3((D + 127) / 128, (unsigned)tiles_max), dim3(256), 0, s,  \
                       (const bf16_t*)hid, order, tile_expert, num_tiles, (const bf16_t*)down_t, part, D, ff)
    if (RT == 16) { TLI_GROUPED(1, 2); }
    else if (RT == 32) { TLI_GROUPED(2, 2); }
    else if (RT == 64) { TLI_GROUPED(4, 2); }
    else { TLI_GROUPED(8, 1); }
#undef TLI_GROUPED
    hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, s, part, pos, weights, (const bf16_t*)shared, shared_gate,
                       (bf16_t*)out, top, D, (const bf16_t*)x);
    return tli_check_launch("moe_grouped");
}
