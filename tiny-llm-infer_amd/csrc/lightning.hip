// Lightning attention: a matrix of state a head that decays by a constant a token.
//
// For the rows of one sequence and head h (key size dk, value size dv, decay c_h from the caller):
//   q_t = silu(proj q),  k_t = silu(proj k),  v_t = silu(proj v)          (float32 from the projections' storage type)
//   S_t = c_h S_(t-1) + k_t v_t^T        S [dk, dv], float32, zero before position 0
//   o_t = S_t^T q_t                      float32
// The state of a sequence lives in its slot between steps, transposed ([head][dv][dk]: the dk elements of a column
// lie together), so that a wave reads and writes it in runs.  A sequence that starts at position 0 does not read its
// slot: slots are never cleared when they change hands.
//
// Columns of S are independent.  A workgroup takes a few columns of one head of one sequence and walks the
// sequence's rows in order; a column belongs to the 16 lanes of a DPP row (a workgroup then has 16 columns), or to
// the 64 lanes of a wave (4 columns), a lane holding R elements of it in registers, in pieces of up to four that lie
// side by side with the other lanes' (R = dk / lanes rounded up to a power of two; elements from dk on stay zero).  A row costs R multiply-adds for the state, R for
// the output and four DPP moves (and two exchanges of rows of lanes, with 64 lanes a column).
//
// Two launches: lightning_prepare takes the silu of every row's q, k and v once and leaves them in float32 in a padded
// layout; lightning_recurrence brings them through LDS in chunks of rows, 16 bytes a copy, which the whole workgroup
// fetches into registers while the chunk before is walked.  Two more where a portion is long enough to be cut into
// segments (lightning_carry, lightning_apply: see LT_SEGMENT below).
//
// lightning_norm: y = o / sqrt(mean(o^2) + eps) * w * sigmoid(gate) over all heads of a row together.
#include "common.h"

#define LT_THREADS 256
#define LT_MAX_DK 256

__device__ __forceinline__ float lt_silu(float z) { return z / (1.0f + expf(-z)); }

// sum over the 16 lanes of a DPP row; every lane gets it
__device__ __forceinline__ float lt_sum16(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));     // neighbours
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));     // pairs of a quad
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));    // halves mirrored
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));    // row mirrored
    return v;
}

// q, k and v of every row and head with the silu taken, in float32 and in the padded layout that the recurrence
// stages with 16-byte copies: qk [T][H][2][DKP] (zeros from dk on), v [T][H][DVP] (zeros from dv on)
template <typename T>
__global__ void lightning_prepare_kernel(const T* __restrict__ proj, int ld, float* __restrict__ qk, float* __restrict__ v,
                                         int H, int dk, int dv, int DKP, int DVP) {
    const size_t row = blockIdx.x;
    const int h = blockIdx.y;
    const T* src = proj + row * ld;
    float* qk_dst = qk + (row * H + h) * 2 * DKP;
    float* v_dst = v + (row * H + h) * DVP;
    for (int e = threadIdx.x; e < 2 * DKP + DVP; e += blockDim.x) {
        if (e < 2 * DKP) {
            const int i = e < DKP ? e : e - DKP;
            const size_t at = (e < DKP ? 0 : (size_t)H * dk) + (size_t)h * dk + i;
            qk_dst[e] = i < dk ? lt_silu(to_f32(src[at])) : 0.f;
        } else {
            const int jj = e - 2 * DKP;
            v_dst[jj] = jj < dv ? lt_silu(to_f32(src[(size_t)2 * H * dk + (size_t)h * dv + jj])) : 0.f;
        }
    }
}

// A long portion of a prompt is cut into segments of LT_SEGMENT rows that are walked side by side (`seg_rows` > 0):
// every segment but a portion's first starts from a state of zero and leaves its end state in `carry`; a second
// launch adds the end states up along the portion (P_1 = E_0, P_(s+1) = c^rows(s) P_s + E_s: what segment s + 1 should
// have started from; the last sum is the sequence's new state); a third (lightning_apply) adds to every row of segment
// s >= 1 what the state it should have started from contributes, c^(t + 1) P_s^T q_t for the segment's row t.  The sums are the
// recurrence's own, in another order.
#define LT_SEGMENT 256

struct LtSegment {
    int seq, first, rows, index, count;                  // the sequence; the first row (within the step's rows of the
};                                                       // sequence) and the rows; which of how many segments

// segment z of the step, counted sequence by sequence (seg_rows 0: every sequence is one segment); false past the last
__device__ __forceinline__ bool lt_segment_of(int z, const int* __restrict__ row_start, int num_seqs, int seg_rows,
                                              LtSegment& s) {
    if (seg_rows <= 0) {
        if (z >= num_seqs) return false;
        s.seq = z, s.first = 0, s.rows = row_start[z + 1] - row_start[z], s.index = 0, s.count = 1;
        return true;
    }
    int before = 0;
    for (int i = 0; i < num_seqs; ++i) {
        const int n = row_start[i + 1] - row_start[i];
        const int c = max(1, (n + seg_rows - 1) / seg_rows);
        if (z < before + c) {
            s.seq = i, s.index = z - before, s.count = c, s.first = s.index * seg_rows;
            s.rows = min(seg_rows, n - s.first);
            return true;
        }
        before += c;
    }
    return false;
}

// L lanes a column (16 or 64), R elements of it a lane, CH rows a chunk
template <int L, int R, int CH>
__global__ __launch_bounds__(LT_THREADS) void lightning_recurrence_kernel(
    const float* __restrict__ qk, const float* __restrict__ vals, int DVP, const float* __restrict__ decay,
    float* __restrict__ state, float* __restrict__ out, const int* __restrict__ row_start,
    const int* __restrict__ seq_start, const int* __restrict__ slots, int H, int dk, int dv, int num_seqs, int seg_rows,
    float* __restrict__ carry) {
    constexpr int DKP = L * R;
    constexpr int NC = LT_THREADS / L;                   // columns a workgroup
    constexpr int W = 2 * DKP + NC;                      // floats of a staged row: q, k, the workgroup's values
    constexpr int PQ = CH * 2 * DKP / 4 / LT_THREADS;    // 16-byte pieces of q and k that a thread brings a chunk
    constexpr int PV = CH * NC / 4;                      // pieces of v a chunk, one a thread for the first threads
    constexpr int VW = R % 4 == 0 ? 4 : R % 2 == 0 ? 2 : 1;   // floats of a piece: what a lane reads or writes at once
    static_assert(PQ * LT_THREADS * 4 == CH * 2 * DKP && PV <= LT_THREADS, "a chunk is shared out evenly");
    __shared__ __align__(16) float rows_s[CH * W];
    const int h = blockIdx.y, j0 = blockIdx.x * NC;
    const int tid = threadIdx.x;
    const int sub = tid % L, jl = tid / L;
    const int j = j0 + jl;
    // Element r of a lane is element at(r) of the column: the lanes' pieces of VW floats lie side by side (piece p of
    // lane s at (p L + s) VW), so that what the column's lanes read from LDS or from the state in one instruction is
    // one run of memory, which no two of them find in the same bank.
    auto at = [&](int r) { return (r / VW) * (L * VW) + sub * VW + r % VW; };
    LtSegment seg;
    if (!lt_segment_of(blockIdx.z, row_start, num_seqs, seg_rows, seg)) return;      // (the grid's slack)
    const int seq = seg.seq, n = seg.rows;
    const int r0 = row_start[seq] + seg.first;
    if (n <= 0) return;
    const float lam = decay[h];
    // where the state comes from and goes to: the sequence's slot, or the segment's place in `carry`
    const size_t column = ((size_t)h * dv + (j < dv ? j : 0)) * dk;
    float* slot_col = state + (size_t)slots[seq] * H * dv * dk + column;
    float* carry_col = carry + (size_t)blockIdx.z * H * dv * dk + column;
    const float* from = slot_col;
    const bool read = seg.index == 0 && seq_start[seq] != 0;
    float* to = seg.count == 1 ? slot_col : carry_col;
    const bool whole = dk == DKP && dk % 4 == 0;         // every lane's elements exist, and its pieces are aligned
    float S[R];
#pragma unroll
    for (int r = 0; r < R; ++r) S[r] = 0.f;
    if (read && j < dv) {
        if (whole) {
#pragma unroll
            for (int r = 0; r < R; r += VW) {
                if constexpr (VW == 4) {
                    const float4 v = *reinterpret_cast<const float4*>(from + at(r));
                    S[r] = v.x, S[r + 1] = v.y, S[r + 2] = v.z, S[r + 3] = v.w;
                } else if constexpr (VW == 2) {
                    const float2 v = *reinterpret_cast<const float2*>(from + at(r));
                    S[r] = v.x, S[r + 1] = v.y;
                } else {
                    S[r] = from[at(r)];
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (at(r) < dk) S[r] = from[at(r)];
        }
    }
    // A chunk is fetched into registers, every load issued before any is used, while the chunk before is walked:
    // piece p of q and k is 4 floats of row p / (2 DKP / 4) of the chunk; rows past the segment's end are zeros.
    const float* qk_seq = qk + ((size_t)r0 * H + h) * 2 * DKP;
    const float* v_seq = vals + ((size_t)r0 * H + h) * DVP + j0;
    float4 pq[PQ], pv;
    auto fetch = [&](int first) {
#pragma unroll
        for (int u = 0; u < PQ; ++u) {
            const int p = tid + u * LT_THREADS;
            const int rr = p / (2 * DKP / 4), c4 = p - rr * (2 * DKP / 4);
            pq[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (first + rr < n) pq[u] = *reinterpret_cast<const float4*>(qk_seq + (size_t)(first + rr) * H * 2 * DKP + c4 * 4);
        }
        pv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (tid < PV) {
            const int rr = tid / (NC / 4), c4 = tid - rr * (NC / 4);
            if (first + rr < n) pv = *reinterpret_cast<const float4*>(v_seq + (size_t)(first + rr) * H * DVP + c4 * 4);
        }
    };
    fetch(0);
    float* o_col = out + (size_t)r0 * H * dv + (size_t)h * dv + j;
    for (int t0 = 0; t0 < n; t0 += CH) {
        __syncthreads();                                 // the chunk before has been walked by every wave
#pragma unroll
        for (int u = 0; u < PQ; ++u) {
            const int p = tid + u * LT_THREADS;
            const int rr = p / (2 * DKP / 4), c4 = p - rr * (2 * DKP / 4);
            *reinterpret_cast<float4*>(rows_s + rr * W + c4 * 4) = pq[u];
        }
        if (tid < PV) {
            const int rr = tid / (NC / 4), c4 = tid - rr * (NC / 4);
            *reinterpret_cast<float4*>(rows_s + rr * W + 2 * DKP + c4 * 4) = pv;
        }
        __syncthreads();
        if (t0 + CH < n) fetch(t0 + CH);
        const int cnt = min(CH, n - t0);
#pragma unroll 4
        for (int t = 0; t < cnt; ++t) {
            const float* row = rows_s + t * W;
            const float v = row[2 * DKP + jl];
            float acc = 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                S[r] = fmaf(lam, S[r], row[DKP + at(r)] * v);
                acc = fmaf(S[r], row[at(r)], acc);
            }
            acc = lt_sum16(acc);
            if constexpr (L == 64) acc = quad_rows_sum(acc);
            if (sub == 0 && j < dv) o_col[(size_t)(t0 + t) * H * dv] = acc;
        }
    }
    if (j >= dv) return;
    if (whole) {
#pragma unroll
        for (int r = 0; r < R; r += VW) {
            if constexpr (VW == 4) *reinterpret_cast<float4*>(to + at(r)) = make_float4(S[r], S[r + 1], S[r + 2], S[r + 3]);
            else if constexpr (VW == 2) *reinterpret_cast<float2*>(to + at(r)) = make_float2(S[r], S[r + 1]);
            else to[at(r)] = S[r];
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (at(r) < dk) to[at(r)] = S[r];
    }
}

// The second launch of a step with segments: one thread an element of a sequence's state.  carry[z] holds the end
// state E of segment z and is left holding the state P that the segment should have started from; the sequence's slot
// gets its new state.
__global__ void lightning_carry_kernel(float* __restrict__ carry, float* __restrict__ state, const float* __restrict__ decay,
                                       const int* __restrict__ row_start, const int* __restrict__ slots, int num_seqs,
                                       int seg_rows, int H, int dv, int dk) {
    const int seq = blockIdx.y;
    const size_t per = (size_t)H * dv * dk;
    const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= per) return;
    int z0 = 0;
    for (int i = 0; i < seq; ++i) z0 += max(1, (row_start[i + 1] - row_start[i] + seg_rows - 1) / seg_rows);
    const int n = row_start[seq + 1] - row_start[seq];
    const int count = max(1, (n + seg_rows - 1) / seg_rows);
    if (count == 1) return;                              // (its one segment wrote the slot itself)
    const float lam = decay[e / ((size_t)dv * dk)];
    const float whole = powf(lam, (float)seg_rows), last = powf(lam, (float)(n - (count - 1) * seg_rows));
    float p = carry[(size_t)z0 * per + e];
    for (int s = 1; s < count; ++s) {
        float* at = carry + (size_t)(z0 + s) * per + e;
        const float end = *at;
        *at = p;
        p = fmaf(s == count - 1 ? last : whole, p, end);
    }
    state[(size_t)slots[seq] * per + e] = p;
}

// The third launch of a step with segments: out[t, :] += c^(t + 1) P^T q_t for the rows t of every segment but a
// portion's first, P the state that the segment should have started from (left in `carry` by the second launch, a
// head's [dv][dk]).  A product of float32 matrices: a wave takes 16 rows of a segment and NT tiles of 16 columns (a
// workgroup 64 rows), and
// multiplies on the matrix cores with v_mfma_f32_16x16x4_f32, which takes float32 as it is (A: lane l has row l % 16,
// k = l / 16; B: k = l / 16, column l % 16; the sums: rows 4 (l / 16) .. + 3 of column l % 16).  Of 16 consecutive k,
// lane group c takes 4 c .. 4 c + 3 in four instructions (the order of k does not matter as long as q and P agree),
// so that a lane loads its four elements of q, and of P, in one piece of 16 bytes, straight from memory: both were
// written by the launches before and lie in the cache.
typedef float lt_f32x4 __attribute__((ext_vector_type(4)));

template <int NT>
__global__ __launch_bounds__(LT_THREADS) void lightning_apply_kernel(
    const float* __restrict__ qk, int DKP, const float* __restrict__ decay, float* __restrict__ out,
    const int* __restrict__ row_start, int H, int dk, int dv, int num_seqs, int seg_rows, const float* __restrict__ carry) {
    LtSegment seg;
    if (!lt_segment_of(blockIdx.z, row_start, num_seqs, seg_rows, seg)) return;      // (the grid's slack)
    if (seg.count == 1 || seg.index == 0) return;
    // (a workgroup: 64 rows of the segment, 16 a wave, and 16 NT columns; blockIdx.x counts the groups of rows first)
    constexpr int ROW_GROUPS = LT_SEGMENT / 64;
    const int h = blockIdx.y, jb = (blockIdx.x / ROW_GROUPS) * 16 * NT;
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE, r = lane % 16, c = lane / 16;
    const int r0 = row_start[seg.seq] + seg.first, n = seg.rows;
    const float lam = decay[h];
    const float* P = carry + ((size_t)blockIdx.z * H + h) * dv * dk;
    const bool whole = dk % 4 == 0;                      // a lane's four elements of a column exist together, aligned
    const int t0 = (blockIdx.x % ROW_GROUPS) * 64 + wave * 16;
    if (t0 < n) {
        const bool live = t0 + r < n;
        const float* q_row = qk + ((size_t)(r0 + (live ? t0 + r : 0)) * H + h) * 2 * DKP;    // (zeros from dk on)
        lt_f32x4 acc[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[nt] = (lt_f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
        for (int kb = 0; kb < DKP; kb += 16) {
            const int i = kb + 4 * c;
            float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
            if (live) a = *reinterpret_cast<const float4*>(q_row + i);
            float4 b[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int j = jb + nt * 16 + r;
                b[nt] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (j < dv && i < dk) {
                    const float* p = P + (size_t)j * dk + i;
                    if (whole) {
                        b[nt] = *reinterpret_cast<const float4*>(p);
                    } else {
                        b[nt].x = p[0];
                        if (i + 1 < dk) b[nt].y = p[1];
                        if (i + 2 < dk) b[nt].z = p[2];
                        if (i + 3 < dk) b[nt].w = p[3];
                    }
                }
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b[nt].x, acc[nt], 0, 0, 0);
                acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b[nt].y, acc[nt], 0, 0, 0);
                acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b[nt].z, acc[nt], 0, 0, 0);
                acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b[nt].w, acc[nt], 0, 0, 0);
            }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int t = t0 + 4 * c + v;
            if (t >= n) continue;
            const float power = powf(lam, (float)(t + 1));
            float* o = out + (size_t)(r0 + t) * H * dv + (size_t)h * dv;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int j = jb + nt * 16 + r;
                if (j < dv) o[j] += power * acc[nt][v];
            }
        }
    }
}

static int lt_pow2_at_least(int n) {
    int p = 1;
    while (p < n) p *= 2;
    return p;
}

// How many lanes hold a column of the state (`lanes` 0: 16, where a wave has four columns and a quarter of the additions
// across lanes a column; 64 lanes a column give one long prompt four times the waves, and were measured level with 16
// at 16 heads of 128 x 128 and a third slower at 32 heads and in decode steps), and the padded key size DKP of that layout.
static int lt_plan(int dk, int lanes, int* dkp) {
    if (lanes == 0) lanes = 16;
    *dkp = lanes * lt_pow2_at_least((dk + lanes - 1) / lanes);
    return lanes;
}

// The rows of a segment, or 0 where the step's portions are walked whole: segments pay from about one and a half of
// them on (a second and a third launch, and the third walks the rows once more).
static int lt_segment_rows(int longest) { return longest > LT_SEGMENT + LT_SEGMENT / 2 ? LT_SEGMENT : 0; }

// float32 elements of scratch that tli_lightning_recurrence wants for a step of `rows` rows in `seqs` sequences whose
// longest portion has `longest` rows
extern "C" long long tli_lightning_scratch_floats(int rows, int seqs, int longest, int H, int dk, int dv) {
    int a = 0, b = 0;
    lt_plan(dk, 16, &a);
    lt_plan(dk, 64, &b);
    const int seg = lt_segment_rows(longest);
    const long long segments = seg ? rows / seg + seqs : 0;
    return (long long)rows * H * (2LL * (a > b ? a : b) + (dv + 15) / 16 * 16) + segments * H * dv * dk;
}

// proj: [T, ld] raw projections, q (H dk), k (H dk), v (H dv) first; decay: float32 [H]; state: float32
// [slots, H, dv, dk]; out: float32 [T, H dv]; row_start [seqs + 1], seq_start, slots [seqs]; scratch: float32,
// tli_lightning_scratch_floats(T, ...) elements; longest: the most rows that a sequence brings (an upper bound will do);
// lanes: 16 or 64 lanes a column, or 0 for the launch rule
extern "C" int tli_lightning_recurrence(const void* proj, int ld, const float* decay, float* state, float* out,
                                        float* scratch, const int* row_start, const int* seq_start, const int* slots,
                                        int T, int seqs, int longest, int H, int dk, int dv, int dtype, int lanes,
                                        void* stream) {
    if (seqs <= 0 || T <= 0) return 0;
    if (H <= 0 || dk <= 0 || dv <= 0 || dk > LT_MAX_DK)
        return tli_fail("lightning: bad sizes (heads %d, keys of %d (at most %d), values of %d)", H, dk, LT_MAX_DK, dv);
    if (ld < 2 * H * dk + H * dv) return tli_fail("lightning: rows of %d hold fewer than q, k and v", ld);
    if (H > 65535 || seqs > 65535) return tli_fail("lightning: too many heads or sequences for one launch");
    if (lanes != 0 && lanes != 16 && lanes != 64) return tli_fail("lightning: 16 or 64 lanes a column, not %d", lanes);
    if (((uintptr_t)scratch | (uintptr_t)state) & 15) return tli_fail("lightning: scratch and state must be 16-byte aligned");
    int DKP = 0;
    lanes = lt_plan(dk, lanes, &DKP);
    const int DVP = (dv + 15) / 16 * 16;
    float* qk = scratch;
    float* vals = qk + (size_t)T * H * 2 * DKP;
    float* carry = vals + (size_t)T * H * DVP;
    const int seg = lt_segment_rows(longest);
    const int zs = seg ? T / seg + seqs : seqs;          // (an upper bound of the segments; a workgroup past the last leaves)
    if (zs > 65535) return tli_fail("lightning: too many segments for one launch");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TLI_F32)
        hipLaunchKernelGGL((lightning_prepare_kernel<float>), dim3(T, H), dim3(256), 0, s, (const float*)proj, ld, qk, vals, H, dk,
                           dv, DKP, DVP);
    else if (dtype == TLI_BF16)
        hipLaunchKernelGGL((lightning_prepare_kernel<bf16_t>), dim3(T, H), dim3(256), 0, s, (const bf16_t*)proj, ld, qk, vals, H,
                           dk, dv, DKP, DVP);
    else
        return tli_fail("lightning: unknown dtype %d", dtype);
    const int cols = LT_THREADS / lanes;
    const dim3 grid((dv + cols - 1) / cols, H, zs);
    const int R = DKP / lanes;
#define LT_LAUNCH(L, R, CH)                                                                                         \
    hipLaunchKernelGGL((lightning_recurrence_kernel<L, R, CH>), grid, dim3(LT_THREADS), 0, s, qk, vals, DVP, decay, \
                       state, out, row_start, seq_start, slots, H, dk, dv, seqs, seg, carry)
    if (lanes == 64) {
        if (R == 1) LT_LAUNCH(64, 1, 32);
        else if (R == 2) LT_LAUNCH(64, 2, 32);
        else LT_LAUNCH(64, 4, 16);
    } else if (R == 1) LT_LAUNCH(16, 1, 32);
    else if (R == 2) LT_LAUNCH(16, 2, 32);
    else if (R == 4) LT_LAUNCH(16, 4, 32);
    else if (R == 8) LT_LAUNCH(16, 8, 32);
    else LT_LAUNCH(16, 16, 16);
#undef LT_LAUNCH
    if (seg) {
        const size_t per = (size_t)H * dv * dk;
        hipLaunchKernelGGL(lightning_carry_kernel, dim3((unsigned)((per + 255) / 256), seqs), dim3(256), 0, s, carry, state, decay,
                           row_start, slots, seqs, seg, H, dv, dk);
        // (four tiles of 16 columns a wave where the head has them: q is then loaded once for 64 columns)
        if (dv > 32)
            hipLaunchKernelGGL((lightning_apply_kernel<4>), dim3((dv + 63) / 64 * (LT_SEGMENT / 64), H, zs), dim3(LT_THREADS), 0, s, qk, DKP, decay, out,
                               row_start, H, dk, dv, seqs, seg, carry);
        else
            hipLaunchKernelGGL((lightning_apply_kernel<2>), dim3((dv + 31) / 32 * (LT_SEGMENT / 64), H, zs), dim3(LT_THREADS), 0, s, qk, DKP, decay, out,
                               row_start, H, dk, dv, seqs, seg, carry);
    }
    return tli_check_launch("lightning_recurrence");
}

// one workgroup a row
template <typename T>
__global__ void lightning_norm_kernel(const float* __restrict__ o, const T* __restrict__ gate, int gate_ld,
                                      const float* __restrict__ weight, T* __restrict__ out, int n, float eps) {
    __shared__ float red[16];
    const size_t row = blockIdx.x;
    const float* x = o + row * n;
    const T* g = gate + row * gate_ld;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss += x[i] * x[i];
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += blockDim.x)
        from_f32(out + row * n + i, x[i] * scale * weight[i] / (1.0f + expf(-to_f32(g[i]))));
}

// o: float32 [T, n]; gate: [T, gate_ld] (its first n columns); weight: float32 [n]; out: [T, n]
extern "C" int tli_lightning_norm(const float* o, const void* gate, int gate_ld, const float* weight, void* out, int T,
                                  int n, float eps, int dtype, void* stream) {
    if (T <= 0) return 0;
    if (n <= 0 || gate_ld < n) return tli_fail("lightning_norm: bad sizes");
    hipStream_t s = (hipStream_t)stream;
    const int threads = n >= 2048 ? 512 : 256;
    if (dtype == TLI_F32)
        hipLaunchKernelGGL((lightning_norm_kernel<float>), dim3(T), dim3(threads), 0, s, o, (const float*)gate, gate_ld, weight,
                           (float*)out, n, eps);
    else if (dtype == TLI_BF16)
        hipLaunchKernelGGL((lightning_norm_kernel<bf16_t>), dim3(T), dim3(threads), 0, s, o, (const bf16_t*)gate, gate_ld,
                           weight, (bf16_t*)out, n, eps);
    else
        return tli_fail("lightning_norm: unknown dtype %d", dtype);
    return tli_check_launch("lightning_norm");
}
