// Attention over the paged cache for heads whose keys and values have sizes of their own: the matrix-core kernels
// for bfloat16, key and value sizes in sixteens.  What they compute is what attention_sized_plain.hip computes
// (maps of a head, values from a cache of their own or the first elements of the keys, a window with kept first
// keys).  Two kernels:
//
// attention_sized_shared_kernel (further down): portions of prompts, and single rows whose values are their keys'
//   first elements (all heads read the one latent vector): four waves with 16 columns each share every tile of keys.
// attention_sized_mfma_kernel (first): single decoded rows whose values have a cache of their own.  A workgroup of
//   four waves takes one row and one (key head, map); its 16 columns are query heads that read that key head.  The keys
//   the row can see (from the first one it sees to itself, and the kept first ones before them) are walked 16 at a
//   time, the waves taking every fourth 16 each with a running maximum and sums of their own, merged through LDS at
//   the end.  (It also takes tiles of 16 rows of a sequence and one head, as it did before the other kernel was there.)
//
// In both everything is transposed: S^T = K Q^T and O^T = V^T P^T with v_mfma_f32_16x16x16_bf16, so that a row's
// scores lie in the four lanes of a column and its weights are already the second operand of the output's product.
// Every (row, key) pair is masked on its own.  Keys come into LDS with 16-byte loads, the next tile's in flight
// meanwhile, and their fragments are read from there; a value cache lies transposed ([dim][slot]), so that a lane's
// four keys of one dim are 8 bytes (a tile of 16 keys lies inside one page: pages of 16 slots and more).
//
// The sizes are arguments, not template parameters, but for the common sizes, which have kernels of their own (EXACT
// below): the registers for the query's fragments and the output's sums are those of the largest size of a variant
// (keys up to 128 / 256 / 640 elements, values up to 128 / 256 / 512).
#include "common.h"

typedef __attribute__((ext_vector_type(4))) short bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

union SFrag4 {
    uint2 u;
    bf16_t e[4];
    bf16x4 v;
};

#define ASM_WAVES 4
#define ASM_PAD 8          // bfloat16 elements between the rows of a key tile in LDS

__device__ __forceinline__ void asm_store4(float* dst, const f32x4& a, float f) {
    *reinterpret_cast<float4*>(dst) = make_float4(a[0] * f, a[1] * f, a[2] * f, a[3] * f);
}
__device__ __forceinline__ void asm_store4(bf16_t* dst, const f32x4& a, float f) {
    uint2 st;
    st.x = pack_bf16x2(a[0] * f, a[1] * f);
    st.y = pack_bf16x2(a[2] * f, a[3] * f);
    *reinterpret_cast<uint2*>(dst) = st;
}

static inline size_t asm_lds_bytes(int DK, int DV) {
    const size_t tiles = (size_t)ASM_WAVES * 16 * (DK + ASM_PAD) * 2;
    const size_t merge = (size_t)(ASM_WAVES - 1) * (16 * DV + 32) * 4;
    return tiles > merge ? tiles : merge;
}

// EXACT: the sizes are NKM and NVM themselves (nk, nv are not read), so that the loops over a head's sixteens have
// no conditions left and the compiler orders the LDS reads of one sixteen ahead of the matrix instruction of another;
// with conditions every sixteen is a block of its own that waits for its own reads.
// A sink: a learned logit a (head, map) that stands in the softmax's denominator with no key and no value.  With the
// running maximum m and sum l (of exp(s - m)) over a row's keys, the row's output is acc / (l + exp(sink - m)); the
// factor that the accumulators are multiplied with, written so that neither exponential overflows.
__device__ __forceinline__ float asm_sink_factor(float sink, float m, float l) {
    const float top = fmaxf(m, sink);
    const float keys = (m == -INFINITY) ? 0.f : __expf(m - top);
    return keys / (l * keys + __expf(sink - top));
}

template <int NKM, int NVM, bool VKEY, typename TO, bool EXACT>
__global__ __launch_bounds__(64 * ASM_WAVES) void attention_sized_mfma_kernel(
    const bf16_t* __restrict__ q, TO* __restrict__ out, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ row_start, const int* __restrict__ seq_start,
    int num_seqs, const int* __restrict__ tables, int table_width, int page_size, int num_pages, int heads,
    int kv_heads, int maps, int nk_arg, int nv_arg, float scale, int window, int keep_first, int grouped, int col_groups,
    const float* __restrict__ sinks) {
    const int nk = EXACT ? NKM : nk_arg, nv = EXACT ? NVM : nv_arg;
    const int DK = nk * 16, DV = nv * 16, LD = DK + ASM_PAD;
    const int pieces = 2 * nk;                                          // 16-byte pieces of one key
    const int chunks = 16 * pieces;                                     // of a key tile
    constexpr int PASSES = (16 * 2 * NKM + 63) / 64;
    extern __shared__ __align__(16) unsigned char asm_lds[];
    const int lane = threadIdx.x % 64, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int col = lane % 16, grp = lane / 16;
    const int per_tile = grouped ? 1 : 16;
    int tile = blockIdx.x, seq = 0, first_row = 0, count = 0;
    for (; seq < num_seqs; ++seq) {
        first_row = row_start[seq];
        count = row_start[seq + 1] - first_row;
        const int nt = (count + per_tile - 1) / per_tile;
        if (tile < nt) break;
        tile -= nt;
    }
    if (seq >= num_seqs) return;                                        // (the whole workgroup)
    const int per_kv = heads / kv_heads;
    int kh, unit, live_cols;
    if (grouped) {
        kh = blockIdx.y / col_groups;                                   // key head * maps + map
        const int c0 = (blockIdx.y % col_groups) * 16;
        live_cols = min(16, per_kv - c0);
        const int head = (kh / maps) * per_kv + c0 + min(col, live_cols - 1);
        unit = head * maps + kh % maps;
    } else {
        unit = blockIdx.y;
        kh = ((unit / maps) / per_kv) * maps + unit % maps;
        live_cols = 0;                                                  // (set below: the tile's rows)
    }
    const int g = kh / maps;                                            // the values' head
    const int units = heads * maps;
    const int* table = tables + (size_t)seq * table_width;
    const int live = min(per_tile, count - tile * per_tile);            // rows of this tile
    if (!grouped) live_cols = live;
    const int row0 = first_row + tile * per_tile;
    const int pos0 = seq_start[seq] + tile * per_tile;
    const int lo = window > 0 ? max(0, pos0 - window + 1) : 0, hi = pos0 + live - 1;
    const int kept_hi = window > 0 ? min(keep_first, lo) : 0;           // keys 0..kept_hi-1 are seen beside lo..hi
    const size_t k_page = (size_t)kv_heads * maps * page_size * DK;
    const size_t v_page = (size_t)kv_heads * page_size * DV;
    const int page_shift = __builtin_ctz(page_size), page_mask = page_size - 1;

    const int my = grouped ? 0 : min(col, live - 1);                    // (idle columns repeat the last row; never stored)
    const int qpos = pos0 + my;
    const int qlo = window > 0 ? max(0, qpos - window + 1) : 0;
    SFrag4 qf[NKM];
    f32x4 acc[NVM];
    {
        const bf16_t* q_row = q + ((size_t)(row0 + my) * units + unit) * DK;
#pragma unroll
        for (int j = 0; j < NKM; ++j) {
            qf[j].u = make_uint2(0, 0);
            if (j < nk) qf[j].u = *reinterpret_cast<const uint2*>(q_row + j * 16 + grp * 4);
            // the fragments stay in registers for the whole walk: without this the compiler is free to fetch them
            // again inside the loop over the keys, one load (and its wait) in front of every matrix instruction
            asm volatile("" : "+v"(qf[j].u.x), "+v"(qf[j].u.y));
        }
#pragma unroll
        for (int j = 0; j < NVM; ++j) acc[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    float m = -INFINITY, l = 0.f;
    bf16_t* kt = reinterpret_cast<bf16_t*>(asm_lds) + (size_t)wave * 16 * LD;     // this wave's key tile [16][LD]

    // the tiles of keys, nearest first: those of lo..hi, then those of the kept first keys that lie before them
    const int k_low = lo - lo % 16, k_top = hi - hi % 16;
    const int n_main = (k_top - k_low) / 16 + 1;
    const int n_kept = (min(kept_hi, k_low) + 15) / 16;
    const int n_tiles = n_main + n_kept;
    auto tile_key = [&](int i) { return i < n_main ? k_top - 16 * i : 16 * (i - n_main); };

    uint4 next[PASSES];
    // chunk c = 64 ps + lane is piece c % pieces of key c / pieces: one division a lane, then steps of 64 chunks
    const int key_first = lane / pieces, piece_first = lane - key_first * pieces;
    const int key_step = 64 / pieces, piece_step = 64 - key_step * pieces;
    auto fetch = [&](int k0) {
        int ck = key_first, cp = piece_first;
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            const int c = ps * 64 + lane;
            next[ps] = make_uint4(0, 0, 0, 0);
            if (c < chunks) {
                const int key = k0 + ck;
                if (key <= hi && (key >= lo || key < kept_hi)) {
                    const int page = table[key >> page_shift];
                    if (page >= 0 && page < num_pages)
                        next[ps] = *reinterpret_cast<const uint4*>(k_cache + (size_t)page * k_page +
                                                                   ((size_t)kh * page_size + (key & page_mask)) * DK + cp * 8);
                }
            }
            ck += key_step;
            cp += piece_step;
            if (cp >= pieces) {
                cp -= pieces;
                ++ck;
            }
        }
    };
    if (wave < n_tiles) fetch(tile_key(wave));
    for (int it = wave; it < n_tiles; it += ASM_WAVES) {
        const int k0 = tile_key(it);
        {
            int ck = key_first, cp = piece_first;
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps) {
                const int c = ps * 64 + lane;
                if (c < chunks) *reinterpret_cast<uint4*>(kt + ck * LD + cp * 8) = next[ps];
                ck += key_step;
                cp += piece_step;
                if (cp >= pieces) {
                    cp -= pieces;
                    ++ck;
                }
            }
        }
        if (it + ASM_WAVES < n_tiles) fetch(tile_key(it + ASM_WAVES));
        // the values of this tile's keys from their own cache: dim 16 j + col of the keys k0 + 4 grp + i
        SFrag4 vf[VKEY ? 1 : NVM];
        if (!VKEY) {
            const int key = k0 + grp * 4;
            const bf16_t* vp = nullptr;
            if (key <= hi && (key + 3 >= lo || key < kept_hi)) {
                const int page = table[key >> page_shift];
                if (page >= 0 && page < num_pages)
                    vp = v_cache + (size_t)page * v_page + ((size_t)g * DV + col) * page_size + (key & page_mask);
            }
#pragma unroll
            for (int j = 0; j < NVM; ++j) {
                vf[j].u = make_uint2(0, 0);
                if (j < nv && vp) vf[j].u = *reinterpret_cast<const uint2*>(vp + (size_t)j * 16 * page_size);
            }
        }
        wave_lds_sync();
        // scores: A = the key k0 + col, this lane group's dims
        // (two sums in turn, so that a matrix instruction does not wait for the one before it)
        f32x4 s = (f32x4){0.f, 0.f, 0.f, 0.f}, s_odd = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < NKM; ++j) {
            if (j < nk) {
                SFrag4 a;
                a.u = *reinterpret_cast<const uint2*>(kt + col * LD + j * 16 + grp * 4);
                if (j % 2)
                    s_odd = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, qf[j].v, s_odd, 0, 0, 0);
                else
                    s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, qf[j].v, s, 0, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] += s_odd[i];
        // this lane: keys k0 + 4 grp + i of column col
        SFrag4 p;
        float w[4];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = k0 + grp * 4 + i;
            const bool seen = key <= qpos && (key >= qlo || key < keep_first);
            w[i] = seen ? s[i] * scale : -INFINITY;
            mx = fmaxf(mx, w[i]);
        }
        mx = quad_rows_max(mx);
        const float m_new = fmaxf(m, mx);
        // (a column whose keys so far are all hidden keeps m = -inf: its weights and its correction are 0)
        const float corr = (m_new == -INFINITY) ? 0.f : __expf(m - m_new);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float e = (w[i] == -INFINITY) ? 0.f : __expf(w[i] - m_new);
            p.e[i] = f32_to_bf16(e);
            sum += bf16_to_f32(p.e[i]);                 // the weights as the values meet them
        }
        l = l * corr + quad_rows_sum(sum);
        m = m_new;
        const bool rescale = __any(corr != 1.0f);       // (the same for the whole wave)
#pragma unroll
        for (int j = 0; j < NVM; ++j) {
            if (j < nv) {
                SFrag4 a;
                if (VKEY) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) a.e[i] = kt[(grp * 4 + i) * LD + j * 16 + col];
                } else {
                    a = vf[j];
                }
                if (rescale) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[j][i] *= corr;
                }
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, p.v, acc[j], 0, 0, 0);
            }
        }
        wave_lds_sync();                                // the tile is read before the next one is written over it
    }
    // the four waves' sums into wave 0: each of the others leaves (m, l) a column and its accumulators
    __syncthreads();
    float* merge = reinterpret_cast<float*>(asm_lds);
    const int per_wave = 16 * DV + 32;
    if (wave > 0) {
        float* mine = merge + (size_t)(wave - 1) * per_wave;
        if (grp == 0) {
            mine[col] = m;
            mine[16 + col] = l;
        }
#pragma unroll
        for (int j = 0; j < NVM; ++j)
            if (j < nv) *reinterpret_cast<f32x4*>(mine + 32 + ((size_t)j * 64 + lane) * 4) = acc[j];
    }
    __syncthreads();
    if (wave > 0) return;
    float mt = m;
#pragma unroll
    for (int w = 0; w < ASM_WAVES - 1; ++w) mt = fmaxf(mt, merge[(size_t)w * per_wave + col]);
    const float f0 = (m == -INFINITY) ? 0.f : __expf(m - mt);
    float lt = l * f0;
    float fw[ASM_WAVES - 1];
#pragma unroll
    for (int w = 0; w < ASM_WAVES - 1; ++w) {
        const float* theirs = merge + (size_t)w * per_wave;
        const float mw = theirs[col];
        fw[w] = (mw == -INFINITY) ? 0.f : __expf(mw - mt);
        lt += theirs[16 + col] * fw[w];
    }
    if (col >= live_cols) return;
    float inv = lt > 0.f ? 1.0f / lt : 0.f;
    if (sinks) inv = asm_sink_factor(sinks[unit], mt, lt);
    int out_unit = unit, out_row = row0 + my;
    TO* o_row = out + ((size_t)out_row * units + out_unit) * DV;
#pragma unroll
    for (int j = 0; j < NVM; ++j) {
        if (j < nv) {
            f32x4 a = acc[j];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] *= f0;
#pragma unroll
            for (int w = 0; w < ASM_WAVES - 1; ++w) {
                const f32x4 t = *reinterpret_cast<const f32x4*>(merge + (size_t)w * per_wave + 32 + ((size_t)j * 64 + lane) * 4);
#pragma unroll
                for (int i = 0; i < 4; ++i) a[i] += t[i] * fw[w];
            }
            asm_store4(o_row + j * 16 + grp * 4, a, inv);
        }
    }
}

// ---- steps with portions of prompts: four waves share every tile of keys ----------------------------------------
//
// A workgroup takes four "column tiles" that read the same key head: a column tile is 16 consecutive rows of one
// sequence for one query head, numbered row tile by row tile and, within a row tile, head by head of the key head's
// query heads.  (Four query heads a key head: one row tile, its four heads; one: four row tiles of the head; sixteen:
// a quarter of a row tile's heads.)  Every wave has one column tile, with its queries' fragments, its running
// maxima and sums and its output in registers, and walks ALL the tiles of 16 keys that the workgroup's rows see;
// a wave whose rows see nothing of a tile leaves its arithmetic out.  The 256 threads bring a tile of keys into LDS
// together (a thread has one key of the tile and every sixteenth 16-byte piece of it, so one look into the block
// table a thread and tile and no division), the next tile's loads in flight while the current one is multiplied,
// two LDS buffers taking turns with one barrier a tile.  Beside the keys' rows [16][dim + 8] lies V^T
// [value dim][16 keys + 4]: copied from the value cache (which is stored transposed) 16 bytes at a time, or, where
// the values are the keys' first elements, written two bytes at a time from the registers that hold the keys, so
// that both operands of both products are 8-byte LDS reads.
#define AST_VLD 20         // bfloat16 elements a row of V^T in LDS

static inline size_t ast_lds_bytes(int DK, int DV) {
    return 2 * ((size_t)16 * (DK + ASM_PAD) + (size_t)DV * AST_VLD) * 2;
}

template <int NKM, int NVM, bool VKEY, typename TO, bool EXACT, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void attention_sized_shared_kernel(
    const bf16_t* __restrict__ q, TO* __restrict__ out, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ row_start, const int* __restrict__ seq_start,
    int num_seqs, const int* __restrict__ tables, int table_width, int page_size, int num_pages, int heads,
    int kv_heads, int maps, int nk_arg, int nv_arg, float scale, int window, int keep_first, int grouped,
    const float* __restrict__ sinks) {
    const int nk = EXACT ? NKM : nk_arg, nv = EXACT ? NVM : nv_arg;
    const int DK = nk * 16, DV = nv * 16, LD = DK + ASM_PAD;
    const int pieces = 2 * nk;                                          // 16-byte pieces of one key
    constexpr int KPASS = (2 * NKM + 4 * WAVES - 1) / (4 * WAVES);                          // pieces of its key a thread brings
    constexpr int VPASS = VKEY ? 1 : (32 * NVM + 64 * WAVES - 1) / (64 * WAVES);            // 16-byte pieces of V^T a thread brings
    extern __shared__ __align__(16) unsigned char ast_lds[];
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int col = lane % 16, grp = lane / 16;
    const int per_kv = heads / kv_heads;
    // grouped (steps of single rows): a column tile is one row, its columns 16 of the key head's query heads
    const int per_tile = grouped ? 1 : 16;
    const int cts_a_tile = grouped ? (per_kv + 15) / 16 : per_kv;       // column tiles that share a tile of rows
    int wg = blockIdx.x, seq = 0, first_row = 0, count = 0, n_ct = 0;
    for (; seq < num_seqs; ++seq) {
        first_row = row_start[seq];
        count = row_start[seq + 1] - first_row;
        n_ct = ((count + per_tile - 1) / per_tile) * cts_a_tile;
        const int n_wg = (n_ct + WAVES - 1) / WAVES;
        if (wg < n_wg) {
            // a sequence's last rows see the most keys: their workgroups start first, and the short ones fill in
            // behind them as compute units come free
            wg = n_wg - 1 - wg;
            break;
        }
        wg -= n_wg;
    }
    if (seq >= num_seqs) return;                                        // (the whole workgroup)
    const int kh = blockIdx.y;                                          // key head * maps + map
    const int g = kh / maps;                                            // the values' head
    const int units = heads * maps;
    const int ct_last = min(wg * WAVES + WAVES - 1, n_ct - 1);
    const int ct = min(wg * WAVES + wave, n_ct - 1);
    const bool stores = wg * WAVES + wave < n_ct;                           // (a wave without a column tile only fetches)
    const int rt = ct / cts_a_tile, hc = ct % cts_a_tile;
    const int base_pos = seq_start[seq];
    const int* table = tables + (size_t)seq * table_width;
    // the keys the workgroup's rows see: lo..hi and the kept first ones before them
    const int rt_first = (wg * WAVES) / cts_a_tile, rt_last = ct_last / cts_a_tile;
    const int hi = base_pos + min(count, rt_last * per_tile + per_tile) - 1;
    const int lo = window > 0 ? max(0, base_pos + rt_first * per_tile - window + 1) : 0;
    const int kept_hi = window > 0 ? min(keep_first, lo) : 0;
    // this wave's rows and columns
    const int live_rows = min(per_tile, count - rt * per_tile);
    const int live = grouped ? min(16, per_kv - hc * 16) : live_rows;   // columns that are stored
    const int my = grouped ? 0 : min(col, live - 1);                    // (idle columns repeat the last; never stored)
    const int head = g * per_kv + (grouped ? hc * 16 + min(col, live - 1) : hc);
    const int unit = head * maps + kh % maps;
    const int row = first_row + rt * per_tile + my;
    const int qpos = base_pos + rt * per_tile + my;
    const int qlo = window > 0 ? max(0, qpos - window + 1) : 0;
    const int w_hi = base_pos + rt * per_tile + live_rows - 1;
    const int w_lo = window > 0 ? max(0, base_pos + rt * per_tile - window + 1) : 0;
    const size_t k_page = (size_t)kv_heads * maps * page_size * DK;
    const size_t v_page = (size_t)kv_heads * page_size * DV;
    const int page_shift = __builtin_ctz(page_size), page_mask = page_size - 1;

    SFrag4 qf[NKM];
    f32x4 acc[NVM];
    {
        const bf16_t* q_row = q + ((size_t)row * units + unit) * DK;
#pragma unroll
        for (int j = 0; j < NKM; ++j) {
            qf[j].u = make_uint2(0, 0);
            if (j < nk) qf[j].u = *reinterpret_cast<const uint2*>(q_row + j * 16 + grp * 4);
        }
#pragma unroll
        for (int j = 0; j < NVM; ++j) acc[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    float m = -INFINITY, l = 0.f;
    const size_t buf_elems = (size_t)16 * LD + (size_t)DV * AST_VLD;
    bf16_t* const lds = reinterpret_cast<bf16_t*>(ast_lds);

    // the tiles of keys, nearest first: those of lo..hi, then those of the kept first keys that lie before them
    const int k_low = lo - lo % 16, k_top = hi - hi % 16;
    const int n_main = (k_top - k_low) / 16 + 1;
    const int n_kept = (min(kept_hi, k_low) + 15) / 16;
    const int n_tiles = n_main + n_kept;
    auto tile_key = [&](int i) { return i < n_main ? k_top - 16 * i : 16 * (i - n_main); };

    const int kk = tid % 16, p0 = tid / 16;                             // this thread's key of a tile, its first piece
    uint4 next_k[KPASS];
    uint4 next_v[VPASS];
    auto fetch = [&](int k0) {
        // (a tile of 16 keys lies inside one page)
        const int page = table[k0 >> page_shift];
        const bool there = page >= 0 && page < num_pages;
        const bf16_t* src = k_cache + (size_t)(there ? page : 0) * k_page + ((size_t)kh * page_size + ((k0 + kk) & page_mask)) * DK;
#pragma unroll
        for (int ps = 0; ps < KPASS; ++ps) {
            const int p = ps * (4 * WAVES) + p0;
            next_k[ps] = make_uint4(0, 0, 0, 0);
            if (there && p < pieces) next_k[ps] = *reinterpret_cast<const uint4*>(src + p * 8);
        }
        if (!VKEY) {
            const bf16_t* vsrc = v_cache + (size_t)(there ? page : 0) * v_page + (size_t)g * DV * page_size + (k0 & page_mask);
#pragma unroll
            for (int ps = 0; ps < VPASS; ++ps) {
                const int c = ps * (64 * WAVES) + tid;                           // dim c / 2, keys 8 (c % 2) .. + 7 of the tile
                next_v[ps] = make_uint4(0, 0, 0, 0);
                if (there && c < 2 * DV) next_v[ps] = *reinterpret_cast<const uint4*>(vsrc + (size_t)(c >> 1) * page_size + (c & 1) * 8);
            }
        }
    };
    auto store = [&](bf16_t* buf) {
        bf16_t* kt = buf;
        bf16_t* vt = buf + (size_t)16 * LD;
#pragma unroll
        for (int ps = 0; ps < KPASS; ++ps) {
            const int p = ps * (4 * WAVES) + p0;
            if (p < pieces) {
                *reinterpret_cast<uint4*>(kt + kk * LD + p * 8) = next_k[ps];
                if (VKEY && p * 8 < DV) {
                    const uint32_t w[4] = {next_k[ps].x, next_k[ps].y, next_k[ps].z, next_k[ps].w};
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        vt[(p * 8 + e) * AST_VLD + kk] = (bf16_t)(e % 2 ? w[e / 2] >> 16 : w[e / 2] & 0xFFFFu);
                }
            }
        }
        if (!VKEY) {
#pragma unroll
            for (int ps = 0; ps < VPASS; ++ps) {
                const int c = ps * (64 * WAVES) + tid;
                if (c < 2 * DV) {
                    bf16_t* dst = vt + (c >> 1) * AST_VLD + (c & 1) * 8;    // (8-byte aligned, not 16)
                    *reinterpret_cast<uint2*>(dst) = make_uint2(next_v[ps].x, next_v[ps].y);
                    *reinterpret_cast<uint2*>(dst + 4) = make_uint2(next_v[ps].z, next_v[ps].w);
                }
            }
        }
    };

    fetch(tile_key(0));
    store(lds);
    __syncthreads();
    for (int it = 0; it < n_tiles; ++it) {
        const int k0 = tile_key(it);
        const bool more = it + 1 < n_tiles;
        if (more) fetch(tile_key(it + 1));
        const bf16_t* kt = lds + (size_t)(it & 1) * buf_elems;
        const bf16_t* vt = kt + (size_t)16 * LD;
        if (stores && k0 <= w_hi && (k0 + 15 >= w_lo || k0 < keep_first)) {   // (the same for the whole wave)
            // scores, transposed: A = the key k0 + col, this lane group's dims; two sums in turn, so that a matrix
            // instruction does not wait for the one before it
            f32x4 s = (f32x4){0.f, 0.f, 0.f, 0.f}, s_odd = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < NKM; ++j) {
                if (j < nk) {
                    SFrag4 a;
                    a.u = *reinterpret_cast<const uint2*>(kt + col * LD + j * 16 + grp * 4);
                    if (j % 2)
                        s_odd = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, qf[j].v, s_odd, 0, 0, 0);
                    else
                        s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, qf[j].v, s, 0, 0, 0);
                }
            }
            // this lane: keys k0 + 4 grp + i of column col
            SFrag4 p;
            float w[4];
            float mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = k0 + grp * 4 + i;
                const bool seen = key <= qpos && (key >= qlo || key < keep_first);
                w[i] = seen ? (s[i] + s_odd[i]) * scale : -INFINITY;
                mx = fmaxf(mx, w[i]);
            }
            mx = quad_rows_max(mx);
            const float m_new = fmaxf(m, mx);
            // (a column whose keys so far are all hidden keeps m = -inf: its weights and its correction are 0)
            const float corr = (m_new == -INFINITY) ? 0.f : __expf(m - m_new);
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = (w[i] == -INFINITY) ? 0.f : __expf(w[i] - m_new);
                p.e[i] = f32_to_bf16(e);
                sum += bf16_to_f32(p.e[i]);             // the weights as the values meet them
            }
            l = l * corr + quad_rows_sum(sum);
            m = m_new;
            const bool rescale = __any(corr != 1.0f);   // (the same for the whole wave)
#pragma unroll
            for (int j = 0; j < NVM; ++j) {
                if (j < nv) {
                    SFrag4 a;
                    a.u = *reinterpret_cast<const uint2*>(vt + (j * 16 + col) * AST_VLD + grp * 4);
                    if (rescale) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) acc[j][i] *= corr;
                    }
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, p.v, acc[j], 0, 0, 0);
                }
            }
        }
        if (more) store(lds + (size_t)((it + 1) & 1) * buf_elems);
        __syncthreads();                                // the next tile is written; this one is read by all
    }
    if (!stores || col >= live) return;
    float inv = l > 0.f ? 1.0f / l : 0.f;
    if (sinks) inv = asm_sink_factor(sinks[unit], m, l);
    TO* o_row = out + ((size_t)row * units + unit) * DV;
#pragma unroll
    for (int j = 0; j < NVM; ++j)
        if (j < nv) asm_store4(o_row + j * 16 + grp * 4, acc[j], inv);
}

// Whether the kernel takes these sizes (else the plain one serves).
extern "C" int tli_attention_sized_mfma_takes(int key_dim, int value_dim, int page_size, int has_values) {
    if (key_dim % 16 || value_dim % 16 || key_dim < 16 || value_dim < 16 || key_dim > 640 || value_dim > 512) return 0;
    if (page_size < 16 || (page_size & (page_size - 1))) return 0;
    if (!has_values && value_dim > key_dim) return 0;
    return 1;
}

// q [rows, heads * maps, key_dim]; out [rows, heads * maps, value_dim] (float32 with out_f32, else bfloat16);
// k_cache [pages][kv_heads * maps][slot][key_dim]; v_cache [pages][kv_heads][value_dim][slot] or null;
// tiles: an upper bound of the sum over the sequences of ceil(rows / 16) (of the rows, with `grouped`);
// grouped: a tile is one row and its columns are the query heads of one key head, 16 at a time;
// sinks: float32 [heads * maps] or null
extern "C" int tli_attention_sized_mfma_bf16(
    const void* q, void* out, const void* k_cache, const void* v_cache, const int* row_start, const int* seq_start,
    int num_seqs, int tiles, const int* tables, int table_width, int page_size, int num_pages, int heads, int kv_heads,
    int maps, int key_dim, int value_dim, float scale, int window, int keep_first, int grouped, int out_f32,
    const float* sinks, void* stream) {
    if (num_seqs <= 0 || tiles <= 0) return 0;
    if (!tli_attention_sized_mfma_takes(key_dim, value_dim, page_size, v_cache != nullptr))
        return tli_fail("attention: the matrix-core kernel does not take keys of %d and values of %d in pages of %d", key_dim,
                        value_dim, page_size);
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || maps <= 0)
        return tli_fail("attention: heads %d must be a multiple of kv heads %d", heads, kv_heads);
    if (table_width <= 0 || num_pages <= 0) return tli_fail("attention: bad cache geometry");
    if (window < 0 || keep_first < 0) return tli_fail("attention: bad window %d with %d kept", window, keep_first);
    if ((((uintptr_t)q | (uintptr_t)out | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15))
        return tli_fail("attention: operands must be 16-byte aligned");
    const int per_kv = heads / kv_heads;
    const int col_groups = grouped ? (per_kv + 15) / 16 : 1;
    const long long gy = grouped ? (long long)kv_heads * maps * col_groups : (long long)heads * maps;
    if (gy > 65535) return tli_fail("attention: %lld heads exceed the grid limit 65535", gy);
    hipStream_t s = (hipStream_t)stream;
    const int nk = key_dim / 16, nv = value_dim / 16;
    // Steps of single rows whose values have a cache of their own go to the kernel whose waves share out the keys
    // (measured at 64 rows over 150 keys, 4 query heads a key head: 21 us against 28); everything else to the one
    // whose waves share the tiles of keys.
    if (!(grouped && v_cache)) {
        // (a sequence's column tiles are rounded up to whole workgroups: at most one more a sequence; a workgroup
        // without column tiles leaves)
        // (eight waves a workgroup, two a SIMD, for portions of prompts over the large latent vector, where that
        // still leaves two workgroups and more a compute unit to even out the rows that see few keys)
        const int waves = (!grouped && !v_cache && !out_f32 && nk == 36 && nv == 32 && (long long)tiles * per_kv >= 8 * 512) ? 8 : 4;
        const long long wgs = ((long long)tiles * (grouped ? col_groups : per_kv) + waves - 1) / waves + num_seqs;
        if (wgs > 0x7fffffffLL || kv_heads * maps > 65535) return tli_fail("attention: too many tiles for one launch");
        const dim3 sgrid((unsigned)wgs, (unsigned)(kv_heads * maps));
        const size_t sbytes = ast_lds_bytes(key_dim, value_dim);
#define AST_ONE(NKM, NVM, VKEY, TO, EXACT, WAVES)                                                                                        \
    {                                                                                                                      \
        auto kernel = attention_sized_shared_kernel<NKM, NVM, VKEY, TO, EXACT, WAVES>;                                                   \
        static bool allowed = false;                                                                                       \
        if (sbytes > 65536 && !allowed) {                                                                                  \
            if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) !=        \
                hipSuccess)                                                                                                \
                return tli_fail("attention: cannot have %zu bytes of LDS", sbytes);                                        \
            allowed = true;                                                                                                \
        }                                                                                                                  \
        kernel<<<sgrid, 64 * WAVES, sbytes, s>>>((const bf16_t*)q, (TO*)out, (const bf16_t*)k_cache, (const bf16_t*)v_cache,      \
                                          row_start, seq_start, num_seqs, tables, table_width, page_size, num_pages,      \
                                          heads, kv_heads, maps, nk, nv, scale, window, keep_first, grouped, sinks);      \
    }
#define AST_SIZES(VKEY, TO)                                                   \
    if (nk <= 8 && nv <= 8) AST_ONE(8, 8, VKEY, TO, false, 4)                 \
    else if (nk <= 16 && nv <= 16) AST_ONE(16, 16, VKEY, TO, false, 4)        \
    else AST_ONE(40, 32, VKEY, TO, false, 4)
        // (sizes with a kernel of their own: heads of 64 and 128 with values of 64 to 256 in float32, for the
        // attention with two maps; a latent vector of 512 beside a turned part of 64)
        if (v_cache && out_f32 && nk == 4 && nv == 4) AST_ONE(4, 4, false, float, true, 4)
        else if (v_cache && out_f32 && nk == 4 && nv == 8) AST_ONE(4, 8, false, float, true, 4)
        else if (v_cache && out_f32 && nk == 8 && nv == 8) AST_ONE(8, 8, false, float, true, 4)
        else if (v_cache && out_f32 && nk == 8 && nv == 16) AST_ONE(8, 16, false, float, true, 4)
        else if (waves == 8) AST_ONE(36, 32, true, bf16_t, true, 8)
        else if (!v_cache && !out_f32 && nk == 36 && nv == 32) AST_ONE(36, 32, true, bf16_t, true, 4)
        else if (v_cache) {
            if (out_f32) { AST_SIZES(false, float) } else { AST_SIZES(false, bf16_t) }
        } else {
            if (out_f32) { AST_SIZES(true, float) } else { AST_SIZES(true, bf16_t) }
        }
#undef AST_SIZES
#undef AST_ONE
        return tli_check_launch("attention_sized_shared");
    }
    const dim3 grid(tiles, (unsigned)gy);
    const size_t bytes = asm_lds_bytes(key_dim, value_dim);
#define ASM_ARGS (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, row_start, seq_start, num_seqs, tables, \
        table_width, page_size, num_pages, heads, kv_heads, maps, nk, nv, scale, window, keep_first, grouped, col_groups
#define ASM_ONE(NKM, NVM, VKEY, TO, EXACT)                                                                                        \
    {                                                                                                                      \
        auto kernel = attention_sized_mfma_kernel<NKM, NVM, VKEY, TO, EXACT>;                                                     \
        static bool allowed = false;                                                                                       \
        if (bytes > 65536 && !allowed) {                                                                                   \
            if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) !=        \
                hipSuccess)                                                                                                \
                return tli_fail("attention: cannot have %zu bytes of LDS", bytes);                                         \
            allowed = true;                                                                                                \
        }                                                                                                                  \
        kernel<<<grid, 64 * ASM_WAVES, bytes, s>>>((const bf16_t*)q, (TO*)out, (const bf16_t*)k_cache,                      \
                                                   (const bf16_t*)v_cache, row_start, seq_start, num_seqs, tables,         \
                                                   table_width, page_size, num_pages, heads, kv_heads, maps, nk, nv,       \
                                                   scale, window, keep_first, grouped, col_groups, sinks);                 \
    }
#define ASM_SIZES(VKEY, TO)                                                   \
    if (nk <= 8 && nv <= 8) ASM_ONE(8, 8, VKEY, TO, false)                    \
    else if (nk <= 16 && nv <= 16) ASM_ONE(16, 16, VKEY, TO, false)           \
    else ASM_ONE(40, 32, VKEY, TO, false)
    if (out_f32 && nk == 4 && nv == 4) ASM_ONE(4, 4, false, float, true)
    else if (out_f32 && nk == 4 && nv == 8) ASM_ONE(4, 8, false, float, true)
    else if (out_f32 && nk == 8 && nv == 8) ASM_ONE(8, 8, false, float, true)
    else if (out_f32 && nk == 8 && nv == 16) ASM_ONE(8, 16, false, float, true)
    else if (out_f32) { ASM_SIZES(false, float) } else { ASM_SIZES(false, bf16_t) }
#undef ASM_SIZES
#undef ASM_ONE
#undef ASM_ARGS
    return tli_check_launch("attention_sized_mfma");
}
