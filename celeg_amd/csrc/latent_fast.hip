// Attention over a latent cache on the matrix cores (bfloat16).
//
// A cached row holds `rank` compressed values and `rot` rotated key values, D = rank + rot.  A
// score is q_lat . row over D; the weighted sum runs over the first `rank` values of the same
// rows.  A workgroup of four wavefronts brings 64 cached rows at a time into LDS, as they lie
// (sK [key][D], the operand of the scores) and, copied from there, turned over (sVt [value][key],
// the operand of the weighted sum); every wavefront owns 16 query columns.  Scores are computed
// transposed (S^T = K Q^T) with the keys of a block dealt to the accumulator registers so that a
// lane's eight registers of two score tiles are eight neighbouring keys of one query: they are
// the operand of O^T = V^T P^T as they stand, no exchange between lanes.  Softmax state (running
// maximum in the base-2 domain, sum) and the output accumulators are 32-bit.
//
// Form 0, portions of prompts: a workgroup owns 64 rows of one sequence and one head (a wavefront
// 16 of the rows), keys 0..position of its last row.  Form 1, single tokens: a workgroup owns one
// row, 16 heads (the columns of one wavefront; all four load) and one share of the row's keys;
// the shares' partial results meet in a second kernel, which also adds the sink.
#include "common.h"

typedef __bf16 lat_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 lat_bf16x4 __attribute__((ext_vector_type(4)));
typedef float lat_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int lat_u32x4 __attribute__((ext_vector_type(4)));

#define LATF_KEYS 64
#define LATF_VROW (LATF_KEYS + 8)
#define LOG2E 1.4426950408889634f

__device__ __forceinline__ float quad_max(float v) {      // over the four lanes that share a column
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    return fmaxf(v, __shfl_xor(v, 32, 64));
}
__device__ __forceinline__ float quad_sum(float v) {
    v += __shfl_xor(v, 16, 64);
    return v + __shfl_xor(v, 32, 64);
}

template <int FORM, int KSMAX, int DTMAX, int RT>
__global__ __launch_bounds__(256, (KSMAX <= 9 ? 2 : 1)) void latent_attention_mfma_kernel(
    const __bf16* __restrict__ q, int ldq, const __bf16* __restrict__ pool, const int* __restrict__ table, int table_stride,
    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot, const int* __restrict__ seq_start, int n_seqs,
    const int* __restrict__ token_slot, const int* __restrict__ positions, const float* __restrict__ sink,
    __bf16* __restrict__ out, int ldo, float* __restrict__ ws_o, float* __restrict__ ws_ml, int n_splits,
    int blocks_per_split, int heads, int rank, int rot, int page_tokens, int n_layers, int layer, float scale_log2e) {
    extern __shared__ __attribute__((aligned(16))) unsigned char latf_lds[];
    const int D = rank + rot, KS = (D + 31) / 32, Dpad = KS * 32, KROW = Dpad + 8, DT = rank / 16;
    __bf16* sK = reinterpret_cast<__bf16*>(latf_lds);                 // [64][KROW]
    __bf16* sVt = sK + LATF_KEYS * KROW;                              // [rank][LATF_VROW]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 15, qd = lane >> 4;
    constexpr int TILE = 64 * RT;          // rows of a workgroup (form 0); a wavefront owns RT tiles of 16 columns

    // ---- which columns this workgroup owns
    int slot, first_block, end_block;      // key blocks [first_block, end_block)
    int wg_limit;                          // the last key any column of the workgroup sees
    int col_row[RT], col_head, col_limit[RT];   // this lane's columns: row of q / out, head, last key seen (-1: none)
    bool wave_computes;
    if (FORM == 0) {
        int tile = blockIdx.x, s = 0, len = 0, row0 = 0;
        for (; s < n_seqs; ++s) {
            row0 = cu_seqlens[s];
            len = cu_seqlens[s + 1] - row0;
            const int tiles = len > 1 ? (len + TILE - 1) / TILE : 0;     // single tokens go to the other form
            if (tile < tiles) break;
            tile -= tiles;
        }
        if (s >= n_seqs) return;
        slot = seq_slot[s];
        const int start = seq_start[s];
        col_head = blockIdx.y;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const int r = tile * TILE + (wave * RT + rt) * 16 + c;     // row within the sequence
            col_row[rt] = row0 + min(r, len - 1);
            col_limit[rt] = r < len ? start + r : -1;
        }
        const int last = min(len, tile * TILE + TILE) - 1;
        first_block = 0;
        wg_limit = start + last;
        end_block = wg_limit / LATF_KEYS + 1;
        wave_computes = tile * TILE + wave * RT * 16 < len;
    } else {
        const int t = blockIdx.x;
        slot = token_slot[t];
        const int pos = positions[t];
        col_head = blockIdx.y * 16 + c;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            col_row[rt] = t;
            col_limit[rt] = col_head < heads ? pos : -1;
        }
        wg_limit = pos;
        first_block = blockIdx.z * blocks_per_split;
        end_block = min(pos / LATF_KEYS + 1, first_block + blocks_per_split);
        wave_computes = wave == 0;
    }
    const int* pages = table + static_cast<size_t>(slot) * table_stride;
    const size_t page_stride = static_cast<size_t>(n_layers) * page_tokens * D;
    const __bf16* layer_base = pool + static_cast<size_t>(layer) * page_tokens * D;
    // a tile's last key (blocks beyond it hold nothing for its columns) and the first key that some column does not see
    int tile_limit[RT], tile_min_limit[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        tile_limit[rt] = col_limit[rt];
        tile_min_limit[rt] = col_limit[rt] < 0 ? 0x7fffffff : col_limit[rt];
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
            tile_limit[rt] = max(tile_limit[rt], __shfl_xor(tile_limit[rt], off, 64));
            tile_min_limit[rt] = min(tile_min_limit[rt], __shfl_xor(tile_min_limit[rt], off, 64));
        }
    }

    // ---- the queries of this lane's columns, as the operand of the scores
    lat_bf16x8 qreg[RT][KSMAX];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const __bf16* qrow = q + static_cast<size_t>(col_row[rt]) * ldq + static_cast<size_t>(min(col_head, heads - 1)) * D;
#pragma unroll
        for (int st = 0; st < KSMAX; ++st) {
            lat_u32x4 v = {0u, 0u, 0u, 0u};
            const int d = st * 32 + qd * 8;
            if (st < KS && d < D && col_limit[rt] >= 0) v = *reinterpret_cast<const lat_u32x4*>(qrow + d);
            qreg[rt][st] = __builtin_bit_cast(lat_bf16x8, v);
        }
    }
    lat_f32x4 oacc[RT][DTMAX];
    float m[RT], l[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m[rt] = -INFINITY;
        l[rt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DTMAX; ++dt) oacc[rt][dt] = lat_f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const int chunks = Dpad / 8;          // 16-byte pieces of a padded row
    const int page_shift = 31 - __clz(page_tokens);     // page_tokens is a power of two

    // this thread's pieces of a block (piece j is piece tid + 256 j of the block's 64 x chunks): the same in every block
    int piece_key[KSMAX], piece_ch[KSMAX];
#pragma unroll
    for (int j = 0; j < KSMAX; ++j) {
        const int i = tid + 256 * j;
        piece_key[j] = i / chunks;
        piece_ch[j] = i - piece_key[j] * chunks;
    }
    __shared__ int s_page[LATF_KEYS];
    for (int blk = first_block; blk < end_block; ++blk) {
        const int kb = blk * LATF_KEYS;
        // ---- 64 cached rows into sK (zeros beyond D and beyond the last key any column sees: pages there may not be the
        // request's): first the rows' pages, then every piece asked for before the first is stored.  (Asking for them a
        // block ahead was measured slower: the registers it holds leave room for one workgroup a compute unit, not two.)
        __syncthreads();
        if (tid < LATF_KEYS) {
            const int pos = kb + tid;
            s_page[tid] = pos <= wg_limit ? pages[pos >> page_shift] : -1;
        }
        __syncthreads();
        {
            lat_u32x4 staged[KSMAX];
#pragma unroll
            for (int j = 0; j < KSMAX; ++j) {
                staged[j] = lat_u32x4{0u, 0u, 0u, 0u};
                if (j < KS) {
                    const int page = s_page[piece_key[j]];
                    if (page >= 0 && piece_ch[j] * 8 < D)
                        staged[j] = *reinterpret_cast<const lat_u32x4*>(
                            layer_base + static_cast<size_t>(page) * page_stride +
                            static_cast<size_t>((kb + piece_key[j]) & (page_tokens - 1)) * D + piece_ch[j] * 8);
                }
            }
#pragma unroll
            for (int j = 0; j < KSMAX; ++j)
                if (j < KS) *reinterpret_cast<lat_u32x4*>(sK + piece_key[j] * KROW + piece_ch[j] * 8) = staged[j];
        }
        __syncthreads();
        // ---- the first `rank` values of every row, turned over, into sVt: a thread takes 8 values of two
        // neighbouring keys and stores them as 8 pairs
#pragma unroll
        for (int j = 0; j < DTMAX / 4; ++j) {
            const int i = tid + 256 * j;
            if (i < (LATF_KEYS / 2) * (rank / 8)) {
                const int pair = i & (LATF_KEYS / 2 - 1), ch = i >> 5;
                const lat_bf16x8 v0 = *reinterpret_cast<const lat_bf16x8*>(sK + (2 * pair) * KROW + ch * 8);
                const lat_bf16x8 v1 = *reinterpret_cast<const lat_bf16x8*>(sK + (2 * pair + 1) * KROW + ch * 8);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    typedef __bf16 lat_bf16x2 __attribute__((ext_vector_type(2)));
                    *reinterpret_cast<lat_bf16x2*>(sVt + (ch * 8 + e) * LATF_VROW + 2 * pair) = lat_bf16x2{v0[e], v1[e]};
                }
            }
        }
        __syncthreads();
        if (!wave_computes) continue;
        // ---- scores, transposed: register r of lane quad qd, tile kt, is key 32 (kt / 2) + 8 qd + 4 (kt % 2) + r
        lat_f32x4 sacc[RT][4];
        bool live[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            live[rt] = kb <= tile_limit[rt];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) sacc[rt][kt] = lat_f32x4{0.f, 0.f, 0.f, 0.f};
        }
        if (!live[0] && !live[RT - 1]) continue;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            const int key = 32 * (kt >> 1) + 8 * (c >> 2) + 4 * (kt & 1) + (c & 3);
            const __bf16* kp = sK + key * KROW + qd * 8;
#pragma unroll
            for (int st = 0; st < KSMAX; ++st)
                if (st < KS) {
                    const lat_bf16x8 kf = *reinterpret_cast<const lat_bf16x8*>(kp + st * 32);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        if (live[rt]) sacc[rt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qreg[rt][st], sacc[rt][kt], 0, 0, 0);
                }
        }
        lat_bf16x8 pb[RT][2];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            if (kb + LATF_KEYS - 1 > tile_min_limit[rt]) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (kb + 32 * (kt >> 1) + 8 * qd + 4 * (kt & 1) + r > col_limit[rt]) sacc[rt][kt][r] = -INFINITY;
            }
            float mx = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) mx = fmaxf(mx, sacc[rt][kt][r]);
            mx = quad_max(mx) * scale_log2e;          // the scale is positive
            const float m_new = fmaxf(m[rt], mx);
            const float alpha = __builtin_amdgcn_exp2f(m[rt] - (m_new == -INFINITY ? 0.f : m_new));
            l[rt] *= alpha;
            m[rt] = m_new;
#pragma unroll
            for (int dt = 0; dt < DTMAX; ++dt)
                if (dt < DT) oacc[rt][dt] *= alpha;
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            float psum = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(sacc[rt][kt][r], scale_log2e, -m_use));
                    sacc[rt][kt][r] = p;
                    psum += p;
                }
            l[rt] += psum;
#pragma unroll
            for (int kp = 0; kp < 2; ++kp)
                pb[rt][kp] = lat_bf16x8{static_cast<__bf16>(sacc[rt][2 * kp][0]),     static_cast<__bf16>(sacc[rt][2 * kp][1]),
                                        static_cast<__bf16>(sacc[rt][2 * kp][2]),     static_cast<__bf16>(sacc[rt][2 * kp][3]),
                                        static_cast<__bf16>(sacc[rt][2 * kp + 1][0]), static_cast<__bf16>(sacc[rt][2 * kp + 1][1]),
                                        static_cast<__bf16>(sacc[rt][2 * kp + 1][2]), static_cast<__bf16>(sacc[rt][2 * kp + 1][3])};
        }
        // ---- O^T += V^T P^T
#pragma unroll
        for (int dt = 0; dt < DTMAX; ++dt)
            if (dt < DT) {
#pragma unroll
                for (int kp = 0; kp < 2; ++kp) {
                    const lat_bf16x8 vf = *reinterpret_cast<const lat_bf16x8*>(sVt + (dt * 16 + c) * LATF_VROW + 32 * kp + 8 * qd);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        if (live[rt]) oacc[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[rt][kp], oacc[rt][dt], 0, 0, 0);
                }
            }
    }
    if (!wave_computes) return;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (col_limit[rt] < 0) continue;
        float l_all = quad_sum(l[rt]);
        if (FORM == 0) {
            float corr = 1.f;
            if (sink) {
                const float sk = sink[col_head] * LOG2E;
                const float m_all = fmaxf(m[rt], sk);
                corr = exp2f(m[rt] - m_all);
                l_all = l_all * corr + exp2f(sk - m_all);
            }
            const float f = corr / l_all;
            __bf16* orow = out + static_cast<size_t>(col_row[rt]) * ldo + static_cast<size_t>(col_head) * rank + qd * 4;
#pragma unroll
            for (int dt = 0; dt < DTMAX; ++dt)
                if (dt < DT)
                    *reinterpret_cast<lat_bf16x4*>(orow + dt * 16) =
                        lat_bf16x4{static_cast<__bf16>(oacc[rt][dt][0] * f), static_cast<__bf16>(oacc[rt][dt][1] * f),
                                   static_cast<__bf16>(oacc[rt][dt][2] * f), static_cast<__bf16>(oacc[rt][dt][3] * f)};
        } else {
            const size_t part = (static_cast<size_t>(col_row[rt]) * heads + col_head) * n_splits + blockIdx.z;
            float* o = ws_o + part * rank + qd * 4;
#pragma unroll
            for (int dt = 0; dt < DTMAX; ++dt)
                if (dt < DT) *reinterpret_cast<lat_f32x4*>(o + dt * 16) = oacc[rt][dt];
            if (qd == 0) {
                ws_ml[part * 2] = m[rt];
                ws_ml[part * 2 + 1] = l_all;
            }
        }
    }
}

// The shares of a single token's keys meet: out = sum_i o_i 2^(m_i - M) / (sum_i l_i 2^(m_i - M) + 2^(sink - M)).
#define LATF_MAX_SPLITS 64
__global__ void latent_attention_join_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml, int n_splits,
                                             const float* __restrict__ sink, __bf16* __restrict__ out, int ldo, int heads,
                                             int rank) {
    __shared__ float factor[LATF_MAX_SPLITS];
    __shared__ float inv_total;
    const int t = blockIdx.x, h = blockIdx.y;
    const size_t part0 = (static_cast<size_t>(t) * heads + h) * n_splits;
    if (threadIdx.x < CELEG_WAVE) {
        const int i = threadIdx.x;
        const float mi = i < n_splits ? ws_ml[(part0 + i) * 2] : -INFINITY;
        const float sk = sink ? sink[h] * LOG2E : -INFINITY;
        const float M = fmaxf(wave_max(mi), sk);
        const float f = mi == -INFINITY ? 0.f : exp2f(mi - M);
        const float L = wave_sum(i < n_splits ? ws_ml[(part0 + i) * 2 + 1] * f : 0.f) + (sink ? exp2f(sk - M) : 0.f);
        if (i < n_splits) factor[i] = f;
        if (i == 0) inv_total = 1.0f / L;
    }
    __syncthreads();
    for (int d = threadIdx.x; d < rank; d += blockDim.x) {
        float acc = 0.f;
        for (int i = 0; i < n_splits; ++i) acc = fmaf(ws_o[(part0 + i) * rank + d], factor[i], acc);
        out[static_cast<size_t>(t) * ldo + static_cast<size_t>(h) * rank + d] = static_cast<__bf16>(acc * inv_total);
    }
}

template <int FORM, int KSMAX, int DTMAX, int RT>
static int latent_mfma_launch(dim3 grid, size_t lds, hipStream_t stream, const void* q, int ldq, const void* pool,
                              const int* table, int table_stride, const int* cu_seqlens, const int* seq_slot,
                              const int* seq_start, int n_seqs, const int* token_slot, const int* positions,
                              const float* sink, void* out, int ldo, float* ws_o, float* ws_ml, int n_splits,
                              int blocks_per_split, int heads, int rank, int rot, int page_tokens, int n_layers, int layer,
                              float scale_log2e) {
    auto kernel = latent_attention_mfma_kernel<FORM, KSMAX, DTMAX, RT>;
    if (lds > 64 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 static_cast<int>(lds));
        if (e != hipSuccess) return static_cast<int>(e);
    }
    hipLaunchKernelGGL(kernel, grid, dim3(256), lds, stream, static_cast<const __bf16*>(q), ldq,
                       static_cast<const __bf16*>(pool), table, table_stride, cu_seqlens, seq_slot, seq_start, n_seqs,
                       token_slot, positions, sink, static_cast<__bf16*>(out), ldo, ws_o, ws_ml, n_splits, blocks_per_split,
                       heads, rank, rot, page_tokens, n_layers, layer, scale_log2e);
    return CELEG_LAUNCH_RESULT();
}

// rank a multiple of 16 up to 512, rank + rot a multiple of 8 up to 576
// rows of a workgroup's tile in form 0
extern "C" int celeg_latent_attention_tile_rows(int rank, int rot) {
    (void)rank;
    (void)rot;
    return 64;        // one tile of 16 columns a wavefront (two were measured slower: half the workgroups, and no more overlap)
}

extern "C" int celeg_latent_attention_fast_ok(int rank, int rot) {
    return rank > 0 && rank % 16 == 0 && rank <= 512 && rot >= 0 && (rank + rot) % 8 == 0 && rank + rot <= 576;
}

// form 0: rows of the sequences of more than one token (max_tiles: a bound on their tiles of 64 rows);
// form 1: rows [0, n_single), each one token of its request, keys in n_splits shares of blocks_per_split
// blocks of 64; ws_o [n_single, heads, n_splits, rank] and ws_ml [n_single, heads, n_splits, 2] 32-bit.
extern "C" int celeg_latent_attention_fast(int form, const void* q, int ldq, const void* pool, const int* table,
                                           int table_stride, const int* cu_seqlens, const int* seq_slot,
                                           const int* seq_start, int n_seqs, int max_tiles, const int* token_slot,
                                           const int* positions, int n_single, const float* sink, void* out, int ldo,
                                           float* ws_o, float* ws_ml, int n_splits, int blocks_per_split, int heads,
                                           int rank, int rot, int page_tokens, int n_layers, int layer, float scale,
                                           hipStream_t stream) {
    if (!celeg_latent_attention_fast_ok(rank, rot) || (form == 1 && n_splits > LATF_MAX_SPLITS) || page_tokens <= 0 ||
        (page_tokens & (page_tokens - 1)))
        return static_cast<int>(hipErrorInvalidValue);
    const int D = rank + rot, KS = (D + 31) / 32, DT = rank / 16;
    const size_t lds = (static_cast<size_t>(LATF_KEYS) * (KS * 32 + 8) + static_cast<size_t>(rank) * LATF_VROW) * 2;
    const float scale_log2e = scale * LOG2E;
    if (form == 0 ? max_tiles <= 0 : n_single <= 0) return 0;
    const dim3 grid = form == 0 ? dim3(max_tiles, heads) : dim3(n_single, (heads + 15) / 16, n_splits);
#define LATF_GO(FORM, KSM, DTM, RT)                                                                                            \
    return latent_mfma_launch<FORM, KSM, DTM, RT>(grid, lds, stream, q, ldq, pool, table, table_stride, cu_seqlens, seq_slot,  \
                                              seq_start, n_seqs, token_slot, positions, sink, out, ldo, ws_o, ws_ml,       \
                                              n_splits, blocks_per_split, heads, rank, rot, page_tokens, n_layers, layer,  \
                                              scale_log2e)
    if (form == 0) {
        if (KS <= 5 && DT <= 8) LATF_GO(0, 5, 8, 1);
        if (KS <= 9 && DT <= 16) LATF_GO(0, 9, 16, 1);
        LATF_GO(0, 18, 32, 1);
    }
    int rc;
    if (KS <= 5 && DT <= 8)
        rc = latent_mfma_launch<1, 5, 8, 1>(grid, lds, stream, q, ldq, pool, table, table_stride, cu_seqlens, seq_slot, seq_start,
                                         n_seqs, token_slot, positions, sink, out, ldo, ws_o, ws_ml, n_splits, blocks_per_split,
                                         heads, rank, rot, page_tokens, n_layers, layer, scale_log2e);
    else if (KS <= 9 && DT <= 16)
        rc = latent_mfma_launch<1, 9, 16, 1>(grid, lds, stream, q, ldq, pool, table, table_stride, cu_seqlens, seq_slot, seq_start,
                                          n_seqs, token_slot, positions, sink, out, ldo, ws_o, ws_ml, n_splits, blocks_per_split,
                                          heads, rank, rot, page_tokens, n_layers, layer, scale_log2e);
    else
        rc = latent_mfma_launch<1, 18, 32, 1>(grid, lds, stream, q, ldq, pool, table, table_stride, cu_seqlens, seq_slot,
                                           seq_start, n_seqs, token_slot, positions, sink, out, ldo, ws_o, ws_ml, n_splits,
                                           blocks_per_split, heads, rank, rot, page_tokens, n_layers, layer, scale_log2e);
    if (rc) return rc;
    hipLaunchKernelGGL(latent_attention_join_kernel, dim3(n_single, heads), dim3(128), 0, stream, ws_o, ws_ml, n_splits, sink,
                       static_cast<__bf16*>(out), ldo, heads, rank);
    return CELEG_LAUNCH_RESULT();
#undef LATF_GO
}
