// Attention whose weights are sigmoids, not a softmax: the weight of a visible key is
//     sigmoid((q . k) * scale * temp[h] + bias[h])
// with a temperature and a bias per query head (either may be absent), weights are not
// normalised over the keys, and the head's sum of weighted values is multiplied by
// sigmoid(gate[row, h]) if a gate is given.  Keys at positions [first, pos] of the row's
// request, first = max(0, pos - window + 1) with a window, else 0.
//
// Cache layout as in attention.hip: K [pages, layers, kv_heads, page_tokens, head_dim],
// V [pages, layers, kv_heads, head_dim, page_tokens].
//
// The general kernel: one wavefront per (row, query head), 64 keys at a time, a lane scores one
// key, all sums in 32-bit in an order that depends on the row's own position only.
#include "common.h"

namespace {

__device__ __forceinline__ size_t sa_cache_offset(int page, int n_layers, int layer, int kv_heads, int head, int page_tokens,
                                                  int in_page, int head_dim) {
    return (((static_cast<size_t>(page) * n_layers + layer) * kv_heads + head) * page_tokens + in_page) * head_dim;
}

__device__ __forceinline__ float sa_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

// 1 / (1 + 2^x) by the hardware's exponential and reciprocal (the matrix-core kernels round the weight
// to bfloat16 right after): 0 for large x, 1 for very negative x
__device__ __forceinline__ float sa_sigmoid2(float x) { return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x)); }

#define SA_MAX_DIM_CHUNKS 4  // head_dim <= 256

template <typename T>
__global__ __launch_bounds__(CELEG_WAVE) void sigmoid_attention_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int* __restrict__ table, int table_stride, const int* __restrict__ token_slot, const int* __restrict__ positions,
    const float* __restrict__ temp, const float* __restrict__ bias, const T* __restrict__ gate, int ldg, T* __restrict__ out,
    int ldo, int q_heads, int kv_heads, int head_dim, int page_tokens, int n_layers, int layer, float scale, int window) {
    extern __shared__ float lds[];  // head_dim floats of q, then 64 weights
    float* qs = lds;
    float* ps = lds + head_dim;
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int kvh = h / (q_heads / kv_heads);
    const int pos = positions[t];
    const int* pages = table + static_cast<size_t>(token_slot[t]) * table_stride;
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const float tau = temp ? temp[h] : 1.0f, beta = bias ? bias[h] : 0.0f;

    const T* qrow = q + static_cast<size_t>(t) * ldq + static_cast<size_t>(h) * head_dim;
    for (int d = lane; d < head_dim; d += CELEG_WAVE) qs[d] = to_float(qrow[d]);
    __syncthreads();

    float acc[SA_MAX_DIM_CHUNKS];
#pragma unroll
    for (int j = 0; j < SA_MAX_DIM_CHUNKS; ++j) acc[j] = 0.f;

    for (int base = first; base <= pos; base += CELEG_WAVE) {
        const int key = base + lane;
        float p = 0.f;
        if (key <= pos) {
            const T* kp = k_pool + sa_cache_offset(pages[key / page_tokens], n_layers, layer, kv_heads, kvh, page_tokens,
                                                   key % page_tokens, head_dim);
            float dot = 0.f;
            for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], to_float(kp[d]), dot);
            p = sa_sigmoid(dot * scale * tau + beta);
        }
        ps[lane] = p;
        __syncthreads();
        const int n_keys = min(CELEG_WAVE, pos - base + 1);
        for (int kk = 0; kk < n_keys; ++kk) {
            const int key2 = base + kk;
            const T* vp = v_pool + sa_cache_offset(pages[key2 / page_tokens], n_layers, layer, kv_heads, kvh, page_tokens, 0,
                                                   head_dim) + key2 % page_tokens;
            const float pk = ps[kk];
#pragma unroll
            for (int j = 0; j < SA_MAX_DIM_CHUNKS; ++j) {
                const int d = lane + j * CELEG_WAVE;
                if (d < head_dim) acc[j] = fmaf(pk, to_float(vp[static_cast<size_t>(d) * page_tokens]), acc[j]);
            }
        }
        __syncthreads();
    }
    const float g = gate ? sa_sigmoid(to_float(gate[static_cast<size_t>(t) * ldg + h])) : 1.0f;
    T* orow = out + static_cast<size_t>(t) * ldo + static_cast<size_t>(h) * head_dim;
#pragma unroll
    for (int j = 0; j < SA_MAX_DIM_CHUNKS; ++j) {
        const int d = lane + j * CELEG_WAVE;
        if (d < head_dim) orow[d] = from_float<T>(acc[j] * g);
    }
}

// ---------------------------------------------------------------- bfloat16 on the matrix cores
// One workgroup of four wavefronts (eight for heads of up to 64 values, whose staging areas fit)
// per (16 rows of one request's step, query head).  The keys
// the rows can see, from the first key of the first row's window (rounded down to 8, which stays
// inside that key's page) to the last row's position, are walked in blocks of 64, the wavefronts
// taking the blocks in turn and adding their sums at the end (a single token with a window of a
// thousand keys is then four chains of four blocks, not one of sixteen).  A block's keys [64][D]
// and values [D][64] (as the pages hold them) go through the wavefront's own part of LDS, and are
// asked for from memory while the block before is multiplied.  Scores are computed transposed (keys as the
// first operand), so a lane ends up with four neighbouring keys of one row in each of the block's
// four tiles; two tiles' weights, rounded to bfloat16, are then a lane's second operand of the
// product with the values as they are, the eight keys dealt to the instruction in the order the
// lane holds them, and the values' operand reads the same eight keys.  Sums are 32-bit; the
// order of a row's additions depends on the row's place in its 16 rows and its position only.
typedef __bf16 sa_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 sa_bf16x4 __attribute__((ext_vector_type(4)));
typedef float sa_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int sa_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int sa_u32x2 __attribute__((ext_vector_type(2)));

#define SA_WAVES 4
#define SA_KEYS 64

template <int D, int WAVES>
__global__ __launch_bounds__(WAVES * CELEG_WAVE) void sigmoid_attention_mfma_kernel(
    const bf16* __restrict__ q, int ldq, const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
    const int* __restrict__ table, int table_stride, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, int n_seqs, const float* __restrict__ temp, const float* __restrict__ bias,
    const bf16* __restrict__ gate, int ldg, bf16* __restrict__ out, int ldo, int q_heads, int kv_heads, int page_tokens,
    int n_layers, int layer, float scale, int window) {
    constexpr int KROW = D + 8, VROW = SA_KEYS + 8;      // padded rows: neighbouring rows start in different banks
    constexpr int KS = D / 32, DT = D / 16;
    extern __shared__ __attribute__((aligned(16))) unsigned char sa_lds[];
    const int wave = threadIdx.x / CELEG_WAVE, lane = threadIdx.x % CELEG_WAVE;
    __bf16* ks = reinterpret_cast<__bf16*>(sa_lds) + static_cast<size_t>(wave) * (SA_KEYS * KROW + D * VROW);
    __bf16* vs = ks + SA_KEYS * KROW;
    // which 16 rows: tiles of all requests of the step, one after the other
    int tile = blockIdx.x, s = 0, row0 = 0, n = 0;
    for (; s < n_seqs; ++s) {
        row0 = cu_seqlens[s];
        n = cu_seqlens[s + 1] - row0;
        const int tiles = (n + 15) / 16;
        if (tile < tiles) break;
        tile -= tiles;
    }
    if (s >= n_seqs) return;
    const int h = blockIdx.y, kvh = h / (q_heads / kv_heads);
    const int r = lane & 15, quad = lane >> 4;
    const int first_row = tile * 16, rows_here = min(16, n - first_row);
    const int pos0 = seq_start[s] + first_row, pos_last = pos0 + rows_here - 1;
    const int my_row = first_row + min(r, rows_here - 1);      // rows past the end repeat the last one (not stored)
    const int my_pos = seq_start[s] + my_row;
    const int* pages = table + static_cast<size_t>(seq_slot[s]) * table_stride;
    // (sigmoid(x) = 1 / (1 + 2^(-x log2 e)): the factor goes into the scale and the bias)
    const float tau2 = -1.44269504089f * scale * (temp ? temp[h] : 1.0f), beta2 = bias ? -1.44269504089f * bias[h] : 0.0f;
    // this lane's operand of q: row r, values 32 st + 8 quad .. + 8
    sa_bf16x8 qreg[KS];
    const bf16* qrow = q + static_cast<size_t>(row0 + my_row) * ldq + static_cast<size_t>(h) * D;
#pragma unroll
    for (int st = 0; st < KS; ++st) qreg[st] = __builtin_bit_cast(sa_bf16x8, *reinterpret_cast<const sa_u32x4*>(qrow + 32 * st + 8 * quad));
    sa_f32x4 oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = sa_f32x4{0.f, 0.f, 0.f, 0.f};
    const int key_first = window > 0 ? max(0, pos0 - window + 1) : 0;
    const size_t head_stride = static_cast<size_t>(page_tokens) * D;
    // (pages hold a power of two of tokens here: a key's page and place by a shift and a mask, not a division)
    const int page_shift = 31 - __builtin_clz(page_tokens), page_mask = page_tokens - 1;
    constexpr int KCH = SA_KEYS * (D / 8) / CELEG_WAVE, VCH = D * (SA_KEYS / 8) / CELEG_WAVE;   // 16-byte pieces a lane
    sa_u32x4 kpre[KCH], vpre[VCH];
    // a block's pieces from memory into registers: keys kb .. kb + 63 (those past pos_last: the last
    // one again), values with zeros past pos_last
    auto fetch = [&](int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            const int c = lane + CELEG_WAVE * i, key_in = c / (D / 8), part = c % (D / 8);
            const int key = min(kb + key_in, pos_last);
            const bf16* src = k_pool + ((static_cast<size_t>(pages[key >> page_shift]) * n_layers + layer) * kv_heads + kvh) * head_stride +
                              static_cast<size_t>((key & page_mask)) * D + 8 * part;
            kpre[i] = *reinterpret_cast<const sa_u32x4*>(src);
        }
#pragma unroll
        for (int i = 0; i < VCH; ++i) {
            const int c = lane + CELEG_WAVE * i, d = c / (SA_KEYS / 8), part = c % (SA_KEYS / 8);
            const int key = kb + 8 * part;         // eight keys that lie side by side in one page
            sa_u32x4 val = {0u, 0u, 0u, 0u};
            if (key <= pos_last) {
                const bf16* src = v_pool + ((static_cast<size_t>(pages[key >> page_shift]) * n_layers + layer) * kv_heads + kvh) * head_stride +
                                  static_cast<size_t>(d) * page_tokens + (key & page_mask);
                val = *reinterpret_cast<const sa_u32x4*>(src);
                const int live = pos_last - key + 1;       // keys of this piece that exist
                if (live < 8) {
                    if (live <= 6) val[3] = 0u; else val[3] &= 0x0000ffffu;
                    if (live <= 4) val[2] = 0u; else if (live == 5) val[2] &= 0x0000ffffu;
                    if (live <= 2) val[1] = 0u; else if (live == 3) val[1] &= 0x0000ffffu;
                    if (live == 1) val[0] &= 0x0000ffffu;
                }
            }
            vpre[i] = val;
        }
    };
    const int kb0 = (key_first & ~7) + wave * SA_KEYS;
    if (kb0 <= pos_last) fetch(kb0);
    for (int kb = kb0; kb <= pos_last; kb += WAVES * SA_KEYS) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            const int c = lane + CELEG_WAVE * i;
            *reinterpret_cast<sa_u32x4*>(ks + (c / (D / 8)) * KROW + 8 * (c % (D / 8))) = kpre[i];
        }
#pragma unroll
        for (int i = 0; i < VCH; ++i) {
            const int c = lane + CELEG_WAVE * i;
            *reinterpret_cast<sa_u32x4*>(vs + (c / (SA_KEYS / 8)) * VROW + 8 * (c % (SA_KEYS / 8))) = vpre[i];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (kb + WAVES * SA_KEYS <= pos_last) fetch(kb + WAVES * SA_KEYS);
        // scores, transposed: tile kt holds keys kb + 16 kt + 4 quad + i of row r
        sa_f32x4 sacc[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            sacc[kt] = sa_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int st = 0; st < KS; ++st) {
                const sa_bf16x8 kf = __builtin_bit_cast(sa_bf16x8, *reinterpret_cast<const sa_u32x4*>(ks + (16 * kt + r) * KROW + 32 * st + 8 * quad));
                sacc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qreg[st], sacc[kt], 0, 0, 0);
            }
        }
        // weights: sigmoid inside the row's window, nothing outside
        sa_bf16x4 w[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + 16 * kt + 4 * quad + i;
                const bool seen = key <= my_pos && (window <= 0 || key > my_pos - window);
                w[kt][i] = static_cast<__bf16>(seen ? sa_sigmoid2(fmaf(sacc[kt][i], tau2, beta2)) : 0.0f);
            }
        // output, transposed: tile dt holds values 16 dt + 4 quad + i of row r
#pragma unroll
        for (int pair = 0; pair < 2; ++pair) {
            const sa_bf16x8 pw = __builtin_shufflevector(w[2 * pair], w[2 * pair + 1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const __bf16* vrow = vs + (16 * dt + r) * VROW + 32 * pair + 4 * quad;
                const sa_u32x2 lo = *reinterpret_cast<const sa_u32x2*>(vrow), hi = *reinterpret_cast<const sa_u32x2*>(vrow + 16);
                const sa_bf16x8 vf = __builtin_bit_cast(sa_bf16x8, sa_u32x4{lo[0], lo[1], hi[0], hi[1]});
                oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pw, oacc[dt], 0, 0, 0);
            }
        }
    }
    // the wavefronts' sums meet in LDS (every wavefront's staging area is its own again after the
    // barrier), the first one adds them in the order of the wavefronts and stores
    __syncthreads();
    float* sums = reinterpret_cast<float*>(sa_lds);
    if (wave > 0) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) sums[(((wave - 1) * DT + dt) * 4 + i) * CELEG_WAVE + lane] = oacc[dt][i];
    }
    __syncthreads();
    if (wave > 0 || r >= rows_here) return;
#pragma unroll
    for (int w = 1; w < WAVES; ++w)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) oacc[dt][i] += sums[(((w - 1) * DT + dt) * 4 + i) * CELEG_WAVE + lane];
    const float g = gate ? sa_sigmoid(to_float(gate[static_cast<size_t>(row0 + my_row) * ldg + h])) : 1.0f;
    bf16* orow = out + static_cast<size_t>(row0 + my_row) * ldo + static_cast<size_t>(h) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const sa_bf16x4 o4 = {static_cast<__bf16>(oacc[dt][0] * g), static_cast<__bf16>(oacc[dt][1] * g),
                              static_cast<__bf16>(oacc[dt][2] * g), static_cast<__bf16>(oacc[dt][3] * g)};
        *reinterpret_cast<sa_bf16x4*>(orow + 16 * dt + 4 * quad) = o4;
    }
}

// The form for portions of prompts: a workgroup per (64 rows of one request's step, query head),
// 16 rows a wavefront.  The tile's key blocks are staged once for all four wavefronts, by all of
// them, into one of two buffers in turn (the next block is asked for from memory while this one
// is multiplied, and one barrier a block is enough: a buffer is written again only after every
// wavefront has passed the barrier behind the block that read it).  A wavefront leaves out the
// blocks none of its rows can see.  The arithmetic is the single-tile form's.
template <int D>
__global__ __launch_bounds__(SA_WAVES * CELEG_WAVE) void sigmoid_attention_rows_kernel(
    const bf16* __restrict__ q, int ldq, const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
    const int* __restrict__ table, int table_stride, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, int n_seqs, const float* __restrict__ temp, const float* __restrict__ bias,
    const bf16* __restrict__ gate, int ldg, bf16* __restrict__ out, int ldo, int q_heads, int kv_heads, int page_tokens,
    int n_layers, int layer, float scale, int window) {
    constexpr int KROW = D + 8, VROW = SA_KEYS + 8, KS = D / 32, DT = D / 16, BUF = SA_KEYS * KROW + D * VROW;
    constexpr int THREADS = SA_WAVES * CELEG_WAVE, KCH = SA_KEYS * (D / 8) / THREADS, VCH = D * (SA_KEYS / 8) / THREADS;
    extern __shared__ __attribute__((aligned(16))) unsigned char sa_lds[];
    __bf16* lds = reinterpret_cast<__bf16*>(sa_lds);
    const int wave = threadIdx.x / CELEG_WAVE, lane = threadIdx.x % CELEG_WAVE, tid = threadIdx.x;
    int tile = blockIdx.x, s = 0, row0 = 0, n = 0;
    for (; s < n_seqs; ++s) {
        row0 = cu_seqlens[s];
        n = cu_seqlens[s + 1] - row0;
        const int tiles = (n + 63) / 64;
        if (tile < tiles) break;
        tile -= tiles;
    }
    if (s >= n_seqs) return;
    const int h = blockIdx.y, kvh = h / (q_heads / kv_heads);
    const int r = lane & 15, quad = lane >> 4;
    const int tile_row = tile * 64, tile_rows = min(64, n - tile_row);
    const int tile_pos0 = seq_start[s] + tile_row, pos_last = tile_pos0 + tile_rows - 1;
    const int first_row = tile_row + 16 * wave, rows_here = min(16, n - first_row);      // <= 0: this wavefront only stages
    const int my_row = first_row + max(0, min(r, rows_here - 1));
    const int safe_row = min(my_row, n - 1);
    const int my_pos = seq_start[s] + safe_row;
    const int wave_pos0 = seq_start[s] + first_row, wave_last = wave_pos0 + rows_here - 1;
    const int* pages = table + static_cast<size_t>(seq_slot[s]) * table_stride;
    // (sigmoid(x) = 1 / (1 + 2^(-x log2 e)): the factor goes into the scale and the bias)
    const float tau2 = -1.44269504089f * scale * (temp ? temp[h] : 1.0f), beta2 = bias ? -1.44269504089f * bias[h] : 0.0f;
    sa_bf16x8 qreg[KS];
    const bf16* qrow = q + static_cast<size_t>(row0 + safe_row) * ldq + static_cast<size_t>(h) * D;
#pragma unroll
    for (int st = 0; st < KS; ++st) qreg[st] = __builtin_bit_cast(sa_bf16x8, *reinterpret_cast<const sa_u32x4*>(qrow + 32 * st + 8 * quad));
    sa_f32x4 oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = sa_f32x4{0.f, 0.f, 0.f, 0.f};
    const int key_first = window > 0 ? max(0, tile_pos0 - window + 1) : 0;
    const size_t head_stride = static_cast<size_t>(page_tokens) * D;
    // (pages hold a power of two of tokens here: a key's page and place by a shift and a mask, not a division)
    const int page_shift = 31 - __builtin_clz(page_tokens), page_mask = page_tokens - 1;
    sa_u32x4 kpre[KCH], vpre[VCH];
    auto fetch = [&](int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            const int c = tid + THREADS * i, key_in = c / (D / 8), part = c % (D / 8);
            const int key = min(kb + key_in, pos_last);
            const bf16* src = k_pool + ((static_cast<size_t>(pages[key >> page_shift]) * n_layers + layer) * kv_heads + kvh) * head_stride +
                              static_cast<size_t>((key & page_mask)) * D + 8 * part;
            kpre[i] = *reinterpret_cast<const sa_u32x4*>(src);
        }
#pragma unroll
        for (int i = 0; i < VCH; ++i) {
            const int c = tid + THREADS * i, d = c / (SA_KEYS / 8), part = c % (SA_KEYS / 8);
            const int key = kb + 8 * part;
            sa_u32x4 val = {0u, 0u, 0u, 0u};
            if (key <= pos_last) {
                const bf16* src = v_pool + ((static_cast<size_t>(pages[key >> page_shift]) * n_layers + layer) * kv_heads + kvh) * head_stride +
                                  static_cast<size_t>(d) * page_tokens + (key & page_mask);
                val = *reinterpret_cast<const sa_u32x4*>(src);
                const int live = pos_last - key + 1;
                if (live < 8) {
                    if (live <= 6) val[3] = 0u; else val[3] &= 0x0000ffffu;
                    if (live <= 4) val[2] = 0u; else if (live == 5) val[2] &= 0x0000ffffu;
                    if (live <= 2) val[1] = 0u; else if (live == 3) val[1] &= 0x0000ffffu;
                    if (live == 1) val[0] &= 0x0000ffffu;
                }
            }
            vpre[i] = val;
        }
    };
    const int kb0 = key_first & ~7;
    fetch(kb0);
    int turn = 0;
    for (int kb = kb0; kb <= pos_last; kb += SA_KEYS, turn ^= 1) {
        __bf16* ks = lds + turn * BUF;
        __bf16* vs = ks + SA_KEYS * KROW;
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            const int c = tid + THREADS * i;
            *reinterpret_cast<sa_u32x4*>(ks + (c / (D / 8)) * KROW + 8 * (c % (D / 8))) = kpre[i];
        }
#pragma unroll
        for (int i = 0; i < VCH; ++i) {
            const int c = tid + THREADS * i;
            *reinterpret_cast<sa_u32x4*>(vs + (c / (SA_KEYS / 8)) * VROW + 8 * (c % (SA_KEYS / 8))) = vpre[i];
        }
        __syncthreads();
        if (kb + SA_KEYS <= pos_last) fetch(kb + SA_KEYS);
        // blocks none of this wavefront's rows can see
        if (rows_here <= 0 || kb > wave_last || (window > 0 && kb + SA_KEYS - 1 < wave_pos0 - window + 1)) continue;
        sa_f32x4 sacc[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            sacc[kt] = sa_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int st = 0; st < KS; ++st) {
                const sa_bf16x8 kf = __builtin_bit_cast(sa_bf16x8, *reinterpret_cast<const sa_u32x4*>(ks + (16 * kt + r) * KROW + 32 * st + 8 * quad));
                sacc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qreg[st], sacc[kt], 0, 0, 0);
            }
        }
        sa_bf16x4 w[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + 16 * kt + 4 * quad + i;
                const bool seen = key <= my_pos && (window <= 0 || key > my_pos - window);
                w[kt][i] = static_cast<__bf16>(seen ? sa_sigmoid2(fmaf(sacc[kt][i], tau2, beta2)) : 0.0f);
            }
#pragma unroll
        for (int pair = 0; pair < 2; ++pair) {
            const sa_bf16x8 pw = __builtin_shufflevector(w[2 * pair], w[2 * pair + 1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const __bf16* vrow = vs + (16 * dt + r) * VROW + 32 * pair + 4 * quad;
                const sa_u32x2 lo = *reinterpret_cast<const sa_u32x2*>(vrow), hi = *reinterpret_cast<const sa_u32x2*>(vrow + 16);
                const sa_bf16x8 vf = __builtin_bit_cast(sa_bf16x8, sa_u32x4{lo[0], lo[1], hi[0], hi[1]});
                oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pw, oacc[dt], 0, 0, 0);
            }
        }
    }
    if (r >= rows_here) return;
    const float g = gate ? sa_sigmoid(to_float(gate[static_cast<size_t>(row0 + my_row) * ldg + h])) : 1.0f;
    bf16* orow = out + static_cast<size_t>(row0 + my_row) * ldo + static_cast<size_t>(h) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const sa_bf16x4 o4 = {static_cast<__bf16>(oacc[dt][0] * g), static_cast<__bf16>(oacc[dt][1] * g),
                              static_cast<__bf16>(oacc[dt][2] * g), static_cast<__bf16>(oacc[dt][3] * g)};
        *reinterpret_cast<sa_bf16x4*>(orow + 16 * dt + 4 * quad) = o4;
    }
}

}  // namespace

extern "C" int celeg_sigmoid_attention(const void* q, int ldq, const void* k_pool, const void* v_pool, int dtype,
                                       const int* table, int table_stride, const int* token_slot, const int* positions,
                                       const float* temp, const float* bias, const void* gate, int ldg, void* out, int ldo,
                                       int n_tokens, int q_heads, int kv_heads, int head_dim, int page_tokens, int n_layers,
                                       int layer, float scale, int window, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (head_dim > SA_MAX_DIM_CHUNKS * CELEG_WAVE || q_heads % kv_heads) return static_cast<int>(hipErrorInvalidValue);
    dim3 grid(n_tokens, q_heads), block(CELEG_WAVE);
    const size_t lds = static_cast<size_t>(head_dim + CELEG_WAVE) * sizeof(float);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(sigmoid_attention_kernel<float>, grid, block, lds, stream, static_cast<const float*>(q), ldq,
                           static_cast<const float*>(k_pool), static_cast<const float*>(v_pool), table, table_stride,
                           token_slot, positions, temp, bias, static_cast<const float*>(gate), ldg, static_cast<float*>(out),
                           ldo, q_heads, kv_heads, head_dim, page_tokens, n_layers, layer, scale, window);
    else
        hipLaunchKernelGGL(sigmoid_attention_kernel<bf16>, grid, block, lds, stream, static_cast<const bf16*>(q), ldq,
                           static_cast<const bf16*>(k_pool), static_cast<const bf16*>(v_pool), table, table_stride, token_slot,
                           positions, temp, bias, static_cast<const bf16*>(gate), ldg, static_cast<bf16*>(out), ldo, q_heads,
                           kv_heads, head_dim, page_tokens, n_layers, layer, scale, window);
    return CELEG_LAUNCH_RESULT();
}

// head sizes the matrix-core kernel takes
extern "C" int celeg_sigmoid_attention_fast_ok(int head_dim) { return head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128; }

// bfloat16 on the matrix cores; form 0: tiles of 16 rows whose key blocks the wavefronts share out
// (single tokens, short portions), form 1: tiles of 64 rows that stage a key block once for four
// wavefronts (portions of prompts); max_tiles: an upper bound on the step's tiles (sum over
// requests of ceil(rows / 16 or 64)); pages of a power of two of at least 8 tokens
extern "C" int celeg_sigmoid_attention_fast(int form, const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
                                            int table_stride, const int* cu_seqlens, const int* seq_slot, const int* seq_start,
                                            int n_seqs, int max_tiles, const float* temp, const float* bias, const void* gate,
                                            int ldg, void* out, int ldo, int q_heads, int kv_heads, int head_dim, int page_tokens,
                                            int n_layers, int layer, float scale, int window, hipStream_t stream) {
    if (max_tiles <= 0 || n_seqs <= 0) return 0;
    if (!celeg_sigmoid_attention_fast_ok(head_dim) || q_heads % kv_heads || page_tokens % 8 || (page_tokens & (page_tokens - 1)) ||
        ldq % 8 || ldo % 4)
        return static_cast<int>(hipErrorInvalidValue);
    // (single tiles: eight wavefronts share out the key blocks where their staging areas fit LDS)
    const int waves = form == 1 ? SA_WAVES : head_dim <= 64 ? 8 : SA_WAVES;
    dim3 grid(max_tiles, q_heads), block(waves * CELEG_WAVE);
    const size_t lds = static_cast<size_t>(form == 1 ? 2 : waves) * (SA_KEYS * (head_dim + 8) + head_dim * (SA_KEYS + 8)) * 2;
#define CELEG_SA_FAST(D_)                                                                                                        \
    hipLaunchKernelGGL((form == 1 ? sigmoid_attention_rows_kernel<D_> : sigmoid_attention_mfma_kernel<D_, (D_ <= 64 ? 8 : SA_WAVES)>), grid, block, lds, stream, static_cast<const bf16*>(q), ldq,               \
                       static_cast<const bf16*>(k_pool), static_cast<const bf16*>(v_pool), table, table_stride, cu_seqlens, seq_slot, \
                       seq_start, n_seqs, temp, bias, static_cast<const bf16*>(gate), ldg, static_cast<bf16*>(out), ldo, q_heads,    \
                       kv_heads, page_tokens, n_layers, layer, scale, window)
    if (head_dim == 32) CELEG_SA_FAST(32);
    else if (head_dim == 64) CELEG_SA_FAST(64);
    else if (head_dim == 96) CELEG_SA_FAST(96);
    else CELEG_SA_FAST(128);
#undef CELEG_SA_FAST
    return CELEG_LAUNCH_RESULT();
}
