// Attention over a latent cache.  A token leaves one row in the pages: its compressed
// key/value vector c [rank] (RMS-normed) followed by one rotated key part [rot] that all heads
// share.  A head's key is (W_uk c, rotated part) and its value W_uv c; neither is ever formed:
// the query side takes W_uk in (q_lat = (W_uk^T q_plain, q_rotated), so that a score is one
// dot product of q_lat with the cached row), the weighted sum runs over c, and W_uv is applied
// to the result.  A learned number per head (the sink) may join the softmax's denominator; it
// has no key and no value.
#include "mfma_rows.h"
#include "small_gemm.h"

__device__ __forceinline__ size_t latent_row(int page, int n_layers, int layer, int page_tokens, int in_page, int row_dim) {
    return ((static_cast<size_t>(page) * n_layers + layer) * page_tokens + in_page) * row_dim;
}

// rotation of a pair by the position's angle, 32-bit: angle = float(pos) * inv_freq[i]
__device__ __forceinline__ void turn(float& u, float& v, float angle) {
    float s, c;
    sincosf(angle, &s, &c);
    const float nu = u * c - v * s, nv = v * c + u * s;
    u = nu;
    v = nv;
}
// the two members of pair i among `rotary` rotated values: halves (i, i + rotary/2) or neighbours (2i, 2i+1)
__device__ __forceinline__ void pair_of(int i, int rotary, int pairing, int& a, int& b) {
    if (pairing) { a = 2 * i; b = 2 * i + 1; } else { a = i; b = i + rotary / 2; }
}

// ---------------------------------------------------------------- prepare
// One workgroup per row.  proj[t] holds (q | dkv | ...): q is [heads, dim + rot] at column q_off,
// dkv is [rank + rot] at column dkv_off.  The first `rank` values of dkv are RMS-normed with
// `weight` and, with the rotated last `rot` values, written to the row's place in the pages; the
// rotated part of every query head is turned in place.  The first `rotary` of the `rot` values
// turn, the rest pass unchanged.
template <typename T>
__global__ void latent_prepare_kernel(T* __restrict__ proj, int ld, int q_off, int dkv_off, int heads, int dim, int rot,
                                      int rank, const float* __restrict__ weight, float eps,
                                      const float* __restrict__ inv_freq, int rotary, int pairing,
                                      const int* __restrict__ positions, const int* __restrict__ token_slot,
                                      const int* __restrict__ table, int table_stride, T* __restrict__ pool, int n_layers,
                                      int layer, int page_tokens, int write) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const int pos = positions[t];
    const float fpos = static_cast<float>(pos);
    T* row = proj + static_cast<size_t>(t) * ld;
    const int half = rotary / 2;
    // queries: pair i of head h
    for (int j = threadIdx.x; j < heads * half; j += blockDim.x) {
        const int h = j / half, i = j - h * half;
        int a, b;
        pair_of(i, rotary, pairing, a, b);
        T* qr = row + q_off + static_cast<size_t>(h) * (dim + rot) + dim;
        float u = to_float(qr[a]), v = to_float(qr[b]);
        turn(u, v, fpos * inv_freq[i]);
        qr[a] = from_float<T>(u);
        qr[b] = from_float<T>(v);
    }
    if (!write) return;
    const T* dkv = row + dkv_off;
    float sq = 0.f;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) {
        const float x = to_float(dkv[i]);
        sq += x * x;
    }
    sq = block_sum(sq, scratch);
    const float inv = 1.0f / sqrtf(sq / static_cast<float>(rank) + eps);
    const int page = table[static_cast<size_t>(token_slot[t]) * table_stride + pos / page_tokens];
    T* dst = pool + latent_row(page, n_layers, layer, page_tokens, pos % page_tokens, rank + rot);
    for (int i = threadIdx.x; i < rank; i += blockDim.x) dst[i] = from_float<T>(to_float(dkv[i]) * inv * weight[i]);
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        int a, b;
        pair_of(i, rotary, pairing, a, b);
        float u = to_float(dkv[rank + a]), v = to_float(dkv[rank + b]);
        turn(u, v, fpos * inv_freq[i]);
        dst[rank + a] = from_float<T>(u);
        dst[rank + b] = from_float<T>(v);
    }
    for (int i = rotary + threadIdx.x; i < rot; i += blockDim.x) dst[rank + i] = dkv[rank + i];
}

// ---------------------------------------------------------------- a matrix per head
// out[t, h, n] = sum_k x[t, h, k] w[h, n, k] for n < N; then, if tail > 0, out[t, h, N + j] =
// x[t, h, K + j] (values that pass by the matrix); with gate: out *= sigmoid(gate[t, h, n]).
// x: head h of row t starts at x + t * ldx + h * x_head; out likewise with ldo and o_head.
template <typename T>
__global__ __launch_bounds__(256) void headwise_linear_kernel(const T* __restrict__ x, int ldx, int x_head,
                                                              const T* __restrict__ w, int N, int K, T* __restrict__ out,
                                                              int ldo, int o_head, int tail, const T* __restrict__ gate,
                                                              int ldg, int rows) {
    __shared__ float as[SG_ROWS][SG_K + 1], ws[SG_COLS][SG_K + 1];
    const int h = blockIdx.z;
    const int row0 = blockIdx.x * SG_ROWS, col0 = blockIdx.y * SG_COLS;
    const int rows_valid = min(SG_ROWS, rows - row0), cols_valid = min(SG_COLS, N - col0);
    const T* a = x + static_cast<size_t>(row0) * ldx + static_cast<size_t>(h) * x_head;
    SmallTileSums sums;
    small_tile_product(a, ldx, rows_valid, w + (static_cast<size_t>(h) * N + col0) * K, K, cols_valid, K, as, ws, sums);
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = ty + 16 * i;
        if (r >= rows_valid) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = tx + 16 * j;
            if (c >= cols_valid) continue;
            float v = sums.v[i][j];
            if (gate) {
                const float g = to_float(gate[static_cast<size_t>(row0 + r) * ldg + static_cast<size_t>(h) * N + col0 + c]);
                v = to_float(from_float<T>(v)) * (1.0f / (1.0f + expf(-g)));
            }
            out[static_cast<size_t>(row0 + r) * ldo + static_cast<size_t>(h) * o_head + col0 + c] = from_float<T>(v);
        }
    }
    if (tail > 0 && blockIdx.y == 0)
        for (int i = threadIdx.x; i < rows_valid * tail; i += 256) {
            const int r = i / tail, j = i - r * tail;
            out[static_cast<size_t>(row0 + r) * ldo + static_cast<size_t>(h) * o_head + N + j] =
                a[static_cast<size_t>(r) * ldx + K + j];
        }
}

// The same on the matrix cores (bfloat16; K a multiple of 32, N of 16, heads and rows 16-byte aligned).
__global__ __launch_bounds__(256) void headwise_linear_mfma_kernel(const __bf16* __restrict__ x, int ldx, int x_head,
                                                                   const __bf16* __restrict__ w, int N, int K,
                                                                   __bf16* __restrict__ out, int ldo, int o_head, int tail,
                                                                   const __bf16* __restrict__ gate, int ldg, int rows) {
    const int h = blockIdx.z, row0 = blockIdx.x * MR_ROWS;
    const int rows_valid = min(MR_ROWS, rows - row0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, qd = lane >> 4;
    const int col0 = blockIdx.y * MR_COLS + wave * 16;
    const __bf16* a = x + static_cast<size_t>(row0) * ldx + static_cast<size_t>(h) * x_head;
    if (tail > 0 && blockIdx.y == 0)
        for (int i = threadIdx.x; i < rows_valid * tail; i += 256) {
            const int r = i / tail, j = i - r * tail;
            out[static_cast<size_t>(row0 + r) * ldo + static_cast<size_t>(h) * o_head + N + j] = a[static_cast<size_t>(r) * ldx + K + j];
        }
    if (col0 >= N) return;
    const __bf16* w_row[1][1] = {{col0 + c < N ? w + (static_cast<size_t>(h) * N + col0 + c) * K : nullptr}};
    const __bf16* a_row[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) a_row[rt] = rt * 16 + c < rows_valid ? a + static_cast<size_t>(rt * 16 + c) * ldx : nullptr;
    mr_f32x4 sums[1][1][4];
    mfma_rows_product<1, 1>(a_row, (rows_valid + 15) / 16, w_row, K, sums);
    if (col0 + 4 * qd >= N) return;
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        const int r = rt * 16 + c;
        if (r >= rows_valid) continue;
        mr_bf16x4 v;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float s = sums[0][0][rt][j];
            if (gate) {
                const float g = static_cast<float>(gate[static_cast<size_t>(row0 + r) * ldg + static_cast<size_t>(h) * N + col0 + 4 * qd + j]);
                s = static_cast<float>(static_cast<__bf16>(s)) * (1.0f / (1.0f + expf(-g)));
            }
            v[j] = static_cast<__bf16>(s);
        }
        *reinterpret_cast<mr_bf16x4*>(out + static_cast<size_t>(row0 + r) * ldo + static_cast<size_t>(h) * o_head + col0 + 4 * qd) = v;
    }
}

// ---------------------------------------------------------------- attention, general form
// One wavefront per (row, head).  The row's q_lat [rank + rot] against the cached rows of its
// request at positions 0..pos, 64 keys at a time: a lane scores one key, the chunk joins a
// running (max, sum, accumulator) in 32-bit, the accumulator running over the first `rank`
// values of the cached rows.  The chunking depends on the row's own position only.
#define LAT_MAX_CHUNKS 16     // rank <= 1024

template <typename T>
__global__ void latent_attention_kernel(const T* __restrict__ q, int ldq, const T* __restrict__ pool,
                                        const int* __restrict__ table, int table_stride,
                                        const int* __restrict__ token_slot, const int* __restrict__ positions,
                                        const float* __restrict__ sink, T* __restrict__ out, int ldo, int heads, int rank,
                                        int rot, int page_tokens, int n_layers, int layer, float scale) {
    extern __shared__ float lds[];      // rank + rot floats of q, then 64 weights
    const int D = rank + rot;
    float* qs = lds;
    float* ps = lds + D;
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[t];
    const int* pages = table + static_cast<size_t>(token_slot[t]) * table_stride;
    const T* qrow = q + static_cast<size_t>(t) * ldq + static_cast<size_t>(h) * D;
    for (int d = lane; d < D; d += CELEG_WAVE) qs[d] = to_float(qrow[d]);
    __syncthreads();
    float m = -INFINITY, l = 0.f;
    float acc[LAT_MAX_CHUNKS];
#pragma unroll
    for (int j = 0; j < LAT_MAX_CHUNKS; ++j) acc[j] = 0.f;
    for (int base = 0; base <= pos; base += CELEG_WAVE) {
        const int key = base + lane;
        const bool valid = key <= pos;
        float s = -INFINITY;
        if (valid) {
            const T* kp = pool + latent_row(pages[key / page_tokens], n_layers, layer, page_tokens, key % page_tokens, D);
            float dot = 0.f;
            for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_float(kp[d]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);
        l = l * corr + wave_sum(p);
        ps[lane] = p;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < LAT_MAX_CHUNKS; ++j) acc[j] *= corr;
        const int n_keys = min(CELEG_WAVE, pos - base + 1);
        for (int kk = 0; kk < n_keys; ++kk) {
            const int key2 = base + kk;
            const T* vp = pool + latent_row(pages[key2 / page_tokens], n_layers, layer, page_tokens, key2 % page_tokens, D);
            const float pk = ps[kk];
#pragma unroll
            for (int j = 0; j < LAT_MAX_CHUNKS; ++j) {
                const int d = lane + j * CELEG_WAVE;
                if (d < rank) acc[j] = fmaf(pk, to_float(vp[d]), acc[j]);
            }
        }
        __syncthreads();
        m = m_new;
    }
    if (sink) {
        // the sink joins the denominator once, unscaled
        const float sk = sink[h];
        const float m_all = fmaxf(m, sk);
        const float corr = expf(m - m_all);
        l = l * corr + expf(sk - m_all);
#pragma unroll
        for (int j = 0; j < LAT_MAX_CHUNKS; ++j) acc[j] *= corr;
    }
    T* orow = out + static_cast<size_t>(t) * ldo + static_cast<size_t>(h) * rank;
    const float inv_l = 1.0f / l;
#pragma unroll
    for (int j = 0; j < LAT_MAX_CHUNKS; ++j) {
        const int d = lane + j * CELEG_WAVE;
        if (d < rank) orow[d] = from_float<T>(acc[j] * inv_l);
    }
}

// ---------------------------------------------------------------- entry points
extern "C" int celeg_latent_prepare(void* proj, int ld, int dtype, int q_off, int dkv_off, int heads, int dim, int rot,
                                    int rank, const float* weight, float eps, const float* inv_freq, int rotary, int pairing,
                                    const int* positions, const int* token_slot, const int* table, int table_stride,
                                    void* pool, int n_layers, int layer, int page_tokens, int write, int n_tokens,
                                    hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (rotary < 0 || rotary % 2 || rotary > rot || (rotary > 0 && !inv_freq)) return static_cast<int>(hipErrorInvalidValue);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(latent_prepare_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, static_cast<float*>(proj), ld,
                           q_off, dkv_off, heads, dim, rot, rank, weight, eps, inv_freq, rotary, pairing, positions,
                           token_slot, table, table_stride, static_cast<float*>(pool), n_layers, layer, page_tokens, write);
    else
        hipLaunchKernelGGL(latent_prepare_kernel<bf16>, dim3(n_tokens), dim3(256), 0, stream, static_cast<bf16*>(proj), ld,
                           q_off, dkv_off, heads, dim, rot, rank, weight, eps, inv_freq, rotary, pairing, positions,
                           token_slot, table, table_stride, static_cast<bf16*>(pool), n_layers, layer, page_tokens, write);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_headwise_linear(const void* x, int ldx, int x_head, const void* w, int dtype, int heads, int N, int K,
                                     void* out, int ldo, int o_head, int tail, const void* gate, int ldg, int rows,
                                     int matrix_cores, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (matrix_cores) {
        if (dtype != CELEG_BF16 || K % 32 || N % 16 || ldx % 8 || x_head % 8 || ldo % 4 || o_head % 4)
            return static_cast<int>(hipErrorInvalidValue);
        dim3 mgrid((rows + MR_ROWS - 1) / MR_ROWS, (N + MR_COLS - 1) / MR_COLS, heads);
        hipLaunchKernelGGL(headwise_linear_mfma_kernel, mgrid, dim3(256), 0, stream, static_cast<const __bf16*>(x), ldx, x_head,
                           static_cast<const __bf16*>(w), N, K, static_cast<__bf16*>(out), ldo, o_head, tail,
                           static_cast<const __bf16*>(gate), ldg, rows);
        return CELEG_LAUNCH_RESULT();
    }
    dim3 grid((rows + SG_ROWS - 1) / SG_ROWS, (N + SG_COLS - 1) / SG_COLS, heads);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(headwise_linear_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(x), ldx,
                           x_head, static_cast<const float*>(w), N, K, static_cast<float*>(out), ldo, o_head, tail,
                           static_cast<const float*>(gate), ldg, rows);
    else
        hipLaunchKernelGGL(headwise_linear_kernel<bf16>, grid, dim3(256), 0, stream, static_cast<const bf16*>(x), ldx,
                           x_head, static_cast<const bf16*>(w), N, K, static_cast<bf16*>(out), ldo, o_head, tail,
                           static_cast<const bf16*>(gate), ldg, rows);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_latent_attention(const void* q, int ldq, const void* pool, int dtype, const int* table,
                                      int table_stride, const int* token_slot, const int* positions, const float* sink,
                                      void* out, int ldo, int n_tokens, int heads, int rank, int rot, int page_tokens,
                                      int n_layers, int layer, float scale, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (rank > LAT_MAX_CHUNKS * CELEG_WAVE) return static_cast<int>(hipErrorInvalidValue);
    dim3 grid(n_tokens, heads), block(CELEG_WAVE);
    const size_t lds = static_cast<size_t>(rank + rot + CELEG_WAVE) * sizeof(float);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(latent_attention_kernel<float>, grid, block, lds, stream, static_cast<const float*>(q), ldq,
                           static_cast<const float*>(pool), table, table_stride, token_slot, positions, sink,
                           static_cast<float*>(out), ldo, heads, rank, rot, page_tokens, n_layers, layer, scale);
    else
        hipLaunchKernelGGL(latent_attention_kernel<bf16>, grid, block, lds, stream, static_cast<const bf16*>(q), ldq,
                           static_cast<const bf16*>(pool), table, table_stride, token_slot, positions, sink,
                           static_cast<bf16*>(out), ldo, heads, rank, rot, page_tokens, n_layers, layer, scale);
    return CELEG_LAUNCH_RESULT();
}
