// A routed feed-forward: every row goes to `top` of E expert feed-forwards.
//   route:   scores from the router's 32-bit logits, the `top` largest chosen per row;
//   plan:    rows sorted by expert (a row's place among its expert's rows is its order in the
//            batch), and the list of row tiles that the products walk;
//   gather:  the rows laid in that order, each times its weight if the weight goes on the input;
//   product: out[p] = a[p] w[expert of p]^T over the tiles;
//   combine: a row's `top` results summed (times the weight if it goes on the output).
// Nothing is planned on the host: grids are sized by bounds, so a recorded step replays.
#include "small_gemm.h"

#define MOE_MAX_PER_LANE 8        // experts <= 512

// ---------------------------------------------------------------- route
// One wavefront per row.  score 0: sigmoid of the logit; 1: softmax over all experts.
// The chosen experts' scores are the weights; with `renorm` they are divided by their sum.
__global__ void moe_route_kernel(const float* __restrict__ logits, int experts, int top, int score, int renorm,
                                 int* __restrict__ ids, float* __restrict__ weights) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + static_cast<size_t>(t) * experts;
    float v[MOE_MAX_PER_LANE];
    float zmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < MOE_MAX_PER_LANE; ++j) {
        const int e = lane + j * CELEG_WAVE;
        v[j] = e < experts ? z[e] : -INFINITY;
        zmax = fmaxf(zmax, v[j]);
    }
    float denom = 1.f;
    if (score == 1) {
        zmax = wave_max(zmax);
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < MOE_MAX_PER_LANE; ++j)
            if (lane + j * CELEG_WAVE < experts) s += expf(v[j] - zmax);
        denom = wave_sum(s);
    }
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        // the largest logit left, the lowest expert among equal ones
        float best = -INFINITY;
        int best_e = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < MOE_MAX_PER_LANE; ++j) {
            const int e = lane + j * CELEG_WAVE;
            if (e < experts && (v[j] > best || (v[j] == best && e < best_e))) { best = v[j]; best_e = e; }
        }
#pragma unroll
        for (int off = CELEG_WAVE / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, CELEG_WAVE);
            const int oe = __shfl_xor(best_e, off, CELEG_WAVE);
            if (ob > best || (ob == best && oe < best_e)) { best = ob; best_e = oe; }
        }
#pragma unroll
        for (int j = 0; j < MOE_MAX_PER_LANE; ++j)
            if (lane + j * CELEG_WAVE == best_e) v[j] = -INFINITY;
        const float s = score == 1 ? expf(best - zmax) / denom : 1.0f / (1.0f + expf(-best));
        total += s;
        if (lane == 0) {
            ids[static_cast<size_t>(t) * top + k] = best_e;
            weights[static_cast<size_t>(t) * top + k] = s;
        }
    }
    if (renorm && lane == 0)
        for (int k = 0; k < top; ++k) weights[static_cast<size_t>(t) * top + k] /= total;
}

// ---------------------------------------------------------------- plan
// One workgroup.  ids [n] -> offsets [E + 1], place_of [n] (entry -> place), entry_at [n] (place ->
// entry), and the tiles of `tile_rows` rows: tile_expert, tile_row0 [max_tiles], n_tiles.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ ids, int n, int experts, int tile_rows,
                                                        int* __restrict__ offsets, int* __restrict__ place_of,
                                                        int* __restrict__ entry_at, int* __restrict__ tile_expert,
                                                        int* __restrict__ tile_row0, int* __restrict__ n_tiles) {
    extern __shared__ int plan_lds[];     // counts [E], starts [E + 1]
    int* counts = plan_lds;
    int* starts = plan_lds + experts;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
    // an entry's rank among the entries of its expert, in batch order
    for (int e = wave; e < experts; e += n_waves) {
        int running = 0;
        for (int base = 0; base < n; base += CELEG_WAVE) {
            const int i = base + lane;
            const bool mine = i < n && ids[i] == e;
            const unsigned long long mask = __ballot(mine);
            if (mine) place_of[i] = running + __popcll(mask & ((1ull << lane) - 1ull));
            running += __popcll(mask);
        }
        if (lane == 0) counts[e] = running;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, tiles = 0;
        for (int e = 0; e < experts; ++e) {
            starts[e] = at;
            offsets[e] = at;
            for (int r = 0; r < counts[e]; r += tile_rows) {
                tile_expert[tiles] = e;
                tile_row0[tiles] = at + r;
                ++tiles;
            }
            at += counts[e];
        }
        starts[experts] = at;
        offsets[experts] = at;
        n_tiles[0] = tiles;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int e = ids[i];
        const int place = (e >= 0 && e < experts ? starts[e] : 0) + place_of[i];
        place_of[i] = place;
        entry_at[place] = i;
    }
}

// ---------------------------------------------------------------- gather
// a[p, :] = x[entry_at[p] / top, :] (* weight of the entry)
template <typename T>
__global__ void moe_gather_kernel(const T* __restrict__ x, const int* __restrict__ entry_at,
                                  const float* __restrict__ weights, T* __restrict__ a, int top, int width) {
    const int p = blockIdx.x;
    const int entry = entry_at[p];
    const float wgt = weights ? weights[entry] : 1.f;
    const T* src = x + static_cast<size_t>(entry / top) * width;
    T* dst = a + static_cast<size_t>(p) * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = weights ? from_float<T>(wgt * to_float(src[i])) : src[i];
}

// ---------------------------------------------------------------- product over the tiles
// w: [E, N, K]; a: [n, K]; out: [n, N].  gated: w holds, per expert, N gate rows then N up rows, and
// out = silu(a gate^T) * (a up^T) (the two sums rounded to T first, as where they are tensors).
template <typename T>
__global__ __launch_bounds__(256) void moe_product_kernel(const T* __restrict__ a, const T* __restrict__ w,
                                                          T* __restrict__ out, int N, int K, int gated,
                                                          const int* __restrict__ offsets,
                                                          const int* __restrict__ tile_expert,
                                                          const int* __restrict__ tile_row0,
                                                          const int* __restrict__ n_tiles) {
    __shared__ float as[SG_ROWS][SG_K + 1], ws[SG_COLS][SG_K + 1];
    const int tile = blockIdx.x;
    if (tile >= n_tiles[0]) return;
    const int e = tile_expert[tile], row0 = tile_row0[tile];
    const int rows_valid = min(SG_ROWS, offsets[e + 1] - row0);
    const int col0 = blockIdx.y * SG_COLS, cols_valid = min(SG_COLS, N - col0);
    const size_t per_expert = static_cast<size_t>(gated ? 2 : 1) * N * K;
    const T* we = w + static_cast<size_t>(e) * per_expert + static_cast<size_t>(col0) * K;
    SmallTileSums sums, ups;
    small_tile_product(a + static_cast<size_t>(row0) * K, K, rows_valid, we, K, cols_valid, K, as, ws, sums);
    if (gated) small_tile_product(a + static_cast<size_t>(row0) * K, K, rows_valid, we + static_cast<size_t>(N) * K, K, cols_valid, K, as, ws, ups);
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
            if (gated) {
                const float g = to_float(from_float<T>(v)), u = to_float(from_float<T>(ups.v[i][j]));
                v = (g / (1.0f + expf(-g))) * u;
            }
            out[static_cast<size_t>(row0 + r) * N + col0 + c] = from_float<T>(v);
        }
    }
}

// ---------------------------------------------------------------- combine
// out[t, :] = sum_k (weight of entry (t, k)) * y[place_of[t * top + k], :], summed in 32-bit
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, const int* __restrict__ place_of,
                                   const float* __restrict__ weights, T* __restrict__ out, int top, int width) {
    const int t = blockIdx.x;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const int entry = t * top + k;
            const float v = to_float(y[static_cast<size_t>(place_of[entry]) * width + i]);
            acc += weights ? weights[entry] * v : v;
        }
        out[static_cast<size_t>(t) * width + i] = from_float<T>(acc);
    }
}

// ---------------------------------------------------------------- entry points
extern "C" int celeg_moe_route(const float* logits, int rows, int experts, int top, int score, int renorm, int* ids,
                               float* weights, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (experts <= 0 || experts > MOE_MAX_PER_LANE * CELEG_WAVE || top <= 0 || top > experts)
        return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(moe_route_kernel, dim3(rows), dim3(CELEG_WAVE), 0, stream, logits, experts, top, score, renorm, ids,
                       weights);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_moe_tile_rows() { return SG_ROWS; }

extern "C" int celeg_moe_plan(const int* ids, int n, int experts, int* offsets, int* place_of, int* entry_at,
                              int* tile_expert, int* tile_row0, int* n_tiles, hipStream_t stream) {
    if (n <= 0) return 0;
    const size_t lds = static_cast<size_t>(2 * experts + 1) * sizeof(int);
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), lds, stream, ids, n, experts, SG_ROWS, offsets, place_of,
                       entry_at, tile_expert, tile_row0, n_tiles);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_moe_gather(const void* x, int dtype, const int* entry_at, const float* weights, void* a, int n,
                                int top, int width, hipStream_t stream) {
    if (n <= 0) return 0;
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(moe_gather_kernel<float>, dim3(n), dim3(256), 0, stream, static_cast<const float*>(x), entry_at,
                           weights, static_cast<float*>(a), top, width);
    else
        hipLaunchKernelGGL(moe_gather_kernel<bf16>, dim3(n), dim3(256), 0, stream, static_cast<const bf16*>(x), entry_at,
                           weights, static_cast<bf16*>(a), top, width);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_moe_product(const void* a, const void* w, void* out, int dtype, int N, int K, int gated,
                                 const int* offsets, const int* tile_expert, const int* tile_row0, const int* n_tiles,
                                 int max_tiles, hipStream_t stream) {
    if (max_tiles <= 0) return 0;
    dim3 grid(max_tiles, (N + SG_COLS - 1) / SG_COLS);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(moe_product_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(a),
                           static_cast<const float*>(w), static_cast<float*>(out), N, K, gated, offsets, tile_expert,
                           tile_row0, n_tiles);
    else
        hipLaunchKernelGGL(moe_product_kernel<bf16>, grid, dim3(256), 0, stream, static_cast<const bf16*>(a),
                           static_cast<const bf16*>(w), static_cast<bf16*>(out), N, K, gated, offsets, tile_expert,
                           tile_row0, n_tiles);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_moe_combine(const void* y, int dtype, const int* place_of, const float* weights, void* out, int rows,
                                 int top, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(moe_combine_kernel<float>, dim3(rows), dim3(256), 0, stream, static_cast<const float*>(y),
                           place_of, weights, static_cast<float*>(out), top, width);
    else
        hipLaunchKernelGGL(moe_combine_kernel<bf16>, dim3(rows), dim3(256), 0, stream, static_cast<const bf16*>(y), place_of,
                           weights, static_cast<bf16*>(out), top, width);
    return CELEG_LAUNCH_RESULT();
}
