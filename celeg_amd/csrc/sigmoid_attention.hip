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
