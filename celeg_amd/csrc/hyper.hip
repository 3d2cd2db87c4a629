// Several residual streams ("hyper-connections"): instead of one residual vector a row keeps S
// of them, xs [rows, S, width] in 32-bit.  A sub-layer reads the mixture u = sum_s in[s] x_s,
// and its output y comes back as x_t <- sum_s mix[s, t] x_s + out[t] y, all streams at once
// from the old ones.  One kernel does, for a row: the write-back of the previous sub-layer's
// output (if one is pending), the mixture for the next sub-layer and its RMS norm.
#include "common.h"

#define HC_MAX_STREAMS 8

// xs[t, s, :] = h[t, :]
__global__ void streams_spread_kernel(const float* __restrict__ h, float* __restrict__ xs, int streams, int width) {
    const size_t t = blockIdx.x;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = h[t * width + i];
        for (int s = 0; s < streams; ++s) xs[(t * streams + s) * width + i] = v;
    }
}

// h[t, :] = sum_s xs[t, s, :]
__global__ void streams_sum_kernel(const float* __restrict__ xs, float* __restrict__ h, int streams, int width) {
    const size_t t = blockIdx.x;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float v = 0.f;
        for (int s = 0; s < streams; ++s) v += xs[(t * streams + s) * width + i];
        h[t * width + i] = v;
    }
}

// y: the pending sub-layer output [rows, width] with mix [S, S] (from, to) and out [S], or null;
// in: the next sub-layer's read weights [S], or null (then nothing is normalised);
// w: the norm's weight [width] (the factor itself), or null: the mixture leaves as it is.
template <typename TY, typename TO>
__global__ void hyper_step_kernel(float* __restrict__ xs, const TY* __restrict__ y, const float* __restrict__ mix,
                                  const float* __restrict__ out_w, const float* __restrict__ in_w,
                                  const float* __restrict__ w, float eps, TO* __restrict__ normed, int streams, int width) {
    extern __shared__ float u_row[];       // width floats
    __shared__ float scratch[16];
    __shared__ float c_mix[HC_MAX_STREAMS * HC_MAX_STREAMS], c_out[HC_MAX_STREAMS], c_in[HC_MAX_STREAMS];
    const size_t t = blockIdx.x;
    if (threadIdx.x < streams * streams && y) c_mix[threadIdx.x] = mix[threadIdx.x];
    if (threadIdx.x < streams) {
        if (y) c_out[threadIdx.x] = out_w[threadIdx.x];
        if (in_w) c_in[threadIdx.x] = in_w[threadIdx.x];
    }
    __syncthreads();
    float* row = xs + t * streams * width;
    float sq = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float x[HC_MAX_STREAMS];
#pragma unroll
        for (int s = 0; s < HC_MAX_STREAMS; ++s)
            if (s < streams) x[s] = row[static_cast<size_t>(s) * width + i];
        if (y) {
            const float yv = to_float(y[t * width + i]);
            float nx[HC_MAX_STREAMS];
#pragma unroll
            for (int to = 0; to < HC_MAX_STREAMS; ++to) {
                if (to >= streams) break;
                float acc = 0.f;
#pragma unroll
                for (int s = 0; s < HC_MAX_STREAMS; ++s)
                    if (s < streams) acc += c_mix[s * streams + to] * x[s];
                nx[to] = acc + c_out[to] * yv;
            }
#pragma unroll
            for (int s = 0; s < HC_MAX_STREAMS; ++s)
                if (s < streams) {
                    x[s] = nx[s];
                    row[static_cast<size_t>(s) * width + i] = nx[s];
                }
        }
        if (in_w) {
            float u = 0.f;
#pragma unroll
            for (int s = 0; s < HC_MAX_STREAMS; ++s)
                if (s < streams) u += c_in[s] * x[s];
            u_row[i] = u;
            sq += u * u;
        }
    }
    if (!in_w) return;
    float inv = 1.f;
    if (w) {
        sq = block_sum(sq, scratch);
        inv = 1.0f / sqrtf(sq / static_cast<float>(width) + eps);
    }
    TO* dst = normed + t * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = from_float<TO>(w ? u_row[i] * inv * w[i] : u_row[i]);
}

extern "C" int celeg_streams_spread(const float* h, float* xs, int rows, int streams, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(streams_spread_kernel, dim3(rows), dim3(256), 0, stream, h, xs, streams, width);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_streams_sum(const float* xs, float* h, int rows, int streams, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(streams_sum_kernel, dim3(rows), dim3(256), 0, stream, xs, h, streams, width);
    return CELEG_LAUNCH_RESULT();
}

template <typename TY>
static int hyper_step_out(float* xs, const TY* y, const float* mix, const float* out_w, const float* in_w, const float* w,
                          float eps, void* normed, int out_dtype, int rows, int streams, int width, hipStream_t stream) {
    const size_t lds = static_cast<size_t>(width) * sizeof(float);
    if (out_dtype == CELEG_F32)
        hipLaunchKernelGGL((hyper_step_kernel<TY, float>), dim3(rows), dim3(256), lds, stream, xs, y, mix, out_w, in_w, w, eps,
                           static_cast<float*>(normed), streams, width);
    else
        hipLaunchKernelGGL((hyper_step_kernel<TY, bf16>), dim3(rows), dim3(256), lds, stream, xs, y, mix, out_w, in_w, w, eps,
                           static_cast<bf16*>(normed), streams, width);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_hyper_step(float* xs, const void* y, int y_dtype, const float* mix, const float* out_w,
                                const float* in_w, const float* w, float eps, void* normed, int out_dtype, int rows,
                                int streams, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (streams <= 0 || streams > HC_MAX_STREAMS || width > 16384) return static_cast<int>(hipErrorInvalidValue);
    if (y_dtype == CELEG_F32)
        return hyper_step_out<float>(xs, static_cast<const float*>(y), mix, out_w, in_w, w, eps, normed, out_dtype, rows,
                                     streams, width, stream);
    return hyper_step_out<bf16>(xs, static_cast<const bf16*>(y), mix, out_w, in_w, w, eps, normed, out_dtype, rows, streams,
                                width, stream);
}
