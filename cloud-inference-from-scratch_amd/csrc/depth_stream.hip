// The float32 stream of a decoder whose layers add their branches in parallel and whose next input is a
// weighted average over the depth: one kernel per layer boundary.
//
//   v      = x + mult * (branch_a + branch_b)        (each branch optional; float32 sum)
//   history[newest] = v                              (what the layer left, before any averaging)
//   v      = sum_j weights[j] * history[j], j < terms (terms = 0: no averaging)
//   stream = v
//   out1   = v / sqrt(mean(v^2) + eps) * gain1       (RMS norms with one gain for all coordinates; each optional)
//   out2   = v / sqrt(mean(v^2) + eps) * gain2
//
// x [rows, hidden] float32; branches and outputs in the activation type; history [layers + 1, rows, hidden]
// float32.  One workgroup per row; the row passes through LDS, so hidden * 4 bytes must fit in 64 KB.
#include "common.h"

template <typename T>
__global__ void depth_stream_kernel(const float* __restrict__ x, const T* __restrict__ branch_a,
                                    const T* __restrict__ branch_b, float mult, float* __restrict__ history,
                                    long layer_stride, int newest, const float* __restrict__ weights, int terms,
                                    float* __restrict__ stream, T* __restrict__ out1, float gain1,
                                    T* __restrict__ out2, float gain2, int hidden, float eps) {
    extern __shared__ float staged[];
    __shared__ float scratch[16];
    const size_t row = static_cast<size_t>(blockIdx.x) * hidden;
    float sum_sq = 0.f;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
        float v = x[row + h];
        if (branch_a) {
            float s = to_float(branch_a[row + h]);
            if (branch_b) s += to_float(branch_b[row + h]);
            v = v + mult * s;
        }
        if (newest >= 0) history[static_cast<size_t>(newest) * layer_stride + row + h] = v;
        if (terms > 0) {
            // (the loads of the earlier layers' rows do not depend on one another: none stands behind a condition,
            // so that they travel together; the row just made comes from its register, last)
            float acc = 0.f;
            const float* past = history + row + h;
            const int own = (newest >= 0 && newest < terms) ? newest : terms;
#pragma unroll 4
            for (int j = 0; j < own; ++j) acc = fmaf(weights[j], past[static_cast<size_t>(j) * layer_stride], acc);
#pragma unroll 4
            for (int j = own + 1; j < terms; ++j) acc = fmaf(weights[j], past[static_cast<size_t>(j) * layer_stride], acc);
            if (own < terms) acc = fmaf(weights[own], v, acc);
            v = acc;
        }
        if (stream) stream[row + h] = v;
        staged[h] = v;
        sum_sq += v * v;
    }
    if (!out1 && !out2) return;
    const float total = block_sum(sum_sq, scratch);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
        const float unit = staged[h] * inv;
        if (out1) out1[row + h] = from_float<T>(unit * gain1);
        if (out2) out2[row + h] = from_float<T>(unit * gain2);
    }
}

CIE_API int cie_depth_stream(void* stream_handle, int dtype, const float* x, const void* branch_a, const void* branch_b,
                             float mult, float* history, long layer_stride, int newest, const float* weights,
                             int terms, float* stream, void* out1, float gain1, void* out2, float gain2, int rows,
                             int hidden, float eps) {
    if (rows < 0 || hidden <= 0 || hidden * sizeof(float) > 64 * 1024 || !(eps > 0.f) || terms < 0) return CIE_BAD_ARGUMENT;
    if ((newest >= 0 || terms > 0) && (!history || layer_stride < static_cast<long>(rows) * hidden)) return CIE_BAD_ARGUMENT;
    if (terms > 0 && !weights) return CIE_BAD_ARGUMENT;
    if (branch_b && !branch_a) return CIE_BAD_ARGUMENT;
    if (rows == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream_handle);
    // few rows (a decode step): a row is one workgroup's, so its width is spread over as many threads as it has
    // numbers, up to 1,024; many rows fill the GPU with smaller workgroups
    int threads = hidden >= 1024 ? 256 : 128;
    if (rows <= 128) threads = hidden >= 1024 ? 1024 : hidden >= 512 ? 512 : threads;
    if (dtype == CIE_F32)
        depth_stream_kernel<float><<<rows, threads, hidden * sizeof(float), s>>>(
            x, static_cast<const float*>(branch_a), static_cast<const float*>(branch_b), mult, history, layer_stride,
            newest, weights, terms, stream, static_cast<float*>(out1), gain1, static_cast<float*>(out2), gain2, hidden, eps);
    else if (dtype == CIE_BF16)
        depth_stream_kernel<bf16_t><<<rows, threads, hidden * sizeof(float), s>>>(
            x, static_cast<const bf16_t*>(branch_a), static_cast<const bf16_t*>(branch_b), mult, history, layer_stride,
            newest, weights, terms, stream, static_cast<bf16_t*>(out1), gain1, static_cast<bf16_t*>(out2), gain2, hidden, eps);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
