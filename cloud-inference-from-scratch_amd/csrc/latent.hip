// Attention over compressed keys: what lies between the down projection and the paged attention kernels.
//
// A token's cache entry is one vector that every head shares: [turned part (R) | normed latent (C) | zeros], as wide
// as the attention kernels' head size D.  A query head is folded into the same space, [its turned part (R) | its plain
// part times the key expansion (C) | zeros], so that the kernels see one key head and as many query heads as the
// layer has, and a head's weighted sum of cache entries holds, in its latent part, what the value expansion reads.
//
// This kernel lays the rows out for the rotation-and-cache-write kernel that follows it:
//
//   proj  [tokens, ldp]: heads x [plain (P) | turned (R)] queries, then [latent (C) | turned key part (R)]
//   rows  [tokens, (heads + 2) * D]:
//     query head h : [0, R) = its turned part as projected (the next kernel turns it)   [R + C, D) = 0
//                    ([R, R + C) is filled by the block-diagonal product with the key expansion)
//     key          : [0, R) = the shared key part as projected   [R, R + C) = latent / rms(latent) * weight   rest 0
//     value        : [0, R) = 0                                  [R, R + C) = the same normed latent         rest 0
//
// The latent's mean square, the division and the weight are float32; one rounding to the activation type.
#include "common.h"

template <typename T, typename W>
__global__ void __launch_bounds__(256)
latent_rows_kernel(const T* __restrict__ proj, long ldp, const W* __restrict__ weight, T* __restrict__ rows,
                   int heads, int plain, int turned, int latent, int width, float eps) {
    __shared__ float scratch[16];
    const int token = blockIdx.x;
    const T* src = proj + static_cast<size_t>(token) * ldp;
    T* dst = rows + static_cast<size_t>(token) * (heads + 2) * width;
    const T* down = src + static_cast<size_t>(heads) * (plain + turned);
    float sum_sq = 0.f;
    for (int i = threadIdx.x; i < latent; i += blockDim.x) {
        const float c = to_float(down[i]);
        sum_sq += c * c;
    }
    const float inv = 1.0f / sqrtf(block_sum(sum_sq, scratch) / static_cast<float>(latent) + eps);
    T* key = dst + static_cast<size_t>(heads) * width;
    T* value = key + width;
    const T zero = from_float<T>(0.f);
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        T k = zero, v = zero;
        if (i < turned) {
            k = down[latent + i];
        } else if (i < turned + latent) {
            const int c = i - turned;
            k = v = from_float<T>((to_float(down[c]) * inv) * to_float(weight[c]));
        }
        key[i] = k;
        value[i] = v;
    }
    const int tail = width - turned - latent;
    for (int i = threadIdx.x; i < heads * (turned + tail); i += blockDim.x) {
        const int head = i / (turned + tail);
        const int j = i - head * (turned + tail);
        T* q = dst + static_cast<size_t>(head) * width;
        if (j < turned)
            q[j] = src[static_cast<size_t>(head) * (plain + turned) + plain + j];
        else
            q[turned + latent + (j - turned)] = zero;
    }
}

CIE_API int cie_latent_rows(void* stream, int dtype, int wdtype, const void* proj, long ldp, const void* weight,
                            void* rows, int tokens, int heads, int plain, int turned, int latent, int width, float eps) {
    if (tokens < 0 || heads <= 0 || plain <= 0 || turned < 0 || latent <= 0 || width < turned + latent || !(eps > 0.f) ||
        ldp < static_cast<long>(heads) * (plain + turned) + latent + turned)
        return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CIE_F32 && wdtype == CIE_F32)
        latent_rows_kernel<float, float><<<tokens, 256, 0, s>>>(
            static_cast<const float*>(proj), ldp, static_cast<const float*>(weight), static_cast<float*>(rows), heads, plain,
            turned, latent, width, eps);
    else if (dtype == CIE_BF16 && wdtype == CIE_BF16)
        latent_rows_kernel<bf16_t, bf16_t><<<tokens, 256, 0, s>>>(
            static_cast<const bf16_t*>(proj), ldp, static_cast<const bf16_t*>(weight), static_cast<bf16_t*>(rows), heads,
            plain, turned, latent, width, eps);
    else if (dtype == CIE_BF16 && wdtype == CIE_F32)
        latent_rows_kernel<bf16_t, float><<<tokens, 256, 0, s>>>(
            static_cast<const bf16_t*>(proj), ldp, static_cast<const float*>(weight), static_cast<bf16_t*>(rows), heads,
            plain, turned, latent, width, eps);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
