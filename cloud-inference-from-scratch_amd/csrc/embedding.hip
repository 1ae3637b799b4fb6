// Embedding gather: residual[t, :] = table[ids[t], :] * scale, widened to float32 (scale 1: as stored).
// The residual stream is float32 in both engine dtypes.  With `rows`, the same values are also written in the
// table's storage type, for a first layer whose products read the stream itself.
// With `feed` (int32 [tokens]) and `pool`: row t takes its token from pool[feed[t]] where feed[t] >= 0, so
// that a decode step can start from the tokens the step before it sampled, before the host has seen them.
#include "common.h"

template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             const int* __restrict__ feed, const int* __restrict__ pool,
                             float* __restrict__ out, T* __restrict__ rows, int hidden, int vocab, float scale) {
    const int token = blockIdx.x;
    int id = ids[token];
    if (feed != nullptr && feed[token] >= 0) id = pool[feed[token]];
    // Ids are validated on the host; clamp so that a stale padding row can never read outside.
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const T* row = table + static_cast<size_t>(id) * hidden;
    float* dst = out + static_cast<size_t>(token) * hidden;
    T* copy = rows ? rows + static_cast<size_t>(token) * hidden : nullptr;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
        const float x = to_float(row[h]) * scale;
        dst[h] = x;
        if (copy) copy[h] = from_float<T>(x);
    }
}

CIE_API int cie_embed(void* stream, int dtype, const void* table, const int* ids, const int* feed,
                      const int* pool, float* out, void* rows, int tokens, int hidden, int vocab, float scale) {
    if (tokens < 0 || hidden <= 0 || vocab <= 0 || (feed && !pool)) return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CIE_F32)
        embed_kernel<float><<<tokens, 256, 0, s>>>(static_cast<const float*>(table), ids, feed, pool, out, static_cast<float*>(rows), hidden, vocab, scale);
    else if (dtype == CIE_BF16)
        embed_kernel<bf16_t><<<tokens, 256, 0, s>>>(static_cast<const bf16_t*>(table), ids, feed, pool, out, static_cast<bf16_t*>(rows), hidden, vocab, scale);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
