// A block-diagonal product: B independent small products side by side on the column axis, one weight each.
//
//   C[m, b, n] = sum_k A[m, b, k] * W[b, n, k] (+ bias[b, n])  (* sigmoid(gate[m, b, n]) if a gate is given)
//
//   A    rows lda apart, block b's K numbers start a_block elements after block b - 1's
//   W    [B, N, K] contiguous;  bias [B, N] or none
//   C    rows ldc apart, block b's N results start c_block elements after block b - 1's
//   gate like C, rows ldg apart, blocks g_block apart (in A's type)
//
// It serves per-head products (a query folded into a shared latent space and back out of it) and gates made from
// a channel's own block.  Operands are float32 or bfloat16, sums are float32 fused multiply-adds in one fixed order
// of k (blocks of 256 summed, then the blocks' sums), so a row's result does not depend on the other rows; the
// result is float32 or the operands' type.  64 x 64 results per workgroup, slices of 16 k through LDS; up to 16 rows
// take a form of their own (below) whose sums have another fixed order, again the same for every row, and bfloat16
// operands of more than four rows go to the matrix cores (further below) where their addresses allow 16-byte loads.
#include "common.h"

namespace {
constexpr int TM = 64, TN = 64, TK = 16;
constexpr int kSlices = 16;

template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
block_linear_kernel(const TA* __restrict__ A, long lda, long a_block, const TA* __restrict__ W,
                    const TA* __restrict__ bias, TC* __restrict__ C, long ldc, long c_block,
                    const TA* __restrict__ gate, long ldg, long g_block, int M, int N, int K) {
    __shared__ float a_tile[TK][TM + 4];
    __shared__ float w_tile[TK][TN + 4];
    const int b = blockIdx.z;
    const int m0 = blockIdx.y * TM;
    const int n0 = blockIdx.x * TN;
    const int tx = threadIdx.x % 16;
    const int ty = threadIdx.x / 16;
    const TA* a_base = A + static_cast<size_t>(b) * a_block;
    const TA* w_base = W + static_cast<size_t>(b) * N * K;
    float acc[4][4] = {}, total[4][4] = {};
    int slice = 0;
    for (int k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int idx = threadIdx.x + 256 * r;
            const int row = idx / TK;
            const int kk = idx % TK;
            const int k = k0 + kk;
            const int m = m0 + row;
            const int n = n0 + row;
            a_tile[kk][row] = (m < M && k < K) ? to_float(a_base[static_cast<size_t>(m) * lda + k]) : 0.f;
            w_tile[kk][row] = (n < N && k < K) ? to_float(w_base[static_cast<size_t>(n) * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = a_tile[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = w_tile[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        if (++slice == kSlices) {
            slice = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    total[i][j] += acc[i][j];
                    acc[i][j] = 0.f;
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = total[i][j] + acc[i][j];
            if (bias) v += to_float(bias[static_cast<size_t>(b) * N + n]);
            if (gate) {
                const float g = to_float(gate[static_cast<size_t>(m) * ldg + static_cast<size_t>(b) * g_block + n]);
                v *= 1.0f / (1.0f + expf(-g));
            }
            C[static_cast<size_t>(m) * ldc + static_cast<size_t>(b) * c_block + n] = from_float<TC>(v);
        }
    }
}
// Up to 16 rows (a decode step): the weights are the traffic.  One wave per result column (a column's work is a chain
// of a few dependent loads and a sum across lanes, so what counts is how many columns are under way at once): its lanes
// stride over k, so a weight row is read in whole segments, the few rows of A come through the cache, and the lanes'
// shares meet in a wave-wide sum; lane m stores row m's result.
constexpr int kRowsOutputs = 4;
constexpr int kRowsMost = 16;  // rows up to which this form runs (in sets of 16)

template <typename TA, typename TC, int MR>
__global__ void __launch_bounds__(256)
block_linear_rows_kernel(const TA* __restrict__ A, long lda, long a_block, const TA* __restrict__ W,
                         const TA* __restrict__ bias, TC* __restrict__ C, long ldc, long c_block,
                         const TA* __restrict__ gate, long ldg, long g_block, int M, int N, int K) {
    const int b = blockIdx.y;
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    // (more than 16 rows: sets of 16 side by side, each reading the weights again, from the cache)
    const int m0 = blockIdx.z * 16;
    M = min(M - m0, 16);
    const TA* a_base = A + static_cast<size_t>(b) * a_block + static_cast<size_t>(m0) * lda;
    C += static_cast<size_t>(m0) * ldc;
    if (gate) gate += static_cast<size_t>(m0) * ldg;
    for (int turn = 0; turn < kRowsOutputs / 4; ++turn) {
        const int n = blockIdx.x * kRowsOutputs + turn * 4 + wave;
        if (n >= N) return;  // (a wave leaves whole)
        const TA* w_row = W + (static_cast<size_t>(b) * N + n) * K;
        float acc[MR];
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[m] = 0.f;
        for (int k = lane; k < K; k += kWave) {
            const float w = to_float(w_row[k]);
#pragma unroll
            for (int m = 0; m < MR; ++m)
                if (m < M) acc[m] = fmaf(to_float(a_base[static_cast<size_t>(m) * lda + k]), w, acc[m]);
        }
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            const float total = wave_sum(acc[m]);
            if (lane == m && m < M) {
                float v = total;
                if (bias) v += to_float(bias[static_cast<size_t>(b) * N + n]);
                if (gate) {
                    const float g = to_float(gate[static_cast<size_t>(m) * ldg + static_cast<size_t>(b) * g_block + n]);
                    v *= 1.0f / (1.0f + expf(-g));
                }
                C[static_cast<size_t>(m) * ldc + static_cast<size_t>(b) * c_block + n] = from_float<TC>(v);
            }
        }
    }
}

template <typename TA, typename TC>
int launch_rows(hipStream_t s, const void* A, long lda, long a_block, const void* W, const void* bias, void* C, long ldc,
                long c_block, const void* gate, long ldg, long g_block, int M, int N, int K, int B) {
    dim3 grid((N + kRowsOutputs - 1) / kRowsOutputs, B, (M + 15) / 16);
#define CIE_ROWS(MR)                                                                                                   \
    block_linear_rows_kernel<TA, TC, MR><<<grid, 256, 0, s>>>(                                                         \
        static_cast<const TA*>(A), lda, a_block, static_cast<const TA*>(W), static_cast<const TA*>(bias),              \
        static_cast<TC*>(C), ldc, c_block, static_cast<const TA*>(gate), ldg, g_block, M, N, K)
    if (M <= 1) CIE_ROWS(1);
    else if (M <= 2) CIE_ROWS(2);
    else if (M <= 4) CIE_ROWS(4);
    else if (M <= 8) CIE_ROWS(8);
    else CIE_ROWS(16);
#undef CIE_ROWS
    return cie_after_launch();
}
// bfloat16 operands with more than four rows: the matrix cores.  A wave owns 16 result columns and up to four tiles
// of 16 rows; a workgroup's four waves take 64 columns side by side.  Per slice of 32 k a lane loads the 8 numbers of
// its weight row (column n0 + lane % 16, k from 8 * (lane / 16)) and of its row of A in each tile as 16 bytes, which
// is the operand layout of v_mfma_f32_16x16x32_bf16 as it is; the rows of A come through the cache (the weights of a
// block are small, the four waves read the same rows).  Sums are float32 in the matrix cores' own order of k, the
// same for every row.  K, the rows' distances and the blocks' distances have to be multiples of 8.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

template <typename TC>
__global__ void __launch_bounds__(256)
block_linear_mfma_kernel(const bf16_t* __restrict__ A, long lda, long a_block, const bf16_t* __restrict__ W,
                         const bf16_t* __restrict__ bias, TC* __restrict__ C, long ldc, long c_block,
                         const bf16_t* __restrict__ gate, long ldg, long g_block, int M, int N, int K) {
    const int b = blockIdx.z;
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int n0 = (blockIdx.x * 4 + wave) * 16;
    const int m0 = blockIdx.y * 64;
    if (n0 >= N) return;  // (a wave leaves whole)
    const int tiles = min(4, (M - m0 + 15) / 16);
    const bf16_t* w_row = W + (static_cast<size_t>(b) * N + min(n0 + r, N - 1)) * K;
    const bf16_t* a_base = A + static_cast<size_t>(b) * a_block;
    const bf16_t* a_row[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) a_row[t] = a_base + static_cast<size_t>(min(m0 + t * 16 + r, M - 1)) * lda;
    floatx4_t acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    const u32x4_t nothing = {0u, 0u, 0u, 0u};
    for (int k0 = 0; k0 < K; k0 += 32) {
        // (a group of 8 past the end of K reads the last group again and counts as zeros: no load under a condition)
        const int k = k0 + g * 8;
        const int at = min(k, K - 8);
        u32x4_t wt = *reinterpret_cast<const u32x4_t*>(w_row + at);
        if (k >= K) wt = nothing;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (t < tiles) {
                u32x4_t av = *reinterpret_cast<const u32x4_t*>(a_row[t] + at);
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                                 __builtin_bit_cast(bf16x8_t, wt), acc[t], 0, 0, 0);
            }
        }
    }
    const int n = n0 + r;
    if (n >= N) return;
    const float add = bias ? to_float(bias[static_cast<size_t>(b) * N + n]) : 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + t * 16 + g * 4 + i;
            if (t < tiles && m < M) {
                float v = acc[t][i] + add;
                if (gate) {
                    const float gv = to_float(gate[static_cast<size_t>(m) * ldg + static_cast<size_t>(b) * g_block + n]);
                    v *= 1.0f / (1.0f + expf(-gv));
                }
                C[static_cast<size_t>(m) * ldc + static_cast<size_t>(b) * c_block + n] = from_float<TC>(v);
            }
        }
    }
}
}  // namespace

// dtype: type of A, W, bias and gate; out_f32: the result is float32 whatever the operands' type
CIE_API int cie_block_linear(void* stream, int dtype, int out_f32, const void* A, long lda, long a_block, const void* W,
                             const void* bias, void* C, long ldc, long c_block, const void* gate, long ldg, long g_block,
                             int M, int N, int K, int B) {
    if (M < 0 || N <= 0 || K <= 0 || B <= 0 || B > 65535 || lda < K || ldc < N) return CIE_BAD_ARGUMENT;
    if (M == 0) return CIE_OK;
    const int grid_y = (M + TM - 1) / TM;
    if (grid_y > 65535) return CIE_BAD_ARGUMENT;
    dim3 grid((N + TN - 1) / TN, grid_y, B);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool cores = dtype == CIE_BF16 && K % 8 == 0 && lda % 8 == 0 && a_block % 8 == 0 &&
                       reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0;
    // (measured at the 3B widths, a decode step of 12 layers: 8 rows 1.26 ms in the few-row form, 1.19 ms on the matrix
    // cores; one row 1.08 against 1.10)
    if (M <= kRowsMost && !(cores && M > 4)) {
        if (dtype == CIE_F32) return launch_rows<float, float>(s, A, lda, a_block, W, bias, C, ldc, c_block, gate, ldg, g_block, M, N, K, B);
        if (dtype == CIE_BF16 && out_f32) return launch_rows<bf16_t, float>(s, A, lda, a_block, W, bias, C, ldc, c_block, gate, ldg, g_block, M, N, K, B);
        if (dtype == CIE_BF16) return launch_rows<bf16_t, bf16_t>(s, A, lda, a_block, W, bias, C, ldc, c_block, gate, ldg, g_block, M, N, K, B);
        return CIE_BAD_ARGUMENT;
    }
    if (cores) {
        dim3 tiles((N + 63) / 64, grid_y, B);
        if (out_f32)
            block_linear_mfma_kernel<float><<<tiles, 256, 0, s>>>(
                static_cast<const bf16_t*>(A), lda, a_block, static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias),
                static_cast<float*>(C), ldc, c_block, static_cast<const bf16_t*>(gate), ldg, g_block, M, N, K);
        else
            block_linear_mfma_kernel<bf16_t><<<tiles, 256, 0, s>>>(
                static_cast<const bf16_t*>(A), lda, a_block, static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias),
                static_cast<bf16_t*>(C), ldc, c_block, static_cast<const bf16_t*>(gate), ldg, g_block, M, N, K);
        return cie_after_launch();
    }
    if (dtype == CIE_F32)
        block_linear_kernel<float, float><<<grid, 256, 0, s>>>(
            static_cast<const float*>(A), lda, a_block, static_cast<const float*>(W), static_cast<const float*>(bias),
            static_cast<float*>(C), ldc, c_block, static_cast<const float*>(gate), ldg, g_block, M, N, K);
    else if (dtype == CIE_BF16 && out_f32)
        block_linear_kernel<bf16_t, float><<<grid, 256, 0, s>>>(
            static_cast<const bf16_t*>(A), lda, a_block, static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias),
            static_cast<float*>(C), ldc, c_block, static_cast<const bf16_t*>(gate), ldg, g_block, M, N, K);
    else if (dtype == CIE_BF16)
        block_linear_kernel<bf16_t, bf16_t><<<grid, 256, 0, s>>>(
            static_cast<const bf16_t*>(A), lda, a_block, static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias),
            static_cast<bf16_t*>(C), ldc, c_block, static_cast<const bf16_t*>(gate), ldg, g_block, M, N, K);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
