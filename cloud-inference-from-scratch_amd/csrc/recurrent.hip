// Mixers that carry a state of fixed size from token to token instead of a growing cache.  Every state lives in
// float32 rows of a state tensor, one row per request slot; a step reads the row its earlier steps left, runs its
// tokens in order and writes the row back, so a sequence may be cut into steps anywhere.
//
// 1. retention: a memory S [dim, vdim] per head that fades by a fixed factor per token,
//        S_t = decay * S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
//    q and k turned by the token's position (the first `rot` dimensions of a head, pair (i, i + rot/2)), k scaled
//    after the turn; o_t divided by its root mean square over the head and multiplied by silu(gate) (a second kernel).
// 2. a causal convolution over each channel's own last `taps` inputs, the inputs of the tokens before the step taken
//    from the state.
// 3. a gated linear recurrence per channel,
//        a = exp(c * sigmoid(r)),  S_t = a * S_(t-1) + sqrt(1 - a^2) * sigmoid(i) * u_t,   out_t = S_t * gelu(y_t),
//    with c = -8 softplus(lambda) < 0 made once per model; it also moves the convolution's state on.
//
// Sequence s of the step brings tokens q_start_loc[s] .. q_start_loc[s + 1] - 1 of the flat token axis, the first at
// position seq_start[s]; its state row is seq_slot[s].
#include "common.h"

namespace {

__device__ __forceinline__ float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ float gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ---------------------------------------------------------------------------------------------- retention
// A column of the memory never meets another column, so one workgroup takes (sequence, head, slice of up to 64
// value columns).  Thread (column v, group g) keeps rows g * DS .. g * DS + DS - 1 of column v in registers.
// Tokens go in chunks: the chunk's turned queries and keys (rows padded with zeros to groups * DS numbers, so that
// a thread reads its DS numbers as 16-byte pieces without a condition) and its values are staged in LDS as float32,
// every thread walks the chunk's tokens in order (no barrier between tokens), and the groups' shares of o_t are
// summed into a float32 buffer [tokens, heads * vdim].  The head's norm and the gate are a second, small kernel:
// they need all slices of a head.
template <typename T, int DS>
__global__ void __launch_bounds__(1024)
retention_kernel(const T* __restrict__ proj, long ldp, int q_off, int k_off, int v_off,
                 const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot,
                 const float* __restrict__ decay, float* __restrict__ state, const int* __restrict__ seq_slot,
                 const int* __restrict__ seq_start, const int* __restrict__ q_start_loc, float* __restrict__ raw,
                 int heads, int dim, int vdim, int slice, int groups, int chunk, float key_scale) {
    extern __shared__ float4 lds4[];
    float* lds = reinterpret_cast<float*>(lds4);
    const int padded = groups * DS;
    float* q_s = lds;                          // [chunk][padded]
    float* k_s = q_s + chunk * padded;         // [chunk][padded]
    float* v_s = k_s + chunk * padded;         // [chunk][slice]
    float* o_s = v_s + chunk * slice;          // [groups][chunk][slice]
    const int seq = blockIdx.x;
    const int head = blockIdx.y;
    const int v0 = blockIdx.z * slice;
    const int first = q_start_loc[seq];
    const int count = q_start_loc[seq + 1] - first;
    const int start = seq_start[seq];
    const int slot = seq_slot[seq];
    const int col = threadIdx.x % slice;
    const int grp = threadIdx.x / slice;
    const bool owner = grp < groups && v0 + col < vdim;
    const int d0 = grp * DS;
    const float fade = decay[head];
    const int half = rot / 2;
    float* mem = state + ((static_cast<size_t>(slot) * heads + head) * dim) * vdim + v0 + col;
    float S[DS];
#pragma unroll
    for (int r = 0; r < DS; ++r) S[r] = (owner && d0 + r < dim) ? mem[static_cast<size_t>(d0 + r) * vdim] : 0.f;
    for (int c0 = 0; c0 < count; c0 += chunk) {
        const int cn = min(chunk, count - c0);
        for (int idx = threadIdx.x; idx < cn * padded; idx += blockDim.x) {
            const int t = idx / padded;
            const int d = idx - t * padded;
            float qv = 0.f, kv = 0.f;
            if (d < dim) {
                const T* row = proj + static_cast<size_t>(first + c0 + t) * ldp;
                const T* qh = row + q_off + head * dim;
                const T* kh = row + k_off + head * dim;
                qv = to_float(qh[d]);
                kv = to_float(kh[d]);
                if (d < rot) {
                    const int i = d < half ? d : d - half;
                    const size_t at = static_cast<size_t>(start + c0 + t) * half + i;
                    const float c = cos_table[at], s = sin_table[at];
                    if (d < half) {
                        qv = qv * c - to_float(qh[d + half]) * s;
                        kv = kv * c - to_float(kh[d + half]) * s;
                    } else {
                        qv = qv * c + to_float(qh[i]) * s;
                        kv = kv * c + to_float(kh[i]) * s;
                    }
                }
            }
            q_s[idx] = qv;
            k_s[idx] = kv * key_scale;
        }
        for (int idx = threadIdx.x; idx < cn * slice; idx += blockDim.x) {
            const int t = idx / slice;
            const int c = idx - t * slice;
            v_s[idx] = v0 + c < vdim
                           ? to_float(proj[static_cast<size_t>(first + c0 + t) * ldp + v_off + head * vdim + v0 + c]) : 0.f;
        }
        __syncthreads();
        if (owner) {
            for (int t = 0; t < cn; ++t) {
                const float vt = v_s[t * slice + col];
                const float4* qt = reinterpret_cast<const float4*>(q_s + t * padded + d0);
                const float4* kt = reinterpret_cast<const float4*>(k_s + t * padded + d0);
                float acc = 0.f;
#pragma unroll
                for (int r = 0; r < DS / 4; ++r) {
                    const float4 k4 = kt[r], q4 = qt[r];
                    S[4 * r + 0] = fmaf(fade, S[4 * r + 0], k4.x * vt);
                    S[4 * r + 1] = fmaf(fade, S[4 * r + 1], k4.y * vt);
                    S[4 * r + 2] = fmaf(fade, S[4 * r + 2], k4.z * vt);
                    S[4 * r + 3] = fmaf(fade, S[4 * r + 3], k4.w * vt);
                    acc = fmaf(S[4 * r + 0], q4.x, acc);
                    acc = fmaf(S[4 * r + 1], q4.y, acc);
                    acc = fmaf(S[4 * r + 2], q4.z, acc);
                    acc = fmaf(S[4 * r + 3], q4.w, acc);
                }
                o_s[(grp * chunk + t) * slice + col] = acc;
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < cn * slice; idx += blockDim.x) {
            const int t = idx / slice;
            const int c = idx - t * slice;
            if (v0 + c >= vdim) continue;
            float o = 0.f;
            for (int g = 0; g < groups; ++g) o += o_s[(g * chunk + t) * slice + c];
            raw[static_cast<size_t>(first + c0 + t) * heads * vdim + head * vdim + v0 + c] = o;
        }
        __syncthreads();
    }
    if (owner)
#pragma unroll
        for (int r = 0; r < DS; ++r)
            if (d0 + r < dim) mem[static_cast<size_t>(d0 + r) * vdim] = S[r];
}

// o / sqrt(mean(o^2) over the head + eps) * silu(gate): one wave per (token, head)
template <typename T>
__global__ void __launch_bounds__(256)
retention_norm_kernel(const float* __restrict__ raw, const T* __restrict__ proj, long ldp, int g_off,
                      T* __restrict__ out, int tokens, int heads, int vdim, float eps) {
    const int item = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (item >= tokens * heads) return;  // (whole waves leave together)
    const int lane = threadIdx.x % kWave;
    const int token = item / heads;
    const int head = item - token * heads;
    const float* o = raw + static_cast<size_t>(token) * heads * vdim + head * vdim;
    float sum_sq = 0.f;
    for (int c = lane; c < vdim; c += kWave) sum_sq += o[c] * o[c];
    const float inv = 1.0f / sqrtf(wave_sum(sum_sq) / static_cast<float>(vdim) + eps);
    const T* gate = proj + static_cast<size_t>(token) * ldp + g_off + head * vdim;
    T* dst = out + static_cast<size_t>(token) * heads * vdim + head * vdim;
    for (int c = lane; c < vdim; c += kWave) {
        const float g = to_float(gate[c]);
        dst[c] = from_float<T>((o[c] * inv) * (g * sigmoidf(g)));
    }
}

template <typename T, int DS>
int launch_retention(hipStream_t s, dim3 grid, int threads, size_t lds, const void* proj, long ldp, int q_off, int k_off,
                     int v_off, const float* cos_table, const float* sin_table, int rot, const float* decay,
                     float* state, const int* seq_slot, const int* seq_start, const int* q_start_loc, float* raw, int heads,
                     int dim, int vdim, int slice, int groups, int chunk, float key_scale) {
    retention_kernel<T, DS><<<grid, threads, lds, s>>>(
        static_cast<const T*>(proj), ldp, q_off, k_off, v_off, cos_table, sin_table, rot, decay, state, seq_slot,
        seq_start, q_start_loc, raw, heads, dim, vdim, slice, groups, chunk, key_scale);
    return cie_after_launch();
}

// ---------------------------------------------------------------------------------------------- convolution
template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ x, long ldx, const T* __restrict__ taps_w, const T* __restrict__ bias,
                   const float* __restrict__ past, const int* __restrict__ seq_of_token, const int* __restrict__ seq_slot,
                   const int* __restrict__ q_start_loc, T* __restrict__ out, int channels, int taps) {
    const int token = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int seq = seq_of_token[token];
    const int first = q_start_loc[seq];
    const int t = token - first;
    const float* before = past + static_cast<size_t>(seq_slot[seq]) * max(taps - 1, 1) * channels;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int src = t - (taps - 1) + j;  // the last tap is this token's input
        const float in = src >= 0 ? to_float(x[static_cast<size_t>(first + src) * ldx + c])
                                  : before[static_cast<size_t>(taps - 1 + src) * channels + c];
        acc = fmaf(to_float(taps_w[static_cast<size_t>(c) * taps + j]), in, acc);
    }
    if (bias) acc += to_float(bias[c]);
    out[static_cast<size_t>(token) * channels + c] = from_float<T>(acc);
}

// ---------------------------------------------------------------------------------------------- gated recurrence
// S_t = a_t S_(t-1) + x_t is linear in S, so a sequence's tokens are cut into `segments` stretches that run side by
// side: thread (channel, stretch) first folds its stretch into (A, B) with S_out = A S_in + B, the stretches before
// it give its S_in (a chain of at most `segments` multiply-adds), and a second walk over the stretch makes the
// outputs.  With one stretch this is the plain walk in order.  64 channels per workgroup.
constexpr int kMaxTaps = 16;
constexpr int kMaxSegments = 16;
constexpr int kScanChannels = 64;

template <typename T>
__global__ void __launch_bounds__(kScanChannels * kMaxSegments)
gated_recurrence_kernel(const T* __restrict__ y_pre, long ldy, const T* __restrict__ x_in, long ldx,
                        const T* __restrict__ u, const float* __restrict__ gates, int block_width,
                        const float* __restrict__ rate, float* __restrict__ state, float* __restrict__ past,
                        const int* __restrict__ seq_slot, const int* __restrict__ q_start_loc, T* __restrict__ out,
                        int channels, int taps, int segments) {
    __shared__ float a_s[kMaxSegments][kScanChannels];
    __shared__ float b_s[kMaxSegments][kScanChannels];
    const int seq = blockIdx.y;
    const int lane = threadIdx.x % kScanChannels;
    const int seg = threadIdx.x / kScanChannels;
    const int c = blockIdx.x * kScanChannels + lane;
    const bool live = c < channels;
    const int first = q_start_loc[seq];
    const int count = q_start_loc[seq + 1] - first;
    const int slot = seq_slot[seq];
    const int per = (count + segments - 1) / segments;
    const int t0 = min(seg * per, count), t1 = min(t0 + per, count);
    const int block = live ? c / block_width : 0;
    const size_t r_at = static_cast<size_t>(block) * 2 * block_width + (c - block * block_width);
    const size_t i_at = r_at + block_width;
    const float coef = live ? rate[c] : 0.f;
    // a_t and x_t of one token
    auto step = [&](int t, float& a, float& x) {
        const size_t token = static_cast<size_t>(first + t);
        const float r = sigmoidf(gates[token * 2 * channels + r_at]);
        const float i = sigmoidf(gates[token * 2 * channels + i_at]);
        const float log_a = coef * r;
        a = expf(log_a);
        x = sqrtf(-expm1f(2.0f * log_a)) * (i * to_float(u[token * channels + c]));  // sqrt(1 - a^2), no cancellation
    };
    float S = live ? state[static_cast<size_t>(slot) * channels + c] : 0.f;
    if (segments > 1) {
        float A = 1.f, B = 0.f;
        if (live)
            for (int t = t0; t < t1; ++t) {
                float a, x;
                step(t, a, x);
                B = fmaf(a, B, x);
                A *= a;
            }
        a_s[seg][lane] = A;
        b_s[seg][lane] = B;
        __syncthreads();
        for (int before = 0; before < seg; ++before) S = fmaf(a_s[before][lane], S, b_s[before][lane]);
    }
    if (!live) return;
    for (int t = t0; t < t1; ++t) {
        float a, x;
        step(t, a, x);
        S = fmaf(a, S, x);
        const size_t token = static_cast<size_t>(first + t);
        out[token * channels + c] = from_float<T>(S * gelu_tanh(to_float(y_pre[token * ldy + c])));
    }
    if (seg != segments - 1) return;
    state[static_cast<size_t>(slot) * channels + c] = S;  // (the last stretch ends where the sequence ends)
    // the convolution's last taps - 1 inputs: those of this step, and behind them what the state held
    const int keep_n = taps - 1;
    if (keep_n <= 0) return;
    float* before = past + static_cast<size_t>(slot) * keep_n * channels;
    float old[kMaxTaps];
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) old[j] = j < keep_n ? before[static_cast<size_t>(j) * channels + c] : 0.f;
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) {
        if (j >= keep_n) break;
        const int src = count + j;  // index into [old (keep_n), new (count)]
        before[static_cast<size_t>(j) * channels + c] =
            src < keep_n ? old[src < kMaxTaps ? src : 0] : to_float(x_in[static_cast<size_t>(first + src - keep_n) * ldx + c]);
    }
}

}  // namespace

CIE_API int cie_retention(void* stream, int dtype, const void* proj, long ldp, int q_off, int k_off, int v_off, int g_off,
                          const float* cos_table, const float* sin_table, int rot, const float* decay, float* state,
                          const int* seq_slot, const int* seq_start, const int* q_start_loc, float* raw, void* out,
                          int tokens, int sequences, int heads, int dim, int vdim, int rows_per_thread, int groups,
                          int slice, int chunk, float eps, float key_scale) {
    if (sequences < 0 || tokens < 0 || heads <= 0 || heads > 65535 || dim <= 0 || vdim <= 0 || groups <= 0 || chunk <= 0 ||
        slice <= 0 || slice > vdim || rot < 0 || rot % 2 || rot > dim || (rot > 0 && (!cos_table || !sin_table)) ||
        !(eps > 0.f) || static_cast<long>(rows_per_thread) * groups < dim || !raw)
        return CIE_BAD_ARGUMENT;
    const int slices = (vdim + slice - 1) / slice;
    const int threads = ((slice * groups + kWave - 1) / kWave) * kWave;
    const size_t lds = sizeof(float) * static_cast<size_t>(chunk) *
                       (2 * static_cast<size_t>(groups) * rows_per_thread + slice + static_cast<size_t>(groups) * slice);
    if (threads > 1024 || lds > 64 * 1024 || slices > 65535) return CIE_BAD_ARGUMENT;
    if (sequences == 0 || tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(sequences, heads, slices);
    int code = CIE_BAD_ARGUMENT;
#define CIE_RETENTION(T, DS)                                                                                          \
    code = launch_retention<T, DS>(s, grid, threads, lds, proj, ldp, q_off, k_off, v_off, cos_table, sin_table, rot,  \
                                   decay, state, seq_slot, seq_start, q_start_loc, raw, heads, dim, vdim, slice,      \
                                   groups, chunk, key_scale)
    if (dtype == CIE_F32) {
        if (rows_per_thread == 4) CIE_RETENTION(float, 4);
        else if (rows_per_thread == 8) CIE_RETENTION(float, 8);
        else if (rows_per_thread == 16) CIE_RETENTION(float, 16);
        else if (rows_per_thread == 32) CIE_RETENTION(float, 32);
    } else if (dtype == CIE_BF16) {
        if (rows_per_thread == 4) CIE_RETENTION(bf16_t, 4);
        else if (rows_per_thread == 8) CIE_RETENTION(bf16_t, 8);
        else if (rows_per_thread == 16) CIE_RETENTION(bf16_t, 16);
        else if (rows_per_thread == 32) CIE_RETENTION(bf16_t, 32);
    }
#undef CIE_RETENTION
    if (code != CIE_OK) return code;
    const int items = tokens * heads;
    const int blocks = (items + 3) / 4;
    if (dtype == CIE_F32)
        retention_norm_kernel<float><<<blocks, 256, 0, s>>>(raw, static_cast<const float*>(proj), ldp, g_off,
                                                           static_cast<float*>(out), tokens, heads, vdim, eps);
    else
        retention_norm_kernel<bf16_t><<<blocks, 256, 0, s>>>(raw, static_cast<const bf16_t*>(proj), ldp, g_off,
                                                            static_cast<bf16_t*>(out), tokens, heads, vdim, eps);
    return cie_after_launch();
}

CIE_API int cie_causal_conv(void* stream, int dtype, const void* x, long ldx, const void* taps_w, const void* bias,
                            const float* past, const int* seq_of_token, const int* seq_slot, const int* q_start_loc,
                            void* out, int tokens, int channels, int taps) {
    if (tokens < 0 || tokens > 65535 * 1 || channels <= 0 || taps < 1 || taps > kMaxTaps || ldx < channels) return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid((channels + 255) / 256, tokens);
    if (dtype == CIE_F32)
        causal_conv_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(x), ldx, static_cast<const float*>(taps_w),
                                                      static_cast<const float*>(bias), past, seq_of_token, seq_slot,
                                                      q_start_loc, static_cast<float*>(out), channels, taps);
    else if (dtype == CIE_BF16)
        causal_conv_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(x), ldx, static_cast<const bf16_t*>(taps_w),
                                                       static_cast<const bf16_t*>(bias), past, seq_of_token, seq_slot,
                                                       q_start_loc, static_cast<bf16_t*>(out), channels, taps);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

CIE_API int cie_gated_recurrence(void* stream, int dtype, const void* y_pre, long ldy, const void* x_in, long ldx,
                                 const void* u, const float* gates, int block_width, const float* rate, float* state,
                                 float* past, const int* seq_slot, const int* q_start_loc, void* out, int sequences,
                                 int channels, int taps, int segments) {
    if (sequences < 0 || sequences > 65535 || channels <= 0 || block_width <= 0 || channels % block_width || taps < 1 ||
        taps > kMaxTaps || ldy < channels || ldx < channels || segments < 1 || segments > kMaxSegments)
        return CIE_BAD_ARGUMENT;
    if (sequences == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid((channels + kScanChannels - 1) / kScanChannels, sequences);
    const int threads = kScanChannels * segments;
    if (dtype == CIE_F32)
        gated_recurrence_kernel<float><<<grid, threads, 0, s>>>(
            static_cast<const float*>(y_pre), ldy, static_cast<const float*>(x_in), ldx, static_cast<const float*>(u), gates,
            block_width, rate, state, past, seq_slot, q_start_loc, static_cast<float*>(out), channels, taps, segments);
    else if (dtype == CIE_BF16)
        gated_recurrence_kernel<bf16_t><<<grid, threads, 0, s>>>(
            static_cast<const bf16_t*>(y_pre), ldy, static_cast<const bf16_t*>(x_in), ldx, static_cast<const bf16_t*>(u),
            gates, block_width, rate, state, past, seq_slot, q_start_loc, static_cast<bf16_t*>(out), channels, taps, segments);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
