// A selective state-space mixer (the recurrence of Mamba-2) on a flat batch of segments: the short
// causal convolution with its carried inputs, the recurrence with its carried state, and the gated
// norm in groups behind it.  A segment is the next tokens of one request; what a request carries from
// step to step lies in one float32 row of `state` per request (row state_slots[segment]):
//   [heads, N, P] the recurrence's state S, then [taps - 1, channels] the convolution's last inputs
//   (the oldest first).
// A fresh request's row is all zeros, which is both "S starts at zero" and "zeros before the start".
// Everything that enters the recurrence is float32: step sizes, decays, the state, the sums.
#include "common.h"

// ---- convolution: out[t, c] = silu(bias[c] + sum_k w[c, k] * in[t - (taps - 1) + k, c]), the inputs
// before the segment's first token taken from the carried rows.  in is a band of a wider row. ----
template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ in, long long in_stride, const float* __restrict__ weight,
                   const float* __restrict__ bias, const float* __restrict__ state, long long state_stride,
                   long long carried_offset, const int* __restrict__ token_segment, const int* __restrict__ seg_q_start,
                   const int* __restrict__ state_slots, T* __restrict__ out, int channels, int taps) {
    const int token = blockIdx.x;
    const int seg = token_segment[token];
    const int local = token - seg_q_start[seg];
    const float* carried = state + static_cast<size_t>(state_slots[seg]) * state_stride + carried_offset;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
        float acc = bias[c];
        for (int k = 0; k < taps; ++k) {
            const int src = local - (taps - 1) + k;          // place in the segment; negative: a carried input
            const float v = src >= 0 ? to_float(in[static_cast<size_t>(token - local + src) * in_stride + c])
                                     : carried[static_cast<size_t>(taps - 1 + src) * channels + c];
            acc = fmaf(weight[static_cast<size_t>(c) * taps + k], v, acc);
        }
        out[static_cast<size_t>(token) * channels + c] = from_float<T>(acc / (1.f + expf(-acc)));
    }
}

// ---- after the convolution of a step: the carried rows take the segment's last taps - 1 inputs (of
// a segment shorter than that, the carried rows move up).  Row j's new value comes from a row above
// it or from the step's inputs, so a thread that walks j upwards never reads what it wrote. ----
template <typename T>
__global__ void __launch_bounds__(256)
conv_carry_kernel(const T* __restrict__ in, long long in_stride, float* __restrict__ state, long long state_stride,
                  long long carried_offset, const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                  const int* __restrict__ state_slots, int channels, int taps) {
    const int seg = blockIdx.x;
    const int q_len = seg_q_len[seg], q_start = seg_q_start[seg];
    if (q_len <= 0) return;
    float* carried = state + static_cast<size_t>(state_slots[seg]) * state_stride + carried_offset;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
        for (int j = 0; j < taps - 1; ++j) {
            const int src = q_len - (taps - 1) + j;
            carried[static_cast<size_t>(j) * channels + c] =
                src >= 0 ? to_float(in[static_cast<size_t>(q_start + src) * in_stride + c])
                         : carried[static_cast<size_t>(j + q_len) * channels + c];
        }
    }
}

WLLM_API int wllm_causal_conv(const void* in, long long in_stride, const float* weight, const float* bias, float* state,
                              long long state_stride, long long carried_offset, const int* token_segment,
                              const int* seg_q_start, const int* seg_q_len, const int* state_slots, void* out,
                              int is_bf16, int tokens, int segments, int channels, int taps, hipStream_t stream) {
    if (tokens <= 0 || segments <= 0) return 0;
    if (channels <= 0 || taps < 1 || taps > 64) return -1;
    const int tiles = (channels + 255) / 256 < 64 ? (channels + 255) / 256 : 64;
    const dim3 grid(tokens, tiles), carry_grid(segments, tiles);
    if (is_bf16)
        causal_conv_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(in), in_stride, weight, bias, state,
                                                           state_stride, carried_offset, token_segment, seg_q_start,
                                                           state_slots, static_cast<bf16*>(out), channels, taps);
    else
        causal_conv_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(in), in_stride, weight, bias, state,
                                                            state_stride, carried_offset, token_segment, seg_q_start,
                                                            state_slots, static_cast<float*>(out), channels, taps);
    if (const int err = launch_status()) return err;
    if (taps == 1) return 0;
    if (is_bf16)
        conv_carry_kernel<bf16><<<carry_grid, 256, 0, stream>>>(static_cast<const bf16*>(in), in_stride, state, state_stride,
                                                                carried_offset, seg_q_start, seg_q_len, state_slots, channels,
                                                                taps);
    else
        conv_carry_kernel<float><<<carry_grid, 256, 0, stream>>>(static_cast<const float*>(in), in_stride, state,
                                                                 state_stride, carried_offset, seg_q_start, seg_q_len,
                                                                 state_slots, channels, taps);
    return launch_status();
}

// ---- the recurrence.  Per head h (group g = h / (heads / groups)), token by token:
//   dt = softplus(dt_in + dt_bias[h]);  S = exp(-exp(A_log[h]) * dt) * S + dt * B_t x_t^T;  y_t = S^T C_t + D[h] x_t
// with S [N, P], B_t and C_t [N] of the group, x_t [P] of the head.  xbc [tokens, heads*P + 2*groups*N]
// holds x, then B, then C.  A workgroup owns (head, segment, 64 columns of P) and walks the segment's
// tokens in order; lane = column p, the four wavefronts split N, each keeping its rows of S in
// registers (R a wavefront).  Tokens are staged 16 at a time through shared memory; a token's y is
// the wavefronts' partial sums added in wavefront order, so it has the same bits whether the token
// came alone or inside a prompt. ----
constexpr int kScanTokens = 16;
constexpr int kScanWaves = 4;

__device__ __forceinline__ float softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

template <typename T, int R>
__global__ void __launch_bounds__(kWave * kScanWaves)
ssm_scan_kernel(const T* __restrict__ xbc, const T* __restrict__ dt_in, long long dt_stride,
                const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
                float* __restrict__ state, long long state_stride, const int* __restrict__ seg_q_start,
                const int* __restrict__ seg_q_len, const int* __restrict__ state_slots, float* __restrict__ y, int heads,
                int groups, int n_state, int p_dim) {
    extern __shared__ float smem[];
    const int h = blockIdx.x, seg = blockIdx.y, p0 = blockIdx.z * kWave;
    const int q_len = seg_q_len[seg], q_start = seg_q_start[seg];
    if (q_len <= 0) return;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int p = p0 + lane;
    const bool live = p < p_dim;
    const int g = h / (heads / groups);
    const int inner = heads * p_dim, channels = inner + 2 * groups * n_state;
    const int b_col = inner + g * n_state, c_col = inner + groups * n_state + g * n_state;
    float* b_s = smem;                                   // [kScanTokens][n_state]
    float* c_s = b_s + kScanTokens * n_state;            // [kScanTokens][n_state]
    float* x_s = c_s + kScanTokens * n_state;            // [kScanTokens][kWave]
    float* dt_s = x_s + kScanTokens * kWave;             // [kScanTokens]
    float* decay_s = dt_s + kScanTokens;                 // [kScanTokens]
    float* part_s = decay_s + kScanTokens;               // [kScanTokens][kScanWaves][kWave]
    float* s_rows = state + static_cast<size_t>(state_slots[seg]) * state_stride + static_cast<size_t>(h) * n_state * p_dim;
    const int n0 = wave * R;
    float s[R];
#pragma unroll
    for (int i = 0; i < R; ++i) s[i] = (live && n0 + i < n_state) ? s_rows[static_cast<size_t>(n0 + i) * p_dim + p] : 0.f;
    const float a = -expf(a_log[h]), bias = dt_bias[h], skip = d_skip[h];
    for (int t0 = 0; t0 < q_len; t0 += kScanTokens) {
        const int count = min(kScanTokens, q_len - t0);
        __syncthreads();                                 // the chunk before is read out
        for (int e = threadIdx.x; e < count * n_state; e += blockDim.x) {
            const int t = e / n_state, n = e - t * n_state;
            const T* row = xbc + static_cast<size_t>(q_start + t0 + t) * channels;
            b_s[e] = to_float(row[b_col + n]);
            c_s[e] = to_float(row[c_col + n]);
        }
        for (int e = threadIdx.x; e < count * kWave; e += blockDim.x) {
            const int t = e / kWave, l = e % kWave;
            x_s[e] = p0 + l < p_dim ? to_float(xbc[static_cast<size_t>(q_start + t0 + t) * channels + h * p_dim + p0 + l]) : 0.f;
        }
        if (threadIdx.x < count) {
            const float dt = softplus(to_float(dt_in[static_cast<size_t>(q_start + t0 + threadIdx.x) * dt_stride + h]) + bias);
            dt_s[threadIdx.x] = dt;
            decay_s[threadIdx.x] = expf(a * dt);
        }
        __syncthreads();
        for (int t = 0; t < count; ++t) {
            const float decay = decay_s[t], dx = dt_s[t] * x_s[t * kWave + lane];
            const float* bt = b_s + t * n_state + n0;
            const float* ct = c_s + t * n_state + n0;
            float part = 0.f;
#pragma unroll
            for (int i = 0; i < R; ++i) {
                if (n0 + i < n_state) {
                    s[i] = fmaf(decay, s[i], dx * bt[i]);
                    part = fmaf(s[i], ct[i], part);
                }
            }
            part_s[(t * kScanWaves + wave) * kWave + lane] = part;
        }
        __syncthreads();
        for (int e = threadIdx.x; e < count * kWave; e += blockDim.x) {
            const int t = e / kWave, l = e % kWave;
            if (p0 + l >= p_dim) continue;
            float total = part_s[(t * kScanWaves) * kWave + l];
#pragma unroll
            for (int w = 1; w < kScanWaves; ++w) total += part_s[(t * kScanWaves + w) * kWave + l];
            total = fmaf(skip, x_s[e], total);
            y[static_cast<size_t>(q_start + t0 + t) * inner + h * p_dim + p0 + l] = total;
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < R; ++i)
            if (n0 + i < n_state) s_rows[static_cast<size_t>(n0 + i) * p_dim + p] = s[i];
    }
}

WLLM_API int wllm_ssm_scan(const void* xbc, const void* dt_in, long long dt_stride, const float* dt_bias, const float* a_log,
                           const float* d_skip, float* state, long long state_stride, const int* seg_q_start,
                           const int* seg_q_len, const int* state_slots, float* y, int is_bf16, int segments, int heads,
                           int groups, int n_state, int p_dim, hipStream_t stream) {
    if (segments <= 0) return 0;
    if (heads <= 0 || groups <= 0 || heads % groups != 0 || n_state <= 0 || n_state > 64 * kScanWaves || p_dim <= 0) return -1;
    if (heads > 65535 * 32 || segments > 65535) return -1;
    const int r = (n_state + kScanWaves - 1) / kScanWaves;
    const dim3 grid(heads, segments, (p_dim + kWave - 1) / kWave);
    const size_t smem = sizeof(float) * (2 * kScanTokens * n_state + kScanTokens * kWave + 2 * kScanTokens +
                                         kScanTokens * kScanWaves * kWave);
#define LAUNCH(T, R)                                                                                                \
    ssm_scan_kernel<T, R><<<grid, kWave * kScanWaves, smem, stream>>>(                                              \
        static_cast<const T*>(xbc), static_cast<const T*>(dt_in), dt_stride, dt_bias, a_log, d_skip, state,         \
        state_stride, seg_q_start, seg_q_len, state_slots, y, heads, groups, n_state, p_dim)
#define LAUNCH_R(T)                        \
    if (r <= 8) LAUNCH(T, 8);              \
    else if (r <= 16) LAUNCH(T, 16);       \
    else if (r <= 32) LAUNCH(T, 32);       \
    else LAUNCH(T, 64)
    if (is_bf16) { LAUNCH_R(bf16); } else { LAUNCH_R(float); }
#undef LAUNCH_R
#undef LAUNCH
    return launch_status();
}

// ---- out = rms_norm_in_groups(y * silu(z)) * weight: the recurrence's result (float32) gated by
// z (a band of a wider row, the activation type), then every one of `groups` equal parts of the row
// divided by its own root mean square, times the weight; out in the activation type.  One workgroup
// a (token, part). ----
template <typename T>
__global__ void __launch_bounds__(256)
gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ z, long long z_stride,
                        const float* __restrict__ weight, T* __restrict__ out, int width, int groups, float eps) {
    __shared__ float scratch[16];
    const int token = blockIdx.x, part = blockIdx.y;
    const int size = width / groups, c0 = part * size;
    const float* yr = y + static_cast<size_t>(token) * width + c0;
    const T* zr = z + static_cast<size_t>(token) * z_stride + c0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < size; i += blockDim.x) {
        const float zv = to_float(zr[i]);
        const float v = yr[i] * (zv / (1.f + expf(-zv)));
        ss += v * v;
    }
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(size) + eps);
    T* o = out + static_cast<size_t>(token) * width + c0;
    for (int i = threadIdx.x; i < size; i += blockDim.x) {
        const float zv = to_float(zr[i]);
        const float v = yr[i] * (zv / (1.f + expf(-zv)));
        o[i] = from_float<T>(v * inv * weight[c0 + i]);
    }
}

WLLM_API int wllm_gated_group_norm(const float* y, const void* z, long long z_stride, const float* weight, void* out,
                                   int is_bf16, int tokens, int width, int groups, float eps, hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (width <= 0 || groups <= 0 || width % groups != 0 || groups > 65535) return -1;
    const dim3 grid(tokens, groups);
    if (is_bf16)
        gated_group_norm_kernel<bf16><<<grid, 256, 0, stream>>>(y, static_cast<const bf16*>(z), z_stride, weight,
                                                                static_cast<bf16*>(out), width, groups, eps);
    else
        gated_group_norm_kernel<float><<<grid, 256, 0, stream>>>(y, static_cast<const float*>(z), z_stride, weight,
                                                                 static_cast<float*>(out), width, groups, eps);
    return launch_status();
}
