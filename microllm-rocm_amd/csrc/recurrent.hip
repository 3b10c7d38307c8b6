// A recurrent block with a real-gated linear recurrent unit: a short causal convolution per channel, two gates from
// block-diagonal products, and S_t = a_t S_(t-1) + sqrt(1 - a_t^2) (i_t u_t) with a_t = exp(-c r_t softplus(lam)).
// What a request keeps between steps: the convolution's last taps - 1 inputs and S, both float32, in its state slot.
// Everything here is float32 but the result, which is rounded once for the output projection.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

// u[t][c] = conv_bias[c] + sum_j taps[c][j] * input(t - (n_taps - 1 - j), c), where input(s, c) = proj[s][x_at + c] +
// x_bias[c] for a token of this step and the request's kept inputs before the step's first token (zeros before the
// request's first token: a fresh slot is zero). One thread a (token, channel).
template <typename W>
__global__ void __launch_bounds__(256)
rglru_conv_kernel(const float* __restrict__ proj, int64_t proj_stride, int x_at, const float* __restrict__ x_bias,
                  const W* __restrict__ taps, const float* __restrict__ conv_bias, const float* __restrict__ kept,
                  const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ cu_tokens,
                  const int32_t* __restrict__ slots, float* __restrict__ u, int width, int n_taps) {
    const int token = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const int seq = seq_of_token[token];
    if (seq < 0) {
        u[static_cast<int64_t>(token) * width + c] = 0.0f;
        return;
    }
    const int local = token - cu_tokens[seq];
    const int before = n_taps - 1;
    const float* tail = kept + static_cast<int64_t>(slots[seq]) * before * width;
    float sum = 0.0f;
    for (int j = 0; j < n_taps; ++j) {
        const int back = before - j;            // how many tokens before this one
        float value;
        if (back <= local) value = proj[static_cast<int64_t>(token - back) * proj_stride + x_at + c] + (x_bias ? x_bias[c] : 0.0f);
        else value = tail[static_cast<int64_t>(before - (back - local)) * width + c];      // the (back - local)-th newest kept input
        sum = fmaf(to_float(taps[static_cast<int64_t>(c) * n_taps + j]), value, sum);
    }
    u[static_cast<int64_t>(token) * width + c] = sum + (conv_bias ? conv_bias[c] : 0.0f);
}

__device__ inline float softplus_f(float x) { return fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x))); }
__device__ inline float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ inline float gelu_tanh_f(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// One thread a (request, channel) walks the request's tokens of the step in order. gates[t] = [blocks][r (size) | i (size)]
// before bias and sigmoid. out[t][c] = S_t * gelu_tanh(proj[t][y_at + c] + y_bias[c]) in T. At the end S and the
// convolution's newest inputs go back into the slot. A request without tokens is passed over.
template <typename T>
__global__ void __launch_bounds__(256)
rglru_scan_kernel(const float* __restrict__ proj, int64_t proj_stride, int x_at, const float* __restrict__ x_bias, int y_at,
                  const float* __restrict__ y_bias, const float* __restrict__ u, const float* __restrict__ gates,
                  const float* __restrict__ r_bias, const float* __restrict__ i_bias, const float* __restrict__ lam,
                  float decay_scale, float* __restrict__ state, float* __restrict__ kept, const int32_t* __restrict__ cu_tokens,
                  const int32_t* __restrict__ slots, T* __restrict__ out, int width, int blocks, int n_taps) {
    const int seq = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    if (last <= first) return;
    const int slot = slots[seq];
    const int size = width / blocks;
    const int gate_at = (c / size) * 2 * size + c % size;
    const float rb = r_bias ? r_bias[c] : 0.0f, ib = i_bias ? i_bias[c] : 0.0f;
    const float rate = -decay_scale * softplus_f(lam[c]);
    float s = state[static_cast<int64_t>(slot) * width + c];
    for (int token = first; token < last; ++token) {
        const float* g = gates + static_cast<int64_t>(token) * 2 * width + gate_at;
        const float r = sigmoid_f(g[0] + rb), i = sigmoid_f(g[size] + ib);
        const float log_a = rate * r;
        const float a = expf(log_a);
        const float step = sqrtf(-expm1f(2.0f * log_a));       // sqrt(1 - a^2) without the cancellation near a = 1
        s = fmaf(a, s, step * (i * u[static_cast<int64_t>(token) * width + c]));
        const float y = gelu_tanh_f(proj[static_cast<int64_t>(token) * proj_stride + y_at + c] + (y_bias ? y_bias[c] : 0.0f));
        out[static_cast<int64_t>(token) * width + c] = from_float<T>(s * y);
    }
    state[static_cast<int64_t>(slot) * width + c] = s;
    const int before = n_taps - 1, count = last - first;
    float* tail = kept + static_cast<int64_t>(slot) * before * width;
    // the newest `before` inputs of (kept inputs, then this step's): entry n of the new tail, n = 0 the oldest
    for (int n = 0; n < before; ++n) {
        const int back = before - n;            // it lies this many inputs before the end
        float value;
        if (back <= count) value = proj[static_cast<int64_t>(last - back) * proj_stride + x_at + c] + (x_bias ? x_bias[c] : 0.0f);
        else value = tail[static_cast<int64_t>(before - (back - count)) * width + c];      // an older kept input; n + count < before, read before it is overwritten
        tail[static_cast<int64_t>(n) * width + c] = value;
    }
}

}  // namespace mll

using namespace mll;

extern "C" {

int mll_rglru_conv(const float* proj, int64_t proj_stride, int x_at, const float* x_bias, const void* taps, int taps_dtype,
                   const float* conv_bias, const float* kept, const int32_t* seq_of_token, const int32_t* cu_tokens,
                   const int32_t* slots, float* u, int n_tokens, int width, int n_taps, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && width > 0 && n_taps >= 1, "rglru_conv: sizes must be positive");
    MLL_REQUIRE(n_taps == 1 || kept != nullptr, "rglru_conv: a convolution of several taps needs the kept inputs");
    MLL_REQUIRE(n_tokens < 65536, "rglru_conv: too many rows for one launch");
    if (n_tokens == 0) return 0;
    const dim3 grid((width + 255) / 256, n_tokens);
    if (taps_dtype == kF32) {
        rglru_conv_kernel<float><<<grid, 256, 0, stream>>>(proj, proj_stride, x_at, x_bias, static_cast<const float*>(taps), conv_bias,
                                                           kept, seq_of_token, cu_tokens, slots, u, width, n_taps);
    } else if (taps_dtype == kBF16) {
        rglru_conv_kernel<bf16><<<grid, 256, 0, stream>>>(proj, proj_stride, x_at, x_bias, static_cast<const bf16*>(taps), conv_bias,
                                                          kept, seq_of_token, cu_tokens, slots, u, width, n_taps);
    } else {
        return fail("rglru_conv: unknown dtype");
    }
    return check_launch("rglru_conv");
}

int mll_rglru_scan(const float* proj, int64_t proj_stride, int x_at, const float* x_bias, int y_at, const float* y_bias,
                   const float* u, const float* gates, const float* r_bias, const float* i_bias, const float* lam,
                   float decay_scale, float* state, float* kept, const int32_t* cu_tokens, const int32_t* slots, void* out,
                   int dtype, int n_seqs, int width, int blocks, int n_taps, hipStream_t stream) {
    MLL_REQUIRE(n_seqs >= 0 && width > 0 && blocks > 0 && width % blocks == 0 && n_taps >= 1, "rglru_scan: the width must divide into blocks");
    MLL_REQUIRE(n_taps == 1 || kept != nullptr, "rglru_scan: a convolution of several taps needs the kept inputs");
    MLL_REQUIRE(n_seqs < 65536, "rglru_scan: too many requests for one launch");
    if (n_seqs == 0) return 0;
    const int threads = width >= 256 ? 256 : 64;
    const dim3 grid((width + threads - 1) / threads, n_seqs);
    if (dtype == kF32) {
        rglru_scan_kernel<float><<<grid, threads, 0, stream>>>(proj, proj_stride, x_at, x_bias, y_at, y_bias, u, gates, r_bias, i_bias, lam,
                                                               decay_scale, state, kept, cu_tokens, slots, static_cast<float*>(out), width, blocks, n_taps);
    } else if (dtype == kBF16) {
        rglru_scan_kernel<bf16><<<grid, threads, 0, stream>>>(proj, proj_stride, x_at, x_bias, y_at, y_bias, u, gates, r_bias, i_bias, lam,
                                                              decay_scale, state, kept, cu_tokens, slots, static_cast<bf16*>(out), width, blocks, n_taps);
    } else {
        return fail("rglru_scan: unknown dtype");
    }
    return check_launch("rglru_scan");
}

}  // extern "C"
