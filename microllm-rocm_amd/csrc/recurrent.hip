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

// ---- long portions: the recurrence in chunks ---------------------------------------------------------------------
// S_t = a_t S_(t-1) + b_t is cut into chunks of kScanChunk tokens of one request. First every chunk is walked from
// S = 0 (its a and b are formed and kept on the way), which gives its product of decays and what it adds; then one
// thread a (request, channel) carries the state from chunk to chunk; then every chunk is walked again from the state
// it starts with. The grid has a chunk for every case (tokens / chunk + requests); which request a chunk belongs to is
// found from cu_tokens on the device, and chunks beyond the last request's leave at once.
constexpr int kScanChunk = 64;

__device__ inline bool find_chunk(const int32_t* __restrict__ cu_tokens, int n_seqs, int chunk, int* seq, int* first, int* last) {
    int before = 0;
    for (int s = 0; s < n_seqs; ++s) {
        const int begin = cu_tokens[s], end = cu_tokens[s + 1];
        const int chunks = (end - begin + kScanChunk - 1) / kScanChunk;
        if (chunk < before + chunks) {
            *seq = s;
            *first = begin + (chunk - before) * kScanChunk;
            *last = min(*first + kScanChunk, end);
            return true;
        }
        before += chunks;
    }
    return false;
}

__global__ void __launch_bounds__(256)
rglru_chunk_first_kernel(const float* __restrict__ u, const float* __restrict__ gates, const float* __restrict__ r_bias,
                         const float* __restrict__ i_bias, const float* __restrict__ lam, float decay_scale,
                         const int32_t* __restrict__ cu_tokens, int n_seqs, float* __restrict__ decay, float* __restrict__ added,
                         float* __restrict__ chunk_decay, float* __restrict__ chunk_added, int width, int blocks) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    int seq, first, last;
    if (c >= width || !find_chunk(cu_tokens, n_seqs, blockIdx.y, &seq, &first, &last)) return;
    const int size = width / blocks;
    const int gate_at = (c / size) * 2 * size + c % size;
    const float rb = r_bias ? r_bias[c] : 0.0f, ib = i_bias ? i_bias[c] : 0.0f;
    const float rate = -decay_scale * softplus_f(lam[c]);
    float product = 1.0f, s = 0.0f;
    for (int token = first; token < last; ++token) {
        const float* g = gates + static_cast<int64_t>(token) * 2 * width + gate_at;
        const float r = sigmoid_f(g[0] + rb), i = sigmoid_f(g[size] + ib);
        const float log_a = rate * r;
        const float a = expf(log_a);
        const float b = sqrtf(-expm1f(2.0f * log_a)) * (i * u[static_cast<int64_t>(token) * width + c]);
        decay[static_cast<int64_t>(token) * width + c] = a;
        added[static_cast<int64_t>(token) * width + c] = b;
        product *= a;
        s = fmaf(a, s, b);
    }
    chunk_decay[static_cast<int64_t>(blockIdx.y) * width + c] = product;
    chunk_added[static_cast<int64_t>(blockIdx.y) * width + c] = s;
}

// One thread a (request, channel): the state each of the request's chunks starts with (written over chunk_added),
// the request's state after the step, and the convolution's newest inputs.
__global__ void __launch_bounds__(256)
rglru_chunk_carry_kernel(const float* __restrict__ proj, int64_t proj_stride, int x_at, const float* __restrict__ x_bias,
                         const float* __restrict__ chunk_decay, float* __restrict__ chunk_added, float* __restrict__ state,
                         float* __restrict__ kept, const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ slots,
                         int width, int n_taps) {
    const int seq = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    if (last <= first) return;
    int chunk = 0;
    for (int s = 0; s < seq; ++s) chunk += (cu_tokens[s + 1] - cu_tokens[s] + kScanChunk - 1) / kScanChunk;
    const int slot = slots[seq];
    float s = state[static_cast<int64_t>(slot) * width + c];
    for (int begin = first; begin < last; begin += kScanChunk, ++chunk) {
        const int64_t at = static_cast<int64_t>(chunk) * width + c;
        const float starts_with = s;
        s = fmaf(chunk_decay[at], s, chunk_added[at]);
        chunk_added[at] = starts_with;
    }
    state[static_cast<int64_t>(slot) * width + c] = s;
    const int before = n_taps - 1, count = last - first;
    float* tail = kept + static_cast<int64_t>(slot) * before * width;
    for (int n = 0; n < before; ++n) {
        const int back = before - n;
        float value;
        if (back <= count) value = proj[static_cast<int64_t>(last - back) * proj_stride + x_at + c] + (x_bias ? x_bias[c] : 0.0f);
        else value = tail[static_cast<int64_t>(before - (back - count)) * width + c];
        tail[static_cast<int64_t>(n) * width + c] = value;
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
rglru_chunk_second_kernel(const float* __restrict__ proj, int64_t proj_stride, int y_at, const float* __restrict__ y_bias,
                          const float* __restrict__ decay, const float* __restrict__ added, const float* __restrict__ chunk_start,
                          const int32_t* __restrict__ cu_tokens, int n_seqs, T* __restrict__ out, int width) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    int seq, first, last;
    if (c >= width || !find_chunk(cu_tokens, n_seqs, blockIdx.y, &seq, &first, &last)) return;
    float s = chunk_start[static_cast<int64_t>(blockIdx.y) * width + c];
    const float yb = y_bias ? y_bias[c] : 0.0f;
    for (int token = first; token < last; ++token) {
        const int64_t at = static_cast<int64_t>(token) * width + c;
        s = fmaf(decay[at], s, added[at]);
        out[at] = from_float<T>(s * gelu_tanh_f(proj[static_cast<int64_t>(token) * proj_stride + y_at + c] + yb));
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

int mll_rglru_scan_chunked(const float* proj, int64_t proj_stride, int x_at, const float* x_bias, int y_at, const float* y_bias,
                           const float* u, const float* gates, const float* r_bias, const float* i_bias, const float* lam,
                           float decay_scale, float* state, float* kept, const int32_t* cu_tokens, const int32_t* slots, void* out,
                           float* scratch, int dtype, int n_tokens, int n_seqs, int width, int blocks, int n_taps, hipStream_t stream) {
    MLL_REQUIRE(n_seqs >= 0 && n_tokens >= 0 && width > 0 && blocks > 0 && width % blocks == 0 && n_taps >= 1,
                "rglru_scan_chunked: the width must divide into blocks");
    MLL_REQUIRE(n_taps == 1 || kept != nullptr, "rglru_scan_chunked: a convolution of several taps needs the kept inputs");
    MLL_REQUIRE(scratch != nullptr, "rglru_scan_chunked: scratch of mll_rglru_scan_scratch floats is needed");
    if (n_seqs == 0 || n_tokens == 0) return 0;
    const int chunks = (n_tokens + kScanChunk - 1) / kScanChunk + n_seqs;
    MLL_REQUIRE(n_seqs < 65536 && chunks < 65536, "rglru_scan_chunked: too many requests or chunks for one launch");
    float* decay = scratch;
    float* added = decay + static_cast<int64_t>(n_tokens) * width;
    float* chunk_decay = added + static_cast<int64_t>(n_tokens) * width;
    float* chunk_added = chunk_decay + static_cast<int64_t>(chunks) * width;
    const int threads = width >= 256 ? 256 : 64;
    const dim3 by_chunk((width + threads - 1) / threads, chunks), by_request((width + threads - 1) / threads, n_seqs);
    rglru_chunk_first_kernel<<<by_chunk, threads, 0, stream>>>(u, gates, r_bias, i_bias, lam, decay_scale, cu_tokens, n_seqs, decay, added,
                                                              chunk_decay, chunk_added, width, blocks);
    rglru_chunk_carry_kernel<<<by_request, threads, 0, stream>>>(proj, proj_stride, x_at, x_bias, chunk_decay, chunk_added, state, kept,
                                                                cu_tokens, slots, width, n_taps);
    if (dtype == kF32) {
        rglru_chunk_second_kernel<float><<<by_chunk, threads, 0, stream>>>(proj, proj_stride, y_at, y_bias, decay, added, chunk_added, cu_tokens,
                                                                          n_seqs, static_cast<float*>(out), width);
    } else if (dtype == kBF16) {
        rglru_chunk_second_kernel<bf16><<<by_chunk, threads, 0, stream>>>(proj, proj_stride, y_at, y_bias, decay, added, chunk_added, cu_tokens,
                                                                         n_seqs, static_cast<bf16*>(out), width);
    } else {
        return fail("rglru_scan_chunked: unknown dtype");
    }
    return check_launch("rglru_scan_chunked");
}

int64_t mll_rglru_scan_scratch(int n_tokens, int n_seqs, int width) {
    const int64_t chunks = (n_tokens + kScanChunk - 1) / kScanChunk + n_seqs;
    return 2 * (static_cast<int64_t>(n_tokens) + chunks) * width;
}

}  // extern "C"
