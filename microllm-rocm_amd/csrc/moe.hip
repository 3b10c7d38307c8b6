// A mixture of experts: the choice of every token's experts from router logits, and the experts' gated
// feed-forwards for (token, choice) pairs whose expert is only known on the device.
//
// Choice: scores are sigmoid(z) or softmax(z) over the experts, the `top` largest are taken (ties: the lower
// index), their weights are the scores, optionally divided by their sum. Everything float32.
//
// Experts, plain kernels: a workgroup takes one (token, choice) pair and a stretch of the expert's output rows; a
// wave forms one output at a time with its lanes along the reduction (16-byte loads of the weight's row), so a
// pair's sums never depend on the other pairs. These serve every dtype and number of tokens; their cost per pair is
// one reading of the expert's weights, which is what decoding a few tokens costs anyway.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

constexpr int kMaxTop = 16;

// One thread a token. z: float32 rows, z_stride apart, experts first; a further column `shared_at` (negative: none)
// holds the logit of the shared expert's gate, whose sigmoid goes to shared_gate[t].
__global__ void __launch_bounds__(64)
moe_route_kernel(const float* __restrict__ z, int64_t z_stride, int n_tokens, int experts, int top, int softmax_scores,
                 int renormalize, int shared_at, int32_t* __restrict__ ids, float* __restrict__ weights,
                 float* __restrict__ shared_gate) {
    const int token = blockIdx.x * blockDim.x + threadIdx.x;
    if (token >= n_tokens) return;
    const float* row = z + static_cast<int64_t>(token) * z_stride;
    float peak = -INFINITY, total = 1.0f;
    if (softmax_scores) {
        for (int e = 0; e < experts; ++e) peak = fmaxf(peak, row[e]);
        total = 0.0f;
        for (int e = 0; e < experts; ++e) total += expf(row[e] - peak);
    }
    int chosen[kMaxTop];
    float taken[kMaxTop];
    float sum = 0.0f;
    for (int n = 0; n < top; ++n) {
        int best = -1;
        float best_logit = 0.0f;
        for (int e = 0; e < experts; ++e) {
            bool used = false;
            for (int m = 0; m < n; ++m) used = used || chosen[m] == e;
            if (used) continue;
            // the scores rise with the logits, so the largest logit is the largest score; a logit that is no number is never larger
            if (best < 0 || row[e] > best_logit) {
                best = e;
                best_logit = row[e];
            }
        }
        chosen[n] = best;
        taken[n] = softmax_scores ? expf(best_logit - peak) / total : 1.0f / (1.0f + expf(-best_logit));
        sum += taken[n];
    }
    for (int n = 0; n < top; ++n) {
        ids[static_cast<int64_t>(token) * top + n] = chosen[n];
        weights[static_cast<int64_t>(token) * top + n] = renormalize ? taken[n] / sum : taken[n];
    }
    if (shared_at >= 0 && shared_gate != nullptr) shared_gate[token] = 1.0f / (1.0f + expf(-row[shared_at]));
}

template <typename T> __device__ inline float row_dot(const T* __restrict__ w, const float* __restrict__ x, int k, int lane);

template <> __device__ inline float row_dot<float>(const float* __restrict__ w, const float* __restrict__ x, int k, int lane) {
    float sum = 0.0f;
    if ((k & 3) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
        for (int c = lane * 4; c < k; c += kWave * 4) {
            const float4 v = *reinterpret_cast<const float4*>(w + c);
            sum = fmaf(v.x, x[c], sum);
            sum = fmaf(v.y, x[c + 1], sum);
            sum = fmaf(v.z, x[c + 2], sum);
            sum = fmaf(v.w, x[c + 3], sum);
        }
    } else {
        for (int c = lane; c < k; c += kWave) sum = fmaf(w[c], x[c], sum);
    }
    return wave_sum(sum);
}

template <> __device__ inline float row_dot<bf16>(const bf16* __restrict__ w, const float* __restrict__ x, int k, int lane) {
    float sum = 0.0f;
    if ((k & 7) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
        for (int c = lane * 8; c < k; c += kWave * 8) {
            const uint4 raw = *reinterpret_cast<const uint4*>(w + c);
            const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sum = fmaf(__builtin_bit_cast(float, words[i] << 16), x[c + 2 * i], sum);
                sum = fmaf(__builtin_bit_cast(float, words[i] & 0xffff0000u), x[c + 2 * i + 1], sum);
            }
        }
    } else {
        for (int c = lane; c < k; c += kWave) sum = fmaf(to_float(w[c]), x[c], sum);
    }
    return wave_sum(sum);
}

constexpr int kExpertWaves = 4;
constexpr int kExpertRowsAWave = 8;     // outputs a wave forms one after the other
constexpr int kExpertRowsABlock = kExpertWaves * kExpertRowsAWave;

// act[pair][f] = silu(Wg_e[f] . xs) * (Wu_e[f] . xs), xs = x[token] * weight[pair] rounded to T (the weight
// multiplies the expert's input) or x[token] (weight_on_input 0). gate_up: [experts][2 * ff][width], gate rows first.
template <typename T>
__global__ void __launch_bounds__(kExpertWaves * kWave)
moe_gate_up_kernel(const T* __restrict__ x, const int32_t* __restrict__ ids, const float* __restrict__ weights, int top,
                   const T* __restrict__ gate_up, T* __restrict__ act, int width, int ff, int weight_on_input) {
    extern __shared__ float xs[];
    const int pair = blockIdx.y;
    const int token = pair / top;
    const int expert = ids[pair];
    const float factor = weight_on_input ? weights[pair] : 1.0f;
    for (int c = threadIdx.x; c < width; c += blockDim.x)
        xs[c] = to_float(from_float<T>(to_float(x[static_cast<int64_t>(token) * width + c]) * factor));
    __syncthreads();
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const T* base = gate_up + static_cast<int64_t>(expert) * 2 * ff * width;
    for (int n = 0; n < kExpertRowsAWave; ++n) {
        const int f = blockIdx.x * kExpertRowsABlock + wave * kExpertRowsAWave + n;
        if (f >= ff) break;
        const float g = row_dot<T>(base + static_cast<int64_t>(f) * width, xs, width, lane);
        const float u = row_dot<T>(base + static_cast<int64_t>(ff + f) * width, xs, width, lane);
        if (lane == 0) act[static_cast<int64_t>(pair) * ff + f] = from_float<T>(g / (1.0f + expf(-g)) * u);
    }
}

// out[choice][token][c] = (Wd_e[c] . act[pair]) (* weight[pair] with weight_on_input 0): float32 [top][tokens][width],
// partial sums that the reader adds in order. down: [experts][width][ff].
template <typename T>
__global__ void __launch_bounds__(kExpertWaves * kWave)
moe_down_kernel(const T* __restrict__ act, const int32_t* __restrict__ ids, const float* __restrict__ weights, int top,
                const T* __restrict__ down, float* __restrict__ out, int n_tokens, int width, int ff, int weight_on_input) {
    extern __shared__ float as[];
    const int pair = blockIdx.y;
    const int token = pair / top, choice = pair % top;
    const int expert = ids[pair];
    for (int c = threadIdx.x; c < ff; c += blockDim.x) as[c] = to_float(act[static_cast<int64_t>(pair) * ff + c]);
    __syncthreads();
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const T* base = down + static_cast<int64_t>(expert) * width * ff;
    const float factor = weight_on_input ? 1.0f : weights[pair];
    for (int n = 0; n < kExpertRowsAWave; ++n) {
        const int c = blockIdx.x * kExpertRowsABlock + wave * kExpertRowsAWave + n;
        if (c >= width) break;
        const float value = row_dot<T>(base + static_cast<int64_t>(c) * ff, as, ff, lane);
        if (lane == 0) out[(static_cast<int64_t>(choice) * n_tokens + token) * width + c] = value * factor;
    }
}

// out[t][c] = factor[t] * sum over parts of in[part][t][c], float32.
__global__ void __launch_bounds__(256)
scale_rows_kernel(const float* __restrict__ in, int n_parts, int64_t part_stride, const float* __restrict__ factor,
                  float* __restrict__ out, int width) {
    const int token = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const int64_t at = static_cast<int64_t>(token) * width + c;
    float value = in[at];
    for (int part = 1; part < n_parts; ++part) value += in[part * part_stride + at];
    out[at] = value * factor[token];
}

}  // namespace mll

using namespace mll;

extern "C" {

int mll_moe_route(const float* z, int64_t z_stride, int n_tokens, int experts, int top, int softmax_scores, int renormalize,
                  int shared_at, int32_t* ids, float* weights, float* shared_gate, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && experts > 0 && top > 0 && top <= experts, "moe_route: 1 <= top <= experts");
    MLL_REQUIRE(top <= kMaxTop, "moe_route: more than 16 experts a token are not supported");
    MLL_REQUIRE(shared_at < 0 || shared_gate != nullptr, "moe_route: the shared expert's gate needs a place");
    if (n_tokens == 0) return 0;
    moe_route_kernel<<<(n_tokens + 63) / 64, 64, 0, stream>>>(z, z_stride, n_tokens, experts, top, softmax_scores, renormalize,
                                                            shared_at, ids, weights, shared_gate);
    return check_launch("moe_route");
}

int mll_moe_gate_up(const void* x, const int32_t* ids, const float* weights, int top, const void* gate_up, void* act,
                    int dtype, int n_tokens, int width, int ff, int weight_on_input, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && top > 0 && width > 0 && ff > 0, "moe_gate_up: sizes must be positive");
    MLL_REQUIRE(static_cast<int64_t>(n_tokens) * top < 65536, "moe_gate_up: too many (token, expert) pairs for one launch");
    MLL_REQUIRE(static_cast<size_t>(width) * sizeof(float) <= 64 * 1024, "moe_gate_up: rows wider than 16384 are not supported");
    if (n_tokens == 0) return 0;
    const dim3 grid((ff + kExpertRowsABlock - 1) / kExpertRowsABlock, n_tokens * top);
    const size_t lds = static_cast<size_t>(width) * sizeof(float);
    if (dtype == kF32) {
        moe_gate_up_kernel<float><<<grid, kExpertWaves * kWave, lds, stream>>>(
            static_cast<const float*>(x), ids, weights, top, static_cast<const float*>(gate_up), static_cast<float*>(act), width, ff, weight_on_input);
    } else if (dtype == kBF16) {
        moe_gate_up_kernel<bf16><<<grid, kExpertWaves * kWave, lds, stream>>>(
            static_cast<const bf16*>(x), ids, weights, top, static_cast<const bf16*>(gate_up), static_cast<bf16*>(act), width, ff, weight_on_input);
    } else {
        return fail("moe_gate_up: unknown dtype");
    }
    return check_launch("moe_gate_up");
}

int mll_moe_down(const void* act, const int32_t* ids, const float* weights, int top, const void* down, float* out, int dtype,
                 int n_tokens, int width, int ff, int weight_on_input, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && top > 0 && width > 0 && ff > 0, "moe_down: sizes must be positive");
    MLL_REQUIRE(static_cast<int64_t>(n_tokens) * top < 65536, "moe_down: too many (token, expert) pairs for one launch");
    MLL_REQUIRE(static_cast<size_t>(ff) * sizeof(float) <= 64 * 1024, "moe_down: experts wider than 16384 are not supported");
    if (n_tokens == 0) return 0;
    const dim3 grid((width + kExpertRowsABlock - 1) / kExpertRowsABlock, n_tokens * top);
    const size_t lds = static_cast<size_t>(ff) * sizeof(float);
    if (dtype == kF32) {
        moe_down_kernel<float><<<grid, kExpertWaves * kWave, lds, stream>>>(
            static_cast<const float*>(act), ids, weights, top, static_cast<const float*>(down), out, n_tokens, width, ff, weight_on_input);
    } else if (dtype == kBF16) {
        moe_down_kernel<bf16><<<grid, kExpertWaves * kWave, lds, stream>>>(
            static_cast<const bf16*>(act), ids, weights, top, static_cast<const bf16*>(down), out, n_tokens, width, ff, weight_on_input);
    } else {
        return fail("moe_down: unknown dtype");
    }
    return check_launch("moe_down");
}

int mll_scale_rows(const float* in, int n_parts, int64_t part_stride, const float* factor, float* out, int n_tokens, int width,
                   hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && width > 0 && n_parts >= 1, "scale_rows: sizes must be positive");
    MLL_REQUIRE(n_tokens < 65536, "scale_rows: too many rows for one launch");
    if (n_tokens == 0) return 0;
    scale_rows_kernel<<<dim3((width + 255) / 256, n_tokens), 256, 0, stream>>>(in, n_parts, part_stride, factor, out, width);
    return check_launch("scale_rows");
}

}  // extern "C"
