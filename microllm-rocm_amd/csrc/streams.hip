// The residual stream in several copies (hyper-connections), the norms that read it, a sinusoidal position
// vector added to the embedding, and a gated activation with clamped inputs.
//
// Streams: instead of one row x a token has S rows x_0 .. x_(S-1). A sublayer reads u = sum_s in[s] x_s, and its
// result y comes back as x_t <- sum_s mix[s, t] x_s + out[t] y for every t at once. One kernel does the write of
// one sublayer, the read of the next and the norm between them, as the residual sum and the norm are one kernel
// for a single stream; with S = 1 and no weights it is that plain sum. Everything is float32 here; only the
// norm's result has the engine's element type.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

constexpr int kMaxStreams = 8;
// Threads of a row's workgroup, by the row's width alone (the order of a row's sums follows the workgroup's size, so
// it must not follow the batch): few columns a thread keep a row of a decode step from waiting for its loads in turn.
inline int norm_threads(int width) { return width >= 2048 ? 1024 : (width >= 1024 ? 512 : 256); }

template <typename T>
__global__ void embedding_sinusoid_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids,
                                          const int32_t* __restrict__ positions, const double* __restrict__ rates,
                                          float* __restrict__ out, int width, int vocab) {
    const int token = blockIdx.x;
    const int id = ids[token];
    const bool valid = id >= 0 && id < vocab;
    const double position = static_cast<double>(positions[token]);
    const T* row = table + static_cast<int64_t>(valid ? id : 0) * width;
    float* to = out + static_cast<int64_t>(token) * width;
    for (int column = threadIdx.x; column < width; column += blockDim.x) {
        // entry 2i: sin(p * rates[i]), entry 2i + 1: cos of the same angle; the angle in float64
        const double angle = position * rates[column / 2];
        const float wave = static_cast<float>((column & 1) ? cos(angle) : sin(angle));
        to[column] = valid ? to_float(row[column]) + wave : __builtin_nanf("");
    }
}

__global__ void stream_copies_kernel(const float* __restrict__ in, float* __restrict__ out, int width, int copies) {
    const int token = blockIdx.x;
    const float* from = in + static_cast<int64_t>(token) * width;
    float* to = out + static_cast<int64_t>(token) * copies * width;
    for (int column = threadIdx.x; column < width; column += blockDim.x) {
        const float value = from[column];
        for (int copy = 0; copy < copies; ++copy) to[copy * width + column] = value;
    }
}

// One workgroup a row. u is kept in LDS (width floats) between the passes over it.
template <typename T>
__global__ void stream_norm_kernel(float* __restrict__ x, const float* __restrict__ y, int n_parts, int64_t part_stride,
                                   const float* __restrict__ mix, const float* __restrict__ give,
                                   const float* __restrict__ take, const int32_t* __restrict__ rows,
                                   const float* __restrict__ weight, float eps, int rms, T* __restrict__ out, int streams,
                                   int width, int write_x) {
    extern __shared__ float u_row[];
    __shared__ float scratch[16];
    const int row = rows ? rows[blockIdx.x] : blockIdx.x;
    float* base = x + static_cast<int64_t>(row) * streams * width;
    float local_sum = 0.0f;
    for (int column = threadIdx.x; column < width; column += blockDim.x) {
        float old[kMaxStreams];
#pragma unroll
        for (int s = 0; s < kMaxStreams; ++s) old[s] = s < streams ? base[s * width + column] : 0.0f;
        float u = 0.0f;
        if (y != nullptr) {
            float delta = y[static_cast<int64_t>(row) * width + column];
            for (int part = 1; part < n_parts; ++part) delta += y[part * part_stride + static_cast<int64_t>(row) * width + column];
#pragma unroll
            for (int t = 0; t < kMaxStreams; ++t) {
                if (t >= streams) break;
                float fresh;
                if (mix != nullptr) {
                    fresh = 0.0f;
#pragma unroll
                    for (int s = 0; s < kMaxStreams; ++s)
                        if (s < streams) fresh += mix[s * streams + t] * old[s];
                } else {
                    fresh = old[t];
                }
                fresh += (give ? give[t] : 1.0f) * delta;
                if (write_x) base[t * width + column] = fresh;
                u += (take ? take[t] : 1.0f) * fresh;
            }
        } else {
#pragma unroll
            for (int s = 0; s < kMaxStreams; ++s)
                if (s < streams) u += (take ? take[s] : 1.0f) * old[s];
        }
        u_row[column] = u;
        local_sum += rms ? u * u : u;
    }
    if (out == nullptr) return;
    const float total = block_sum(local_sum, scratch);
    float mean = 0.0f, factor;
    if (rms) {
        factor = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
    } else {
        mean = total / static_cast<float>(width);
        float spread = 0.0f;
        for (int column = threadIdx.x; column < width; column += blockDim.x) {
            const float d = u_row[column] - mean;
            spread += d * d;
        }
        factor = 1.0f / sqrtf(block_sum(spread, scratch) / static_cast<float>(width) + eps);
    }
    T* to = out + static_cast<int64_t>(blockIdx.x) * width;
    for (int column = threadIdx.x; column < width; column += blockDim.x)
        to[column] = from_float<T>((u_row[column] - mean) * factor * weight[column]);
}

// gu[t] = [gate (width) | up (width)] in float32: g = min(gate, limit), u = clamp(up, -limit, limit),
// out = g * sigmoid(slope * g) * (u + 1).
template <typename T>
__global__ void clamped_glu_kernel(const float* __restrict__ gu, T* __restrict__ out, int width, float limit, float slope) {
    const int token = blockIdx.y;
    const int column = blockIdx.x * blockDim.x + threadIdx.x;
    if (column >= width) return;
    const float* row = gu + static_cast<int64_t>(token) * 2 * width;
    const float g = fminf(row[column], limit);
    const float u = fminf(fmaxf(row[width + column], -limit), limit);
    const float gate = g / (1.0f + expf(-slope * g));
    out[static_cast<int64_t>(token) * width + column] = from_float<T>(gate * (u + 1.0f));
}

}  // namespace mll

using namespace mll;

extern "C" {

int mll_embedding_sinusoid(const void* table, int table_dtype, const int32_t* ids, const int32_t* positions,
                           const double* rates, float* out, int n_tokens, int width, int vocab, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && width > 0 && vocab > 0 && rates != nullptr, "embedding_sinusoid: sizes must be positive");
    if (n_tokens == 0) return 0;
    if (table_dtype == kF32) {
        embedding_sinusoid_kernel<float><<<n_tokens, 256, 0, stream>>>(static_cast<const float*>(table), ids, positions, rates,
                                                                      out, width, vocab);
    } else if (table_dtype == kBF16) {
        embedding_sinusoid_kernel<bf16><<<n_tokens, 256, 0, stream>>>(static_cast<const bf16*>(table), ids, positions, rates,
                                                                     out, width, vocab);
    } else {
        return fail("embedding_sinusoid: unknown table dtype");
    }
    return check_launch("embedding_sinusoid");
}

int mll_stream_copies(const float* in, float* out, int n_tokens, int width, int copies, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && width > 0 && copies >= 1, "stream_copies: sizes must be positive");
    if (n_tokens == 0) return 0;
    stream_copies_kernel<<<n_tokens, 256, 0, stream>>>(in, out, width, copies);
    return check_launch("stream_copies");
}

int mll_stream_norm(float* x, const float* y, int n_parts, int64_t part_stride, const float* mix, const float* give,
                    const float* take, const int32_t* rows, const float* weight, float eps, int rms, void* out, int dtype,
                    int n_rows, int streams, int width, int write_x, hipStream_t stream) {
    MLL_REQUIRE(n_rows >= 0 && width > 0, "stream_norm: sizes must be positive");
    MLL_REQUIRE(streams >= 1 && streams <= kMaxStreams, "stream_norm: between 1 and 8 streams");
    MLL_REQUIRE(n_parts >= 1, "stream_norm: the delta needs at least one part");
    MLL_REQUIRE(!(write_x && rows), "stream_norm: cannot write the streams through a row selection");
    MLL_REQUIRE(out == nullptr || (weight != nullptr && eps > 0.0f), "stream_norm: a norm needs its weight and a positive eps");
    MLL_REQUIRE(static_cast<size_t>(width) * sizeof(float) <= 64 * 1024, "stream_norm: rows wider than 16384 are not supported");
    if (n_rows == 0) return 0;
    const size_t lds = static_cast<size_t>(width) * sizeof(float);
    if (dtype == kF32) {
        stream_norm_kernel<float><<<n_rows, norm_threads(width), lds, stream>>>(x, y, n_parts, part_stride, mix, give, take, rows, weight,
                                                                        eps, rms, static_cast<float*>(out), streams, width, write_x);
    } else if (dtype == kBF16) {
        stream_norm_kernel<bf16><<<n_rows, norm_threads(width), lds, stream>>>(x, y, n_parts, part_stride, mix, give, take, rows, weight,
                                                                       eps, rms, static_cast<bf16*>(out), streams, width, write_x);
    } else {
        return fail("stream_norm: unknown dtype");
    }
    return check_launch("stream_norm");
}

int mll_clamped_glu(const float* gate_up, void* out, int dtype, int n_tokens, int width, float limit, float slope,
                    hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && width > 0, "clamped_glu: sizes must be positive");
    MLL_REQUIRE(limit > 0.0f, "clamped_glu: the limit must be positive");
    if (n_tokens == 0) return 0;
    MLL_REQUIRE(n_tokens <= 65535, "clamped_glu: more than 65535 tokens in one call");
    const dim3 grid((width + 255) / 256, n_tokens);
    if (dtype == kF32) {
        clamped_glu_kernel<float><<<grid, 256, 0, stream>>>(gate_up, static_cast<float*>(out), width, limit, slope);
    } else if (dtype == kBF16) {
        clamped_glu_kernel<bf16><<<grid, 256, 0, stream>>>(gate_up, static_cast<bf16*>(out), width, limit, slope);
    } else {
        return fail("clamped_glu: unknown dtype");
    }
    return check_launch("clamped_glu");
}

}  // extern "C"
