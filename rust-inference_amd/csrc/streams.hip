// Residual streams in several copies (hyper-connections), the norm that reads them, and the embedding that
// starts them.
//
// A model with S streams keeps x_1 .. x_S per token, [tokens][S][dim] float32.  A sublayer reads
//     u = sum_s in[s] x_s,                     y = sublayer(norm(u)),
// and writes all streams at once from the old ones,
//     x_t <- sum_s mix[s][t] x_s + out[t] y    (mix is indexed [from][to]).
// As with the plain residual stream, the write waits for the next read and is done by it, in the same
// kernel: ri_streams_read_norm applies the write that is pending (y, mix, out of the sublayer before), stores
// the new streams, forms u with the coefficients of the sublayer that reads, and norms it.  S = 1 with no
// coefficients (each taken as 1) is the plain residual add and norm, so a norm with mean and bias serves both
// kinds of model.  The norm is a layer norm (mean and variance of the row, variance as the mean of squared
// deviations, gain and optional bias), an RMS norm, or none; statistics and streams are float32 throughout.
#include "api.h"
#include "common.h"

#define ST_MAX_STREAMS 8

enum { ST_NORM_NONE = 0, ST_NORM_RMS = 1, ST_NORM_LAYER = 2 };

// One workgroup a row.  u[] (dynamic LDS, dim floats) holds the row that is normed.
template <typename TP, typename TO>
__global__ void __launch_bounds__(256)
streams_read_norm_kernel(TO* __restrict__ out, float* dst, const float* src, long src_copy_stride, int S,
                         const TP* __restrict__ pending, int parts, size_t part_stride,
                         const float* __restrict__ mix, const float* __restrict__ outw, const float* __restrict__ inw,
                         const float* __restrict__ gain, const float* __restrict__ bias, float eps, int kind,
                         const int32_t* __restrict__ rows, int dim) {
    extern __shared__ float u[];
    __shared__ float scratch[16];
    __shared__ float c_mix[ST_MAX_STREAMS * ST_MAX_STREAMS], c_out[ST_MAX_STREAMS], c_in[ST_MAX_STREAMS];
    const int row = blockIdx.x;
    const size_t at = rows ? (size_t)rows[row] : (size_t)row;
    const bool store = rows == nullptr && (pending != nullptr || dst != src);
    if (threadIdx.x < S * S) c_mix[threadIdx.x] = mix ? mix[threadIdx.x] : (threadIdx.x / S == threadIdx.x % S ? 1.f : 0.f);
    if (threadIdx.x < S) {
        c_out[threadIdx.x] = outw ? outw[threadIdx.x] : 1.f;
        c_in[threadIdx.x] = inw ? inw[threadIdx.x] : 1.f;
    }
    __syncthreads();
    // the row's S copies lie S * dim apart in dst; in src they lie src_copy_stride apart (0: one copy serves
    // all, the streams of a fresh sequence of tokens)
    const float* xs = src + at * (src_copy_stride ? (size_t)S * dim : (size_t)dim);
    float* xd = dst + at * (size_t)S * dim;
    float sum = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        float x[ST_MAX_STREAMS], nx[ST_MAX_STREAMS];
        for (int s = 0; s < S; ++s) x[s] = xs[(size_t)s * src_copy_stride + d];
        if (pending) {
            float y = 0.f;
            for (int p = 0; p < parts; ++p) y += to_f32(pending[p * part_stride + at * dim + d]);
            for (int t = 0; t < S; ++t) {
                float v = 0.f;
                for (int s = 0; s < S; ++s) v += c_mix[s * S + t] * x[s];
                nx[t] = v + c_out[t] * y;
            }
        } else {
            for (int t = 0; t < S; ++t) nx[t] = x[t];
        }
        float r = 0.f;
        for (int t = 0; t < S; ++t) {
            if (store) xd[(size_t)t * dim + d] = nx[t];
            r += c_in[t] * nx[t];
        }
        u[d] = r;
        sum += kind == ST_NORM_RMS ? r * r : r;
    }
    TO* o = out + (size_t)row * dim;
    if (kind == ST_NORM_NONE) {
        for (int d = threadIdx.x; d < dim; d += blockDim.x) from_f32(o + d, u[d]);      // each thread its own elements
        return;
    }
    const float total = block_sum(sum, scratch);
    if (kind == ST_NORM_RMS) {
        const float inv = 1.0f / sqrtf(total / (float)dim + eps);
        for (int d = threadIdx.x; d < dim; d += blockDim.x) from_f32(o + d, u[d] * inv * gain[d]);
        return;
    }
    const float mean = total / (float)dim;
    float dev = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float c = u[d] - mean;
        dev += c * c;
    }
    const float inv = 1.0f / sqrtf(block_sum(dev, scratch) / (float)dim + eps);
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float v = (u[d] - mean) * inv * gain[d];
        from_f32(o + d, bias ? v + bias[d] : v);
    }
}

template <typename TP>
static void launch_streams(void* out, int out_dtype, float* dst, const float* src, long scs, int S, const TP* pending,
                           int parts, size_t ps, const float* mix, const float* outw, const float* inw,
                           const float* gain, const float* bias, float eps, int kind, const int32_t* rows, int n_rows,
                           int dim, hipStream_t s) {
    const size_t lds = (size_t)dim * sizeof(float);
    if (out_dtype == RI_F32)
        streams_read_norm_kernel<TP, float><<<n_rows, 256, lds, s>>>((float*)out, dst, src, scs, S, pending, parts, ps,
                                                                      mix, outw, inw, gain, bias, eps, kind, rows, dim);
    else
        streams_read_norm_kernel<TP, bf16_t><<<n_rows, 256, lds, s>>>((bf16_t*)out, dst, src, scs, S, pending, parts, ps,
                                                                       mix, outw, inw, gain, bias, eps, kind, rows, dim);
}

extern "C" int ri_streams_read_norm(void* out, int out_dtype, float* streams, const float* fresh, int n_streams,
                                    const void* pending, int pending_dtype, int parts, int total_rows,
                                    const float* mix, const float* out_coef, const float* in_coef, const float* gain,
                                    const float* bias, float eps, int norm_kind, const int32_t* rows, int n_rows,
                                    int dim, void* stream) {
    RI_REQUIRE(n_rows > 0 && dim > 0 && total_rows > 0, "streams_read_norm: rows %d of %d, dim %d", n_rows, total_rows, dim);
    RI_REQUIRE(n_streams >= 1 && n_streams <= ST_MAX_STREAMS, "streams_read_norm: %d streams, the kernel takes 1 to %d",
               n_streams, ST_MAX_STREAMS);
    RI_REQUIRE(dim <= 16384, "streams_read_norm: rows of %d elements exceed the kernel's 16384", dim);
    RI_REQUIRE(norm_kind == ST_NORM_NONE || norm_kind == ST_NORM_RMS || norm_kind == ST_NORM_LAYER,
               "streams_read_norm: norm kind %d", norm_kind);
    RI_REQUIRE(norm_kind == ST_NORM_NONE || gain != nullptr, "streams_read_norm: a norm needs its gain");
    RI_REQUIRE(parts >= 1 && parts <= 64, "streams_read_norm: %d parts", parts);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "streams_read_norm: out dtype %d", out_dtype);
    RI_REQUIRE(pending_dtype == RI_F32 || pending_dtype == RI_BF16, "streams_read_norm: pending dtype %d", pending_dtype);
    RI_REQUIRE(streams != nullptr, "streams_read_norm: no streams");
    // fresh: [total_rows][dim], one copy that all streams start from; it is spread into `streams` by this call
    const float* src = fresh ? fresh : streams;
    const long scs = fresh ? 0 : dim;
    const size_t ps = (size_t)total_rows * dim;
    hipStream_t s = (hipStream_t)stream;
    if (pending_dtype == RI_F32)
        launch_streams<float>(out, out_dtype, streams, src, scs, n_streams, (const float*)pending, parts, ps, mix,
                              out_coef, in_coef, gain, bias, eps, norm_kind, rows, n_rows, dim, s);
    else
        launch_streams<bf16_t>(out, out_dtype, streams, src, scs, n_streams, (const bf16_t*)pending, parts, ps, mix,
                               out_coef, in_coef, gain, bias, eps, norm_kind, rows, n_rows, dim, s);
    RI_LAUNCH_CHECK("streams_read_norm");
    return 0;
}

// out[t, :] = norm(table[ids[t], :] + positions[pos[t], :]): a learned row per position added to the token's row
// (neither scaled), then the norm (kinds as above; none: the sum itself).  positions may be NULL.
template <typename TT>
__global__ void __launch_bounds__(256)
embed_positions_norm_kernel(float* __restrict__ out, const TT* __restrict__ table, const TT* __restrict__ positions,
                            const int32_t* __restrict__ ids, const int32_t* __restrict__ tok_pos,
                            const float* __restrict__ gain, const float* __restrict__ bias, float eps, int kind,
                            int dim) {
    extern __shared__ float u[];
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const TT* a = table + (size_t)ids[t] * dim;
    const TT* b = positions ? positions + (size_t)tok_pos[t] * dim : nullptr;
    float sum = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float r = b ? to_f32(a[d]) + to_f32(b[d]) : to_f32(a[d]);
        u[d] = r;
        sum += kind == ST_NORM_RMS ? r * r : r;
    }
    float* o = out + (size_t)t * dim;
    if (kind == ST_NORM_NONE) {
        for (int d = threadIdx.x; d < dim; d += blockDim.x) o[d] = u[d];
        return;
    }
    const float total = block_sum(sum, scratch);
    if (kind == ST_NORM_RMS) {
        const float inv = 1.0f / sqrtf(total / (float)dim + eps);
        for (int d = threadIdx.x; d < dim; d += blockDim.x) o[d] = u[d] * inv * gain[d];
        return;
    }
    const float mean = total / (float)dim;
    float dev = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float c = u[d] - mean;
        dev += c * c;
    }
    const float inv = 1.0f / sqrtf(block_sum(dev, scratch) / (float)dim + eps);
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float v = (u[d] - mean) * inv * gain[d];
        o[d] = bias ? v + bias[d] : v;
    }
}

extern "C" int ri_embed_positions_norm(float* out, const void* table, const void* positions, int table_dtype,
                                       const int32_t* ids, const int32_t* tok_pos, const float* gain,
                                       const float* bias, float eps, int norm_kind, int tokens, int dim, void* stream) {
    RI_REQUIRE(tokens > 0 && dim > 0 && dim <= 16384, "embed_positions_norm: tokens %d, dim %d", tokens, dim);
    RI_REQUIRE(norm_kind == ST_NORM_NONE || norm_kind == ST_NORM_RMS || norm_kind == ST_NORM_LAYER,
               "embed_positions_norm: norm kind %d", norm_kind);
    RI_REQUIRE(norm_kind == ST_NORM_NONE || gain != nullptr, "embed_positions_norm: a norm needs its gain");
    RI_REQUIRE(table_dtype == RI_F32 || table_dtype == RI_BF16, "embed_positions_norm: table dtype %d", table_dtype);
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)dim * sizeof(float);
    if (table_dtype == RI_F32)
        embed_positions_norm_kernel<float><<<tokens, 256, lds, s>>>(out, (const float*)table, (const float*)positions, ids,
                                                                    tok_pos, gain, bias, eps, norm_kind, dim);
    else
        embed_positions_norm_kernel<bf16_t><<<tokens, 256, lds, s>>>(out, (const bf16_t*)table, (const bf16_t*)positions,
                                                                     ids, tok_pos, gain, bias, eps, norm_kind, dim);
    RI_LAUNCH_CHECK("embed_positions_norm");
    return 0;
}
