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

#define ST_MAX_STREAMS 16

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

// The same for rows of up to 8192 elements (a multiple of 4) and up to four streams: every thread asks for all
// its 16-byte pieces of all streams and of the waiting output up front and keeps them in registers, so a row's
// loads are in flight together and a step of one row is one trip to memory, not one per element.  Loads are
// issued whatever the indices are, from a column pulled back inside the row.
__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ld4(const bf16_t* p) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xFFFF0000u), __uint_as_float(w.y << 16),
                       __uint_as_float(w.y & 0xFFFF0000u));
}
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void st4(bf16_t* p, float4 v) {
    uint2 w;
    w.x = pack_bf16x2(v.x, v.y);
    w.y = pack_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = w;
}
__device__ __forceinline__ float4 fma4(float a, float4 x, float4 acc) {
    return make_float4(fmaf(a, x.x, acc.x), fmaf(a, x.y, acc.y), fmaf(a, x.z, acc.z), fmaf(a, x.w, acc.w));
}

template <typename TP, typename TO, int S, int VPT>
__global__ void __launch_bounds__(256)
streams_read_norm_vec_kernel(TO* __restrict__ out, float* dst, const float* src, long src_copy_stride,
                             const TP* __restrict__ pending, int parts, size_t part_stride,
                             const float* __restrict__ mix, const float* __restrict__ outw,
                             const float* __restrict__ inw, const float* __restrict__ gain,
                             const float* __restrict__ bias, float eps, int kind, const int32_t* __restrict__ rows,
                             int dim) {
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    const size_t at = rows ? (size_t)rows[row] : (size_t)row;
    const bool store = rows == nullptr && (pending != nullptr || dst != src);
    float cm[S][S], co[S], ci[S];
#pragma unroll
    for (int a = 0; a < S; ++a) {
#pragma unroll
        for (int b = 0; b < S; ++b) cm[a][b] = mix ? mix[a * S + b] : (a == b ? 1.f : 0.f);
        co[a] = outw ? outw[a] : 1.f;
        ci[a] = inw ? inw[a] : 1.f;
    }
    const float* xs = src + at * (src_copy_stride ? (size_t)S * dim : (size_t)dim);
    float* xd = dst + at * (size_t)S * dim;
    const TP* pend = pending ? pending + at * dim : nullptr;
    float4 x[VPT][S], y[VPT];
    int col[VPT];
    bool ok[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = (threadIdx.x + i * 256) * 4;
        ok[i] = c < dim;
        col[i] = ok[i] ? c : 0;
#pragma unroll
        for (int s = 0; s < S; ++s) x[i][s] = ld4(xs + (size_t)s * src_copy_stride + col[i]);
        y[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (pend) {
        for (int p = 0; p < parts; ++p) {
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                const float4 v = ld4(pend + p * part_stride + col[i]);
                y[i] = make_float4(y[i].x + v.x, y[i].y + v.y, y[i].z + v.z, y[i].w + v.w);
            }
        }
    }
    float4 u[VPT];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int t = 0; t < S; ++t) {
            float4 nx = x[i][t];
            if (pend) {
                nx = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int s = 0; s < S; ++s) nx = fma4(cm[s][t], x[i][s], nx);
                nx = fma4(co[t], y[i], nx);
            }
            if (store && ok[i]) st4(xd + (size_t)t * dim + col[i], nx);
            r = fma4(ci[t], nx, r);
        }
        if (!ok[i]) r = make_float4(0.f, 0.f, 0.f, 0.f);
        u[i] = r;
        sum += kind == ST_NORM_RMS ? (r.x * r.x + r.y * r.y) + (r.z * r.z + r.w * r.w) : (r.x + r.y) + (r.z + r.w);
    }
    TO* o = out + (size_t)row * dim;
    float mean = 0.f, inv = 1.f;
    if (kind != ST_NORM_NONE) {
        const float total = block_sum(sum, scratch);
        if (kind == ST_NORM_RMS) {
            inv = 1.0f / sqrtf(total / (float)dim + eps);
        } else {
            mean = total / (float)dim;
            float dev = 0.f;
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                if (ok[i]) {
                    const float a = u[i].x - mean, b = u[i].y - mean, c = u[i].z - mean, d = u[i].w - mean;
                    dev += (a * a + b * b) + (c * c + d * d);
                }
            }
            inv = 1.0f / sqrtf(block_sum(dev, scratch) / (float)dim + eps);
        }
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        if (!ok[i]) continue;
        float4 v = u[i];
        if (kind != ST_NORM_NONE) {
            const float4 g = ld4(gain + col[i]);
            v = make_float4((v.x - mean) * inv * g.x, (v.y - mean) * inv * g.y, (v.z - mean) * inv * g.z, (v.w - mean) * inv * g.w);
            if (bias) {
                const float4 b = ld4(bias + col[i]);
                v = make_float4(v.x + b.x, v.y + b.y, v.z + b.z, v.w + b.w);
            }
        }
        st4(o + col[i], v);
    }
}

template <typename TP, typename TO, int S>
static void launch_streams_vec(TO* out, float* dst, const float* src, long scs, const TP* pending, int parts, size_t ps,
                               const float* mix, const float* outw, const float* inw, const float* gain,
                               const float* bias, float eps, int kind, const int32_t* rows, int n_rows, int dim,
                               hipStream_t s) {
#define RI_STREAMS_VEC(VPT)                                                                                           \
    streams_read_norm_vec_kernel<TP, TO, S, VPT><<<n_rows, 256, 0, s>>>(out, dst, src, scs, pending, parts, ps, mix, outw, \
                                                                        inw, gain, bias, eps, kind, rows, dim)
    if (dim <= 1024) RI_STREAMS_VEC(1);
    else if (dim <= 2048) RI_STREAMS_VEC(2);
    else if (dim <= 4096) RI_STREAMS_VEC(4);
    else RI_STREAMS_VEC(8);
#undef RI_STREAMS_VEC
}

template <typename TP, typename TO>
static bool try_streams_vec(TO* out, float* dst, const float* src, long scs, int S, const TP* pending, int parts, size_t ps,
                            const float* mix, const float* outw, const float* inw, const float* gain, const float* bias,
                            float eps, int kind, const int32_t* rows, int n_rows, int dim, hipStream_t s) {
    if (dim % 4 || dim > 8192 || S > 4) return false;
#define RI_STREAMS_S(SS)                                                                                             \
    case SS: launch_streams_vec<TP, TO, SS>(out, dst, src, scs, pending, parts, ps, mix, outw, inw, gain, bias, eps, kind, \
                                            rows, n_rows, dim, s); break;
    switch (S) {
        RI_STREAMS_S(1)
        RI_STREAMS_S(2)
        RI_STREAMS_S(3)
        RI_STREAMS_S(4)
    }
#undef RI_STREAMS_S
    return true;
}

template <typename TP>
static void launch_streams(void* out, int out_dtype, float* dst, const float* src, long scs, int S, const TP* pending,
                           int parts, size_t ps, const float* mix, const float* outw, const float* inw,
                           const float* gain, const float* bias, float eps, int kind, const int32_t* rows, int n_rows,
                           int dim, hipStream_t s) {
    if (out_dtype == RI_F32 ? try_streams_vec<TP, float>((float*)out, dst, src, scs, S, pending, parts, ps, mix, outw, inw, gain,
                                                          bias, eps, kind, rows, n_rows, dim, s)
                            : try_streams_vec<TP, bf16_t>((bf16_t*)out, dst, src, scs, S, pending, parts, ps, mix, outw, inw,
                                                           gain, bias, eps, kind, rows, n_rows, dim, s))
        return;
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

// The same with a row's 8- or 16-byte pieces asked for up front (rows of up to 8192 elements, a multiple of 4): a
// step of one token is then two trips to memory (the id and position, the rows), not one per element.
template <typename TT, int VPT>
__global__ void __launch_bounds__(256)
embed_positions_norm_vec_kernel(float* __restrict__ out, const TT* __restrict__ table, const TT* __restrict__ positions,
                                const int32_t* __restrict__ ids, const int32_t* __restrict__ tok_pos,
                                const float* __restrict__ gain, const float* __restrict__ bias, float eps, int kind,
                                int dim) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const TT* a = table + (size_t)ids[t] * dim;
    const TT* b = positions ? positions + (size_t)tok_pos[t] * dim : a;      // (no positions: the load is made and dropped)
    float4 u[VPT];
    int col[VPT];
    bool ok[VPT];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = (threadIdx.x + i * 256) * 4;
        ok[i] = c < dim;
        col[i] = ok[i] ? c : 0;
    }
    float4 ra[VPT], rb[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        ra[i] = ld4(a + col[i]);
        rb[i] = ld4(b + col[i]);
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        float4 r = positions ? make_float4(ra[i].x + rb[i].x, ra[i].y + rb[i].y, ra[i].z + rb[i].z, ra[i].w + rb[i].w) : ra[i];
        if (!ok[i]) r = make_float4(0.f, 0.f, 0.f, 0.f);
        u[i] = r;
        sum += kind == ST_NORM_RMS ? (r.x * r.x + r.y * r.y) + (r.z * r.z + r.w * r.w) : (r.x + r.y) + (r.z + r.w);
    }
    float mean = 0.f, inv = 1.f;
    if (kind != ST_NORM_NONE) {
        const float total = block_sum(sum, scratch);
        if (kind == ST_NORM_RMS) {
            inv = 1.0f / sqrtf(total / (float)dim + eps);
        } else {
            mean = total / (float)dim;
            float dev = 0.f;
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                if (ok[i]) {
                    const float x0 = u[i].x - mean, x1 = u[i].y - mean, x2 = u[i].z - mean, x3 = u[i].w - mean;
                    dev += (x0 * x0 + x1 * x1) + (x2 * x2 + x3 * x3);
                }
            }
            inv = 1.0f / sqrtf(block_sum(dev, scratch) / (float)dim + eps);
        }
    }
    float* o = out + (size_t)t * dim;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        if (!ok[i]) continue;
        float4 v = u[i];
        if (kind != ST_NORM_NONE) {
            const float4 g = ld4(gain + col[i]);
            v = make_float4((v.x - mean) * inv * g.x, (v.y - mean) * inv * g.y, (v.z - mean) * inv * g.z, (v.w - mean) * inv * g.w);
            if (bias) {
                const float4 bb = ld4(bias + col[i]);
                v = make_float4(v.x + bb.x, v.y + bb.y, v.z + bb.z, v.w + bb.w);
            }
        }
        st4(o + col[i], v);
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
    if (dim % 4 == 0 && dim <= 8192) {
#define RI_EMBED_VEC(T, VPT)                                                                                          \
    embed_positions_norm_vec_kernel<T, VPT><<<tokens, 256, 0, s>>>(out, (const T*)table, (const T*)positions, ids, tok_pos,  \
                                                                   gain, bias, eps, norm_kind, dim)
#define RI_EMBED_DIM(T)                                                                                               \
    if (dim <= 1024) RI_EMBED_VEC(T, 1); else if (dim <= 2048) RI_EMBED_VEC(T, 2); else if (dim <= 4096) RI_EMBED_VEC(T, 4); \
    else RI_EMBED_VEC(T, 8)
        if (table_dtype == RI_F32) { RI_EMBED_DIM(float); } else { RI_EMBED_DIM(bf16_t); }
#undef RI_EMBED_DIM
#undef RI_EMBED_VEC
        RI_LAUNCH_CHECK("embed_positions_norm");
        return 0;
    }
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
