// Queries and keys made ready for an attention without rotation, and keys and values into their pages, in one
// pass over the fused projection [tokens][heads * dim | kv_heads * dim | kv_heads * vdim] (the value heads may
// have another size than the query and key heads).
//
//   q, k: optional per-head RMS norm, x / sqrt(mean(x^2) + eps) * gain, one gain of `dim` for all heads;
//   q:    a temperature by position, q *= 1 + coef * ln(floor((p + 1) / every) + 1) (coef 0: none), in place;
//   k:    into k_pages [pages][kv_heads][page_size][dim];
//   v:    copied into v_pages [pages][kv_heads][vdim][page_size] (transposed inside a page).
//
// Norm, logarithm and factor are float32; a q or k element is rounded once.  One wavefront per (token, head).
#include "api.h"
#include "common.h"

#define QT_MAX_PER_LANE 8    // head sizes up to 64 * 8

template <typename TA, typename TC>
__global__ void qk_norm_temper_kv_write_kernel(
    TA* __restrict__ qkv, const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    float temp_coef, int temp_every, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
    const int32_t* __restrict__ page_table, int table_width, TC* __restrict__ k_pages, TC* __restrict__ v_pages,
    int tokens, int heads, int kv_heads, int dim, int vdim, int page_size) {
    const int lane = threadIdx.x & (RI_WAVE - 1);
    const int all_heads = heads + 2 * kv_heads;
    const long item = (long)blockIdx.x * (blockDim.x / RI_WAVE) + threadIdx.x / RI_WAVE;
    if (item >= (long)tokens * all_heads) return;          // whole wavefront leaves together
    const int t = (int)(item / all_heads), hh = (int)(item % all_heads);
    const size_t row_len = (size_t)(heads + kv_heads) * dim + (size_t)kv_heads * vdim;
    TA* row = qkv + (size_t)t * row_len;
    const int pos = tok_pos[t];
    const int page = page_table[(size_t)tok_seq[t] * table_width + pos / page_size];
    if (hh >= heads + kv_heads) {
        const int kvh = hh - heads - kv_heads;
        const TA* x = row + (size_t)(heads + kv_heads) * dim + (size_t)kvh * vdim;
        TC* vt = v_pages + ((size_t)page * kv_heads + kvh) * page_size * vdim + pos % page_size;
        for (int d = lane; d < vdim; d += RI_WAVE) from_f32(vt + (size_t)d * page_size, to_f32(x[d]));
        return;
    }
    TA* x = row + (size_t)hh * dim;
    float v[QT_MAX_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < QT_MAX_PER_LANE; ++j) {
        const int i = lane + j * RI_WAVE;
        v[j] = i < dim ? to_f32(x[i]) : 0.f;
        ss += v[j] * v[j];
    }
    const bool is_q = hh < heads;
    const float* gain = is_q ? q_gain : k_gain;
    float f = 1.0f;
    if (gain) f = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
    float temper = 1.0f;
    if (is_q && temp_coef != 0.f) temper = 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
    TC* dst = is_q ? nullptr
                   : k_pages + (((size_t)page * kv_heads + (hh - heads)) * page_size + pos % page_size) * dim;
#pragma unroll
    for (int j = 0; j < QT_MAX_PER_LANE; ++j) {
        const int i = lane + j * RI_WAVE;
        if (i >= dim) continue;
        float a = v[j];
        if (gain) a = a * f * gain[i];
        if (is_q) from_f32(x + i, a * temper);
        else      from_f32(dst + i, a);
    }
}

extern "C" int ri_qk_norm_temper_kv_write(void* qkv, int act_dtype, const float* q_gain, const float* k_gain, float eps,
                                          float temp_coef, int temp_every, const int32_t* tok_pos,
                                          const int32_t* tok_seq, const int32_t* page_table, int table_width,
                                          void* k_pages, void* v_pages, int cache_dtype, int tokens, int heads,
                                          int kv_heads, int dim, int vdim, int page_size, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0, "qk_norm_temper_kv_write: tokens %d, heads %d, kv heads %d", tokens,
               heads, kv_heads);
    RI_REQUIRE(dim >= 1 && dim <= RI_WAVE * QT_MAX_PER_LANE && vdim >= 1, "qk_norm_temper_kv_write: head sizes %d and %d",
               dim, vdim);
    RI_REQUIRE(act_dtype == cache_dtype && (act_dtype == RI_F32 || act_dtype == RI_BF16),
               "qk_norm_temper_kv_write: activations (%d) and cache (%d) must share float32 or bfloat16", act_dtype,
               cache_dtype);
    RI_REQUIRE(temp_coef == 0.f || temp_every >= 1, "qk_norm_temper_kv_write: a temperature every %d positions", temp_every);
    RI_REQUIRE(page_size > 0 && table_width > 0 && k_pages && v_pages, "qk_norm_temper_kv_write: page geometry");
    const long items = (long)tokens * (heads + 2 * kv_heads);
    const long blocks = (items + 3) / 4;
    RI_REQUIRE(blocks <= 2147483647L, "qk_norm_temper_kv_write: %ld heads exceed one launch", items);
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == RI_F32)
        qk_norm_temper_kv_write_kernel<float, float><<<(unsigned)blocks, 256, 0, s>>>(
            (float*)qkv, q_gain, k_gain, eps, temp_coef, temp_every, tok_pos, tok_seq, page_table, table_width,
            (float*)k_pages, (float*)v_pages, tokens, heads, kv_heads, dim, vdim, page_size);
    else
        qk_norm_temper_kv_write_kernel<bf16_t, bf16_t><<<(unsigned)blocks, 256, 0, s>>>(
            (bf16_t*)qkv, q_gain, k_gain, eps, temp_coef, temp_every, tok_pos, tok_seq, page_table, table_width,
            (bf16_t*)k_pages, (bf16_t*)v_pages, tokens, heads, kv_heads, dim, vdim, page_size);
    RI_LAUNCH_CHECK("qk_norm_temper_kv_write");
    return 0;
}
