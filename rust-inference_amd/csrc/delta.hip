// The gated delta rule: a mixer that keeps, per sequence and head, a float32 state S of dim x vdim and the last
// inputs of three short convolutions.
//
// Per token, with q and k shared by heads / kv_heads value heads each:
//     x <- silu(causal convolution over time of the projection, per channel)       for q, k and v
//     q <- q / sqrt(sum q^2 + 1e-6) * dim^(-1/2),   k <- k / sqrt(sum k^2 + 1e-6)      per head
//     beta = sigmoid(b),   g = exp(-exp(A_log) * softplus(a + dt_bias))               per value head
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q.
// Everything after the projections is float32.  ri_delta_prepare makes q, k, v, g and beta of all tokens of a step
// (one workgroup a token), ri_delta_tails then moves the convolutions' last inputs into the sequences' state, and
// ri_delta_scan walks every sequence's tokens in order.  A token's sums are taken in the same order whatever step
// or block of tokens it falls into.
#include "api.h"
#include "common.h"

#define DELTA_MAX_TAPS 16

__device__ __forceinline__ float silu_f(float v) { return v / (1.f + expf(-v)); }
__device__ __forceinline__ float softplus_f(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// One workgroup a token.  conv[] (dynamic LDS, channels floats) holds the token's activated convolutions.
template <typename T>
__global__ void __launch_bounds__(256)
delta_prepare_kernel(float* __restrict__ qkv, float* __restrict__ gates, const T* __restrict__ proj, int row, int q_off,
                     const float* __restrict__ taps, int ntaps, const float* __restrict__ tails,
                     const float* __restrict__ ab, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                     const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ cu_seqlens,
                     const int32_t* __restrict__ slots, int heads, int kv_heads, int dim, int vdim) {
    extern __shared__ float conv[];
    const int t = blockIdx.x, b = tok_seq[t];
    const int i = t - cu_seqlens[b];                          // the token's place among its sequence's new tokens
    const int qk = kv_heads * dim, channels = 2 * qk + heads * vdim;
    const float* tail = tails + (size_t)slots[b] * (ntaps - 1) * channels;
    for (int c = threadIdx.x; c < channels; c += blockDim.x) {
        float y = 0.f;
        for (int d = ntaps - 1; d >= 0; --d) {                // oldest input first
            const int at = i - d;
            const float x = at >= 0 ? to_f32(proj[(size_t)(t - d) * row + q_off + c])
                                    : tail[(size_t)(ntaps - 1 + at) * channels + c];
            y += taps[(size_t)c * ntaps + (ntaps - 1 - d)] * x;
        }
        conv[c] = silu_f(y);
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    float* out = qkv + (size_t)t * channels;
    for (int h = wave; h < 2 * kv_heads; h += waves) {        // q heads, then k heads
        const float* x = conv + (size_t)h * dim;
        float ss = 0.f;
        for (int d = lane; d < dim; d += 64) ss += x[d] * x[d];
        ss = wave_sum(ss);
        const float f = (h < kv_heads ? rsqrtf((float)dim) : 1.f) / sqrtf(ss + 1e-6f);
        for (int d = lane; d < dim; d += 64) out[(size_t)h * dim + d] = x[d] * f;
    }
    for (int c = 2 * qk + threadIdx.x; c < channels; c += blockDim.x) out[c] = conv[c];
    if (threadIdx.x < heads) {
        const int h = threadIdx.x;
        const float a = ab[(size_t)t * 2 * heads + h], bb = ab[(size_t)t * 2 * heads + heads + h];
        gates[(size_t)t * 2 * heads + h] = expf(-expf(a_log[h]) * softplus_f(a + dt_bias[h]));
        gates[(size_t)t * 2 * heads + heads + h] = 1.f / (1.f + expf(-bb));
    }
}

// The last ntaps - 1 inputs of every sequence after this step's n tokens: row r of the new tail is entry n + r of
// (old tail, then the step's inputs).  One thread a (sequence, channel): it reads all it needs before it writes.
template <typename T>
__global__ void __launch_bounds__(256)
delta_tails_kernel(float* __restrict__ tails, const T* __restrict__ proj, int row, int q_off, int ntaps,
                   const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots, int channels) {
    const int b = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0, keep = ntaps - 1;
    float* tail = tails + (size_t)slots[b] * keep * channels;
    float v[DELTA_MAX_TAPS];
    for (int r = 0; r < keep; ++r) {
        const int at = n + r;                                 // place in (old tail, new inputs)
        v[r] = at < keep ? tail[(size_t)at * channels + c] : to_f32(proj[(size_t)(t0 + at - keep) * row + q_off + c]);
    }
    for (int r = 0; r < keep; ++r) tail[(size_t)r * channels + c] = v[r];
}

// The walk.  A workgroup owns one (sequence, value head) and 64 columns of its state: 64 columns x 4 slices of
// rows; a thread keeps RPT rows of one column in registers (rows r * RPT ..+RPT of slice r; rows past dim are
// zeros that stay zeros).  Tokens come through LDS in blocks of DELTA_BLOCK, the next block's loads in flight
// while a block is walked.  The two sums over rows of a token meet over the four lanes of a column.
template <int RPT>
struct DeltaLds {
    static constexpr int DELTA_BLOCK = RPT >= 64 ? 8 : 16;    // tokens a block: two buffers stay inside 64 KB
    static constexpr int QS = RPT + 4;                        // stride of a slice of q or k: no bank conflicts between the four slices
    float q[DELTA_BLOCK][4][QS];
    float k[DELTA_BLOCK][4][QS];
    float v[DELTA_BLOCK][64];
    float g[DELTA_BLOCK], beta[DELTA_BLOCK];
};

template <int RPT>
__global__ void __launch_bounds__(256)
delta_scan_kernel(float* __restrict__ out, const float* __restrict__ qkv, const float* __restrict__ gates,
                  float* __restrict__ state, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots,
                  int heads, int kv_heads, int dim, int vdim) {
    __shared__ DeltaLds<RPT> lds[2];
    constexpr int DELTA_BLOCK = DeltaLds<RPT>::DELTA_BLOCK;
    constexpr int QR = DELTA_BLOCK * 4 * RPT / 256;           // elements of q (and of k) a thread fetches per block
    constexpr int VR = DELTA_BLOCK * 64 / 256;
    const int b = blockIdx.x / heads, h = blockIdx.x % heads, col0 = blockIdx.y * 64;
    const int hq = h / (heads / kv_heads);
    const int tid = threadIdx.x, r = tid & 3, col = col0 + (tid >> 2);
    const bool has_col = col < vdim;
    const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0;
    if (n <= 0) return;
    const int qk = kv_heads * dim, channels = 2 * qk + heads * vdim;
    float* st = state + (((size_t)slots[b] * heads + h) * dim) * vdim;

    float S[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int rw = r * RPT + i;
        S[i] = (has_col && rw < dim) ? st[(size_t)rw * vdim + col] : 0.f;
    }

    float fq[QR], fk[QR], fv[VR], fg = 0.f;
    auto fetch = [&](int first) {                             // the block of tokens first ..+DELTA_BLOCK, into registers
#pragma unroll
        for (int e = 0; e < QR; ++e) {
            const int at = e * 256 + tid, tk = at / (4 * RPT), rw = at % (4 * RPT);
            const bool ok = first + tk < n && rw < dim;
            const float* p = qkv + (size_t)(t0 + min(first + tk, n - 1)) * channels + (size_t)hq * dim + min(rw, dim - 1);
            const float a = p[0], c = p[qk];
            fq[e] = ok ? a : 0.f;
            fk[e] = ok ? c : 0.f;
        }
#pragma unroll
        for (int e = 0; e < VR; ++e) {
            const int at = e * 256 + tid, tk = at >> 6, cc = col0 + (at & 63);
            const float a = qkv[(size_t)(t0 + min(first + tk, n - 1)) * channels + 2 * qk + (size_t)h * vdim + min(cc, vdim - 1)];
            fv[e] = a;
        }
        if (tid < 2 * DELTA_BLOCK) {
            const int tk = tid >> 1;
            fg = gates[(size_t)(t0 + min(first + tk, n - 1)) * 2 * heads + (tid & 1) * heads + h];
        }
    };
    auto stage = [&](DeltaLds<RPT>& l) {
#pragma unroll
        for (int e = 0; e < QR; ++e) {
            const int at = e * 256 + tid, tk = at / (4 * RPT), rw = at % (4 * RPT);
            l.q[tk][rw / RPT][rw % RPT] = fq[e];
            l.k[tk][rw / RPT][rw % RPT] = fk[e];
        }
#pragma unroll
        for (int e = 0; e < VR; ++e) {
            const int at = e * 256 + tid;
            l.v[at >> 6][at & 63] = fv[e];
        }
        if (tid < 2 * DELTA_BLOCK) {
            if (tid & 1) l.beta[tid >> 1] = fg; else l.g[tid >> 1] = fg;
        }
    };

    fetch(0);
    stage(lds[0]);
    __syncthreads();
    int cur = 0;
    for (int first = 0; first < n; first += DELTA_BLOCK) {
        const bool more = first + DELTA_BLOCK < n;
        fetch(more ? first + DELTA_BLOCK : first);            // (always issued: no load in a branch)
        const DeltaLds<RPT>& l = lds[cur];
        const int count = min(DELTA_BLOCK, n - first);
        for (int tk = 0; tk < count; ++tk) {
            const float g = l.g[tk], beta = l.beta[tk];
            float kk[RPT], dot = 0.f;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                kk[i] = l.k[tk][r][i];
                S[i] *= g;
                dot += S[i] * kk[i];
            }
            dot += __shfl_xor(dot, 1, RI_WAVE);
            dot += __shfl_xor(dot, 2, RI_WAVE);
            const float u = beta * (l.v[tk][tid >> 2] - dot);
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                S[i] += kk[i] * u;
                o += S[i] * l.q[tk][r][i];
            }
            o += __shfl_xor(o, 1, RI_WAVE);
            o += __shfl_xor(o, 2, RI_WAVE);
            if (r == 0 && has_col) out[(size_t)(t0 + first + tk) * heads * vdim + (size_t)h * vdim + col] = o;
        }
        stage(lds[cur ^ 1]);
        __syncthreads();
        cur ^= 1;
    }
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int rw = r * RPT + i;
        if (has_col && rw < dim) st[(size_t)rw * vdim + col] = S[i];
    }
}

extern "C" int ri_delta_prepare(float* qkv, float* gates, const void* proj, int act_dtype, int row, int q_off,
                                const float* taps, int ntaps, float* tails, const float* ab, const float* a_log,
                                const float* dt_bias, const int32_t* tok_seq, const int32_t* cu_seqlens,
                                const int32_t* slots, int seqs, int tokens, int heads, int kv_heads, int dim, int vdim,
                                void* stream) {
    RI_REQUIRE(tokens > 0 && seqs > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0,
               "delta_prepare: tokens %d, sequences %d, heads %d, kv heads %d of %d x %d", tokens, seqs, heads, kv_heads,
               dim, vdim);
    RI_REQUIRE(heads <= 256, "delta_prepare: %d heads, the kernel takes up to 256", heads);
    RI_REQUIRE(ntaps >= 1 && ntaps <= DELTA_MAX_TAPS, "delta_prepare: %d taps, the kernels take 1 to %d", ntaps, DELTA_MAX_TAPS);
    const long channels = 2L * kv_heads * dim + (long)heads * vdim;
    RI_REQUIRE(q_off >= 0 && q_off + channels <= row, "delta_prepare: %ld channels at column %d of rows of %d", channels, q_off, row);
    RI_REQUIRE(channels * 4 <= 64 * 1024, "delta_prepare: %ld channels exceed the workgroup's memory", channels);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "delta_prepare: dtype %d", act_dtype);
    hipStream_t s = (hipStream_t)stream;
    const size_t shared = (size_t)channels * sizeof(float);
    if (act_dtype == RI_F32) {
        delta_prepare_kernel<float><<<tokens, 256, shared, s>>>(qkv, gates, (const float*)proj, row, q_off, taps, ntaps, tails,
                                                               ab, a_log, dt_bias, tok_seq, cu_seqlens, slots, heads,
                                                               kv_heads, dim, vdim);
    } else {
        delta_prepare_kernel<bf16_t><<<tokens, 256, shared, s>>>(qkv, gates, (const bf16_t*)proj, row, q_off, taps, ntaps,
                                                                tails, ab, a_log, dt_bias, tok_seq, cu_seqlens, slots,
                                                                heads, kv_heads, dim, vdim);
    }
    RI_LAUNCH_CHECK("delta_prepare");
    if (ntaps > 1) {
        const dim3 grid((unsigned)((channels + 255) / 256), seqs);
        if (act_dtype == RI_F32)
            delta_tails_kernel<float><<<grid, 256, 0, s>>>(tails, (const float*)proj, row, q_off, ntaps, cu_seqlens, slots, (int)channels);
        else
            delta_tails_kernel<bf16_t><<<grid, 256, 0, s>>>(tails, (const bf16_t*)proj, row, q_off, ntaps, cu_seqlens, slots, (int)channels);
        RI_LAUNCH_CHECK("delta_tails");
    }
    return 0;
}

extern "C" int ri_delta_max_dim() { return 256; }

extern "C" int ri_delta_scan(float* out, const float* qkv, const float* gates, float* state, const int32_t* cu_seqlens,
                             const int32_t* slots, int seqs, int tokens, int heads, int kv_heads, int dim, int vdim,
                             void* stream) {
    RI_REQUIRE(tokens > 0 && seqs > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && vdim > 0,
               "delta_scan: tokens %d, sequences %d, heads %d, kv heads %d", tokens, seqs, heads, kv_heads);
    RI_REQUIRE(dim >= 1 && dim <= 256, "delta_scan: key heads of %d, the kernel takes 1 to 256", dim);
    RI_REQUIRE((long)seqs * heads <= 2147483647L && (vdim + 63) / 64 <= 65535, "delta_scan: the grid");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)(seqs * heads), (unsigned)((vdim + 63) / 64));
    const int need = (dim + 3) / 4;
#define RI_DELTA_GO(R) delta_scan_kernel<R><<<grid, 256, 0, s>>>(out, qkv, gates, state, cu_seqlens, slots, heads, kv_heads, dim, vdim)
    if (need <= 4) RI_DELTA_GO(4);
    else if (need <= 8) RI_DELTA_GO(8);
    else if (need <= 16) RI_DELTA_GO(16);
    else if (need <= 32) RI_DELTA_GO(32);
    else RI_DELTA_GO(64);
#undef RI_DELTA_GO
    RI_LAUNCH_CHECK("delta_scan");
    return 0;
}
