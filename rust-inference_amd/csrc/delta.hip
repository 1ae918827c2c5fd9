// The gated delta rule: a mixer that keeps, per sequence and head, a float32 state S of dim x vdim and the last
// inputs of three short convolutions.
//
// Per token, with q and k shared by heads / kv_heads value heads each:
//     x <- silu(causal convolution over time of the projection, per channel)       for q, k and v
//     q <- q / sqrt(sum q^2 + 1e-6) * dim^(-1/2),   k <- k / sqrt(sum k^2 + 1e-6)      per head
//     beta = sigmoid(b),   g = exp(-exp(A_log) * softplus(a + dt_bias))               per value head
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q.
// Everything after the projections is float32.  ri_delta_prepare makes q, k, v, g and beta of all tokens of a step
// (a workgroup a token and head), ri_delta_tails then moves the convolutions' last inputs into the sequences' state, and
// ri_delta_scan walks every sequence's tokens in order.  A token's sums are taken in the same order whatever step
// or block of tokens it falls into.
#include "api.h"
#include "common.h"

#define DELTA_MAX_TAPS 16

__device__ __forceinline__ float silu_f(float v) { return v / (1.f + expf(-v)); }
__device__ __forceinline__ float softplus_f(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// A workgroup takes one token and one unit of its channels: a q or k head (units 0 .. 2 kv_heads - 1), which it
// norms, or a stretch of DELTA_V_UNIT channels of v.  conv[] (dynamic LDS, max(dim, DELTA_V_UNIT) floats) holds the
// unit's activated convolutions.  (One workgroup a token walked its thousands of channels in turns of 256, each
// turn waiting for its own loads: 22 us for a single token.)
#define DELTA_V_UNIT 256

template <typename T>
__global__ void __launch_bounds__(256)
delta_prepare_kernel(float* __restrict__ qkv, float* __restrict__ gates, const T* __restrict__ proj, int row, int q_off,
                     const float* __restrict__ taps, int ntaps, const float* __restrict__ tails,
                     const float* __restrict__ ab, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                     const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ cu_seqlens,
                     const int32_t* __restrict__ slots, int heads, int kv_heads, int dim, int vdim) {
    extern __shared__ float conv[];
    __shared__ float scratch[16];
    const int t = blockIdx.x, unit = blockIdx.y, b = tok_seq[t];
    const int i = t - cu_seqlens[b];                          // the token's place among its sequence's new tokens
    const int qk = kv_heads * dim, channels = 2 * qk + heads * vdim;
    const bool normed = unit < 2 * kv_heads;
    const int first = normed ? unit * dim : 2 * qk + (unit - 2 * kv_heads) * DELTA_V_UNIT;
    const int count = normed ? dim : min(DELTA_V_UNIT, channels - first);
    const float* tail = tails + (size_t)slots[b] * (ntaps - 1) * channels;
    if (ntaps <= 4) {
        // the usual few taps: all inputs asked for at once, whatever their place (an address that is not used is
        // pulled back to one that exists), so that no load waits for another
        const float* tail_safe = ntaps > 1 ? tail : taps;
        for (int e = threadIdx.x; e < count; e += blockDim.x) {
            const int c = first + e;
            float x[4], w[4];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const int at = i - d;
                const float a = to_f32(proj[(size_t)(t - min(d, i)) * row + q_off + c]);
                const float bb = tail_safe[(size_t)min(max(ntaps - 1 + at, 0), max(ntaps - 2, 0)) * channels + c];
                x[d] = at >= 0 ? a : bb;
                w[d] = d < ntaps ? taps[(size_t)c * ntaps + max(ntaps - 1 - d, 0)] : 0.f;
            }
            float y = 0.f;
#pragma unroll
            for (int d = 3; d >= 0; --d) y += d < ntaps ? w[d] * x[d] : 0.f;           // oldest input first
            conv[e] = silu_f(y);
        }
    } else {
        for (int e = threadIdx.x; e < count; e += blockDim.x) {
            const int c = first + e;
            float y = 0.f;
            for (int d = ntaps - 1; d >= 0; --d) {                // oldest input first
                const int at = i - d;
                const float x = at >= 0 ? to_f32(proj[(size_t)(t - d) * row + q_off + c])
                                        : tail[(size_t)(ntaps - 1 + at) * channels + c];
                y += taps[(size_t)c * ntaps + (ntaps - 1 - d)] * x;
            }
            conv[e] = silu_f(y);
        }
    }
    __syncthreads();
    float* out = qkv + (size_t)t * channels + first;
    if (normed) {                                             // a q head (also times dim^(-1/2)) or a k head
        float ss = 0.f;
        for (int e = threadIdx.x; e < count; e += blockDim.x) ss += conv[e] * conv[e];
        ss = block_sum(ss, scratch);
        const float f = (unit < kv_heads ? rsqrtf((float)dim) : 1.f) / sqrtf(ss + 1e-6f);
        for (int e = threadIdx.x; e < count; e += blockDim.x) out[e] = conv[e] * f;
    } else {
        for (int e = threadIdx.x; e < count; e += blockDim.x) out[e] = conv[e];
    }
    if (unit == 0 && threadIdx.x < heads) {
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

// The sum over the four lanes of a quad, in each of them, by two quad permutations of the vector unit's own data
// path (DPP): [1, 0, 3, 2] then [2, 3, 0, 1].  A shuffle goes through the LDS crossbar instead, and the walk waits
// for four of them in a row at every token.
__device__ __forceinline__ float quad_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));
    return v;
}

// The same over the SL = 4 or 8 lanes of a column: after the quads, the mirror image inside every eight lanes
// (lane i takes lane 7 - i: the other quad, all of whose lanes hold its sum).
template <int SL>
__device__ __forceinline__ float slices_sum(float v) {
    v = quad_sum(v);
    if (SL == 8) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));
    return v;
}

// The walk.  A workgroup owns one (sequence, value head) and 256 / SL columns of its state: that many columns x SL
// slices of rows (4 or 8); a thread keeps RPT rows of one column in registers (rows r * RPT ..+RPT of slice r; rows
// past dim are zeros that stay zeros).  Tokens come through LDS in blocks of DELTA_BLOCK, the next block's loads in
// flight while a block is walked.  The two sums over rows of a token meet over the SL lanes of a column.  A token costs
// a wavefront 4 RPT vector instructions and nothing hides them, so eight slices halve a token's time; they also
// double the workgroups that each stage q and k, which is what counts once the machine is full: the launch chooses.
template <int RPT, int SL>
struct DeltaLds {
    static constexpr int DELTA_BLOCK = RPT * SL >= 256 ? 8 : 16;    // tokens a block: two buffers stay inside 64 KB
    static constexpr int QS = RPT + 4;                        // stride of a slice of q or k: no bank conflicts between the slices
    static constexpr int COLS = 256 / SL;
    float q[DELTA_BLOCK][SL][QS];
    float k[DELTA_BLOCK][SL][QS];
    float v[DELTA_BLOCK][COLS];
    float g[DELTA_BLOCK], beta[DELTA_BLOCK];
};

template <int RPT, int SL>
__global__ void __launch_bounds__(256)
delta_scan_kernel(float* __restrict__ out, const float* __restrict__ qkv, const float* __restrict__ gates,
                  float* __restrict__ state, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots,
                  int heads, int kv_heads, int dim, int vdim) {
    __shared__ DeltaLds<RPT, SL> lds[2];
    constexpr int DELTA_BLOCK = DeltaLds<RPT, SL>::DELTA_BLOCK, COLS = DeltaLds<RPT, SL>::COLS;
    constexpr int QR = DELTA_BLOCK * SL * RPT / 256;          // elements of q (and of k) a thread fetches per block
    constexpr int VR = DELTA_BLOCK * COLS / 256;
    const int b = blockIdx.x / heads, h = blockIdx.x % heads, col0 = blockIdx.y * COLS;
    const int hq = h / (heads / kv_heads);
    const int tid = threadIdx.x, r = tid & (SL - 1), col = col0 + tid / SL;
    const bool has_col = col < vdim;
    const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0;
    if (n <= 0) return;
    const int qk = kv_heads * dim, channels = 2 * qk + heads * vdim;
    float* st = state + (((size_t)slots[b] * heads + h) * dim) * vdim;

    float S[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        // (no load in a branch: the address is pulled back inside the state and the value dropped afterwards)
        const int rw = r * RPT + i;
        const float v = st[(size_t)min(rw, dim - 1) * vdim + min(col, vdim - 1)];
        S[i] = (has_col && rw < dim) ? v : 0.f;
    }

    float fq[QR], fk[QR], fv[VR], fg = 0.f;
    auto fetch = [&](int first) {                             // the block of tokens first ..+DELTA_BLOCK, into registers
#pragma unroll
        for (int e = 0; e < QR; ++e) {
            const int at = e * 256 + tid, tk = at / (SL * RPT), rw = at % (SL * RPT);
            const bool ok = first + tk < n && rw < dim;
            const float* p = qkv + (size_t)(t0 + min(first + tk, n - 1)) * channels + (size_t)hq * dim + min(rw, dim - 1);
            const float a = p[0], c = p[qk];
            fq[e] = ok ? a : 0.f;
            fk[e] = ok ? c : 0.f;
        }
#pragma unroll
        for (int e = 0; e < VR; ++e) {
            const int at = e * 256 + tid, tk = at / COLS, cc = col0 + at % COLS;
            const float a = qkv[(size_t)(t0 + min(first + tk, n - 1)) * channels + 2 * qk + (size_t)h * vdim + min(cc, vdim - 1)];
            fv[e] = a;
        }
        if (tid < 2 * DELTA_BLOCK) {
            const int tk = tid >> 1;
            fg = gates[(size_t)(t0 + min(first + tk, n - 1)) * 2 * heads + (tid & 1) * heads + h];
        }
    };
    auto stage = [&](DeltaLds<RPT, SL>& l) {
#pragma unroll
        for (int e = 0; e < QR; ++e) {
            const int at = e * 256 + tid, tk = at / (SL * RPT), rw = at % (SL * RPT);
            l.q[tk][rw / RPT][rw % RPT] = fq[e];
            l.k[tk][rw / RPT][rw % RPT] = fk[e];
        }
#pragma unroll
        for (int e = 0; e < VR; ++e) {
            const int at = e * 256 + tid;
            l.v[at / COLS][at % COLS] = fv[e];
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
        const DeltaLds<RPT, SL>& l = lds[cur];
        const int count = min(DELTA_BLOCK, n - first);
#pragma unroll 2
        for (int tk = 0; tk < count; ++tk) {
            const float g = l.g[tk], beta = l.beta[tk];
            // four partial sums each: a single one would be a chain of RPT dependent additions
            float kk[RPT], d4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                kk[i] = l.k[tk][r][i];
                S[i] *= g;
                d4[i & 3] += S[i] * kk[i];
            }
            const float dot = slices_sum<SL>((d4[0] + d4[1]) + (d4[2] + d4[3]));
            const float u = beta * (l.v[tk][tid / SL] - dot);
            float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                S[i] += kk[i] * u;
                o4[i & 3] += S[i] * l.q[tk][r][i];
            }
            const float o = slices_sum<SL>((o4[0] + o4[1]) + (o4[2] + o4[3]));
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

// One new token a sequence: the convolutions, the unit norms, the gates, the step on the state, the per-head norm
// and the output gate in one kernel.  A workgroup owns one (sequence, head): `groups` threads across a row of the
// state, four columns each (16-byte loads and stores of whole lines), x 256 / groups slices of rows, a thread RPT rows
// in registers.  The sums over rows meet through LDS, slice after slice.  The convolutions' tails are read here and
// moved on by delta_tails_kernel afterwards (the heads that share a q/k head all read its tail).
template <typename T, int RPT>
__global__ void __launch_bounds__(256)
delta_step_kernel(T* __restrict__ out, const T* __restrict__ proj, int row, int q_off, int g_off,
                  const float* __restrict__ taps, int ntaps, const float* __restrict__ tails, const float* __restrict__ ab,
                  const float* __restrict__ a_log, const float* __restrict__ dt_bias, float* __restrict__ state,
                  const int32_t* __restrict__ slots, const float* __restrict__ gain, float eps, int heads, int kv_heads,
                  int dim, int vdim, int groups) {
    __shared__ float qs[256], ks[256], vs[256], scratch[16];
    __shared__ float4 part[256];
    const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int hq = h / (heads / kv_heads), slot = slots[b];
    const int grp = tid % groups, r = tid / groups, slices = 256 / groups, c0 = grp * 4;
    const bool has_col = c0 < vdim;                           // vdim is a multiple of 4: all four columns or none
    const int qk = kv_heads * dim, channels = 2 * qk + heads * vdim;
    float* st = state + (((size_t)slot * heads + h) * dim) * vdim;
    float4 S[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        // (no load in a branch: the address is pulled back inside the state and the value dropped afterwards)
        const int rw = r * RPT + i;
        const float4 v = *reinterpret_cast<const float4*>(st + (size_t)min(rw, dim - 1) * vdim + min(c0, vdim - 4));
        S[i] = (has_col && rw < dim) ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    const T* x = proj + (size_t)b * row;
    const float* tail = tails + (size_t)slot * (ntaps - 1) * channels;
    // everything the end of the kernel reads from memory is asked for here, so that no load is waited for on its own
    const float a_in = ab[(size_t)b * 2 * heads + h], b_in = ab[(size_t)b * 2 * heads + heads + h];
    const float a_exp = a_log[h], a_bias = dt_bias[h];
    float gate[4], gain_c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        gate[j] = to_f32(x[g_off + h * vdim + min(c0, vdim - 4) + j]);
        gain_c[j] = gain[min(c0, vdim - 4) + j];
    }
    for (int e = tid; e < 2 * dim + vdim; e += 256) {
        const int ch = e < dim ? hq * dim + e : e < 2 * dim ? qk + hq * dim + (e - dim) : 2 * qk + h * vdim + (e - 2 * dim);
        float y = 0.f;
        if (ntaps <= 4) {                                     // the usual few taps: every load asked for before any is used
            const float* tail_safe = ntaps > 1 ? tail : taps;
            float xv[3], wv[3];
#pragma unroll
            for (int d = 1; d <= 3; ++d) {
                xv[d - 1] = tail_safe[(size_t)max(ntaps - 1 - d, 0) * channels + ch];
                wv[d - 1] = taps[(size_t)ch * ntaps + max(ntaps - 1 - d, 0)];
            }
            const float w0 = taps[(size_t)ch * ntaps + ntaps - 1], x0 = to_f32(x[q_off + ch]);
#pragma unroll
            for (int d = 3; d >= 1; --d) y += d < ntaps ? wv[d - 1] * xv[d - 1] : 0.f;
            y += w0 * x0;
        } else {
            for (int d = ntaps - 1; d >= 1; --d) y += taps[(size_t)ch * ntaps + (ntaps - 1 - d)] * tail[(size_t)(ntaps - 1 - d) * channels + ch];
            y += taps[(size_t)ch * ntaps + ntaps - 1] * to_f32(x[q_off + ch]);
        }
        const float a = silu_f(y);
        if (e < dim) qs[e] = a; else if (e < 2 * dim) ks[e - dim] = a; else vs[e - 2 * dim] = a;
    }
    __syncthreads();
    float sq = 0.f, sk = 0.f;
    for (int e = tid; e < dim; e += 256) {
        sq += qs[e] * qs[e];
        sk += ks[e] * ks[e];
    }
    sq = block_sum(sq, scratch);
    sk = block_sum(sk, scratch);
    const float fq = rsqrtf((float)dim) / sqrtf(sq + 1e-6f), fk = 1.f / sqrtf(sk + 1e-6f);
    const float g = expf(-expf(a_exp) * softplus_f(a_in + a_bias));
    const float beta = 1.f / (1.f + expf(-b_in));
    float kk[RPT];
    float4 d = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int rw = r * RPT + i;
        kk[i] = rw < dim ? ks[rw] * fk : 0.f;
        S[i].x *= g; S[i].y *= g; S[i].z *= g; S[i].w *= g;
        d.x += S[i].x * kk[i]; d.y += S[i].y * kk[i]; d.z += S[i].z * kk[i]; d.w += S[i].w * kk[i];
    }
    part[tid] = d;
    __syncthreads();
    float4 dot = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j = 0; j < slices; ++j) {                        // slice after slice: the same order for every column
        const float4 p = part[j * groups + grp];
        dot.x += p.x; dot.y += p.y; dot.z += p.z; dot.w += p.w;
    }
    const int cv = min(c0, vdim - 4);
    const float4 u = make_float4(beta * (vs[cv] - dot.x), beta * (vs[cv + 1] - dot.y), beta * (vs[cv + 2] - dot.z),
                                 beta * (vs[cv + 3] - dot.w));
    __syncthreads();                                          // part is written again
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int rw = r * RPT + i;
        const float qq = rw < dim ? qs[rw] * fq : 0.f;
        S[i].x += kk[i] * u.x; S[i].y += kk[i] * u.y; S[i].z += kk[i] * u.z; S[i].w += kk[i] * u.w;
        o.x += S[i].x * qq; o.y += S[i].y * qq; o.z += S[i].z * qq; o.w += S[i].w * qq;
        if (has_col && rw < dim) *reinterpret_cast<float4*>(st + (size_t)rw * vdim + c0) = S[i];
    }
    part[tid] = o;
    __syncthreads();
    o = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j = 0; j < slices; ++j) {
        const float4 p = part[j * groups + grp];
        o.x += p.x; o.y += p.y; o.z += p.z; o.w += p.w;
    }
    const float ss = block_sum((r == 0 && has_col) ? (o.x * o.x + o.y * o.y) + (o.z * o.z + o.w * o.w) : 0.f, scratch);
    if (r == 0 && has_col) {
        const float inv = 1.f / sqrtf(ss / (float)vdim + eps);
        T* to = out + (size_t)b * heads * vdim + (size_t)h * vdim + c0;
        from_f32(to, o.x * inv * gain_c[0] * silu_f(gate[0]));
        from_f32(to + 1, o.y * inv * gain_c[1] * silu_f(gate[1]));
        from_f32(to + 2, o.z * inv * gain_c[2] * silu_f(gate[2]));
        from_f32(to + 3, o.w * inv * gain_c[3] * silu_f(gate[3]));
    }
}

static int delta_step_cols(int vdim) {
    int cols = 32;
    while (cols < vdim) cols *= 2;
    return cols;
}

extern "C" int ri_delta_step_fits(int dim, int vdim) {
    if (dim < 1 || dim > 256 || vdim < 4 || vdim > 256 || vdim % 4) return 0;
    const int slices = 256 / (delta_step_cols(vdim) / 4);
    return (dim + slices - 1) / slices <= 16;
}

extern "C" int ri_delta_step(void* out, const void* proj, int act_dtype, int row, int q_off, int g_off, const float* taps,
                             int ntaps, float* tails, const float* ab, const float* a_log, const float* dt_bias,
                             float* state, const int32_t* cu_seqlens, const int32_t* slots, const float* gain, float eps,
                             int seqs, int heads, int kv_heads, int dim, int vdim, void* stream) {
    RI_REQUIRE(seqs > 0 && seqs <= 65535 && heads > 0 && heads <= 65535 && kv_heads > 0 && heads % kv_heads == 0,
               "delta_step: %d sequences, %d heads, %d kv heads", seqs, heads, kv_heads);
    RI_REQUIRE(ri_delta_step_fits(dim, vdim), "delta_step: heads of %d x %d", dim, vdim);
    RI_REQUIRE(ntaps >= 1 && ntaps <= DELTA_MAX_TAPS, "delta_step: %d taps, the kernels take 1 to %d", ntaps, DELTA_MAX_TAPS);
    const long channels = 2L * kv_heads * dim + (long)heads * vdim;
    RI_REQUIRE(q_off >= 0 && q_off + channels <= row && g_off >= 0 && g_off + (long)heads * vdim <= row,
               "delta_step: %ld channels at column %d and the gate at %d of rows of %d", channels, q_off, g_off, row);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "delta_step: dtype %d", act_dtype);
    hipStream_t s = (hipStream_t)stream;
    const int groups = delta_step_cols(vdim) / 4, slices = 256 / groups, rpt = (dim + slices - 1) / slices;
    const dim3 grid(heads, seqs);
#define RI_DSTEP_GO(T, R) delta_step_kernel<T, R><<<grid, 256, 0, s>>>((T*)out, (const T*)proj, row, q_off, g_off, taps, ntaps, \
                                                                    tails, ab, a_log, dt_bias, state, slots, gain, eps, heads,   \
                                                                    kv_heads, dim, vdim, groups)
    if (act_dtype == RI_F32) {
        if (rpt <= 4) RI_DSTEP_GO(float, 4); else if (rpt <= 8) RI_DSTEP_GO(float, 8); else RI_DSTEP_GO(float, 16);
    } else {
        if (rpt <= 4) RI_DSTEP_GO(bf16_t, 4); else if (rpt <= 8) RI_DSTEP_GO(bf16_t, 8); else RI_DSTEP_GO(bf16_t, 16);
    }
#undef RI_DSTEP_GO
    RI_LAUNCH_CHECK("delta_step");
    if (ntaps > 1) {
        const dim3 tgrid((unsigned)((channels + 255) / 256), seqs);
        if (act_dtype == RI_F32)
            delta_tails_kernel<float><<<tgrid, 256, 0, s>>>(tails, (const float*)proj, row, q_off, ntaps, cu_seqlens, slots, (int)channels);
        else
            delta_tails_kernel<bf16_t><<<tgrid, 256, 0, s>>>(tails, (const bf16_t*)proj, row, q_off, ntaps, cu_seqlens, slots, (int)channels);
        RI_LAUNCH_CHECK("delta_tails");
    }
    return 0;
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
    RI_REQUIRE(dim <= 8192, "delta_prepare: heads of %d exceed the workgroup's memory", dim);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "delta_prepare: dtype %d", act_dtype);
    hipStream_t s = (hipStream_t)stream;
    const size_t shared = (size_t)(dim > DELTA_V_UNIT ? dim : DELTA_V_UNIT) * sizeof(float);
    const int units = 2 * kv_heads + (heads * vdim + DELTA_V_UNIT - 1) / DELTA_V_UNIT;
    RI_REQUIRE(units <= 65535, "delta_prepare: %d units of channels exceed one launch", units);
    const dim3 pgrid(tokens, units);
    if (act_dtype == RI_F32) {
        delta_prepare_kernel<float><<<pgrid, 256, shared, s>>>(qkv, gates, (const float*)proj, row, q_off, taps, ntaps, tails,
                                                               ab, a_log, dt_bias, tok_seq, cu_seqlens, slots, heads,
                                                               kv_heads, dim, vdim);
    } else {
        delta_prepare_kernel<bf16_t><<<pgrid, 256, shared, s>>>(qkv, gates, (const bf16_t*)proj, row, q_off, taps, ntaps,
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
                             int slices, void* stream) {
    RI_REQUIRE(slices == 0 || slices == 4 || slices == 8, "delta_scan: %d slices of rows (4, 8, or 0 for the launch's choice)", slices);
    RI_REQUIRE(tokens > 0 && seqs > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && vdim > 0,
               "delta_scan: tokens %d, sequences %d, heads %d, kv heads %d", tokens, seqs, heads, kv_heads);
    RI_REQUIRE(dim >= 1 && dim <= 256, "delta_scan: key heads of %d, the kernel takes 1 to 256", dim);
    RI_REQUIRE((long)seqs * heads <= 2147483647L && (vdim + 31) / 32 <= 65535, "delta_scan: the grid");
    hipStream_t s = (hipStream_t)stream;
    // eight slices of rows while the workgroups of four would leave compute units idle (a token's time halves), four
    // once they fill the machine (half the workgroups stage q and k)
    const bool eight = slices ? slices == 8 : (long)seqs * heads * ((vdim + 63) / 64) <= (long)ri_compute_units() && dim >= 8;
    const int sl = eight ? 8 : 4, cols = 256 / sl;
    const dim3 grid((unsigned)(seqs * heads), (unsigned)((vdim + cols - 1) / cols));
    const int need = (dim + sl - 1) / sl;
#define RI_DELTA_GO(R, SL) delta_scan_kernel<R, SL><<<grid, 256, 0, s>>>(out, qkv, gates, state, cu_seqlens, slots, heads, kv_heads, dim, vdim)
    if (eight) {
        if (need <= 4) RI_DELTA_GO(4, 8);
        else if (need <= 8) RI_DELTA_GO(8, 8);
        else if (need <= 16) RI_DELTA_GO(16, 8);
        else RI_DELTA_GO(32, 8);
    } else {
        if (need <= 4) RI_DELTA_GO(4, 4);
        else if (need <= 8) RI_DELTA_GO(8, 4);
        else if (need <= 16) RI_DELTA_GO(16, 4);
        else if (need <= 32) RI_DELTA_GO(32, 4);
        else RI_DELTA_GO(64, 4);
    }
#undef RI_DELTA_GO
    RI_LAUNCH_CHECK("delta_scan");
    return 0;
}
