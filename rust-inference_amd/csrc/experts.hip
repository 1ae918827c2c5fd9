// A mixture of experts: the router's choice and weights, and the experts' activation.
//
// Router: s = sigmoid(z) of the float32 logits; the choice is by s + correction, the weights are the chosen
// experts' s over their sum.  The experts themselves are products: every expert's gate and up branch side by side
// in one matrix, [experts, 2, ff] rows, and every expert's down matrix side by side along K, so that the weighted
// sum over the chosen experts is the one product's sum over K, with the weight of an expert that was not chosen
// being zero.
#include "api.h"
#include "common.h"

#define EXPERTS_MAX 1024

// One thread a token.
__global__ void __launch_bounds__(64)
experts_route_kernel(int32_t* __restrict__ ids, float* __restrict__ weights, float* __restrict__ dense,
                     const float* __restrict__ z, const float* __restrict__ correction, int tokens, int experts, int top) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= tokens) return;
    const float* zt = z + (size_t)t * experts;
    float* dt = dense + (size_t)t * experts;
    for (int e = 0; e < experts; ++e) dt[e] = 0.f;
    float sum = 0.f;
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float best_choice = 0.f, best_s = 0.f;
        for (int e = 0; e < experts; ++e) {
            if (dt[e] != 0.f) continue;                       // chosen already (marked below)
            const float s = 1.f / (1.f + expf(-zt[e]));
            const float c = s + correction[e];
            if (best < 0 || c > best_choice) { best = e; best_choice = c; best_s = s; }
        }
        ids[(size_t)t * top + k] = best;
        weights[(size_t)t * top + k] = best_s;
        dt[best] = -1.f;                                      // a mark that no weight can be
        sum += best_s;
    }
    const float inv = 1.f / (sum + 1e-20f);
    for (int k = 0; k < top; ++k) {
        const float w = weights[(size_t)t * top + k] * inv;
        weights[(size_t)t * top + k] = w;
        dt[ids[(size_t)t * top + k]] = w;
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
experts_activate_kernel(T* __restrict__ out, const T* __restrict__ gu, const float* __restrict__ dense, int experts, int ff,
                        float limit) {
    const int t = blockIdx.x, e = blockIdx.y;
    const float w = dense[(size_t)t * experts + e];
    T* o = out + ((size_t)t * experts + e) * ff;
    const T* g = gu + ((size_t)t * experts + e) * 2 * ff;
    for (int i = threadIdx.x; i < ff; i += blockDim.x) {
        float v = 0.f;
        if (w != 0.f) {
            const float a = fminf(to_f32(g[i]), limit);
            const float u = fminf(fmaxf(to_f32(g[ff + i]), -limit), limit);
            v = w * (a / (1.f + expf(-1.702f * a)) * (u + 1.f));
        }
        from_f32(o + i, v);
    }
}

extern "C" int ri_experts_route(int32_t* ids, float* weights, float* dense, const float* z, const float* correction,
                                int tokens, int experts, int top, void* stream) {
    RI_REQUIRE(tokens > 0 && experts >= 1 && experts <= EXPERTS_MAX && top >= 1 && top <= experts,
               "experts_route: %d tokens, the %d best of %d experts (at most %d)", tokens, top, experts, EXPERTS_MAX);
    experts_route_kernel<<<(tokens + 63) / 64, 64, 0, (hipStream_t)stream>>>(ids, weights, dense, z, correction, tokens,
                                                                             experts, top);
    RI_LAUNCH_CHECK("experts_route");
    return 0;
}

extern "C" int ri_experts_activate(void* out, const void* gu, int dtype, const float* dense, int tokens, int experts,
                                   int ff, float limit, void* stream) {
    RI_REQUIRE(tokens > 0 && experts >= 1 && experts <= 65535 && ff >= 1, "experts_activate: %d tokens, %d experts of %d",
               tokens, experts, ff);
    RI_REQUIRE(dtype == RI_F32 || dtype == RI_BF16, "experts_activate: dtype %d", dtype);
    const dim3 grid(tokens, experts);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == RI_F32)
        experts_activate_kernel<float><<<grid, 256, 0, s>>>((float*)out, (const float*)gu, dense, experts, ff, limit);
    else
        experts_activate_kernel<bf16_t><<<grid, 256, 0, s>>>((bf16_t*)out, (const bf16_t*)gu, dense, experts, ff, limit);
    RI_LAUNCH_CHECK("experts_activate");
    return 0;
}
