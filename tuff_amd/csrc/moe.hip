// Mixture of experts: the choice of experts per token and the chosen experts' two products.
//
// Routing: from router logits z [T][E] (float32) the `top` largest are chosen per token (the lower
// index wins a tie); the weight of a choice is f(z): 0 sigmoid (each score on its own, not
// renormalised), 1 softmax over the chosen.  Everything here is float32.
//
// Experts: y = W_down act(W_up x) with x the token's input, multiplied by the choice's weight before
// (scale_input) or y after; act: 0 relu squared, 1 silu, 2 gelu (tanh form).  A (token, choice) pair is a
// row of the work arrays; the rows of a token are added into the residual stream in the order of
// its choices, so the sum does not depend on what else is in the step.
#include "common.h"
#include <math.h>

namespace {
__device__ __forceinline__ float act_fn(float z, int act) {
    if (act == 0) { const float r = fmaxf(z, 0.f); return r * r; }
    if (act == 1) return z / (1.0f + expf(-z));
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

__global__ void route_kernel(const float* __restrict__ z, int stride, int* __restrict__ ids, float* __restrict__ wts,
                             int n_tokens, int E, int top, int weight_fn) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_tokens) return;
    const float* row = z + (long long)t * stride;
    float last = INFINITY;
    int last_id = -1;
    float zmax = 0.f, den = 0.f;
    for (int s = 0; s < top; ++s) {
        // the largest logit that comes after (last, last_id) in the order (value descending, index ascending)
        float best = -INFINITY;
        int best_id = -1;
        for (int e = 0; e < E; ++e) {
            const float v = row[e];
            const bool after = v < last || (v == last && e > last_id);
            if (after && (best_id < 0 || v > best)) { best = v; best_id = e; }
        }
        if (best_id < 0) { best_id = 0; best = row[0]; }      // NaN logits: still a valid expert
        ids[(long long)t * top + s] = best_id;
        float w;
        if (weight_fn == 0) w = 1.0f / (1.0f + expf(-best));
        else { if (s == 0) zmax = best; w = expf(best - zmax); den += w; }
        wts[(long long)t * top + s] = w;
        last = best; last_id = best_id;
    }
    if (weight_fn == 1)
        for (int s = 0; s < top; ++s) wts[(long long)t * top + s] /= den;
}

constexpr int ROWS_WG = 16;          // output rows a workgroup of four waves computes

// a[row][f] = act(W_up[e][f] . x), x = h[t] (times the choice's weight), rounded to T as the second product takes it
template <typename T>
__global__ __launch_bounds__(256) void expert_up_kernel(const T* __restrict__ h, const T* __restrict__ w_up, const int* __restrict__ ids,
                                                        const float* __restrict__ wts, T* __restrict__ a, int d, int F, int top,
                                                        int act, int scale_input) {
    extern __shared__ float xs[];
    const long long row = blockIdx.x;
    const long long t = row / top;
    const int e = ids[row];
    const float w = scale_input ? wts[row] : 1.f;
    for (int c = threadIdx.x; c < d; c += 256) xs[c] = to_f32(from_f32<T>(to_f32(h[t * d + c]) * w));
    __syncthreads();
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    for (int f = blockIdx.y * ROWS_WG + wave; f < min(F, (int)(blockIdx.y + 1) * ROWS_WG); f += 4) {
        const T* wr = w_up + ((long long)e * F + f) * d;
        float acc = 0.f;
        for (int c = lane; c < d; c += WAVE) acc = fmaf(to_f32(wr[c]), xs[c], acc);
        acc = wave_sum(acc);
        if (lane == 0) a[row * F + f] = from_f32<T>(act_fn(acc, act));
    }
}

// y[row][c] = W_down[e][c] . a[row]  (float32)
template <typename T>
__global__ __launch_bounds__(256) void expert_down_kernel(const T* __restrict__ a, const T* __restrict__ w_down, const int* __restrict__ ids,
                                                          float* __restrict__ y, int d, int F) {
    extern __shared__ float as[];
    const long long row = blockIdx.x;
    const int e = ids[row];
    for (int f = threadIdx.x; f < F; f += 256) as[f] = to_f32(a[row * F + f]);
    __syncthreads();
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    for (int c = blockIdx.y * ROWS_WG + wave; c < min(d, (int)(blockIdx.y + 1) * ROWS_WG); c += 4) {
        const T* wr = w_down + ((long long)e * d + c) * F;
        float acc = 0.f;
        for (int f = lane; f < F; f += WAVE) acc = fmaf(to_f32(wr[f]), as[f], acc);
        acc = wave_sum(acc);
        if (lane == 0) y[row * d + c] = acc;
    }
}

// residual[t][c] += sum over the token's choices, in their order, of y[t * top + s][c] (times the weight)
__global__ void combine_kernel(const float* __restrict__ y, const float* __restrict__ wts, float* __restrict__ residual,
                               long long n, int d, int top, int scale_output) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long long t = i / d;
    const int c = (int)(i - t * d);
    float acc = 0.f;
    for (int s = 0; s < top; ++s) {
        const float v = y[(t * top + s) * d + c];
        acc += scale_output ? v * wts[t * top + s] : v;
    }
    residual[i] += acc;
}
}  // namespace

TUFF_EXPORT int tuff_moe_route(const float* z, int stride, int* ids, float* wts, int n_tokens, int E, int top, int weight_fn,
                               hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (top < 1 || top > E || stride < E) return -2;
    hipLaunchKernelGGL(route_kernel, dim3(ceil_div(n_tokens, 64)), dim3(64), 0, stream, z, stride, ids, wts, n_tokens, E, top, weight_fn);
    return launch_status();
}

// h [T][d], w_up [E][F][d], w_down [E][d][F] of type dt; ids, wts [T][top]; a [T*top][F] (type dt) and
// y [T*top][d] (float32) are work arrays; residual float32 [T][d].
TUFF_EXPORT int tuff_moe_experts(const void* h, const void* w_up, const void* w_down, int dt, const int* ids, const float* wts,
                                 void* a, float* y, float* residual, int n_tokens, int d, int F, int top, int act,
                                 int scale_input, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (d > 16384 || F > 16384) return -2;
    const long long rows = (long long)n_tokens * top;
    dim3 block(256);
    if (dt == DT_F32) {
        hipLaunchKernelGGL(expert_up_kernel<float>, dim3((unsigned)rows, ceil_div(F, ROWS_WG)), block, d * sizeof(float), stream,
                           (const float*)h, (const float*)w_up, ids, wts, (float*)a, d, F, top, act, scale_input);
        hipLaunchKernelGGL(expert_down_kernel<float>, dim3((unsigned)rows, ceil_div(d, ROWS_WG)), block, F * sizeof(float), stream,
                           (const float*)a, (const float*)w_down, ids, y, d, F);
    } else {
        hipLaunchKernelGGL(expert_up_kernel<bf16_t>, dim3((unsigned)rows, ceil_div(F, ROWS_WG)), block, d * sizeof(float), stream,
                           (const bf16_t*)h, (const bf16_t*)w_up, ids, wts, (bf16_t*)a, d, F, top, act, scale_input);
        hipLaunchKernelGGL(expert_down_kernel<bf16_t>, dim3((unsigned)rows, ceil_div(d, ROWS_WG)), block, F * sizeof(float), stream,
                           (const bf16_t*)a, (const bf16_t*)w_down, ids, y, d, F);
    }
    const long long n = (long long)n_tokens * d;
    hipLaunchKernelGGL(combine_kernel, dim3((unsigned)ceil_div_ll(n, 256)), block, 0, stream, y, wts, residual, n, d, top, !scale_input);
    return launch_status();
}
