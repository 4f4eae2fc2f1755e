// Several residual streams (hyper-connections).  A model keeps S copies of the residual stream,
// xs [S][T][d] in float32.  A sublayer reads a weighted sum of them, u = sum_s in[s] xs[s], and its
// output y goes back into all of them at once, from the old values:
//     xs[r] <- sum_s mix[s][r] xs[s] + out[r] y          (mix is indexed [from][to])
//
// One kernel does the write of one sublayer and the read of the next, with the next sublayer's RMS norm:
// per token row it loads the S values of a column once, forms the new ones (where a write is asked for),
// stores them, forms u (where a read is asked for), and, after the row's sum of squares is known, writes
// norm(u) * w in the compute type (or u itself in float32 where no norm weight is given: the sum of the
// streams at the end of the model).  All sums run over s in ascending order, whatever the step holds.
#include "common.h"

namespace {
constexpr int MAX_STREAMS = 8;

template <typename TO>
__global__ __launch_bounds__(256) void hc_step_kernel(float* __restrict__ xs, float* __restrict__ y,
                                                      const float* __restrict__ mix, const float* __restrict__ out_w,
                                                      const float* __restrict__ in_w, const float* __restrict__ norm_w,
                                                      TO* __restrict__ h_out, float* __restrict__ u_out,
                                                      int S, long long T, int d, float eps, int clear_y) {
    extern __shared__ float us[];                      // d floats: the row of u
    __shared__ float scratch[4];
    __shared__ float w_mix[MAX_STREAMS * MAX_STREAMS], w_out[MAX_STREAMS], w_in[MAX_STREAMS];
    const long long t = blockIdx.x;
    const bool write = mix != nullptr, read = in_w != nullptr;
    if (threadIdx.x < S * S && write) w_mix[threadIdx.x] = mix[threadIdx.x];
    if (threadIdx.x < S) {
        if (write) w_out[threadIdx.x] = out_w[threadIdx.x];
        if (read) w_in[threadIdx.x] = in_w[threadIdx.x];
    }
    __syncthreads();
    const long long plane = T * (long long)d;
    float ss = 0.f;
    for (int c = threadIdx.x; c < d; c += 256) {
        const long long at = t * d + c;
        float x[MAX_STREAMS];
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s) x[s] = s < S ? xs[s * plane + at] : 0.f;
        if (write) {
            const float yv = y[at];
            if (clear_y) y[at] = 0.f;              // the sublayers add into y: it is left ready for the next one
            float nx[MAX_STREAMS];
#pragma unroll
            for (int r = 0; r < MAX_STREAMS; ++r) {
                float a = 0.f;
#pragma unroll
                for (int s = 0; s < MAX_STREAMS; ++s)
                    if (s < S && r < S) a = fmaf(w_mix[s * S + r], x[s], a);
                nx[r] = r < S ? fmaf(w_out[r], yv, a) : 0.f;
            }
#pragma unroll
            for (int r = 0; r < MAX_STREAMS; ++r) {
                x[r] = nx[r];
                if (r < S) xs[r * plane + at] = nx[r];
            }
        }
        if (read) {
            float u = 0.f;
#pragma unroll
            for (int s = 0; s < MAX_STREAMS; ++s)
                if (s < S) u = fmaf(w_in[s], x[s], u);
            if (norm_w) { us[c] = u; ss = fmaf(u, u, ss); }
            else u_out[at] = u;
        }
    }
    if (!read || !norm_w) return;
    const float total = block_sum<4>(ss, scratch);
    const float inv = 1.0f / sqrtf(total / (float)d + eps);
    for (int c = threadIdx.x; c < d; c += 256) h_out[t * d + c] = from_f32<TO>(us[c] * inv * norm_w[c]);
}
}  // namespace

// xs float32 [S][T][d].  mix [S][S] and out_w [S] with y [T][d]: the write (all three null: none).  in_w [S]: the
// read (null: none); with norm_w [d] the result norm(u) * norm_w goes to h_out [T][d] of type out_dt, without it
// u goes to u_out [T][d] in float32.  clear_y: y is zero afterwards.
TUFF_EXPORT int tuff_hc_step(float* xs, float* y, const float* mix, const float* out_w, const float* in_w,
                             const float* norm_w, void* h_out, int out_dt, float* u_out, int S, int n_tokens, int d,
                             float eps, int clear_y, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (S < 1 || S > MAX_STREAMS || d < 1 || d > 15360) return -2;
    if ((mix == nullptr) != (out_w == nullptr) || (mix == nullptr) != (y == nullptr)) return -2;
    if (in_w && (norm_w ? h_out == nullptr : u_out == nullptr)) return -2;
    const size_t lds = (size_t)d * sizeof(float);
    if (out_dt == DT_F32)
        hipLaunchKernelGGL(hc_step_kernel<float>, dim3(n_tokens), dim3(256), lds, stream, xs, y, mix, out_w, in_w, norm_w,
                           (float*)h_out, u_out, S, (long long)n_tokens, d, eps, clear_y);
    else
        hipLaunchKernelGGL(hc_step_kernel<bf16_t>, dim3(n_tokens), dim3(256), lds, stream, xs, y, mix, out_w, in_w, norm_w,
                           (bf16_t*)h_out, u_out, S, (long long)n_tokens, d, eps, clear_y);
    return launch_status();
}
