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

// V: neighbouring columns a thread takes at a time (4 where d is a multiple of 4: 16-byte loads and stores; else 1).
template <typename TO, int V>
__global__ __launch_bounds__(256) void hc_step_kernel(float* __restrict__ xs, float* __restrict__ y,
                                                      const float* __restrict__ mix, const float* __restrict__ out_w,
                                                      const float* __restrict__ in_w, const float* __restrict__ norm_w,
                                                      TO* __restrict__ h_out, float* __restrict__ u_out,
                                                      int S, long long T, int d, float eps, int clear_y) {
    extern __shared__ __attribute__((aligned(16))) float us[];     // d floats: the row of u
    __shared__ float scratch[4];
    typedef float vec __attribute__((ext_vector_type(V)));
    const long long t = blockIdx.x;
    const bool write = mix != nullptr, read = in_w != nullptr;
    // the step's few weights are read where they are used: the same address for all lanes, so they come through the
    // scalar unit beside the row's own loads, and no barrier stands before those
    const float* __restrict__ w_mix = mix;
    const float* __restrict__ w_out = out_w;
    const float* __restrict__ w_in = in_w;
    const long long plane = T * (long long)d;
    float ss = 0.f;
    for (int c = threadIdx.x * V; c < d; c += 256 * V) {
        const long long at = t * d + c;
        float x[MAX_STREAMS][V];
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s) {
            vec v = {};
            if (s < S) v = *(const vec*)(xs + s * plane + at);
#pragma unroll
            for (int e = 0; e < V; ++e) x[s][e] = v[e];
        }
        if (write) {
            const vec yv = *(const vec*)(y + at);
            if (clear_y) { const vec z = {}; *(vec*)(y + at) = z; }    // the sublayers add into y: it is left ready for the next one
#pragma unroll
            for (int e = 0; e < V; ++e) {
                float nx[MAX_STREAMS];
#pragma unroll
                for (int r = 0; r < MAX_STREAMS; ++r) {
                    float a = 0.f;
#pragma unroll
                    for (int s = 0; s < MAX_STREAMS; ++s)
                        if (s < S && r < S) a = fmaf(w_mix[s * S + r], x[s][e], a);
                    nx[r] = r < S ? fmaf(w_out[r], yv[e], a) : 0.f;
                }
#pragma unroll
                for (int r = 0; r < MAX_STREAMS; ++r) x[r][e] = nx[r];
            }
#pragma unroll
            for (int r = 0; r < MAX_STREAMS; ++r) {
                if (r < S) {
                    vec v;
#pragma unroll
                    for (int e = 0; e < V; ++e) v[e] = x[r][e];
                    *(vec*)(xs + r * plane + at) = v;
                }
            }
        }
        if (read) {
            vec u;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                float a = 0.f;
#pragma unroll
                for (int s = 0; s < MAX_STREAMS; ++s)
                    if (s < S) a = fmaf(w_in[s], x[s][e], a);
                u[e] = a;
                ss = fmaf(a, a, ss);
            }
            if (norm_w) *(vec*)(us + c) = u;
            else *(vec*)(u_out + at) = u;
        }
    }
    if (!read || !norm_w) return;
    const float total = block_sum<4>(ss, scratch);
    const float inv = 1.0f / sqrtf(total / (float)d + eps);
    for (int c = threadIdx.x * V; c < d; c += 256 * V) {
        const vec u = *(const vec*)(us + c), w = *(const vec*)(norm_w + c);
        typedef TO ovec __attribute__((ext_vector_type(V)));
        ovec o;
#pragma unroll
        for (int e = 0; e < V; ++e) o[e] = from_f32<TO>(u[e] * inv * w[e]);
        *(ovec*)(h_out + t * d + c) = o;
    }
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
    const bool four = d % 4 == 0 && (uintptr_t)xs % 16 == 0 && (!y || (uintptr_t)y % 16 == 0) && (!norm_w || (uintptr_t)norm_w % 16 == 0) &&
                      (!h_out || (uintptr_t)h_out % 16 == 0) && (!u_out || (uintptr_t)u_out % 16 == 0);
#define LAUNCH(TO, V) hipLaunchKernelGGL((hc_step_kernel<TO, V>), dim3(n_tokens), dim3(256), lds, stream, xs, y, mix, out_w, in_w, norm_w, \
                                         (TO*)h_out, u_out, S, (long long)n_tokens, d, eps, clear_y)
    if (out_dt == DT_F32) { if (four) LAUNCH(float, 4); else LAUNCH(float, 1); }
    else { if (four) LAUNCH(bf16_t, 4); else LAUNCH(bf16_t, 1); }
#undef LAUNCH
    return launch_status();
}
