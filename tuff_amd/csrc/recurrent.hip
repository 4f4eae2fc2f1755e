// Kernels of mixers that carry a fixed-size state from token to token: the blend of a token's input
// with the one before it (token shift), a short causal convolution per channel with an activation,
// and two matrix-state recurrences, a decaying outer-product memory with a bonus for the current
// token ("wkv") and a gated delta rule.  States are float32 and live in a slot per request; a step
// brings each request's next tokens (one decoded token or a portion of a prompt of any length),
// tokens flat and ordered by request, and every kernel continues from the slot and leaves it ready
// for the next step.  The recurrences run token by token in one fixed order of operations, so a
// position's result does not depend on how the sequence was cut into steps.
//
// Everything that enters a recurrence besides the projected rows is float32: decays, their
// exponentials and softplus, the write strength, the unit norms of q and k.
//
// Requests with no tokens in the step (q_len 0: a recorded step's padding) are skipped everywhere.
#include "common.h"
#include <math.h>

namespace {

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float siluf_(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// ------------------------------------------------------------------------ token shift
// out[s][t][c] = h[t][c] + (prev - h[t][c]) * mu[s][c], prev = the request's token before (its
// state where t is the first of the step).
template <typename T>
__global__ void shift_mix_kernel(const T* __restrict__ h, const float* __restrict__ prev_state, const float* __restrict__ mu,
                                 T* __restrict__ out, const int* __restrict__ req_of_token, const int* __restrict__ q_start,
                                 const int* __restrict__ state_slot, int n_tokens, int d, int n_mix) {
    const int t = blockIdx.x;
    const int r = req_of_token[t];
    const bool first = t == q_start[r];
    const float* ps = prev_state + (long long)state_slot[r] * d;
    const T* hp = h + (long long)(t - 1) * d;
    const T* hc = h + (long long)t * d;
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
        const float x = to_f32(hc[c]);
        const float p = first ? ps[c] : to_f32(hp[c]);
        for (int s = 0; s < n_mix; ++s)
            out[((long long)s * n_tokens + t) * d + c] = from_f32<T>(fmaf(p - x, mu[(long long)s * d + c], x));
    }
}

// prev_state[slot] = the request's last row of the step
template <typename T>
__global__ void shift_state_kernel(const T* __restrict__ h, float* __restrict__ prev_state, const int* __restrict__ q_start,
                                   const int* __restrict__ q_len, const int* __restrict__ state_slot, int d) {
    const int r = blockIdx.x;
    const int n = q_len[r];
    if (n <= 0) return;
    const T* src = h + (long long)(q_start[r] + n - 1) * d;
    float* dst = prev_state + (long long)state_slot[r] * d;
    for (int c = threadIdx.x; c < d; c += blockDim.x) dst[c] = to_f32(src[c]);
}

// --------------------------------------------------------------- short causal convolution
// y[t][c] = act(sum_j taps[c][j] x[t - (K-1) + j][c]); inputs before the step's first token come from
// the request's state [K-1][C] (zeros for a new request).  act: 0 none, 1 silu.
constexpr int MAX_TAPS = 17;

template <typename T>
__global__ void conv_act_kernel(const T* __restrict__ x, const float* __restrict__ taps, const float* __restrict__ state,
                                T* __restrict__ y, const int* __restrict__ req_of_token, const int* __restrict__ q_start,
                                const int* __restrict__ state_slot, int C, int K, int act) {
    const int t = blockIdx.x;
    const int r = req_of_token[t];
    const int i = t - q_start[r];                     // index within the step's portion
    const float* st = state + (long long)state_slot[r] * (K - 1) * C;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
        float acc = 0.f;
        for (int j = 0; j < K; ++j) {
            const int li = i - (K - 1) + j;
            const float v = li >= 0 ? to_f32(x[(long long)(t - (K - 1) + j) * C + c]) : st[(long long)(i + j) * C + c];
            acc = fmaf(taps[(long long)c * K + j], v, acc);
        }
        y[(long long)t * C + c] = from_f32<T>(act == 1 ? siluf_(acc) : acc);
    }
}

// the state after the step: the last K-1 inputs, from the step's rows and, for a short portion, the old state
template <typename T>
__global__ void conv_state_kernel(const T* __restrict__ x, float* __restrict__ state, const int* __restrict__ q_start,
                                  const int* __restrict__ q_len, const int* __restrict__ state_slot, int C, int K) {
    const int r = blockIdx.x;
    const int n = q_len[r];
    if (n <= 0) return;
    float* st = state + (long long)state_slot[r] * (K - 1) * C;
    const int t0 = q_start[r];
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
        float keep[MAX_TAPS - 1];
#pragma unroll
        for (int m = 0; m < MAX_TAPS - 1; ++m) {
            if (m < K - 1) {
                const int li = n - (K - 1) + m;
                keep[m] = li >= 0 ? to_f32(x[(long long)(t0 + li) * C + c]) : st[(long long)(m + n) * C + c];
            }
        }
#pragma unroll
        for (int m = 0; m < MAX_TAPS - 1; ++m)
            if (m < K - 1) st[(long long)m * C + c] = keep[m];
    }
}

// ------------------------------------------------------------------------ recurrences
// One wave per (request, head, 64 value channels): lane j keeps column j of the head's state,
// S[0..D-1][j], in registers (NI = ceil(D / 4) groups of four rows) and walks the request's tokens in
// order.  What a token brings for the key channels (r or q, k, the decay) is staged by the wave
// through LDS, the token after it is fetched while the current one is computed.
//
// wkv:    o_j = sum_i r_i (S_ij + u_i k_i v_j);   S_ij <- w_i S_ij + k_i v_j
//         w_i = exp(-exp(lw_i + w0_i))
// delta:  S_ij <- g_i S_ij;  e_j = beta (v_j - sum_i k_i S_ij);  S_ij <- S_ij + k_i e_j;  o_j = sum_i q_i S_ij
//         g_i = exp(-exp(A_log) softplus(a_i + dt_bias_i)), beta = sigmoid(b), q and k unit vectors
//         (x / sqrt(sum x^2 + 1e-6)), q also times D^(-1/2)
struct ScanArgs {
    const void *a, *k, *v;          // per token: r or q [T][Ha*D], k [T][Ha*D], v [T][H*Dv]   (Ha: heads of a and k)
    const float* decay_in;          // per token [T][H*D]: lw (wkv) or a (delta)
    const float* decay_bias;        // [H*D]: w0 or dt_bias
    const float* per_head;          // wkv: u [H][D];  delta: A_log [H]
    const float* beta_in;           // delta: b [T][H]
    float* state;                   // [slots][H][D][Dv]
    float* out;                     // [T][H][Dv]
    const int *q_start, *q_len, *state_slot;
    int H, Ha, D, Dv;
};

template <typename T, int NI, bool DELTA>
__global__ __launch_bounds__(WAVE) void scan_kernel(ScanArgs p) {
    constexpr int DP = NI * 4;                         // key channels, padded
    constexpr int PER = (DP + WAVE - 1) / WAVE;        // key channels a lane stages
    __shared__ __attribute__((aligned(16))) float sa[2][DP];
    __shared__ __attribute__((aligned(16))) float sk[2][DP];
    __shared__ __attribute__((aligned(16))) float sw[2][DP];
    const int r = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int n = p.q_len[r];
    if (n <= 0) return;
    const int D = p.D, Dv = p.Dv, H = p.H, Ha = p.Ha;
    const int ha = head / (H / Ha);
    const int j = blockIdx.z * WAVE + lane;
    const bool jv = j < Dv;
    const int t0 = p.q_start[r];
    float* S = p.state + (((long long)p.state_slot[r] * H + head) * D) * Dv + j;
    const T* pa = (const T*)p.a;
    const T* pk = (const T*)p.k;
    const T* pv = (const T*)p.v;

    float s[DP];
#pragma unroll
    for (int i = 0; i < DP; ++i) s[i] = (jv && i < D) ? S[(long long)i * Dv] : 0.f;

    float bias[PER], extra[PER];
#pragma unroll
    for (int e = 0; e < PER; ++e) {
        const int i = lane + e * WAVE;
        bias[e] = i < D ? p.decay_bias[head * D + i] : 0.f;
        extra[e] = (!DELTA && i < D) ? p.per_head[head * D + i] : 0.f;      // u
    }
    const float neg_rate = DELTA ? -expf(p.per_head[head]) : 0.f;
    const float q_scale = DELTA ? 1.0f / sqrtf((float)D) : 1.f;

    // what a token brings, fetched one token ahead
    float fa[PER], fk[PER], fw[PER], fv = 0.f, fb = 0.f;
    auto fetch = [&](int t) {
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int i = lane + e * WAVE;
            const bool ok = i < D;
            fa[e] = ok ? to_f32(pa[((long long)t * Ha + ha) * D + i]) : 0.f;
            fk[e] = ok ? to_f32(pk[((long long)t * Ha + ha) * D + i]) : 0.f;
            fw[e] = ok ? p.decay_in[((long long)t * H + head) * D + i] : 0.f;
        }
        fv = jv ? to_f32(pv[((long long)t * H + head) * Dv + j]) : 0.f;
        if (DELTA) fb = p.beta_in[(long long)t * H + head];
    };
    fetch(t0);
    for (int it = 0; it < n; ++it) {
        const int t = t0 + it, buf = it & 1;
        const float v = fv;
        float beta = 0.f;
        // stage this token's key-channel vectors
        if (DELTA) {
            float qq = 0.f, kk = 0.f;
#pragma unroll
            for (int e = 0; e < PER; ++e) { qq = fmaf(fa[e], fa[e], qq); kk = fmaf(fk[e], fk[e], kk); }
            qq = wave_sum(qq); kk = wave_sum(kk);
            const float qn = q_scale / sqrtf(qq + 1e-6f), kn = 1.0f / sqrtf(kk + 1e-6f);
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                const int i = lane + e * WAVE;
                if (i < DP) {
                    sa[buf][i] = fa[e] * qn;
                    sk[buf][i] = fk[e] * kn;
                    sw[buf][i] = i < D ? expf(neg_rate * softplusf_(fw[e] + bias[e])) : 0.f;
                }
            }
            beta = sigmoidf_(fb);
        } else {
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                const int i = lane + e * WAVE;
                if (i < DP) {
                    sa[buf][i] = fa[e];
                    sk[buf][i] = fk[e];
                    sw[buf][i] = i < D ? expf(-expf(fw[e] + bias[e])) : 0.f;
                }
            }
        }
        float bonus = 0.f;
        if (!DELTA) {
#pragma unroll
            for (int e = 0; e < PER; ++e) bonus = fmaf(fa[e] * extra[e], fk[e], bonus);
            bonus = wave_sum(bonus);
        }
        if (it + 1 < n) fetch(t + 1);
        __syncthreads();                               // one wave: orders the LDS writes before the reads
        float o = 0.f;
        if (DELTA) {
            float kv = 0.f;
#pragma unroll
            for (int g4 = 0; g4 < NI; ++g4) {
                const f32x4 w4 = *(const f32x4*)&sw[buf][g4 * 4];
                const f32x4 k4 = *(const f32x4*)&sk[buf][g4 * 4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s[g4 * 4 + e] *= w4[e];
                    kv = fmaf(k4[e], s[g4 * 4 + e], kv);
                }
            }
            const float err = beta * (v - kv);
#pragma unroll
            for (int g4 = 0; g4 < NI; ++g4) {
                const f32x4 k4 = *(const f32x4*)&sk[buf][g4 * 4];
                const f32x4 q4 = *(const f32x4*)&sa[buf][g4 * 4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s[g4 * 4 + e] = fmaf(k4[e], err, s[g4 * 4 + e]);
                    o = fmaf(q4[e], s[g4 * 4 + e], o);
                }
            }
        } else {
#pragma unroll
            for (int g4 = 0; g4 < NI; ++g4) {
                const f32x4 w4 = *(const f32x4*)&sw[buf][g4 * 4];
                const f32x4 k4 = *(const f32x4*)&sk[buf][g4 * 4];
                const f32x4 r4 = *(const f32x4*)&sa[buf][g4 * 4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    o = fmaf(r4[e], s[g4 * 4 + e], o);
                    s[g4 * 4 + e] = fmaf(w4[e], s[g4 * 4 + e], k4[e] * v);
                }
            }
            o = fmaf(bonus, v, o);
        }
        if (jv) p.out[((long long)t * H + head) * Dv + j] = o;
    }
#pragma unroll
    for (int i = 0; i < DP; ++i)
        if (jv && i < D) S[(long long)i * Dv] = s[i];
}

// ---------------------------------------------------------- per-head unit norm, weight and gate
// y[t][h][j] = o[t][h][j] / sqrt(mean_j o^2 + eps) * w[(h * w_stride) + j] * f(gate[t][h][j]);
// f: 0 identity, 1 silu, 2 sigmoid.  A wave per (token, head).
template <typename TG, typename T>
__global__ __launch_bounds__(WAVE) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w, int w_stride,
                                                              const TG* __restrict__ gate, int gate_fn, T* __restrict__ y,
                                                              int H, int Dv, float eps) {
    const long long row = (long long)blockIdx.x * H + blockIdx.y;
    const float* src = o + row * Dv;
    float ss = 0.f;
    for (int j = threadIdx.x; j < Dv; j += WAVE) ss = fmaf(src[j], src[j], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)Dv + eps);
    for (int j = threadIdx.x; j < Dv; j += WAVE) {
        float g = to_f32(gate[row * Dv + j]);
        if (gate_fn == 1) g = siluf_(g);
        else if (gate_fn == 2) g = sigmoidf_(g);
        y[row * Dv + j] = from_f32<T>(src[j] * inv * w[(long long)blockIdx.y * w_stride + j] * g);
    }
}

template <typename T, bool DELTA>
int launch_scan(const ScanArgs& p, int R, hipStream_t stream) {
    const int ni = (p.D + 3) / 4;
    dim3 grid(R, p.H, ceil_div(p.Dv, WAVE)), block(WAVE);
#define SCAN(NI) hipLaunchKernelGGL((scan_kernel<T, NI, DELTA>), grid, block, 0, stream, p)
    if (ni <= 4) SCAN(4);
    else if (ni <= 8) SCAN(8);
    else if (ni <= 12) SCAN(12);
    else if (ni <= 16) SCAN(16);
    else if (ni <= 24) SCAN(24);
    else if (ni <= 32) SCAN(32);
    else if (ni <= 48) SCAN(48);
    else if (ni <= 64) SCAN(64);
    else return -2;
#undef SCAN
    return launch_status();
}
}  // namespace

TUFF_EXPORT int tuff_shift_mix(const void* h, int dt, const float* prev_state, const float* mu, void* out,
                               const int* req_of_token, const int* q_start, const int* state_slot,
                               int n_tokens, int d, int n_mix, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens), block(256);
    if (dt == DT_F32) hipLaunchKernelGGL(shift_mix_kernel<float>, grid, block, 0, stream, (const float*)h, prev_state, mu, (float*)out, req_of_token, q_start, state_slot, n_tokens, d, n_mix);
    else hipLaunchKernelGGL(shift_mix_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)h, prev_state, mu, (bf16_t*)out, req_of_token, q_start, state_slot, n_tokens, d, n_mix);
    return launch_status();
}

TUFF_EXPORT int tuff_shift_state(const void* h, int dt, float* prev_state, const int* q_start, const int* q_len,
                                 const int* state_slot, int n_requests, int d, hipStream_t stream) {
    if (n_requests <= 0) return 0;
    dim3 grid(n_requests), block(256);
    if (dt == DT_F32) hipLaunchKernelGGL(shift_state_kernel<float>, grid, block, 0, stream, (const float*)h, prev_state, q_start, q_len, state_slot, d);
    else hipLaunchKernelGGL(shift_state_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)h, prev_state, q_start, q_len, state_slot, d);
    return launch_status();
}

// x, y [T][C]; taps float32 [C][K]; state float32 [slots][K-1][C].  q_len null: the state is only read.
TUFF_EXPORT int tuff_conv_act(const void* x, int dt, const float* taps, float* state, void* y,
                              const int* req_of_token, const int* q_start, const int* q_len, const int* state_slot,
                              int n_tokens, int n_requests, int C, int K, int act, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (K < 1 || K > MAX_TAPS) return -2;
    const int cols = ceil_div(C, 256);
    dim3 block(256);
    if (dt == DT_F32) hipLaunchKernelGGL(conv_act_kernel<float>, dim3(n_tokens, cols), block, 0, stream, (const float*)x, taps, state, (float*)y, req_of_token, q_start, state_slot, C, K, act);
    else hipLaunchKernelGGL(conv_act_kernel<bf16_t>, dim3(n_tokens, cols), block, 0, stream, (const bf16_t*)x, taps, state, (bf16_t*)y, req_of_token, q_start, state_slot, C, K, act);
    int rc = launch_status();
    if (rc != 0 || !q_len || K == 1) return rc;
    if (dt == DT_F32) hipLaunchKernelGGL(conv_state_kernel<float>, dim3(n_requests, cols), block, 0, stream, (const float*)x, state, q_start, q_len, state_slot, C, K);
    else hipLaunchKernelGGL(conv_state_kernel<bf16_t>, dim3(n_requests, cols), block, 0, stream, (const bf16_t*)x, state, q_start, q_len, state_slot, C, K);
    return launch_status();
}

// wkv: r, k [T][H*D], v [T][H*D] of type dt; lw float32 [T][H*D]; w0 float32 [H*D]; u float32 [H][D];
// state float32 [slots][H][D][D]; out float32 [T][H][D].
TUFF_EXPORT int tuff_wkv_scan(const void* r, const void* k, const void* v, int dt, const float* lw, const float* w0,
                              const float* u, float* state, float* out, const int* q_start, const int* q_len,
                              const int* state_slot, int n_requests, int H, int D, hipStream_t stream) {
    if (n_requests <= 0) return 0;
    ScanArgs p{r, k, v, lw, w0, u, nullptr, state, out, q_start, q_len, state_slot, H, H, D, D};
    return dt == DT_F32 ? launch_scan<float, false>(p, n_requests, stream) : launch_scan<bf16_t, false>(p, n_requests, stream);
}

// delta: q, k [T][Hk*D], v [T][H*Dv] of type dt (after convolution and activation, not yet unit
// vectors); a float32 [T][H*D]; dt_bias float32 [H*D]; A_log float32 [H]; b float32 [T][H];
// state float32 [slots][H][D][Dv]; out float32 [T][H][Dv].
TUFF_EXPORT int tuff_delta_scan(const void* q, const void* k, const void* v, int dt, const float* a, const float* dt_bias,
                                const float* A_log, const float* b, float* state, float* out, const int* q_start,
                                const int* q_len, const int* state_slot, int n_requests, int H, int Hk, int D, int Dv,
                                hipStream_t stream) {
    if (n_requests <= 0) return 0;
    if (Hk <= 0 || H % Hk) return -2;
    ScanArgs p{q, k, v, a, dt_bias, A_log, b, state, out, q_start, q_len, state_slot, H, Hk, D, Dv};
    return dt == DT_F32 ? launch_scan<float, true>(p, n_requests, stream) : launch_scan<bf16_t, true>(p, n_requests, stream);
}

// gate_dt: type of the gate's rows (float32 sums of a product may come in as they are); dt: type of y.
TUFF_EXPORT int tuff_head_norm_gate(const float* o, const float* w, int w_stride, const void* gate, int gate_dt, int dt, int gate_fn,
                                    void* y, int n_tokens, int H, int Dv, float eps, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens, H), block(WAVE);
    if (dt == DT_F32 && gate_dt == DT_F32) hipLaunchKernelGGL((head_norm_gate_kernel<float, float>), grid, block, 0, stream, o, w, w_stride, (const float*)gate, gate_fn, (float*)y, H, Dv, eps);
    else if (gate_dt == DT_F32) hipLaunchKernelGGL((head_norm_gate_kernel<float, bf16_t>), grid, block, 0, stream, o, w, w_stride, (const float*)gate, gate_fn, (bf16_t*)y, H, Dv, eps);
    else if (dt == DT_BF16) hipLaunchKernelGGL((head_norm_gate_kernel<bf16_t, bf16_t>), grid, block, 0, stream, o, w, w_stride, (const bf16_t*)gate, gate_fn, (bf16_t*)y, H, Dv, eps);
    else return -2;
    return launch_status();
}
