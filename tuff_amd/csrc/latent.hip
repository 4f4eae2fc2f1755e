// Latent attention: what stands between the projections and the attention over the cache, and after it.
//
// A token's cache row is [c | k_rot]: c = RMS norm (with a weight) of the first `rank` projected channels,
// k_rot the rotated last `rot` ones, shared by all heads.  A head's key would be [W_uk,h c | k_rot] and its
// value W_uv,h c; neither is ever formed.  Instead the query is carried into the latent space,
//     q'_h = [W_uk,h^T q_plain,h | rotate(q_rot,h)],   score = q'_h . [c | k_rot],
// attention runs with the cache rows as keys and their first `rank` channels as values (one kv head for all
// query heads), and the head's output is W_uv,h (sum_j p_j c_j), times the head's gate.
//
// tuff_latent_post: norm, rotation, cache write and the rotated part of q'.
// tuff_head_matmul: y[t][h][0..N) = x[t][h][0..K) . W[h] with W [H][K][N], optionally times
// sigmoid(gate[t][h]): both per-head products above (W_uk as stored is [H][dim][rank]; W_uv is transposed per
// head when it is bound).  Sums run over k in ascending order in float32, one chain a (token, head, column).
//
// Rotation: neighbouring pairs (2i, 2i+1) of the first `rot_dims` channels of the rotated part turn by
// pos * inv_freq[i] (float32 angle, cosf and sinf); channels beyond rot_dims pass.
#include "common.h"
#include <math.h>

namespace {
constexpr int POST_THREADS = 256;

template <typename T, typename TW>
__global__ __launch_bounds__(POST_THREADS) void latent_post_kernel(
    const T* __restrict__ proj, int row_stride, int q_off, int ckr_off, T* __restrict__ q_lat, T* __restrict__ cache,
    T* __restrict__ cache_t, int page_size, const TW* __restrict__ norm_w, float eps, const float* __restrict__ inv_freq, int rot_dims,
    const int* __restrict__ positions, const int* __restrict__ slot_mapping, int H, int dim, int rot, int rank) {
    __shared__ float scratch[POST_THREADS / WAVE];
    const long long t = blockIdx.x;
    const T* row = proj + t * row_stride;
    const float pos = (float)positions[t];
    const int lat = rank + rot;
    // the latent row: norm over the first `rank` channels
    float ss = 0.f;
    for (int c = threadIdx.x; c < rank; c += POST_THREADS) { const float v = to_f32(row[ckr_off + c]); ss = fmaf(v, v, ss); }
    const float total = block_sum<POST_THREADS / WAVE>(ss, scratch);
    const float inv = 1.0f / sqrtf(total / (float)rank + eps);
    const long long slot = slot_mapping ? slot_mapping[t] : -1;
    // cache_t: the same row once more with a channel's positions contiguous within the page,
    // [page][channel][offset], as the matrix-core attention kernels read values
    T* dst_t = nullptr;
    if (slot >= 0 && cache_t) dst_t = cache_t + (slot / page_size) * (long long)lat * page_size + slot % page_size;
    if (slot >= 0) {
        T* dst = cache + slot * lat;
        for (int c = threadIdx.x; c < rank; c += POST_THREADS) {
            const T v = from_f32<T>(to_f32(row[ckr_off + c]) * inv * to_f32(norm_w[c]));
            dst[c] = v;
            if (dst_t) dst_t[(long long)c * page_size] = v;
        }
    }
    // rotated parts: item 0 is the shared key part, items 1..H the heads' query parts; a thread a pair
    const int pairs = rot / 2, odd = rot % 2;
    for (int i = threadIdx.x; i < (H + 1) * (pairs + odd); i += POST_THREADS) {
        const int item = i / (pairs + odd), p = i % (pairs + odd);
        const T* src = item == 0 ? row + ckr_off + rank : row + q_off + (long long)(item - 1) * (dim + rot) + dim;
        T* dst = item == 0 ? (slot >= 0 ? cache + slot * lat + rank : nullptr) : q_lat + (t * H + (item - 1)) * lat + rank;
        if (!dst) continue;
        T* dt2 = item == 0 && dst_t ? dst_t + (long long)rank * page_size : nullptr;
        if (p == pairs) {                                                // a last channel without a partner passes
            dst[rot - 1] = src[rot - 1];
            if (dt2) dt2[(long long)(rot - 1) * page_size] = src[rot - 1];
            continue;
        }
        float u = to_f32(src[2 * p]), v = to_f32(src[2 * p + 1]);
        if (2 * p + 1 < rot_dims) {
            const float a = pos * inv_freq[p];
            const float cs = cosf(a), sn = sinf(a);
            const float u2 = u * cs - v * sn, v2 = v * cs + u * sn;
            u = u2; v = v2;
        }
        dst[2 * p] = from_f32<T>(u);
        dst[2 * p + 1] = from_f32<T>(v);
        if (dt2) { dt2[(long long)(2 * p) * page_size] = from_f32<T>(u); dt2[(long long)(2 * p + 1) * page_size] = from_f32<T>(v); }
    }
}

// A workgroup takes TT tokens of one head; a thread owns output columns n = tid, tid + 256, ... (at most NPT of
// them a pass) and walks k with the tokens' x in LDS: W is read once for TT tokens.
constexpr int HM_TT = 8;
constexpr int HM_NPT = 2;

template <typename T>
__global__ __launch_bounds__(256) void head_matmul_kernel(const T* __restrict__ x, long long x_row, long long x_head,
                                                          const T* __restrict__ W, T* __restrict__ y, long long y_row,
                                                          long long y_head, const T* __restrict__ gate, long long gate_row,
                                                          int n_tokens, int K, int N) {
    extern __shared__ float xs[];                      // [HM_TT][K]
    const int h = blockIdx.y;
    const int t0 = blockIdx.x * HM_TT;
    const int nt = min(HM_TT, n_tokens - t0);
    for (int i = threadIdx.x; i < HM_TT * K; i += 256) {
        const int tt = i / K, k = i % K;
        xs[i] = tt < nt ? to_f32(x[(long long)(t0 + tt) * x_row + h * x_head + k]) : 0.f;
    }
    __syncthreads();
    const T* Wh = W + (long long)h * K * N;
    for (int n0 = threadIdx.x; n0 < N; n0 += 256 * HM_NPT) {
        float acc[HM_NPT][HM_TT];
#pragma unroll
        for (int j = 0; j < HM_NPT; ++j)
#pragma unroll
            for (int tt = 0; tt < HM_TT; ++tt) acc[j][tt] = 0.f;
        for (int k = 0; k < K; ++k) {
            float w[HM_NPT];
#pragma unroll
            for (int j = 0; j < HM_NPT; ++j) { const int n = n0 + 256 * j; w[j] = n < N ? to_f32(Wh[(long long)k * N + n]) : 0.f; }
#pragma unroll
            for (int tt = 0; tt < HM_TT; ++tt) {
                const float xv = xs[tt * K + k];
#pragma unroll
                for (int j = 0; j < HM_NPT; ++j) acc[j][tt] = fmaf(xv, w[j], acc[j][tt]);
            }
        }
#pragma unroll
        for (int tt = 0; tt < HM_TT; ++tt) {
            if (tt >= nt) continue;
            float g = 1.f;
            if (gate) g = 1.0f / (1.0f + expf(-to_f32(gate[(long long)(t0 + tt) * gate_row + h])));
#pragma unroll
            for (int j = 0; j < HM_NPT; ++j) {
                const int n = n0 + 256 * j;
                if (n < N) y[(long long)(t0 + tt) * y_row + h * y_head + n] = from_f32<T>(acc[j][tt] * g);
            }
        }
    }
}

// The same product on the matrix cores (bfloat16, K a multiple of 8 up to 32 KC, operands on 16-byte borders).  Wt is
// [H][N][K]: a column's weights lie together, so a lane's eight k of either operand are one 16-byte load.  A workgroup
// takes 16 tokens of one head; their x stays in registers and the four waves share the output's blocks of 16 columns.
// The product is formed transposed (rows: output columns, columns: tokens), which leaves a lane four neighbouring
// columns of one token.  A token's sums do not depend on the tokens beside it.
template <int KC>
__global__ __launch_bounds__(256) void head_matmul_mfma_kernel(const bf16_t* __restrict__ x, long long x_row, long long x_head,
                                                               const bf16_t* __restrict__ Wt, bf16_t* __restrict__ y, long long y_row,
                                                               long long y_head, const bf16_t* __restrict__ gate, long long gate_row,
                                                               int n_tokens, int K, int N, int vec_store) {
    const int h = blockIdx.y, t0 = blockIdx.x * 16;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n16 = lane % 16, g = lane / 16;
    const int t = t0 + n16;
    const bool tok = t < n_tokens;
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const bf16_t* xr = x + (long long)(tok ? t : 0) * x_row + h * x_head;
    bf16x8 xf[KC];
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) {
        const int k = kc * 32 + g * 8;
        xf[kc] = (tok && k < K) ? *(const bf16x8*)(xr + k) : zero;
    }
    float gv = 1.f;
    if (gate && tok) gv = 1.0f / (1.0f + expf(-to_f32(gate[(long long)t * gate_row + h])));
    const bf16_t* Wh = Wt + (long long)h * N * K;
    for (int nb = wave; nb * 16 < N; nb += 4) {
        const int n = nb * 16 + n16;
        const bf16_t* wr = Wh + (long long)(n < N ? n : 0) * K;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) {
            const int k = kc * 32 + g * 8;
            const bf16x8 wf = (n < N && k < K) ? *(const bf16x8*)(wr + k) : zero;
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf[kc], acc, 0, 0, 0);
        }
        if (!tok) continue;
        const int col = nb * 16 + 4 * g;               // acc[e]: column col + e of token t
        bf16_t* dst = y + (long long)t * y_row + h * y_head + col;
        if (vec_store && col + 3 < N) {
            bf16x4 o4;
#pragma unroll
            for (int e = 0; e < 4; ++e) o4[e] = (bf16_t)(acc[e] * gv);
            *(bf16x4*)dst = o4;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col + e < N) dst[e] = (bf16_t)(acc[e] * gv);
        }
    }
}
}  // namespace

// proj [T][row_stride] of type dt holds, a token: the heads' queries [H][dim + rot] from q_off, the latent's raw
// channels [rank] and the shared key part [rot] from ckr_off.  Writes cache row slot_mapping[t] = [norm(c) w | rotate(k)]
// (cache [slots][rank + rot]; slot_mapping null or a negative slot: nothing is written) and q_lat[t][h][rank ..] =
// rotate(q_rot); q_lat [T][H][rank + rot].  norm_w [rank] of type norm_dt; inv_freq float32 [rot_dims / 2].
// cache_t (or null): the rows once more as [pages][rank + rot][page_size], for kernels that read values that way.
TUFF_EXPORT int tuff_latent_post(const void* proj, int row_stride, int q_off, int ckr_off, void* q_lat, void* cache,
                                 void* cache_t, int page_size, int dt,
                                 const void* norm_w, int norm_dt, float eps, const float* inv_freq, int rot_dims,
                                 const int* positions, const int* slot_mapping, int n_tokens, int H, int dim, int rot, int rank,
                                 hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (H < 1 || dim < 0 || rot < 0 || rank < 1 || rot_dims < 0 || rot_dims > rot || rot_dims % 2) return -2;
    if (cache_t && page_size < 1) return -2;
#define LAUNCH(T, TW) hipLaunchKernelGGL((latent_post_kernel<T, TW>), dim3(n_tokens), dim3(POST_THREADS), 0, stream, (const T*)proj, \
        row_stride, q_off, ckr_off, (T*)q_lat, (T*)cache, (T*)cache_t, page_size, (const TW*)norm_w, eps, inv_freq, rot_dims, positions, slot_mapping, H, dim, rot, rank)
    if (dt == DT_F32 && norm_dt == DT_F32) LAUNCH(float, float);
    else if (dt == DT_F32) LAUNCH(float, bf16_t);
    else if (norm_dt == DT_F32) LAUNCH(bf16_t, float);
    else LAUNCH(bf16_t, bf16_t);
#undef LAUNCH
    return launch_status();
}

// y[t][h][n] = sum_k x[t][h][k] W[h][k][n] (times sigmoid(gate[t][h]) where gate is given); x, W, y, gate of type dt.
// x_row, x_head: elements from a token's row to the next and from a head to the next inside a row; the same for y;
// gate_row: elements from a token's gates to the next token's.
TUFF_EXPORT int tuff_head_matmul(const void* x, long long x_row, long long x_head, const void* W, void* y, long long y_row,
                                 long long y_head, const void* gate, long long gate_row, int dt, int n_tokens, int H, int K, int N,
                                 hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (H < 1 || H > 65535 || K < 1 || N < 1 || (long long)HM_TT * K * 4 > 65536) return -2;
    dim3 grid(ceil_div(n_tokens, HM_TT), H), block(256);
    const size_t lds = (size_t)HM_TT * K * sizeof(float);
    if (dt == DT_F32)
        hipLaunchKernelGGL(head_matmul_kernel<float>, grid, block, lds, stream, (const float*)x, x_row, x_head, (const float*)W,
                           (float*)y, y_row, y_head, (const float*)gate, gate_row, n_tokens, K, N);
    else
        hipLaunchKernelGGL(head_matmul_kernel<bf16_t>, grid, block, lds, stream, (const bf16_t*)x, x_row, x_head, (const bf16_t*)W,
                           (bf16_t*)y, y_row, y_head, (const bf16_t*)gate, gate_row, n_tokens, K, N);
    return launch_status();
}

// The matrix-core form of the product above: bfloat16; Wt is the weight as [H][N][K].  K must be a multiple of 8 and at
// most 512, and x, x_row, x_head must keep every head's row on a 16-byte border (returns -2 otherwise: the caller
// takes the other kernel).
TUFF_EXPORT int tuff_head_matmul_mfma(const void* x, long long x_row, long long x_head, const void* Wt, void* y, long long y_row,
                                      long long y_head, const void* gate, long long gate_row, int n_tokens, int H, int K, int N,
                                      hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (H < 1 || H > 65535 || K < 8 || K % 8 || K > 512 || N < 1) return -2;
    if ((uintptr_t)x % 16 || (uintptr_t)Wt % 16 || x_row % 8 || x_head % 8) return -2;
    const int vec_store = ((uintptr_t)y % 8 == 0 && y_row % 4 == 0 && y_head % 4 == 0) ? 1 : 0;
    dim3 grid(ceil_div(n_tokens, 16), H), block(256);
#define LAUNCH(KC) hipLaunchKernelGGL(head_matmul_mfma_kernel<KC>, grid, block, 0, stream, (const bf16_t*)x, x_row, x_head, \
        (const bf16_t*)Wt, (bf16_t*)y, y_row, y_head, (const bf16_t*)gate, gate_row, n_tokens, K, N, vec_store)
    if (K <= 64) LAUNCH(2);
    else if (K <= 128) LAUNCH(4);
    else if (K <= 256) LAUNCH(8);
    else LAUNCH(16);
#undef LAUNCH
    return launch_status();
}
