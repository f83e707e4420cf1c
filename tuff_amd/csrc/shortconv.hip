// Gated short convolution of a mixed batch, with per-request state.
//
//   bcx = in_proj(h): B = bcx[0:d], C = bcx[d:2d], X = bcx[2d:3d];  u = B * X
//   y_t = sum_{k=0}^{K-1} w[c, k] * u_{t-(K-1)+k}      (tap K-1 is the current token)
//   out = C * y;   state <- the last K-1 rows of u
// (src/lfm25_gpu.cu:378-397 for one token, :1056-1079 over a chunk;
//  tools/lfm25_fp64_ref.py:118-126.)
//
// The convolution is a finite filter, not a recurrence: a token needs only the K-1
// values of u before it.  Those come from earlier tokens of the same portion when they
// are in this step, and from the request's state slot otherwise, so all tokens of a
// step run in parallel and the sum  fma(u_2, w_2, fma(u_1, w_1, u_0 * w_0))  is the
// same chain of operations wherever the portion was cut.  The state holds u in float32
// (a product of two bfloat16 values is exact in float32).
//
// The forward kernel comes in two forms.  Reading only: every token is a thread's own, and a second
// kernel (shortconv_state), launched after it on the same stream, rewrites each (slot, channel) column.
// Updating: the thread of a request's first token also computes the other tokens that read the old
// state (the first K-1 of the portion) and then writes the new state, rows in ascending order; no
// other thread touches that column of the state, so nothing races and no second kernel is needed.
#include "common.h"

namespace {
constexpr int MAX_TAPS = 16;

// Token i of its request's portion (row t = t0 + i of the step), channel c.
template <typename T, typename TW>
__device__ __forceinline__ void conv_token(const T* __restrict__ bcx, const TW* __restrict__ conv_w, const float* st,
                                           T* __restrict__ out, int t0, int i, int c, int d, int K) {
    const int t = t0 + i;
    float y = 0.f;
    for (int k = 0; k < K; ++k) {
        const int src = i - (K - 1) + k;
        float u;
        if (src >= 0) {
            const T* row = bcx + (long long)(t0 + src) * 3 * d;
            u = to_f32(row[c]) * to_f32(row[2 * d + c]);
        } else {
            u = st[(long long)(K - 1 + src) * d + c];
        }
        const float w = to_f32(conv_w[(long long)c * K + k]);
        y = (k == 0) ? u * w : fmaf(u, w, y);
    }
    const float cg = to_f32(bcx[(long long)t * 3 * d + d + c]);
    out[(long long)t * d + c] = from_f32<T>(cg * y);
}

template <typename T, typename TW, bool UPDATE>
__global__ void shortconv_fwd_kernel(const T* __restrict__ bcx, const TW* __restrict__ conv_w,
                                     float* state, T* __restrict__ out,
                                     const int* __restrict__ req_of_token, const int* __restrict__ q_start,
                                     const int* __restrict__ q_len, const int* __restrict__ state_slot, int d, int K) {
    const int t = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= d) return;
    const int r = req_of_token[t];
    const int t0 = q_start[r];
    const int i = t - t0;
    float* st = state + (long long)state_slot[r] * (K - 1) * d;
    if (!UPDATE || i >= K - 1) {
        conv_token(bcx, conv_w, st, out, t0, i, c, d, K);
        return;
    }
    if (i > 0) return;                              // done by the thread of the request's first token
    const int n = q_len[r];
    for (int ii = 0; ii < min(n, K - 1); ++ii) conv_token(bcx, conv_w, st, out, t0, ii, c, d, K);
    for (int j = 0; j < K - 1; ++j) {               // row j <- u of token n - (K-1) + j, or the old row j + n (not yet rewritten)
        const int src = n - (K - 1) + j;
        float u;
        if (src >= 0) {
            const T* row = bcx + (long long)(t0 + src) * 3 * d;
            u = to_f32(row[c]) * to_f32(row[2 * d + c]);
        } else {
            u = st[(long long)(j + n) * d + c];
        }
        st[(long long)j * d + c] = u;
    }
}

// The same for bfloat16 activations, eight channels a thread (16-byte loads and stores); d must
// be a multiple of 8.  Every channel goes through the chain of operations of the kernel above.
template <typename TW, int KT, bool UPDATE>       // KT: the kernel length if it is 2, 3 or 4, else 0 (read K)
__global__ void shortconv_fwd_vec_kernel(const bf16_t* __restrict__ bcx, const TW* __restrict__ conv_w,
                                         float* state, bf16_t* __restrict__ out,
                                         const int* __restrict__ req_of_token, const int* __restrict__ q_start,
                                         const int* __restrict__ q_len, const int* __restrict__ state_slot, int d, int K_arg) {
    const int K = KT ? KT : K_arg;
    const int t_own = blockIdx.x;
    const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
    if (c >= d) return;
    const int r = req_of_token[t_own];
    const int t0 = q_start[r];
    const int i_own = t_own - t0;
    if (UPDATE && i_own > 0 && i_own < K - 1) return;      // done by the thread of the request's first token
    float* st = state + (long long)state_slot[r] * (K - 1) * d;
    // the taps of the thread's eight channels are 8 K neighbouring weights: with a known K they come
    // in whole pieces of eight
    float wl[KT ? 8 * KT : 1];
    if (KT) {
#pragma unroll
        for (int p = 0; p < KT; ++p)
#pragma unroll
            for (int e = 0; e < 8; ++e) wl[p * 8 + e] = to_f32(conv_w[(long long)c * KT + p * 8 + e]);
    }
    auto u_of = [&](int src, float (&u)[8]) {       // u of the portion's token src, or of the state's row K-1+src
        if (src >= 0) {
            const bf16_t* row = bcx + (long long)(t0 + src) * 3 * d;
            const bf16x8 b = *(const bf16x8*)(row + c), x = *(const bf16x8*)(row + 2 * d + c);
#pragma unroll
            for (int e = 0; e < 8; ++e) u[e] = (float)b[e] * (float)x[e];
        } else {
            const float* p = st + (long long)(K - 1 + src) * d + c;
            const f32x4 u0 = *(const f32x4*)p, u1 = *(const f32x4*)(p + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) { u[e] = u0[e]; u[4 + e] = u1[e]; }
        }
    };
    auto token = [&](int i) {
        const int t = t0 + i;
        float y[8];
#pragma unroll
        for (int k = 0; k < (KT ? KT : 1) * (KT ? 1 : K); ++k) {
            float u[8];
            u_of(i - (K - 1) + k, u);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float w = KT ? wl[e * (KT ? KT : 1) + k] : to_f32(conv_w[(long long)(c + e) * K + k]);
                y[e] = (k == 0) ? u[e] * w : fmaf(u[e], w, y[e]);
            }
        }
        const bf16x8 cg = *(const bf16x8*)(bcx + (long long)t * 3 * d + d + c);
        bf16x8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (bf16_t)((float)cg[e] * y[e]);
        *(bf16x8*)(out + (long long)t * d + c) = o;
    };
    if (!UPDATE || i_own > 0) {
        token(i_own);
        return;
    }
    const int n = q_len[r];
    for (int ii = 0; ii < min(n, K - 1); ++ii) token(ii);
    for (int j = 0; j < K - 1; ++j) {               // row j <- u of token n - (K-1) + j, or the old row j + n (not yet rewritten)
        float u[8];
        u_of(n - (K - 1) + j, u);
        float* p = st + (long long)j * d + c;
        *(f32x4*)p = f32x4{u[0], u[1], u[2], u[3]};
        *(f32x4*)(p + 4) = f32x4{u[4], u[5], u[6], u[7]};
    }
}

template <typename T>
__global__ void shortconv_state_kernel(const T* __restrict__ bcx, float* __restrict__ state,
                                       const int* __restrict__ q_start, const int* __restrict__ q_len,
                                       const int* __restrict__ state_slot, int d, int K) {
    const int r = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= d) return;
    const int t0 = q_start[r], n = q_len[r];
    if (n <= 0) return;                          // an entry without tokens (padding of a recorded step) owns no state
    float* st = state + (long long)state_slot[r] * (K - 1) * d;
    float tmp[MAX_TAPS];
    for (int j = 0; j < K - 1; ++j) {
        const int src = n - (K - 1) + j;
        if (src >= 0) {
            const T* row = bcx + (long long)(t0 + src) * 3 * d;
            tmp[j] = to_f32(row[c]) * to_f32(row[2 * d + c]);
        } else {
            tmp[j] = st[(long long)(K - 1 + src) * d + c];
        }
    }
    for (int j = 0; j < K - 1; ++j) st[(long long)j * d + c] = tmp[j];
}
// A step of single tokens (every request of the step has exactly one): output and new state in
// one pass.  Thread (r, c) owns column c of request r's state, so reading the old rows and
// writing the new ones needs no second kernel.  Same chain of operations as the two above.
template <typename T, typename TW>
__global__ void shortconv_decode_kernel(const T* __restrict__ bcx, const TW* __restrict__ conv_w, float* __restrict__ state,
                                        T* __restrict__ out, const int* __restrict__ state_slot, int d, int K) {
    const int r = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= d) return;
    float* st = state + (long long)state_slot[r] * (K - 1) * d;
    const T* row = bcx + (long long)r * 3 * d;
    // every load first (a store into the state in between would hold the loads after it back), then
    // the chain, then the stores
    float s[MAX_TAPS], w[MAX_TAPS];
#pragma unroll
    for (int k = 0; k < MAX_TAPS; ++k) {
        s[k] = k < K - 1 ? st[(long long)k * d + c] : 0.f;
        w[k] = k < K - 1 ? to_f32(conv_w[(long long)c * K + k]) : 0.f;
    }
    const float w_last = to_f32(conv_w[(long long)c * K + K - 1]);
    const float u = to_f32(row[c]) * to_f32(row[2 * d + c]);
    const float gate = to_f32(row[d + c]);
    float y = 0.f;
#pragma unroll
    for (int k = 0; k < MAX_TAPS; ++k)
        if (k < K - 1) y = (k == 0) ? s[k] * w[k] : fmaf(s[k], w[k], y);
    y = fmaf(u, w_last, y);
#pragma unroll
    for (int k = 1; k < MAX_TAPS; ++k)
        if (k < K - 1) st[(long long)(k - 1) * d + c] = s[k];
    st[(long long)(K - 2) * d + c] = u;
    out[(long long)r * d + c] = from_f32<T>(gate * y);
}
}  // namespace

TUFF_EXPORT int tuff_shortconv_decode(const void* bcx, const void* conv_w, int w_dt, float* state, void* out, int dt,
                                      const int* state_slot, int n_requests, int d, int K, hipStream_t stream) {
    if (n_requests <= 0) return 0;
    if (K < 2 || K - 1 > MAX_TAPS) return -2;
    dim3 block(256), grid(n_requests, ceil_div(d, 256));
#define LAUNCH(T, TW) hipLaunchKernelGGL((shortconv_decode_kernel<T, TW>), grid, block, 0, stream, (const T*)bcx, (const TW*)conv_w, \
        state, (T*)out, state_slot, d, K)
    if (dt == DT_F32 && w_dt == DT_F32) LAUNCH(float, float);
    else if (dt == DT_F32) LAUNCH(float, bf16_t);
    else if (w_dt == DT_F32) LAUNCH(bf16_t, float);
    else LAUNCH(bf16_t, bf16_t);
#undef LAUNCH
    return launch_status();
}

// q_len: null, the state is only read; else [requests], and the state of every request with tokens in the
// step is rewritten as well (the last K-1 values of u, as tuff_shortconv_state leaves them).
TUFF_EXPORT int tuff_shortconv_fwd(const void* bcx, const void* conv_w, int w_dt, float* state, void* out, int dt,
                                   const int* req_of_token, const int* q_start, const int* q_len, const int* state_slot,
                                   int n_tokens, int d, int K, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (K < 2 || K - 1 > MAX_TAPS) return -2;
    if (dt == DT_BF16 && d % 8 == 0 && n_tokens > 16) {
        const int threads = d / 8 < 256 ? ((d / 8 + 63) / 64) * 64 : 256;
        dim3 vblock(threads), vgrid(n_tokens, ceil_div(d / 8, threads));
#define VEC_U(TW, KT, U) hipLaunchKernelGGL((shortconv_fwd_vec_kernel<TW, KT, U>), vgrid, vblock, 0, stream, (const bf16_t*)bcx, \
                                             (const TW*)conv_w, state, (bf16_t*)out, req_of_token, q_start, q_len, state_slot, d, K)
#define VEC(TW, KT) do { if (q_len) VEC_U(TW, KT, true); else VEC_U(TW, KT, false); } while (0)
#define VEC_K(TW) do { if (K == 2) VEC(TW, 2); else if (K == 3) VEC(TW, 3); else if (K == 4) VEC(TW, 4); else VEC(TW, 0); } while (0)
        if (w_dt == DT_F32) VEC_K(float); else VEC_K(bf16_t);
#undef VEC_K
#undef VEC
#undef VEC_U
        return launch_status();
    }
    dim3 block(256), grid(n_tokens, ceil_div(d, 256));
#define LAUNCH_U(T, TW, U) hipLaunchKernelGGL((shortconv_fwd_kernel<T, TW, U>), grid, block, 0, stream, (const T*)bcx, (const TW*)conv_w, \
        state, (T*)out, req_of_token, q_start, q_len, state_slot, d, K)
#define LAUNCH(T, TW) do { if (q_len) LAUNCH_U(T, TW, true); else LAUNCH_U(T, TW, false); } while (0)
    if (dt == DT_F32 && w_dt == DT_F32) LAUNCH(float, float);
    else if (dt == DT_F32) LAUNCH(float, bf16_t);
    else if (w_dt == DT_F32) LAUNCH(bf16_t, float);
    else LAUNCH(bf16_t, bf16_t);
#undef LAUNCH
#undef LAUNCH_U
    return launch_status();
}

TUFF_EXPORT int tuff_shortconv_state(const void* bcx, int dt, float* state, const int* q_start, const int* q_len,
                                     const int* state_slot, int n_requests, int d, int K, hipStream_t stream) {
    if (n_requests <= 0) return 0;
    if (K < 2 || K - 1 > MAX_TAPS) return -2;
    dim3 block(256), grid(n_requests, ceil_div(d, 256));
    if (dt == DT_F32) hipLaunchKernelGGL(shortconv_state_kernel<float>, grid, block, 0, stream, (const float*)bcx, state, q_start, q_len, state_slot, d, K);
    else hipLaunchKernelGGL(shortconv_state_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)bcx, state, q_start, q_len, state_slot, d, K);
    return launch_status();
}
