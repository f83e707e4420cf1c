// Row-wise kernels of the residual stream: embedding gather, RMSNorm, SwiGLU gate,
// casts and fills.  The residual stream is float32 in every mode; sums of squares
// are taken in float32 in a fixed order.
#include "common.h"

// ------------------------------------------------------------------ embedding
// out[t, :] = table[tokens[t], :] * scale as float32.  Reference: one row gather per token
// with no scale (src/lfm25_gpu.cu:725-741), which is scale = 1: the product with 1 is exact.
template <typename T>
__global__ void embed_rows_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                                  float* __restrict__ out, int d, float scale) {
    const int t = blockIdx.x;
    const long long row = tokens[t];
    const T* src = table + row * (long long)d;
    float* dst = out + (long long)t * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) dst[i] = to_f32(src[i]) * scale;
}

TUFF_EXPORT int tuff_embed_rows(const void* table, int table_dt, const int* tokens, float* out,
                                int n_tokens, int d, float scale, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens), block(256);
    if (table_dt == DT_F32)
        hipLaunchKernelGGL(embed_rows_kernel<float>, grid, block, 0, stream, (const float*)table, tokens, out, d, scale);
    else
        hipLaunchKernelGGL(embed_rows_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)table, tokens, out, d, scale);
    return launch_status();
}

// ----------------------------------------------------------------------- bias
// y[r, c] += bias[c], the sum in float32: for projections with a bias, after their product (the
// products' epilogues have none).
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, const float* __restrict__ bias, long long n, int N) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = from_f32<T>(to_f32(y[i]) + bias[i % N]);
}

TUFF_EXPORT int tuff_add_bias(void* y, int dt, const float* bias, long long rows, int N, hipStream_t stream) {
    const long long n = rows * N;
    if (n <= 0) return 0;
    dim3 grid((unsigned)ceil_div_ll(n, 256)), block(256);
    if (dt == DT_F32) hipLaunchKernelGGL(add_bias_kernel<float>, grid, block, 0, stream, (float*)y, bias, n, N);
    else hipLaunchKernelGGL(add_bias_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)y, bias, n, N);
    return launch_status();
}

// --------------------------------------------------------------- logits: scale and soft cap
// x <- x * scale, then, with cap > 0, x <- cap * tanh(x / cap).
__global__ void scale_cap_kernel(float* __restrict__ x, long long n, float scale, float cap) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = x[i] * scale;
    if (cap > 0.f) v = cap * tanhf(v / cap);
    x[i] = v;
}

TUFF_EXPORT int tuff_scale_cap(float* x, long long n, float scale, float cap, hipStream_t stream) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(scale_cap_kernel, dim3((unsigned)ceil_div_ll(n, 256)), dim3(256), 0, stream, x, n, scale, cap);
    return launch_status();
}

// -------------------------------------------------------------------- RMSNorm
// y_i = x_i * (1 / sqrt(mean_j x_j^2 + eps)) * w_i   (src/lfm25_gpu.cu:235,244).
// `rows` (optional) gathers input rows: output row r is the norm of x[rows[r]].
// Per-thread strided partial sums -> wave butterfly -> wave partials in order; which elements a
// thread takes depends on d alone (multiples of 4: four neighbours a step).
template <typename TW, typename TO, bool VEC>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const TW* __restrict__ w,
                                                      TO* __restrict__ out, const int* __restrict__ rows, int d, float eps) {
    __shared__ float scratch[4];
    const int r = blockIdx.x;
    const long long src = rows ? rows[r] : r;
    const float* xr = x + src * (long long)d;
    TO* o = out + (long long)r * d;
    float ss = 0.f;
    if (VEC) {
        // d is a multiple of 4: four neighbouring elements a thread and step, 16-byte loads
        for (int i = threadIdx.x * 4; i < d; i += 1024) {
            const f32x4 v = *(const f32x4*)(xr + i);
            ss = fmaf(v[0], v[0], ss); ss = fmaf(v[1], v[1], ss); ss = fmaf(v[2], v[2], ss); ss = fmaf(v[3], v[3], ss);
        }
    } else {
        for (int i = threadIdx.x; i < d; i += 256) { const float v = xr[i]; ss += v * v; }
    }
    const float total = block_sum<4>(ss, scratch);
    const float inv = 1.0f / sqrtf(total / (float)d + eps);
    if (VEC) {
        for (int i = threadIdx.x * 4; i < d; i += 1024) {
            const f32x4 v = *(const f32x4*)(xr + i);
            TO y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = from_f32<TO>(v[e] * inv * to_f32(w[i + e]));
            if (sizeof(TO) == 2) *(uint2*)(o + i) = *(const uint2*)y;
            else *(uint4*)(o + i) = *(const uint4*)y;
        }
    } else {
        for (int i = threadIdx.x; i < d; i += 256) o[i] = from_f32<TO>(xr[i] * inv * to_f32(w[i]));
    }
}

TUFF_EXPORT int tuff_rmsnorm(const float* x, const void* w, int w_dt, void* out, int out_dt,
                             const int* rows, int n_rows, int d, float eps, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    dim3 grid(n_rows), block(256);
#define LAUNCH(TW, TO) do { \
        if (d % 4 == 0) hipLaunchKernelGGL((rmsnorm_kernel<TW, TO, true>), grid, block, 0, stream, x, (const TW*)w, (TO*)out, rows, d, eps); \
        else hipLaunchKernelGGL((rmsnorm_kernel<TW, TO, false>), grid, block, 0, stream, x, (const TW*)w, (TO*)out, rows, d, eps); \
    } while (0)
    if (w_dt == DT_F32 && out_dt == DT_F32) LAUNCH(float, float);
    else if (w_dt == DT_F32 && out_dt == DT_BF16) LAUNCH(float, bf16_t);
    else if (w_dt == DT_BF16 && out_dt == DT_F32) LAUNCH(bf16_t, float);
    else LAUNCH(bf16_t, bf16_t);
#undef LAUNCH
    return launch_status();
}

// --------------------------------------------------------------------- SwiGLU
// act[t, f] = g / (1 + exp(-g)) * u with g = gu[t, f], u = gu[t, F + f]
// (src/lfm25_gpu.cu:614-617), evaluated in float32.
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ act, long long n, int F) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long long t = i / F;
    const int f = (int)(i - t * F);
    const float g = to_f32(gu[t * 2 * F + f]);
    const float u = to_f32(gu[t * 2 * F + F + f]);
    act[i] = from_f32<T>(g / (1.0f + expf(-g)) * u);
}

TUFF_EXPORT int tuff_swiglu(const void* gu, void* act, int dt, int n_tokens, int F, hipStream_t stream) {
    const long long n = (long long)n_tokens * F;
    if (n <= 0) return 0;
    dim3 grid((unsigned)ceil_div_ll(n, 256)), block(256);
    if (dt == DT_F32) hipLaunchKernelGGL(swiglu_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)act, n, F);
    else hipLaunchKernelGGL(swiglu_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)act, n, F);
    return launch_status();
}

// ----------------------------------------------------------------------- cast
template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = from_f32<TO>(to_f32(in[i]));
}

TUFF_EXPORT int tuff_cast(const void* in, int in_dt, void* out, int out_dt, long long n, hipStream_t stream) {
    if (n <= 0) return 0;
    dim3 grid((unsigned)ceil_div_ll(n, 256)), block(256);
    if (in_dt == DT_F32 && out_dt == DT_BF16) hipLaunchKernelGGL((cast_kernel<float, bf16_t>), grid, block, 0, stream, (const float*)in, (bf16_t*)out, n);
    else if (in_dt == DT_BF16 && out_dt == DT_F32) hipLaunchKernelGGL((cast_kernel<bf16_t, float>), grid, block, 0, stream, (const bf16_t*)in, (float*)out, n);
    else if (in_dt == DT_F32) hipLaunchKernelGGL((cast_kernel<float, float>), grid, block, 0, stream, (const float*)in, (float*)out, n);
    else hipLaunchKernelGGL((cast_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (const bf16_t*)in, (bf16_t*)out, n);
    return launch_status();
}

// ----------------------------------------------------------------------- fill
// Sets n 32-bit words to `value`; used instead of a memset so that a caller may
// record it into a graph.
__global__ void fill_u32_kernel(uint32_t* __restrict__ p, uint32_t value, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = value;
}

TUFF_EXPORT int tuff_fill_u32(void* p, uint32_t value, long long n, hipStream_t stream) {
    if (n <= 0) return 0;
    dim3 grid((unsigned)ceil_div_ll(n, 256)), block(256);
    hipLaunchKernelGGL(fill_u32_kernel, grid, block, 0, stream, (uint32_t*)p, value, n);
    return launch_status();
}

// -------------------------------------------------------------------- scatter
// dst[idx[i]] = src[idx[n + i]] for i < n, bounds checked (a bad index writes nothing): token ids that
// a sampling kernel has left on the device go into the next step's token buffer without a trip
// to the host.
__global__ void scatter_i32_kernel(int* __restrict__ dst, int n_dst, const int* __restrict__ src, int n_src,
                                   const int* __restrict__ idx, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int d = idx[i], s = idx[n + i];
    if (d >= 0 && d < n_dst && s >= 0 && s < n_src) dst[d] = src[s];
}

TUFF_EXPORT int tuff_scatter_i32(int* dst, int n_dst, const int* src, int n_src, const int* idx, int n, hipStream_t stream) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(scatter_i32_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, stream, dst, n_dst, src, n_src, idx, n);
    return launch_status();
}
