// True float32 matrix product  Y[M,N] (=|+=) X[M,K] * W[N,K]^T  with plain FMAs.
//
// Every output element is one chain  acc = fma(x[m,k], w[n,k], acc)  over k = 0..K-1
// in ascending order, whatever the tile it falls into, so a row of Y does not depend
// on how many other rows were in the call.  No matrix cores, no reduced precision.
#include "common.h"

namespace {
constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4, NT = 256;

template <bool ACCUM>
__global__ __launch_bounds__(NT) void gemm_f32_kernel(const float* __restrict__ X, const float* __restrict__ W,
                                                      float* __restrict__ Y, int M, int N, int K) {
    __shared__ float Xs[BK][BM + 4];
    __shared__ float Ws[BK][BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < (BM * BK) / NT; ++i) {
            const int idx = tid + i * NT;
            const int row = idx / BK, kk = idx % BK;
            const int gm = m0 + row, gn = n0 + row, gk = k0 + kk;
            Xs[kk][row] = (gm < M && gk < K) ? X[(long long)gm * K + gk] : 0.f;
            Ws[kk][row] = (gn < N && gk < K) ? W[(long long)gn * K + gk] : 0.f;
        }
        __syncthreads();
        const int kmax = min(BK, K - k0);      // zero padding would be harmless; skip it anyway
        for (int kk = 0; kk < kmax; ++kk) {
            float a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = Xs[kk][ty * TM + i];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = Ws[kk][tx * TN + j];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int gm = m0 + ty * TM + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int gn = n0 + tx * TN + j;
            if (gn >= N) continue;
            float* y = Y + (long long)gm * N + gn;
            if (ACCUM) *y = *y + acc[i][j]; else *y = acc[i][j];
        }
    }
}
}  // namespace

// accumulate != 0: Y += X W^T (the residual add of the reference, src/lfm25_gpu.cu:171).
TUFF_EXPORT int tuff_gemm_f32(const float* X, const float* W, float* Y, int M, int N, int K,
                              int accumulate, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    dim3 grid(ceil_div(N, BN), ceil_div(M, BM)), block(NT);
    if (accumulate) hipLaunchKernelGGL(gemm_f32_kernel<true>, grid, block, 0, stream, X, W, Y, M, N, K);
    else hipLaunchKernelGGL(gemm_f32_kernel<false>, grid, block, 0, stream, X, W, Y, M, N, K);
    return launch_status();
}
