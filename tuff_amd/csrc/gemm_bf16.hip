// bfloat16 matrix products on the gfx950 matrix cores:  Y[M,N] (=|+=) X[M,K] * W[N,K]^T,
// X and W bfloat16 with K contiguous, products accumulated in float32.
//
// Two kernels, chosen by M on the host:
//  * gemm_bf16_tiled   M > 64: 128x128 block tiles staged through LDS (compute bound);
//  * gemm_bf16_skinny  M <= 64: weights streamed once from HBM straight into MFMA
//    operands, K split over the four waves of a workgroup and summed in wave order
//    (bandwidth bound).
// Both use v_mfma_f32_16x16x32_bf16.  Lane l of a wave supplies row (l % 16) of an
// operand tile and eight consecutive k at 8 * (l / 16); it receives rows
// 4 * (l / 16) + 0..3, column (l % 16) of the 16x16 result.
// Within one kernel the order in which the products of an output element are added
// depends on K alone, never on M, N or the position of the row in the call.
#include "common.h"

enum : int { OUT_BF16 = 0, OUT_F32 = 1, OUT_F32_ACCUM = 2 };

namespace {

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

template <int MODE>
__device__ __forceinline__ void store_out(void* Y, long long idx, float v) {
    if (MODE == OUT_BF16) ((bf16_t*)Y)[idx] = (bf16_t)v;
    else if (MODE == OUT_F32) ((float*)Y)[idx] = v;
    else ((float*)Y)[idx] += v;
}

// 16-byte load of eight bf16 with a guard; out-of-range pieces read as zero.
__device__ __forceinline__ bf16x8 load8(const bf16_t* base, long long row, int nrows, int k, int K) {
    bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
    if (row < nrows && k < K) return *(const bf16x8*)(base + row * (long long)K + k);
    return z;
}

// ------------------------------------------------------------------ tiled kernel
constexpr int TBM = 128, TBN = 128, TBK = 64, TNT = 256;
constexpr int CHUNKS = TBK / 8;                     // 16-byte chunks in one row of a tile

// Chunk c of row r lives at chunk position c ^ (r % CHUNKS): the sixteen lanes that
// read one k-chunk of sixteen rows then hit different LDS banks.
__device__ __forceinline__ int swz(int r, int c) { return r * TBK + ((c ^ (r % CHUNKS)) * 8); }

template <int MODE>
__global__ __launch_bounds__(TNT) void gemm_bf16_tiled_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                              void* __restrict__ Y, int M, int N, int K) {
    __shared__ __attribute__((aligned(16))) bf16_t As[2][TBM * TBK];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[2][TBN * TBK];
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int wm = (wave / 2) * 64, wn = (wave % 2) * 64;
    const int r16 = lane % 16, g = lane / 16;
    const long long m0 = (long long)blockIdx.y * TBM, n0 = (long long)blockIdx.x * TBN;

    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    constexpr int PER_THREAD = (TBM * CHUNKS) / TNT;     // 4 chunks of A and 4 of B per thread
    bf16x8 ra[PER_THREAD], rb[PER_THREAD];

    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            const int id = tid + i * TNT;
            const int row = id / CHUNKS, c = id % CHUNKS;
            ra[i] = load8(X, m0 + row, M, k0 + c * 8, K);
            rb[i] = load8(W, n0 + row, N, k0 + c * 8, K);
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            const int id = tid + i * TNT;
            const int row = id / CHUNKS, c = id % CHUNKS;
            *(bf16x8*)(&As[buf][swz(row, c)]) = ra[i];
            *(bf16x8*)(&Bs[buf][swz(row, c)]) = rb[i];
        }
    };

    const int nk = (K + TBK - 1) / TBK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load_global((kt + 1) * TBK);
#pragma unroll
        for (int ks = 0; ks < TBK / 32; ++ks) {
            bf16x8 a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = *(const bf16x8*)(&As[buf][swz(wm + i * 16 + r16, ks * 4 + g)]);
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = *(const bf16x8*)(&Bs[buf][swz(wn + j * 16 + r16, ks * 4 + g)]);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = mfma16(a[i], b[j], acc[i][j]);
        }
        if (kt + 1 < nk) store_lds(buf ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const long long col = n0 + wn + j * 16 + r16;
            if (col >= N) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const long long row = m0 + wm + i * 16 + g * 4 + e;
                if (row < M) store_out<MODE>(Y, row * N + col, acc[i][j][e]);
            }
        }
}

// ----------------------------------------------------------------- skinny kernel
// One workgroup owns 16 rows of W (16 output columns) and all M <= 16*MT rows of X.
// Wave w takes the k-chunks w, w+4, w+8, ... of 128 elements; in a chunk a lane reads
// 64 contiguous bytes of its W row (and of each X row) and issues four MFMAs.  The four
// wave partials are added in wave order 0,1,2,3 through LDS.
constexpr int SK_CHUNK = 128, SK_NT = 256;

template <int MT, int MODE>
__global__ __launch_bounds__(SK_NT) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                                 void* __restrict__ Y, int M, int N, int K) {
    __shared__ float red[4][MT][WAVE][4];
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int r16 = lane % 16, g = lane / 16;
    const long long n0 = (long long)blockIdx.x * 16;

    f32x4 acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nchunks = (K + SK_CHUNK - 1) / SK_CHUNK;
    for (int c = wave; c < nchunks; c += 4) {
        const int kb = c * SK_CHUNK + g * 32;
        bf16x8 b[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = load8(W, n0 + r16, N, kb + j * 8, K);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            bf16x8 a[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) a[j] = load8(X, i * 16 + r16, M, kb + j * 8, K);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i] = mfma16(a[j], b[j], acc[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) red[wave][i][lane][e] = acc[i][e];
    __syncthreads();
    // 256 threads share the MT*64*4 sums: element id -> (i, lane, e)
    for (int id = tid; id < MT * WAVE * 4; id += SK_NT) {
        const int e = id % 4, l = (id / 4) % WAVE, i = id / (4 * WAVE);
        const float v = ((red[0][i][l][e] + red[1][i][l][e]) + red[2][i][l][e]) + red[3][i][l][e];
        const long long row = i * 16 + (l / 16) * 4 + e, col = n0 + (l % 16);
        if (row < M && col < N) store_out<MODE>(Y, row * N + col, v);
    }
}

template <int MODE>
int launch_mode(const bf16_t* X, const bf16_t* W, void* Y, int M, int N, int K, hipStream_t stream) {
    if (M <= 64) {
        dim3 grid(ceil_div(N, 16)), block(SK_NT);
        const int mt = ceil_div(M, 16);
        if (mt == 1) hipLaunchKernelGGL((gemm_bf16_skinny_kernel<1, MODE>), grid, block, 0, stream, X, W, Y, M, N, K);
        else if (mt == 2) hipLaunchKernelGGL((gemm_bf16_skinny_kernel<2, MODE>), grid, block, 0, stream, X, W, Y, M, N, K);
        else if (mt == 3) hipLaunchKernelGGL((gemm_bf16_skinny_kernel<3, MODE>), grid, block, 0, stream, X, W, Y, M, N, K);
        else hipLaunchKernelGGL((gemm_bf16_skinny_kernel<4, MODE>), grid, block, 0, stream, X, W, Y, M, N, K);
    } else {
        dim3 grid(ceil_div(N, TBN), ceil_div(M, TBM)), block(TNT);
        hipLaunchKernelGGL((gemm_bf16_tiled_kernel<MODE>), grid, block, 0, stream, X, W, Y, M, N, K);
    }
    return launch_status();
}
}  // namespace

// K must be a multiple of 8 (16-byte operand loads); the host wrapper refuses other K.
TUFF_EXPORT int tuff_gemm_bf16(const void* X, const void* W, void* Y, int M, int N, int K, int mode,
                               hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 != 0) return -2;
    const bf16_t* x = (const bf16_t*)X;
    const bf16_t* w = (const bf16_t*)W;
    if (mode == OUT_BF16) return launch_mode<OUT_BF16>(x, w, Y, M, N, K, stream);
    if (mode == OUT_F32) return launch_mode<OUT_F32>(x, w, Y, M, N, K, stream);
    if (mode == OUT_F32_ACCUM) return launch_mode<OUT_F32_ACCUM>(x, w, Y, M, N, K, stream);
    return -3;
}
