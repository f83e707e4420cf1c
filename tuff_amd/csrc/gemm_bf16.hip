// bfloat16 matrix products on the gfx950 matrix cores:  Y[M,N] (=|+=) X[M,K] * W[N,K]^T,
// X bfloat16 with K contiguous, products accumulated in float32.
//
// W is stored tile-major: [ceil(N/16)][ceil(K/32)] blocks of 16 rows x 32 k, each block 1 KB in
// the order a wave's MFMA operand wants it (piece l of 16 bytes = row l % 16, k 8 (l / 16) .. + 7),
// rows and k beyond the matrix zero.  One load instruction of a wave then reads 1 KB in one run
// instead of 64 bytes from each of sixteen rows that lie a whole row apart; measured on streams of
// the shapes of a decode step, the run-wise reads are 17 % faster.
//
// Three kernels, chosen by the sizes on the host:
//  * tiled     M > 64: 128x128 or 256x256 block tiles staged through LDS (compute bound), in two
//    forms: operands loaded straight into LDS (K a multiple of 64) or through registers (other K);
//  * skinny64  up to 64 rows that skinny16 does not take: a workgroup owns 64 rows of W, one MFMA column
//    tile a wave; the activations of a K chunk are staged once in LDS for all four waves (bandwidth bound);
//  * skinny16  M <= 16, and up to 32 rows (two row tiles a wave) where few_rows_kernel() says so:
//    a workgroup owns 8 to 64 rows of W; its waves split K (bandwidth bound), no barrier in the loop.
// The skinny kernels stream each weight byte once from HBM straight into MFMA operands.  Where
// N alone gives too little parallelism to fill 256 CUs, skinny16 uses more waves a workgroup
// (8 or 16, partials added in wave order through LDS) and skinny64 splits K over workgroups
// (partial tiles in a work space, added in slice order by a second kernel, which also does the
// epilogue).  Within a kernel the cut depends on N and K only (and on whether M is beyond 16), so the
// order of additions is fixed.
//
// All use v_mfma_f32_16x16x32_bf16.  Lane l of a wave supplies row (l % 16) of an operand tile
// and eight consecutive k at 8 * (l / 16); it receives rows 4 * (l / 16) + 0..3, column (l % 16)
// of the 16x16 result.
#include "common.h"
#include <stdlib.h>

// OUT_SWIGLU: the rows of W are gate and up rows interleaved (2f: gate f, 2f+1: up f); the
// output is bfloat16 [M, N/2] with y[m, f] = silu(g) * u, silu(g) = g / (1 + exp(-g)).
// OUT_CONV (at most 16 rows, one token a row): W is the input projection of a gated short convolution
// with its rows regrouped, sixteen channels a group, as [B of the group | C of the group | X of the
// group]; the epilogue forms u = B * X, runs the convolution over the row's state, writes
// bfloat16 C * y [M, N/3] and shifts u into the state.  No projected row ever reaches memory.
enum : int { OUT_BF16 = 0, OUT_F32 = 1, OUT_F32_ACCUM = 2, OUT_SWIGLU = 3, OUT_CONV = 4 };

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

__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.0f + expf(-g)) * u; }

// Stores element (row, col) of the product.  For OUT_SWIGLU `partner` is the value of column
// col ^ 1 of the same row; even columns (the gates) write.  Every lane must call it.
template <int MODE>
__device__ __forceinline__ void store_elem(void* Y, long long row, long long col, int M, int N, float v, float partner) {
    if (MODE == OUT_SWIGLU) {
        if ((col & 1) == 0 && row < M && col < N) ((bf16_t*)Y)[row * (N / 2) + col / 2] = (bf16_t)silu_mul(v, partner);
    } else {
        if (row < M && col < N) store_out<MODE>(Y, row * N + col, v);
    }
}

// 16-byte load of eight bf16 with a guard; out-of-range pieces read as zero.
__device__ __forceinline__ bf16x8 load8(const bf16_t* base, long long row, int nrows, int k, int K) {
    bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
    if (row < nrows && k < K) return *(const bf16x8*)(base + row * (long long)K + k);
    return z;
}

// Piece `piece` (0..63) of block (tile, kblock) of a tile-major W with kb blocks a row tile.
// Weights of a skinny product are read once and never again: a streaming (non-temporal) load.
__device__ __forceinline__ bf16x8 load_w(const bf16_t* W, long long tile, int kb, int kblock, int piece) {
    return __builtin_nontemporal_load((const bf16x8*)(W + ((tile * kb + kblock) * 64 + piece) * 8));
}

// ------------------------------------------------------------------ tiled kernel
// A workgroup of WAVES_M x WAVES_N waves computes a block of Y; each wave a (16 TM) x (16 TN) part
// of it as TM x TN MFMA tiles.  K is walked in steps of 64 through two LDS buffers: while a step
// is multiplied out of one buffer, the next step's operands travel from memory to registers and,
// piece by piece between the MFMAs, into the other buffer; one barrier a step.
//
// What the shapes answer to, measured on this part: one wave per SIMD issues MFMAs at little more
// than half the rate two waves reach, the LDS takes about 170 bytes/ns per CU and gives 350 to
// 430, against 8600 flop/ns per CU of the matrix cores.  So
//   large:  256 x 256 blocks of eight waves (2 x 4, 128 x 64 each), 128 KB of LDS: two waves per
//           SIMD, and per flop the least LDS traffic two buffers of 160 KB allow;
//   small:  128 x 128 blocks of eight waves (2 x 4, 64 x 32 each), 64 KB of LDS, where the product
//           has too few large blocks to give every CU one.
// The MFMA takes W as its first operand, so a lane ends up with four neighbouring columns of one
// row of Y and stores them as one piece.
constexpr int TBK = 64;
constexpr int CHUNKS = TBK / 8;                     // 16-byte chunks in one row of a tile

// Chunk c of row r lives at chunk position c ^ (r % CHUNKS): the sixteen lanes that
// read one k-chunk of sixteen rows then hit different LDS banks.
__device__ __forceinline__ int swz(int r, int c) { return r * TBK + ((c ^ (r % CHUNKS)) * 8); }

template <int MODE>
__device__ __forceinline__ void store_quad(void* Y, long long row, long long col, int M, int N, f32x4 v) {
    if (row >= M) return;
    if (MODE == OUT_SWIGLU) {
        bf16_t* out = (bf16_t*)Y + row * (N / 2) + col / 2;
        if (col + 3 < N && N % 4 == 0) {
            bf16x2 o = {(bf16_t)silu_mul(v[0], v[1]), (bf16_t)silu_mul(v[2], v[3])};
            *(bf16x2*)out = o;
        } else {
            if (col + 1 < N) out[0] = (bf16_t)silu_mul(v[0], v[1]);
            if (col + 3 < N) out[1] = (bf16_t)silu_mul(v[2], v[3]);
        }
    } else if (col + 3 < N && N % 4 == 0) {
        if (MODE == OUT_BF16) {
            bf16x4 o = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
            *(bf16x4*)((bf16_t*)Y + row * N + col) = o;
        } else {
            f32x4* out = (f32x4*)((float*)Y + row * N + col);
            if (MODE == OUT_F32_ACCUM) { const f32x4 old = *out; v[0] += old[0]; v[1] += old[1]; v[2] += old[2]; v[3] += old[3]; }
            *out = v;
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (col + e < N) store_out<MODE>(Y, row * N + col + e, v[e]);
    }
}

// What the tiled product can do around an RMSNorm, as the skinny products do (described with them below):
// TILED_SCALED: X is bf16(x * norm weight) and ss_in [n_ss][M] holds sums of squares of each row of x over
// n_ss groups of columns; every row of the result is scaled by 1 / sqrt(sum / K + eps).  TILED_EMIT (adding
// into the float32 residual stream Y): the new Y is also written as bf16(Y * emit_nw[col]) to emit_xw, and
// each workgroup leaves the sums of squares of its rows over its columns in emit_ss [block column][M] (the
// waves that share rows add theirs in the order of their columns).
struct TiledExtra {
    const float* ss_in = nullptr; int n_ss = 0; float eps = 0.f;
    int ss_rows = 0;                      // rows of a group of sums in ss_in (0: M; 64 where a product of at most 64 rows left them)
    const float* emit_nw = nullptr; bf16_t* emit_xw = nullptr; float* emit_ss = nullptr;
};
enum : int { TILED_PLAIN = 0, TILED_SCALED = 1, TILED_EMIT = 2 };

template <int TM, int TN, int WAVES_M, int WAVES_N, int AHEAD, int MODE>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_bf16_tiled_kernel(
        const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, void* __restrict__ Y, int M, int N, int K,
        int steps_per_slice, float* __restrict__ ws) {
    constexpr int NT = 64 * WAVES_M * WAVES_N;
    constexpr int BM = 16 * TM * WAVES_M, BN = 16 * TN * WAVES_N;
    constexpr int PA = BM * CHUNKS / NT, PB = BN * CHUNKS / NT;     // 16-byte pieces of X and of W a thread moves a step
    constexpr int ROWS_PER_PIECE = NT / CHUNKS;
    static_assert(BM * CHUNKS % NT == 0 && BN * CHUNKS % NT == 0, "whole pieces");
    static_assert(TN <= TM, "the fragments of W are fetched over TM inner steps");
    extern __shared__ __attribute__((aligned(16))) bf16_t tiles[];       // [2][BM * TBK] of X then [2][BN * TBK] of W
    bf16_t* As = tiles;
    bf16_t* Bs = tiles + 2 * BM * TBK;
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int wm = (wave / WAVES_N) * 16 * TM, wn = (wave % WAVES_N) * 16 * TN;
    const int r16 = lane % 16, g = lane / 16;
    const long long m0 = (long long)blockIdx.y * BM, n0 = (long long)blockIdx.x * BN;

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Rows beyond the matrix read its last row instead (their results are never stored), so the
    // loads of a full step need no guard.  Offsets are relative to the block's first row.
    // Of W a step holds two blocks (k 0..31, 32..63) of each of the BN / 16 row tiles; thread tid moves
    // piece tid % 64 of block (tid / 64) % 2 of row tile tid / 128, and the same NT / 128 tiles further.
    const int kb = (K + 31) / 32;
    const bf16_t* Xb = X + m0 * K;
    const bf16_t* Wb = W + (n0 / 16) * (long long)kb * 512;
    const int row0 = tid / CHUNKS, c0 = tid % CHUNKS;
    const int last_a = (int)min((long long)BM - 1, (long long)M - 1 - m0);
    const int last_tile = (int)min((long long)BN / 16 - 1, (N - 1 - n0) / 16);
    const int wpiece = tid % 64, wh = (tid / 64) % 2, wtile = tid / 128;
    static_assert(NT % 128 == 0 && ROWS_PER_PIECE == (NT / 128) * 16, "pieces of X and of W advance by the same rows");
    unsigned offa[PA], offb[PB];
#pragma unroll
    for (int i = 0; i < PA; ++i) offa[i] = (unsigned)min(row0 + i * ROWS_PER_PIECE, last_a) * (unsigned)K + c0 * 8;
#pragma unroll
    for (int i = 0; i < PB; ++i)
        offb[i] = ((unsigned)min(wtile + i * (NT / 128), last_tile) * (unsigned)kb + wh) * 512u + wpiece * 8;
    const int lds_st = swz(row0, c0);                    // piece i goes ROWS_PER_PIECE * TBK * i further
    const int lds_st_b = swz(wtile * 16 + wpiece % 16, wh * 4 + wpiece / 16);
    // Memory answers later than a step lasts, so the operands of AHEAD steps are on their way at
    // any time, each in a register set of its own; a set is free again once it went into LDS.
    bf16x8 ra[AHEAD][PA], rb[AHEAD][PB];
    // gridDim.z > 1: the block walks only its slice of K and leaves a float32 partial block in the work
    // space, ws[slice][row][col]; splitk_finish_kernel adds the slices and does the epilogue.
    const int nk = (K + TBK - 1) / TBK;
    const int kt_begin = blockIdx.z * steps_per_slice, kt_end = min(nk, kt_begin + steps_per_slice);

    auto load_global = [&](auto set_tag, int kt) {
        constexpr int set = decltype(set_tag)::value;
        const int k0 = min(kt, nk - 1) * TBK;            // steps past the end read the last one again; nobody uses them
        const unsigned w0 = (unsigned)(k0 / 32) * 512u;  // W: two blocks a step
        if (k0 + TBK <= K) {
#pragma unroll
            for (int i = 0; i < PA; ++i) ra[set][i] = *(const bf16x8*)(Xb + k0 + offa[i]);
#pragma unroll
            for (int i = 0; i < PB; ++i) rb[set][i] = *(const bf16x8*)(Wb + w0 + offb[i]);
        } else {                                         // the last, partial step: zeros beyond K
            const bool in = k0 + c0 * 8 < K, in_w = k0 / 32 + wh < kb;
            const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < PA; ++i) ra[set][i] = in ? *(const bf16x8*)(Xb + k0 + offa[i]) : z;
#pragma unroll
            for (int i = 0; i < PB; ++i) rb[set][i] = in_w ? *(const bf16x8*)(Wb + w0 + offb[i]) : z;
        }
    };
    auto store_piece = [&](auto set_tag, int buf, int p) {             // p counts the pieces of X, then those of W
        constexpr int set = decltype(set_tag)::value;
        if (p < PA) *(bf16x8*)(&As[buf * BM * TBK + lds_st + p * ROWS_PER_PIECE * TBK]) = ra[set][p < PA ? p : 0];
        else *(bf16x8*)(&Bs[buf * BN * TBK + lds_st_b + (p - PA) * ROWS_PER_PIECE * TBK]) = rb[set][p < PA ? 0 : p - PA];
    };
    // fragment offsets inside a buffer: row r16 of MFMA tile 0 of this wave, k-chunk g (+4 for the second half)
    const int fa0 = swz(wm + r16, g), fa1 = swz(wm + r16, 4 + g);
    const int fb0 = swz(wn + r16, g), fb1 = swz(wn + r16, 4 + g);

    // One step out of buffer `buf`: two halves (k 0..31, 32..63) of TM inner steps.  An inner step
    // multiplies one fragment of X with the TN fragments of W; meanwhile the next fragment of X
    // and, in the first half, the fragments of W for the second half are on their way from LDS,
    // and in the second half the pieces of register set `fill` go into the other buffer.
    auto multiply = [&](int buf, auto fill) {
        const bf16_t* Ab = As + buf * BM * TBK;
        const bf16_t* Bb = Bs + buf * BN * TBK;
        bf16x8 b[TN], bn[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[j] = *(const bf16x8*)(Bb + fb0 + j * 16 * TBK);
        bf16x8 a = *(const bf16x8*)(Ab + fa0);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const bf16x8 an = *(const bf16x8*)(Ab + (i + 1 < TM ? fa0 + (i + 1) * 16 * TBK : fa1));
            if (i < TN) bn[i] = *(const bf16x8*)(Bb + fb1 + i * 16 * TBK);
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = mfma16(b[j], a, acc[i][j]);
            a = an;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            bf16x8 an = a;
            if (i + 1 < TM) an = *(const bf16x8*)(Ab + fa1 + (i + 1) * 16 * TBK);
#pragma unroll
            for (int p = 0; p < PA + PB; ++p)
                if (p * TM / (PA + PB) == i) store_piece(fill, buf ^ 1, p);
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = mfma16(bn[j], a, acc[i][j]);
            a = an;
        }
    };

    // set s holds step s, later step s + AHEAD, ...; step kt + 1 is filled in while step kt is multiplied
    static_for<AHEAD>([&](auto s) { load_global(s, kt_begin + decltype(s)::value); });
#pragma unroll
    for (int p = 0; p < PA + PB; ++p) store_piece(std::integral_constant<int, 0>(), 0, p);
    __syncthreads();
    for (int kt0 = kt_begin; kt0 < kt_end; kt0 += AHEAD) {
        static_for<AHEAD>([&](auto u) {
            constexpr int set = decltype(u)::value;
            const int kt = kt0 + set;
            if (kt < kt_end) {
                load_global(u, kt + AHEAD);
                multiply((kt - kt_begin) & 1, std::integral_constant<int, (set + 1) % AHEAD>());
                __syncthreads();
            }
        });
    }

    if (gridDim.z > 1) {
        float* mine = ws + (long long)blockIdx.z * M * N;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                store_quad<OUT_F32>(mine, m0 + wm + i * 16 + r16, n0 + wn + j * 16 + g * 4, M, N, acc[i][j]);
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
            store_quad<MODE>(Y, m0 + wm + i * 16 + r16, n0 + wn + j * 16 + g * 4, M, N, acc[i][j]);
}

// The same product with the operands going from memory straight into LDS (global_load_lds_dwordx4),
// without a stop in registers; used where K is a multiple of 64.  A wave's load instruction fills
// 1 KB of LDS, lane l the 16 bytes at 16 l.  X keeps the swizzled row-major layout above: an
// instruction covers eight rows of 128 bytes, and the lane that fills chunk position p of row r
// fetches chunk p ^ (r % 8) of that row.  W lies in LDS as in memory, one block of 1 KB per (row
// tile, k 32): the fragment of lane l is at 16 l.  STAGES buffers of a step of 64 k each: the
// operands of STAGES - 1 steps are on their way while one is multiplied.
// Measured against the kernel above (M = 2048; N x K): 3072 x 2048 42.8 -> 32.9 us, 2048 x 2048
// 35.1 -> 27.4, 2048 x 8192 102.7 -> 81.3, 16384 x 2048 157.6 -> 148.6, 6144 x 2048 69.0 -> 61.2.
// With all CUs busy and random operands the clock, not the instruction stream, sets the pace: the
// same loop over constant data runs a quarter faster.
template <int VM>
__device__ __forceinline__ void wait_loads_and_lds() {               // s_waitcnt vmcnt(VM) lgkmcnt(0)
    static_assert(VM >= 0 && VM < 64, "vmcnt has six bits");
    __builtin_amdgcn_s_waitcnt((VM & 15) | ((VM >> 4) << 14) | 0x0070);
}

template <int TM, int TN, int WAVES_M, int WAVES_N, int STAGES, int MODE, int AROUND>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_bf16_dma_kernel(
        const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, void* __restrict__ Y, int M, int N, int K,
        int steps_per_slice, float* __restrict__ ws, TiledExtra ex) {
    static_assert(AROUND != TILED_EMIT || MODE == OUT_F32_ACCUM, "the emitting epilogue adds into the residual stream");
    constexpr int NW = WAVES_M * WAVES_N;
    constexpr int BM = 16 * TM * WAVES_M, BN = 16 * TN * WAVES_N;
    constexpr int IA = BM / 8 / NW, IB = BN / 8 / NW;                  // load instructions of X and of W a wave issues a step
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "whole instructions");
    extern __shared__ __attribute__((aligned(16))) bf16_t tiles[];       // [STAGES][BM * TBK] of X then [STAGES][BN * TBK] of W
    bf16_t* As = tiles;
    bf16_t* Bs = tiles + STAGES * BM * TBK;
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int wm = (wave / WAVES_N) * 16 * TM, wn = (wave % WAVES_N) * 16 * TN;
    const int r16 = lane % 16, g = lane / 16;
    const long long m0 = (long long)blockIdx.y * BM, n0 = (long long)blockIdx.x * BN;

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int kb = K / 32;
    const bf16_t* Xb = X + m0 * K;
    const bf16_t* Wb = W + (n0 / 16) * (long long)kb * 512;
    const int last_a = (int)min((long long)BM - 1, (long long)M - 1 - m0);
    const int last_tile = (int)min((long long)BN / 16 - 1, (N - 1 - n0) / 16);
    // instruction q of X (q = wave + NW i) fills rows 8 q .. 8 q + 7; instruction q of W fills block q % 2 of row tile q / 2
    unsigned offa[IA], offb[IB];
#pragma unroll
    for (int i = 0; i < IA; ++i)
        offa[i] = (unsigned)min((wave + NW * i) * 8 + lane / 8, last_a) * (unsigned)K + (((lane % 8) ^ (lane / 8)) * 8);
#pragma unroll
    for (int i = 0; i < IB; ++i) {
        const int q = wave + NW * i;
        offb[i] = ((unsigned)min(q / 2, last_tile) * (unsigned)kb + q % 2) * 512u + lane * 8;
    }
    const int nk = K / TBK;
    const int kt_begin = blockIdx.z * steps_per_slice, kt_end = min(nk, kt_begin + steps_per_slice);

    auto issue = [&](int buf, int kt) {
        const bf16_t* xs = Xb + kt * TBK;
        const bf16_t* wsrc = Wb + (unsigned)(kt * 2) * 512u;
#pragma unroll
        for (int i = 0; i < IA; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xs + offa[i]),
                                             (__attribute__((address_space(3))) void*)(As + buf * BM * TBK + (wave + NW * i) * 512), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < IB; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(wsrc + offb[i]),
                                             (__attribute__((address_space(3))) void*)(Bs + buf * BN * TBK + (wave + NW * i) * 512), 16, 0, 0);
    };
    const int fa0 = swz(wm + r16, g), fa1 = swz(wm + r16, 4 + g);
    const int fb = (wn / 16) * 1024 + lane * 8;                        // block h of MFMA tile j: + (2 j + h) * 512

    // The fragments of half a step (k 0..31 or 32..63: TM of X, TN of W) are read at once into one of
    // two register sets, half a step before the MFMAs that use them: while one set is multiplied the
    // other is on its way from LDS, also across the barrier between two steps.
    bf16x8 fx[2][TM], fw[2][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) fx[1][i] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < TN; ++j) fw[1][j] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    auto read_half = [&](auto set_tag, int buf, auto half_tag) {
        constexpr int set = decltype(set_tag)::value, h = decltype(half_tag)::value;
        const bf16_t* Ab = As + buf * BM * TBK + (h ? fa1 : fa0);
        const bf16_t* Bb = Bs + buf * BN * TBK + fb + h * 512;
#pragma unroll
        for (int j = 0; j < TN; ++j) fw[set][j] = *(const bf16x8*)(Bb + 2 * j * 512);
#pragma unroll
        for (int i = 0; i < TM; ++i) fx[set][i] = *(const bf16x8*)(Ab + i * 16 * TBK);
    };
    auto mult = [&](auto set_tag) {
        constexpr int set = decltype(set_tag)::value;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = mfma16(fw[set][j], fx[set][i], acc[i][j]);
    };
    // asks the instruction scheduler to spread the LDS reads of a half step evenly among its MFMAs
    auto spread = [&]() {
        constexpr int R = TM + TN, Q = TM * TN;
        static_for<R>([&](auto r) {
            constexpr int n = Q / R + (decltype(r)::value < Q % R ? 1 : 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);         // one LDS read
            __builtin_amdgcn_sched_group_barrier(0x008, n, 0);         // n MFMAs
        });
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;

    // Step kt lives in buffer (kt - kt_begin) % STAGES.  Before step kt is multiplied the loads of
    // steps kt .. kt + STAGES - 2 are under way; a wave waits until all but those of the later steps
    // have landed, the barrier then says the same of everybody's and that nobody reads the buffer
    // of step kt - 1 any more, which the loads of step kt + STAGES - 1 go into.
    static_for<STAGES - 1>([&](auto s) {
        constexpr int st = decltype(s)::value;
        if (kt_begin + st < kt_end) issue(st, kt_begin + st);
    });
    // TILED_SCALED: the sum of squares of each of the block's rows, in SS_PARTS parts: thread (part, row) adds the groups
    // part, part + SS_PARTS, ... in that order, sixteen loads at a time (one after the other would be as many trips to
    // memory: a product of few rows leaves 256 groups for 2,048 columns); behind the first barrier of the loop the parts
    // of a row are added in their order and the row's scale is left for the epilogue.  (Up to sixteen groups, as the
    // tiled products of a prompt leave them: one thread a row, the scale at once.)
    constexpr int SS_PARTS = (64 * NW) / BM >= 4 ? 4 : (64 * NW) / BM >= 2 ? 2 : 1;
    __shared__ float row_ss[AROUND == TILED_SCALED ? SS_PARTS : 1][AROUND == TILED_SCALED ? BM : 1];
    __shared__ float row_scale[AROUND == TILED_SCALED ? BM : 1];
    if constexpr (AROUND == TILED_SCALED) {
        // while the first operands are on their way (a product cut along K leaves the scales to the kernel that adds the slices)
        const int ss_rows = ex.ss_rows ? ex.ss_rows : M;
        if (ex.n_ss <= 16) {
            // one trip to memory a row: the scale at once
            if (tid < BM && gridDim.z == 1) {
                const long long row = m0 + tid;
                float v[16], t = 0.f;
#pragma unroll
                for (int u = 0; u < 16; ++u) v[u] = (row < M && u < ex.n_ss) ? ex.ss_in[(long long)u * ss_rows + row] : 0.f;
#pragma unroll
                for (int u = 0; u < 16; ++u) t += v[u];
                row_scale[tid] = 1.0f / sqrtf(t / (float)K + ex.eps);
            }
        } else if (tid < SS_PARTS * BM && gridDim.z == 1) {
            const int r = tid % BM, part = tid / BM;
            const long long row = m0 + r;
            float t = 0.f;
            if (row < M) {
                for (int j0 = part; j0 < ex.n_ss; j0 += 16 * SS_PARTS) {
                    float v[16];
#pragma unroll
                    for (int u = 0; u < 16; ++u) {
                        const int j = j0 + u * SS_PARTS;
                        v[u] = j < ex.n_ss ? ex.ss_in[(long long)j * ss_rows + row] : 0.f;
                    }
#pragma unroll
                    for (int u = 0; u < 16; ++u) t += v[u];
                }
            }
            row_ss[part][r] = t;
        }
        // read in the epilogue, behind the barriers of the loop (every wave waits for its LDS writes before each)
    }
    for (int kt0 = kt_begin; kt0 < kt_end; kt0 += STAGES) {
        static_for<STAGES>([&](auto u) {
            constexpr int buf = decltype(u)::value;
            const int kt = kt0 + buf;
            if (kt < kt_end) {
                const int later = min(STAGES - 2, kt_end - 1 - kt);      // steps after kt whose loads are under way
                bool waited = false;
                static_for<STAGES - 1>([&](auto l) {
                    constexpr int n = decltype(l)::value;
                    if (!waited && later == n) { wait_loads_and_lds<n * (IA + IB)>(); waited = true; }
                });
                __builtin_amdgcn_s_barrier();
                if (kt + STAGES - 1 < kt_end) issue((buf + STAGES - 1) % STAGES, kt + STAGES - 1);
                if constexpr (AROUND == TILED_SCALED) {
                    if (kt == kt_begin && ex.n_ss > 16 && tid < BM && gridDim.z == 1) {
                        float t = row_ss[0][tid];
#pragma unroll
                        for (int q = 1; q < SS_PARTS; ++q) t += row_ss[q][tid];
                        row_scale[tid] = 1.0f / sqrtf(t / (float)K + ex.eps);
                    }
                }
                read_half(S0(), buf, S0());
                mult(S1());                                            // the second half of the step before (zeros at first)
                spread();
                read_half(S1(), buf, S1());
                mult(S0());
                spread();
            }
        });
    }
    if (kt_begin < kt_end) mult(S1());

    if (gridDim.z > 1) {
        float* mine = ws + (long long)blockIdx.z * M * N;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                store_quad<OUT_F32>(mine, m0 + wm + i * 16 + r16, n0 + wn + j * 16 + g * 4, M, N, acc[i][j]);
        return;
    }
    if constexpr (AROUND == TILED_SCALED) {
        if (kt_end - kt_begin < 2) __syncthreads();        // a single step: no barrier has followed the scales yet
    }
    if constexpr (AROUND == TILED_EMIT) {
        // whole blocks of columns only (the host sees to it): Y += acc, the next norm's operand, the row's sum of squares
        float wave_sq[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const long long row = m0 + wm + i * 16 + r16;
            float sq = 0.f;
            if (row < M) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const long long col = n0 + wn + j * 16 + g * 4;
                    f32x4* yp = (f32x4*)((float*)Y + row * N + col);
                    f32x4 y = *yp;
#pragma unroll
                    for (int e = 0; e < 4; ++e) y[e] += acc[i][j][e];
                    *yp = y;
                    const f32x4 nw = *(const f32x4*)(ex.emit_nw + col);
                    bf16x4 o = {(bf16_t)(y[0] * nw[0]), (bf16_t)(y[1] * nw[1]), (bf16_t)(y[2] * nw[2]), (bf16_t)(y[3] * nw[3])};
                    *(bf16x4*)(ex.emit_xw + row * N + col) = o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) sq = fmaf(y[e], y[e], sq);
                }
            }
            sq += __shfl_xor(sq, 16, WAVE);
            sq += __shfl_xor(sq, 32, WAVE);
            wave_sq[i] = sq;
        }
        // the waves that share rows add their sums in the order of their columns, through the LDS the operands
        // have left: one sum per row and block of columns, so that whoever reads them asks only once
        float* red = (float*)tiles;                            // [WAVES_N][BM]
        __syncthreads();                                       // nobody reads operands any more
        if (g == 0) {
#pragma unroll
            for (int i = 0; i < TM; ++i) red[(wave % WAVES_N) * BM + wm + i * 16 + r16] = wave_sq[i];
        }
        __syncthreads();
        for (int r = tid; r < BM; r += 64 * NW) {
            float t = red[r];
#pragma unroll
            for (int w = 1; w < WAVES_N; ++w) t += red[w * BM + r];
            if (m0 + r < M) ex.emit_ss[(long long)blockIdx.x * M + m0 + r] = t;
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        float sc = 1.f;
        if constexpr (AROUND == TILED_SCALED) sc = row_scale[wm + i * 16 + r16];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            f32x4 v = acc[i][j];
            if constexpr (AROUND == TILED_SCALED) { v[0] *= sc; v[1] *= sc; v[2] *= sc; v[3] *= sc; }
            store_quad<MODE>(Y, m0 + wm + i * 16 + r16, n0 + wn + j * 16 + g * 4, M, N, v);
        }
    }
}

// ----------------------------------------------------------------- skinny kernels
constexpr int SK_CHUNK = 128;

// M <= 16.  grid: tiles of 16 columns.  The NW waves of a workgroup split K: wave w takes the
// chunks w, w + NW, w + 2 NW, ... of 128; in a chunk the wave reads four blocks of its row tile of W
// (1 KB each) and 256 bytes of each of the 16 X rows (four loads of 16 rows x 64 contiguous bytes)
// and issues four MFMAs.
// Loads run one chunk ahead.  The wave partials are added in wave order through LDS.  NW is
// chosen from N and K only.
//
// The product may be taken of the RMSNorm of the float32 residual stream x,
//   y[m, n] = (1 / sqrt(mean_k x[m,k]^2 + eps)) * sum_k bf16(x[m,k] * w[k]) W[n,k]:
// the norm weight is applied to the operand, the row's scale to the result.
//  * NORM_INSIDE: X is x itself; the operand is formed and the sum of squares taken from the
//    values the workgroup loads anyway (lane partials in a fixed butterfly, waves in wave
//    order).  `rows` (optional) gathers rows of x.
//  * NORM_SCALED: X is bf16(x * w), made by the product that last added into x (below), and
//    ss_in [n_ss][16] holds that product's per-tile sums of squares of each row; this kernel
//    adds them in tile order and scales its result.  Costs no more than the plain product.
// EMIT (with OUT_F32_ACCUM): after y += ..., the new y is also written as bf16(y * emit_nw[col])
// to emit_xw [M, N], and the tile's sums of squares of each row to emit_ss [tile][16], for the
// NORM_SCALED product that follows.
enum : int { NORM_NONE = 0, NORM_INSIDE = 1, NORM_SCALED = 2 };

// What the OUT_CONV epilogue needs beside the product: the taps [d][taps] (float32 or bfloat16), the
// float32 state [slots][taps - 1][d] and each row's slot.
constexpr int CONV_MAX_TAPS = 16;
struct ConvTail {
    const void* taps_w = nullptr; int taps_dt = DT_F32; int taps = 0;
    float* state = nullptr; const int* state_slot = nullptr;
    __device__ __forceinline__ float tap(int ch, int k) const {
        const long long i = (long long)ch * taps + k;
        return taps_dt == DT_F32 ? ((const float*)taps_w)[i] : (float)((const bf16_t*)taps_w)[i];
    }
};

// MT: row tiles of 16 (1: up to 16 rows, 2: up to 32).  With two, a wave multiplies every block of W
// with two tiles of X rows; the sums of squares that go from product to product then have 64 rows a tile
// in memory (SS_ROWS), as for every product of 17 to 64 rows.
constexpr int SS_ROWS_WIDE = 64;

template <int NW, int MODE, int NORM, bool EMIT, int COLS, int MT>
__global__ __launch_bounds__(NW * WAVE) void gemm_bf16_skinny16_kernel(const void* __restrict__ Xv, const bf16_t* __restrict__ W,
                                                                       void* __restrict__ Y, int M, int N, int K,
                                                                       const float* __restrict__ norm_w, float eps,
                                                                       const int* __restrict__ rows,
                                                                       const float* __restrict__ ss_in, int n_ss,
                                                                       const float* __restrict__ emit_nw,
                                                                       bf16_t* __restrict__ emit_xw, float* __restrict__ emit_ss,
                                                                       ConvTail cv) {
    constexpr bool CONV = MODE == OUT_CONV;
    static_assert(!CONV || COLS == 8, "the convolution's epilogue takes eight channels a workgroup");
    static_assert(MT == 1 || NORM != NORM_INSIDE, "the norm inside is for at most 16 rows");
    constexpr int TN = CONV ? 3 : (COLS > 16 ? COLS / 16 : 1);           // MFMA tiles side by side: they share the rows of X
    static_assert(!EMIT || TN == 1, "the emitting epilogue works on one tile");
    constexpr int ROWS = 16 * MT;
    constexpr int SSR = MT == 1 ? 16 : SS_ROWS_WIDE;                     // rows of a tile of sums of squares in memory
    constexpr int NT_ = NW * WAVE;
    constexpr int PAIRS = (16 * ROWS + NT_ - 1) / NT_;                   // (row, part) sums a thread adds for NORM_SCALED
    __shared__ float red[MT][TN][NW][WAVE][4];
    __shared__ float ssq[16][ROWS];                                      // [wave or part][row]
    extern __shared__ __attribute__((aligned(16))) float nw_lds[];       // NORM_INSIDE: the norm weight, K floats
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int r16 = lane % 16, g = lane / 16;
    // OUT_CONV: workgroup b takes the channels 8 b .. 8 b + 7: half (b % 2) of the three row tiles of group b / 2
    const long long n0 = CONV ? (long long)(blockIdx.x / 2) * 48 + (blockIdx.x % 2) * 8 : (long long)blockIdx.x * COLS;
    const int nchunks = (K + SK_CHUNK - 1) / SK_CHUNK;
    const bf16_t* X = (const bf16_t*)Xv;
    const long long w_rows = min((long long)N, n0 + COLS);               // this tile's rows of W end here
    // tile-major W: this lane's piece of a block; a workgroup of 8 columns owns half a row tile
    const int kb = (K + 31) / 32, n_tiles16 = (N + 15) / 16;
    const long long tile0 = n0 / 16;
    const int wpiece = COLS == 8 ? g * 16 + (int)(n0 % 16) + r16 : lane;
    const bool wlane = COLS == 8 ? r16 < 8 : true;
    const float* xrow = nullptr;
    if (NORM == NORM_INSIDE && r16 < M) xrow = (const float*)Xv + (long long)(rows ? rows[r16] : r16) * K;

    // What the epilogue adds to is read now, not after the last product: a load at the end would
    // cost one more trip to memory.  (Thread t of every 256 -> element (row (t / 64) * 4 + t % 4,
    // column (t / 4) % 16) of a 16 x 16 tile; the groups of 256 threads take the row tiles in turn.)
    constexpr int EPI_GROUPS = NT_ / 256;                                // groups of 256 threads a workgroup
    constexpr int EPI_TILES = (MT + EPI_GROUPS - 1) / EPI_GROUPS;        // row tiles a group finishes
    float y_old[EPI_TILES][TN], emit_w = 0.f;
#pragma unroll
    for (int i = 0; i < EPI_TILES; ++i) {
        const int mt = tid / 256 + i * EPI_GROUPS;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            y_old[i][tn] = 0.f;
            if (MODE == OUT_F32_ACCUM && mt < MT) {
                const int t = tid % 256;
                const long long row = mt * 16 + (t / 64) * 4 + t % 4, col = n0 + tn * 16 + (t / 4) % 16;
                if (row < M && col < w_rows) {
                    y_old[i][tn] = ((const float*)Y)[row * N + col];
                    if (EMIT) emit_w = emit_nw[col];
                }
            }
        }
    }

    // OUT_CONV: likewise the rows of the state and the taps that the convolution reads (slot -> state: two trips to
    // memory one after the other, which now run beside the product instead of behind it); the first CONV_AHEAD rows of the
    // state, which is all of them up to a kernel length of CONV_AHEAD + 1, and the last tap.
    constexpr int CONV_AHEAD = 4;
    float st_ahead[CONV ? EPI_TILES : 1][CONV_AHEAD], tap_ahead[CONV ? EPI_TILES : 1][CONV_AHEAD + 1];
    if constexpr (CONV) {
#pragma unroll
        for (int i = 0; i < EPI_TILES; ++i) {
            const int mt = tid / 256 + i * EPI_GROUPS, t = tid % 256, l = t / 4;
            const int row = mt * 16 + (l / 16) * 4 + t % 4, ch = (int)blockIdx.x * 8 + (l % 16), d = N / 3, Kc = cv.taps;
#pragma unroll
            for (int k = 0; k <= CONV_AHEAD; ++k) tap_ahead[i][k] = 0.f;
#pragma unroll
            for (int k = 0; k < CONV_AHEAD; ++k) st_ahead[i][k] = 0.f;
            if (mt < MT && (l % 16) < 8 && row < M && ch < d) {
                const float* st = cv.state + (long long)cv.state_slot[row] * (Kc - 1) * d;
#pragma unroll
                for (int k = 0; k < CONV_AHEAD; ++k)
                    if (k < Kc - 1) { st_ahead[i][k] = st[(long long)k * d + ch]; tap_ahead[i][k] = cv.tap(ch, k); }
                tap_ahead[i][CONV_AHEAD] = cv.tap(ch, Kc - 1);
            }
        }
    }

    f32x4 acc[MT][TN];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) acc[mt][tn] = f32x4{0.f, 0.f, 0.f, 0.f};
    float ss = 0.f;
    struct Operands { bf16x8 a[MT][4]; bf16x8 b[TN][4]; f32x4 x[NORM == NORM_INSIDE ? 4 : 1][2]; };
    Operands o0, o1;
    auto load = [&](int c, Operands& o) {
        // instruction j of the wave reads block 4 c + j of its row tile (1 KB) and bytes 64 j .. 64 j + 63 of
        // the chunk of each of the rows of X
        const int k0 = c * SK_CHUNK + g * 8;
        const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                o.b[tn][j] = (wlane && tile0 + tn < n_tiles16 && c * 4 + j < kb) ? load_w(W, tile0 + tn, kb, c * 4 + j, wpiece) : z;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + j * 32;
            if (NORM == NORM_INSIDE) {
                const bool ok = xrow != nullptr && k < K;
                o.x[j][0] = ok ? *(const f32x4*)(xrow + k) : f32x4{0.f, 0.f, 0.f, 0.f};
                o.x[j][1] = ok ? *(const f32x4*)(xrow + k + 4) : f32x4{0.f, 0.f, 0.f, 0.f};
            } else {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) o.a[mt][j] = load8(X, mt * 16 + r16, M, k, K);
            }
        }
    };
    auto multiply = [&](int c, Operands& o) {
        if (NORM == NORM_INSIDE) {
            const int k0 = c * SK_CHUNK + g * 8;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = min(k0 + j * 32, K - 8);               // past the end x is zero anyway
                const f32x4 w0 = *(const f32x4*)(&nw_lds[k]), w1 = *(const f32x4*)(&nw_lds[k + 4]);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float x0 = o.x[j][0][e], x1 = o.x[j][1][e];
                    ss = fmaf(x0, x0, ss);
                    ss = fmaf(x1, x1, ss);
                    o.a[0][j][e] = (bf16_t)(x0 * w0[e]);
                    o.a[0][j][4 + e] = (bf16_t)(x1 * w1[e]);
                }
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[mt][tn] = mfma16(o.a[mt][j], o.b[tn][j], acc[mt][tn]);
    };
    // Workgroups start at different chunks (a rotation by the tile index), so that at any moment
    // the chip reads from all columns of W and not from one.  The order of a tile's additions
    // still depends on N and K only.
    const int rot = (int)((blockIdx.x * 5u) % (unsigned)nchunks);
    auto chunk_of = [&](int i) { int c = i + rot; return c >= nchunks ? c - nchunks : c; };
    int i = wave;
    if (i < nchunks) load(chunk_of(i), o0);
    if (NORM == NORM_INSIDE) {
        // the norm weight goes to LDS while the first operands are on their way from HBM
        for (int k = tid * 4; k < K; k += NW * WAVE * 4) *(f32x4*)(&nw_lds[k]) = *(const f32x4*)(norm_w + k);
        __syncthreads();
    }
    // NORM_SCALED: 16 parts x ROWS rows; part p adds the tiles p, p + 16, ... of its row.  The first
    // sixteen of them are only asked for here and added after the products, when they have long
    // arrived; a wider matrix adds the rest right away.
    float ss_part[PAIRS][16], ss_rest[PAIRS];
    if (NORM == NORM_SCALED) {
#pragma unroll
        for (int q = 0; q < PAIRS; ++q) {
            const int pr = tid + q * NT_;
            const int row = pr % ROWS, part = pr / ROWS;
            ss_rest[q] = 0.f;
            if (pr < 16 * ROWS) {
#pragma unroll
                for (int u = 0; u < 16; ++u) ss_part[q][u] = (part + 16 * u < n_ss) ? ss_in[(long long)(part + 16 * u) * SSR + row] : 0.f;
                for (int j = part + 256; j < n_ss; j += 16) ss_rest[q] += ss_in[(long long)j * SSR + row];
            }
        }
    }
    for (; i < nchunks; i += 2 * NW) {
        const bool more = i + NW < nchunks;
        if (more) load(chunk_of(i + NW), o1);
        multiply(chunk_of(i), o0);
        if (more) {
            if (i + 2 * NW < nchunks) load(chunk_of(i + 2 * NW), o0);
            multiply(chunk_of(i + NW), o1);
        }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[mt][tn][wave][lane][e] = acc[mt][tn][e];
    if (NORM == NORM_SCALED) {
#pragma unroll
        for (int q = 0; q < PAIRS; ++q) {
            const int pr = tid + q * NT_;
            if (pr < 16 * ROWS) {
                float t = ss_rest[q];
#pragma unroll
                for (int u = 0; u < 16; ++u) t += ss_part[q][u];
                ssq[pr / ROWS][pr % ROWS] = t;
            }
        }
    }
    if (NORM == NORM_INSIDE) {
        ss += __shfl_xor(ss, 16, WAVE);
        ss += __shfl_xor(ss, 32, WAVE);
        if (g == 0) ssq[wave][r16] = ss;
    }
    __syncthreads();
#pragma unroll
    for (int ei = 0; ei < EPI_TILES; ++ei) {
        const int mt = tid / 256 + ei * EPI_GROUPS;
        if (mt >= MT) break;
        // thread -> (lane l, element e) of each 16x16 tile; the wave partials in wave order
        const int t256 = tid % 256;
        const int e = t256 % 4, l = t256 / 4;
        const int trow = mt * 16 + (l / 16) * 4 + e;                     // the thread's row of the product
        float scale = 1.f;
        if (NORM != NORM_NONE) {
            constexpr int PARTS = NORM == NORM_INSIDE ? NW : 16;
            float total = ssq[0][trow];
#pragma unroll
            for (int w = 1; w < PARTS; ++w) total += ssq[w][trow];
            scale = 1.0f / sqrtf(total / (float)K + eps);
        }
        if constexpr (CONV) {
            // (row, channel): the three tiles hold B, C and X of the channel; the convolution as the kernel
            // for single tokens does it, on the values rounded to bfloat16 as a projected row would hold them
            float bcx[3];
#pragma unroll
            for (int tn = 0; tn < 3; ++tn) {
                float v = red[mt][tn][0][l][e];
#pragma unroll
                for (int w = 1; w < NW; ++w) v += red[mt][tn][w][l][e];
                if (NORM != NORM_NONE) v *= scale;
                bcx[tn] = (float)(bf16_t)v;
            }
            const int row = trow, d = N / 3, Kc = cv.taps;
            const int ch = (int)(blockIdx.x) * 8 + (l % 16);
            if ((l % 16) < 8 && row < M && ch < d) {
                float* st = cv.state + (long long)cv.state_slot[row] * (Kc - 1) * d;
                float sv[CONV_MAX_TAPS], wv[CONV_MAX_TAPS];
#pragma unroll
                for (int k = 0; k < CONV_MAX_TAPS; ++k) {
                    if (k < CONV_AHEAD) { sv[k] = st_ahead[ei][k]; wv[k] = tap_ahead[ei][k]; continue; }   // (zero beyond Kc - 1)
                    sv[k] = k < Kc - 1 ? st[(long long)k * d + ch] : 0.f;
                    wv[k] = k < Kc - 1 ? cv.tap(ch, k) : 0.f;
                }
                const float w_last = tap_ahead[ei][CONV_AHEAD];
                const float u = bcx[0] * bcx[2];
                float y = 0.f;
#pragma unroll
                for (int k = 0; k < CONV_MAX_TAPS; ++k)
                    if (k < Kc - 1) y = (k == 0) ? sv[k] * wv[k] : fmaf(sv[k], wv[k], y);
                y = fmaf(u, w_last, y);
#pragma unroll
                for (int k = 1; k < CONV_MAX_TAPS; ++k)
                    if (k < Kc - 1) st[(long long)(k - 1) * d + ch] = sv[k];
                st[(long long)(Kc - 2) * d + ch] = u;
                ((bf16_t*)Y)[(long long)row * d + ch] = (bf16_t)(bcx[1] * y);
            }
            continue;
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            float v = red[mt][tn][0][l][e];
#pragma unroll
            for (int w = 1; w < NW; ++w) v += red[mt][tn][w][l][e];
            const long long col = n0 + tn * 16 + (l % 16);
            const long long row = col < w_rows ? trow : ROWS;                // columns beyond the tile: no row
            if (NORM != NORM_NONE) v *= scale;
            if (EMIT) {
                // y += v; the new y also as the next norm's operand, and its square into the row's tile sum
                float y = 0.f;
                if (row < M && col < N) {
                    y = y_old[ei][tn] + v;
                    ((float*)Y)[row * N + col] = y;
                    emit_xw[row * N + col] = (bf16_t)(y * emit_w);
                }
                float sq = y * y;                       // t256 = (16 q + c) * 4 + e: the 16 columns c are its bits 2..5
                sq += __shfl_xor(sq, 4, WAVE);
                sq += __shfl_xor(sq, 8, WAVE);
                sq += __shfl_xor(sq, 16, WAVE);
                sq += __shfl_xor(sq, 32, WAVE);
                if ((l % 16) == 0 && row < ROWS) emit_ss[(long long)blockIdx.x * SSR + row] = sq;
            } else if (MODE == OUT_F32_ACCUM) {
                if (row < M && col < N) ((float*)Y)[row * N + col] = y_old[ei][tn] + v;
            } else {
                const float partner = (MODE == OUT_SWIGLU) ? __shfl_xor(v, 4, WAVE) : 0.f;   // thread t ^ 4 holds column col ^ 1
                store_elem<MODE>(Y, row, col, min(M, ROWS), N, v, partner);
            }
        }
    }
}

// 16 < M <= 64.  grid (tiles of 64 columns, K slices).  Wave w owns columns 16w..16w+15 of the
// tile and all MT row tiles.  The X rows of a K chunk (128 wide) go through LDS once for the
// four waves, double buffered; W goes from HBM to registers one chunk ahead.  With more than
// one K slice, or when the epilogue has to leave the next norm's operand, the partial tiles go to
// a work space and splitk_finish_kernel adds them in slice order and does the epilogue.
// NORM_SCALED as above, with the sums of squares per tile of 64 columns: ss_in [n_ss][64].
constexpr int SK_NT = 256;
constexpr int XS_STRIDE = SK_CHUNK + 8;             // bf16 elements; 272 bytes: conflict-free 16-byte reads

template <int MT, int MODE, int NORM>
__global__ __launch_bounds__(SK_NT) void gemm_bf16_skinny64_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                                   void* __restrict__ Y, int M, int N, int K, int chunks_per_slice,
                                                                   float* __restrict__ ws, bool to_ws,
                                                                   const float* __restrict__ ss_in, int n_ss, float eps) {
    static_assert(NORM != NORM_INSIDE, "the norm inside is for at most 16 rows");
    __shared__ __attribute__((aligned(16))) bf16_t xs[2][MT * 16 * XS_STRIDE];
    __shared__ float ss_parts[4][64];
    __shared__ float scale_lds[64];
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int r16 = lane % 16, g = lane / 16;
    const int tile = blockIdx.x, slice = blockIdx.y, n_slices = gridDim.y;
    const long long tile16 = (long long)tile * 4 + wave;                 // this wave's row tile of W
    const int kb = (K + 31) / 32;
    const bool tile_ok = tile16 < (N + 15) / 16;
    const int nchunks = (K + SK_CHUNK - 1) / SK_CHUNK;
    const int c_begin = slice * chunks_per_slice, c_end = min(nchunks, c_begin + chunks_per_slice);

    f32x4 acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // X chunk: MT*16 rows x 16 pieces of 16 bytes = MT*256 pieces, MT a thread
    bf16x8 xr[MT], b0[4], b1[4];
    auto load_x = [&](int c) {
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int id = tid + i * SK_NT;
            xr[i] = load8(X, id / 16, M, c * SK_CHUNK + (id % 16) * 8, K);
        }
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int id = tid + i * SK_NT;
            *(bf16x8*)(&xs[buf][(id / 16) * XS_STRIDE + (id % 16) * 8]) = xr[i];
        }
    };
    auto load_w4 = [&](int c, bf16x8* b) {
        const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = (tile_ok && c * 4 + j < kb) ? load_w(W, tile16, kb, c * 4 + j, lane) : z;
    };
    auto compute = [&](int buf, const bf16x8* b) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bf16x8 a = *(const bf16x8*)(&xs[buf][(i * 16 + r16) * XS_STRIDE + j * 32 + g * 8]);
                acc[i] = mfma16(a, b[j], acc[i]);
            }
    };

    if (c_begin < c_end) {
        load_x(c_begin);
        load_w4(c_begin, b0);
    }
    if (NORM == NORM_SCALED && !to_ws) {
        // thread -> (row tid % 64, part tid / 64): part p adds the tiles p, p + 4, ... of its row
        float t = 0.f;
        for (int j = tid / 64; j < n_ss; j += 4) t += ss_in[(long long)j * 64 + tid % 64];
        ss_parts[tid / 64][tid % 64] = t;
    }
    if (c_begin < c_end) store_x(0);
    __syncthreads();
    if (NORM == NORM_SCALED && !to_ws && tid < 64)    // read in the epilogue, behind the barriers of the loop
        scale_lds[tid] = 1.0f / sqrtf((ss_parts[0][tid] + ss_parts[1][tid] + ss_parts[2][tid] + ss_parts[3][tid]) / (float)K + eps);
    for (int c = c_begin; c < c_end; c += 2) {
        // chunk c from buffer 0 / b0, chunk c+1 from buffer 1 / b1
        const bool more1 = c + 1 < c_end, more2 = c + 2 < c_end;
        if (more1) { load_x(c + 1); load_w4(c + 1, b1); }
        compute(0, b0);
        if (more1) store_x(1);
        __syncthreads();
        if (more1) {
            if (more2) { load_x(c + 2); load_w4(c + 2, b0); }
            compute(1, b1);
            if (more2) store_x(0);
            __syncthreads();
        }
    }

    const long long col = (long long)tile * 64 + wave * 16 + r16;
    if (to_ws) {
        // partial tile of this slice: ws[slice][row][col]
        if (col >= N) return;
        float* mine = ws + (long long)slice * (MT * 16) * N;
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) mine[(long long)(i * 16 + g * 4 + e) * N + col] = acc[i][e];
        return;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const long long row = i * 16 + g * 4 + e;
            float v = acc[i][e];
            if (NORM == NORM_SCALED) v *= scale_lds[row];
            const float partner = (MODE == OUT_SWIGLU) ? __shfl_xor(v, 1, WAVE) : 0.f;
            store_elem<MODE>(Y, row, col, M, N, v, partner);
        }
}

// Finishes a product whose partial tiles lie in the work space: v = sum over slices, in slice
// order, of ws[slice][row][col] (rows_padded rows a slice), scaled per row for NORM_SCALED, then the
// epilogue of MODE; with EMIT, Y += v and from the new Y the operand of the norm that follows, as
// in the kernel for at most 16 rows, with sums of squares per tile of 64 columns: emit_ss [tiles][64].
// grid (tiles of 64 columns, groups of 16 rows), 256 threads: thread -> row tid / 16 of the group and
// four neighbouring columns.
struct FinishExtra {
    const float* ss_in = nullptr; int n_ss = 0; float eps = 0.f; int K = 0;                 // NORM_SCALED
    const float* emit_nw = nullptr; bf16_t* emit_xw = nullptr; float* emit_ss = nullptr;   // EMIT
    int ss_rows = 64;                     // rows of a tile of sums of squares, read or written: 64, or M for the tiled product
};

template <int MODE, int NORM, bool EMIT>
__global__ __launch_bounds__(256) void splitk_finish_kernel(const float* __restrict__ ws, void* __restrict__ Y, int M, int N,
                                                            int rows_padded, int n_slices, FinishExtra ex) {
    static_assert(!EMIT || MODE == OUT_F32_ACCUM, "the emitting epilogue adds into the residual stream");
    const int tid = threadIdx.x, q = tid % 16;
    const long long row = (long long)blockIdx.y * 16 + tid / 16;
    const long long col = (long long)blockIdx.x * 64 + q * 4;
    float scale = 1.f;
    if (NORM == NORM_SCALED) {
        // the sixteen threads of a row add the tiles q, q + 16, ... and then each other, in a fixed butterfly
        float t = 0.f;
        if (row < ex.ss_rows)
            for (int j = q; j < ex.n_ss; j += 16) t += ex.ss_in[(long long)j * ex.ss_rows + row];
        t += __shfl_xor(t, 1, WAVE);
        t += __shfl_xor(t, 2, WAVE);
        t += __shfl_xor(t, 4, WAVE);
        t += __shfl_xor(t, 8, WAVE);
        scale = 1.0f / sqrtf(t / (float)ex.K + ex.eps);
    }
    const bool whole = N % 4 == 0 && col + 3 < N;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (row < M) {
        if (whole) {
            // the slices of a step of eight are asked for together and added in their order
            const long long stride = (long long)rows_padded * N;
            const float* p0 = ws + row * N + col;
            for (int s0 = 0; s0 < n_slices; s0 += 8) {
                f32x4 t[8];
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (s0 + u < n_slices) t[u] = *(const f32x4*)(p0 + (s0 + u) * stride);
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (s0 + u < n_slices) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] += t[u][e];
                    }
            }
        } else {
            for (int s = 0; s < n_slices; ++s) {
                const float* p = ws + ((long long)s * rows_padded + row) * N + col;
#pragma unroll
                for (int e = 0; e < 4; ++e) if (col + e < N) v[e] += p[e];
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] *= scale;
    float sq = 0.f;
    if (row < M) {
        if (MODE == OUT_SWIGLU) {
            bf16_t* out = (bf16_t*)Y + row * (N / 2) + col / 2;
            if (col + 1 < N) out[0] = (bf16_t)silu_mul(v[0], v[1]);
            if (col + 3 < N) out[1] = (bf16_t)silu_mul(v[2], v[3]);
        } else if (EMIT) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col + e < N) {
                    const float y = ((const float*)Y)[row * N + col + e] + v[e];
                    ((float*)Y)[row * N + col + e] = y;
                    ex.emit_xw[row * N + col + e] = (bf16_t)(y * ex.emit_nw[col + e]);
                    sq = fmaf(y, y, sq);
                }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) if (col + e < N) store_out<MODE>(Y, row * N + col + e, v[e]);
        }
    }
    if (EMIT) {
        sq += __shfl_xor(sq, 1, WAVE);
        sq += __shfl_xor(sq, 2, WAVE);
        sq += __shfl_xor(sq, 4, WAVE);
        sq += __shfl_xor(sq, 8, WAVE);
        if (q == 0 && row < ex.ss_rows) ex.emit_ss[(long long)blockIdx.x * ex.ss_rows + row] = sq;   // rows beyond M: zero
    }
}

// The same for the input projection of a gated short convolution over 17 to 64 single tokens (row r is
// request r's token): from the partial tiles of the projection [3 d] wide (B | C | X, as the checkpoint
// has them) the thread of (row, four channels) adds the slices of its twelve columns in slice order,
// scales and rounds them to bfloat16 as a projected row would hold them, and then does what the kernel
// for single tokens does: y = C * (taps . (state, B * X)), the state shifted by one.  The projected
// rows are never written.  grid (tiles of 64 channels, groups of 4 rows), one wave a workgroup: with twelve
// columns a thread there is three times the work of the kernel above in a thread, so more and smaller
// workgroups.  Two trips to memory one after the other remain (the row's slot, then its state beside the
// slices): 7.1 us at 64 rows of 2,048 channels, where the kernel above and the convolution's own took 9.5.
constexpr int FC_ROWS = 4;
template <int NORM>
__global__ __launch_bounds__(FC_ROWS * 16) void splitk_finish_conv_kernel(const float* __restrict__ ws, bf16_t* __restrict__ Y, int M, int d,
                                                                 int rows_padded, int n_slices, FinishExtra ex, ConvTail cv) {
    const int tid = threadIdx.x, q = tid % 16;
    const long long row = (long long)blockIdx.y * FC_ROWS + tid / 16;
    const long long ch0 = (long long)blockIdx.x * 64 + q * 4;
    const int N = 3 * d;
    float scale = 1.f;
    if (NORM == NORM_SCALED) {
        float t = 0.f;
        if (row < ex.ss_rows)
            for (int j = q; j < ex.n_ss; j += 16) t += ex.ss_in[(long long)j * ex.ss_rows + row];
        t += __shfl_xor(t, 1, WAVE);
        t += __shfl_xor(t, 2, WAVE);
        t += __shfl_xor(t, 4, WAVE);
        t += __shfl_xor(t, 8, WAVE);
        scale = 1.0f / sqrtf(t / (float)ex.K + ex.eps);
    }
    if (row >= M || ch0 >= d) return;                      // d is a multiple of 16: four channels or none
    // The state's rows and the taps are asked for now, before the slices: they depend on nothing that is
    // computed here, and a load at the end would cost another trip to memory.  (Up to four older rows are
    // kept in registers; a longer convolution reads the rest when it needs them.)
    const int Kc = cv.taps;
    float* st = cv.state + (long long)cv.state_slot[row] * (Kc - 1) * d;
    constexpr int KEEP = 4;
    f32x4 sv[KEEP];
    float wv[KEEP + 1][4];
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        sv[k] = k < Kc - 1 ? *(const f32x4*)(st + (long long)k * d + ch0) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; ++e) wv[k][e] = k < Kc - 1 ? cv.tap((int)ch0 + e, k) : 0.f;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) wv[KEEP][e] = cv.tap((int)ch0 + e, Kc - 1);
    float v[3][4];
    const long long stride = (long long)rows_padded * N;
#pragma unroll
    for (int part = 0; part < 3; ++part) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[part][e] = 0.f;
        const float* p0 = ws + row * N + (long long)part * d + ch0;
        for (int s0 = 0; s0 < n_slices; s0 += 8) {         // as the kernel above: eight slices asked for together, added in order
            f32x4 t[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (s0 + u < n_slices) t[u] = *(const f32x4*)(p0 + (s0 + u) * stride);
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (s0 + u < n_slices) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[part][e] += t[u][e];
                }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) v[part][e] = (float)(bf16_t)(v[part][e] * scale);
    }
    f32x4 y, u4;
#pragma unroll
    for (int e = 0; e < 4; ++e) { u4[e] = v[0][e] * v[2][e]; y[e] = 0.f; }
    // y = taps . (state rows in order, then u), one chain of operations a channel; row k moves to k - 1
#pragma unroll
    for (int k = 0; k < KEEP; ++k)
        if (k < Kc - 1) {
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = (k == 0) ? sv[k][e] * wv[k][e] : fmaf(sv[k][e], wv[k][e], y[e]);
            if (k > 0) *(f32x4*)(st + (long long)(k - 1) * d + ch0) = sv[k];
        }
    for (int k = KEEP; k < Kc - 1; ++k) {
        const f32x4 s4 = *(const f32x4*)(st + (long long)k * d + ch0);
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = fmaf(s4[e], cv.tap((int)ch0 + e, k), y[e]);
        *(f32x4*)(st + (long long)(k - 1) * d + ch0) = s4;
    }
    bf16x4 o4;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        y[e] = fmaf(u4[e], wv[KEEP][e], y[e]);
        o4[e] = (bf16_t)(v[1][e] * y[e]);
    }
    *(f32x4*)(st + (long long)(Kc - 2) * d + ch0) = u4;
    *(bf16x4*)(Y + row * d + ch0) = o4;
}

struct SkinnyPlan { int tiles, waves, slices, chunks_per_slice, cols; long long ws_floats; };

constexpr int SKINNY_ROWS = 32;     // the most rows of the kernel whose waves split K inside the workgroup (two row tiles)

// 17 to 64 rows and a wide output with a short K (gate and up of a feed-forward): the tiled product with one
// block of 64 x 64 for every 64 columns gives every CU a workgroup without slices of K, so no second kernel
// adds partial tiles, and its time is that of streaming W whatever the rows.  Measured against the two ways
// for few rows, SwiGLU epilogue, 17 to 64 rows: 16,384 x 2,048 18 to 22 us -> 15.5 to 16.5, 13,824 x 1,536 14 to
// 17 -> 11.5, 9,216 x 1,536 12 to 14 -> 11, 24,576 x 2,048 26 to 28.5 -> 24 to 27; no gain at 6,144 and 8,192
// columns nor at 32,768.
int wide64_min_n = 9216, wide64_max_n = 24576, wide64_min_m = 17;      // measurements may move them
bool wide64_shape(int N, int K) { return N >= wide64_min_n && N <= wide64_max_n && K % TBK == 0 && K / TBK <= 48; }
bool rows64_tiled(int M, int N, int K) { return M >= wide64_min_m && M <= 64 && wide64_shape(N, K); }

// Whether a product of M rows goes through that kernel (else, up to 64 rows: K cut over workgroups and a
// second kernel that adds the slices).  Up to 16 rows always.  17 to 32 rows: every workgroup reads all M
// rows of X again, M / (its columns) times the bytes of its share of W, and has half the waves; measured
// on the shapes of a 1.2B model (against the two kernels of the other way, at 32 rows): 2,048 columns
// 14.8 us against 11.9, 3,072 columns 8.8 against 10.7, a conv's input projection with the convolution
// 12.5 against 15.2, 16,384 columns 21.7 against 21.3, 65,536 columns 67.7 against 52.2; at 17 rows
// it wins everywhere.  So: narrow outputs up to 20 rows, medium ones up to 32, wide ones up to 24 (where the
// tiled product does not take them, above).
bool few_rows_kernel(int M, int N, int K, bool conv = false) {
    if (M <= 16) return true;
    if (M > SKINNY_ROWS) return false;
    if (conv) return true;
    if (rows64_tiled(M, N, K)) return false;
    return N <= 2048 ? M <= 20 : N <= 8192 ? true : M <= 24;
}

// How a skinny product is cut.  Depends on N and K (and on which of the two kernels M selects).
SkinnyPlan plan_skinny(int M, int N, int K, int max_waves = 16, bool emit = false, bool conv = false) {
    const int nchunks = ceil_div(K, SK_CHUNK);
    SkinnyPlan p;
    p.slices = 1; p.chunks_per_slice = nchunks; p.ws_floats = 0; p.waves = 4;
    p.cols = 16;
    if (few_rows_kernel(M, N, K, conv)) {
        // Narrow outputs: tiles of 8 columns, where 16 would leave CUs without a workgroup (half of
        // each MFMA idles, which costs nothing here: these products wait for memory).  Wide outputs:
        // 32 or 64 columns, whose MFMA tiles share the rows of X: with 16 columns the rows of X
        // (from the L2, again for every workgroup) are up to as many bytes again as the weights.
        const int tiles16 = ceil_div(N, 16);
        if (tiles16 <= 128) p.cols = 8;
        else if (tiles16 >= 4096) p.cols = 64;
        else if (tiles16 >= 512) p.cols = 32;
        if ((max_waves < 16 || emit) && p.cols > 16) p.cols = 16;       // the norm inside keeps float32 rows in registers;
                                                                        // the emitting epilogue works on one tile
        if (M > 16) {
            // two row tiles: twice the operands of X a wave, so at most two tiles of W side by side and eight waves
            p.cols = min(p.cols, 32);
            max_waves = min(max_waves, 8);
        }
        p.tiles = ceil_div(N, p.cols);
        // enough waves in flight to cover the latency of HBM, at least one chunk a wave
        while (p.waves < max_waves && p.tiles * p.waves < 3072 && nchunks >= 2 * p.waves) p.waves *= 2;
    } else {
        const int mt = ceil_div(M, 16);
        p.tiles = ceil_div(N, 64);
        int s = ceil_div(512, p.tiles);
        s = max(1, min(s, nchunks / 2));
        p.chunks_per_slice = ceil_div(nchunks, s);
        p.slices = ceil_div(nchunks, p.chunks_per_slice);
        p.ws_floats = (p.slices > 1 || emit) ? (long long)p.slices * mt * 16 * N : 0;
    }
    return p;
}

// How a product of more than 64 rows is cut: shape 0: 256 x 256 blocks; 1: 128 x 128 blocks, two a CU;
// 2: 128 x 128 blocks, one a CU, four steps of operands under way; 3: 64 x 64 blocks of four waves;
// 4: 256 x 192 blocks.
// Depends on the sizes only.
struct TiledPlan { int shape, slices, steps_per_slice; long long ws_floats; };

int tiled_shape_forced = -1;       // >= 0: every tiled product takes this shape (measurements only)

TiledPlan plan_tiled(int M, int N, int K) {
    const long long large = (long long)ceil_div(N, 256) * ceil_div(M, 256);
    const long long small = (long long)ceil_div(N, 128) * ceil_div(M, 128);
    const int nk = ceil_div(K, TBK);
    TiledPlan t;
    t.shape = large >= 160 ? 0 : small > 256 ? 1 : 2;
    t.slices = 1; t.steps_per_slice = nk; t.ws_floats = 0;
    if (tiled_shape_forced >= 0 && K % TBK == 0) { t.shape = tiled_shape_forced; return t; }
    // blocks of 256 x 192 where they need fewer rounds of 256 workgroups times columns than 256 x 256
    // (6144 columns and 2048 rows: 256 blocks, one round, instead of 192 blocks that leave a quarter of the CUs idle)
    if (t.shape == 0 && K % TBK == 0) {
        const long long wide = (long long)ceil_div(N, 192) * ceil_div(M, 256);
        if (ceil_div(wide, 256) * 192 < ceil_div(large, 256) * 256) t.shape = 4;
        return t;
    }
    // A little more than one round of pairs of 128 x 128 blocks (512 of them side by side), where blocks of 256 x 256
    // would be too few for the CUs: the blocks beyond the round run a second one almost alone.  Blocks of 256 x 192
    // in one round instead (4608 columns and 2048 rows, K = 1536: 37.1 us instead of 43.8; 256 x 256: 45.7).
    if (t.shape == 1 && small > 512 && K % TBK == 0) {
        const long long wide = (long long)ceil_div(N, 192) * ceil_div(M, 256);
        if (wide <= 256) { t.shape = 4; return t; }
    }
    // few blocks and a short K: blocks of 64 x 64 give enough workgroups without slices of K, whose partial
    // tiles cost a second kernel and as much traffic as the product's own (K = 1536 .. 2048, 96 to 512
    // rows: 9 to 14 us instead of 11 to 19); beyond 48 steps the slices win
    if (t.shape == 2 && small <= 128 && K % TBK == 0 && nk <= 48) { t.shape = 3; return t; }
    if (t.shape == 2 && small <= 128) {
        // as many slices as give every CU at most one block, at least eight steps a slice
        int s = max(1, min((int)(256 / small), nk / 8));
        t.steps_per_slice = ceil_div(nk, s);
        t.slices = ceil_div(nk, t.steps_per_slice);
        if (t.slices > 1) t.ws_floats = (long long)t.slices * M * N;
    }
    return t;
}

struct Skinny16Extra {
    const float* norm_w = nullptr; float eps = 0.f; const int* rows = nullptr;       // NORM_INSIDE
    const float* ss_in = nullptr; int n_ss = 0;                                      // NORM_SCALED (+ eps)
    const float* emit_nw = nullptr; bf16_t* emit_xw = nullptr; float* emit_ss = nullptr;   // EMIT
    ConvTail conv;                                                                   // OUT_CONV
};

template <int MODE, int NORM, bool EMIT>
int launch_skinny16(const void* X, const bf16_t* W, void* Y, int M, int N, int K, const Skinny16Extra& x, hipStream_t stream) {
    // the in-kernel norm needs more registers a wave: at most 8 waves a workgroup
    SkinnyPlan p = plan_skinny(M, N, K, NORM == NORM_INSIDE ? 8 : 16, EMIT, MODE == OUT_CONV);
    const size_t lds = NORM == NORM_INSIDE ? (size_t)K * sizeof(float) : 0;
    const int mt = M > 16 ? 2 : 1;
#define GO_MT(NW, COLS, MT) hipLaunchKernelGGL((gemm_bf16_skinny16_kernel<NW, MODE, NORM, EMIT, COLS, MT>), grid, dim3(NW * WAVE), lds, stream, \
                                        X, W, Y, M, N, K, x.norm_w, x.eps, x.rows, x.ss_in, x.n_ss, x.emit_nw, x.emit_xw, x.emit_ss, \
                                        x.conv)
#define GO(NW, COLS) do { \
        if (mt == 1) GO_MT(NW, COLS, 1); \
        else if constexpr (NW <= 8 && COLS <= 32 && NORM != NORM_INSIDE) GO_MT(NW, COLS, 2); \
        else return -3; \
    } while (0)
    if constexpr (MODE == OUT_CONV) {
        // eight channels a workgroup (three half tiles); the waves split K as always, at most eight of them:
        // sixteen would leave a wave 128 registers, too few for three tiles' operands of two chunks
        const int nchunks = ceil_div(K, SK_CHUNK), groups = N / 3 / 8;
        int waves = 4;
        while (waves < 8 && groups * waves < 3072 && nchunks >= 2 * waves) waves *= 2;
        dim3 grid(groups);
        if (waves == 4) GO(4, 8); else GO(8, 8);
    } else {
        dim3 grid(p.tiles);
        if (p.cols == 16) { if (p.waves == 4) GO(4, 16); else if (p.waves == 8) GO(8, 16); else GO(16, 16); }
        else if (p.cols == 8) { if (p.waves == 4) GO(4, 8); else if (p.waves == 8) GO(8, 8); else GO(16, 8); }
        else if constexpr (!EMIT && NORM != NORM_INSIDE) {
            if (p.cols == 32) { if (p.waves == 4) GO(4, 32); else if (p.waves == 8) GO(8, 32); else GO(16, 32); }
            else if (p.cols == 64) { if (p.waves == 4) GO(4, 64); else if (p.waves == 8) GO(8, 64); else GO(16, 64); }
            else return -3;
        } else return -3;
    }
#undef GO
#undef GO_MT
    return launch_status();
}

template <int NORM>
int launch_skinny16_mode(const void* X, const bf16_t* W, void* Y, int M, int N, int K, int mode, const Skinny16Extra& x,
                         hipStream_t stream) {
    if (mode == OUT_BF16) return launch_skinny16<OUT_BF16, NORM, false>(X, W, Y, M, N, K, x, stream);
    if (mode == OUT_F32) return launch_skinny16<OUT_F32, NORM, false>(X, W, Y, M, N, K, x, stream);
    if (mode == OUT_F32_ACCUM) return launch_skinny16<OUT_F32_ACCUM, NORM, false>(X, W, Y, M, N, K, x, stream);
    if (mode == OUT_SWIGLU) {
        if (N % 2) return -2;
        return launch_skinny16<OUT_SWIGLU, NORM, false>(X, W, Y, M, N, K, x, stream);
    }
    return -3;
}

// 16 < M <= 64.  ws: the work space tuff_gemm_bf16_workspace asks for.
template <int MODE, int NORM, bool EMIT>
int launch_skinny64(const bf16_t* X, const bf16_t* W, void* Y, int M, int N, int K, float* ws, const FinishExtra& ex,
                    hipStream_t stream) {
    const SkinnyPlan p = plan_skinny(M, N, K, 16, EMIT);
    dim3 grid(p.tiles, p.slices), block(SK_NT);
    const bool to_ws = p.ws_floats > 0;
    if (to_ws && !ws) return -4;
    const int mt = ceil_div(M, 16);
#define GO(MT) hipLaunchKernelGGL((gemm_bf16_skinny64_kernel<MT, MODE, NORM>), grid, block, 0, stream, X, W, Y, M, N, K, \
                                  p.chunks_per_slice, ws, to_ws, ex.ss_in, ex.n_ss, ex.eps)
    if (mt == 2) GO(2); else if (mt == 3) GO(3); else GO(4);
#undef GO
    if (to_ws) {
        int rc = launch_status();
        if (rc) return rc;
        // the emitting epilogue writes the sums of squares of all 64 rows of a tile (zero beyond M)
        hipLaunchKernelGGL((splitk_finish_kernel<MODE, NORM, EMIT>), dim3(p.tiles, EMIT ? 4 : mt), dim3(256), 0, stream,
                           (const float*)ws, Y, M, N, mt * 16, p.slices, ex);
    }
    return launch_status();
}

// 16 < M <= 64: the projection's partial tiles into the work space (always: also with one slice), then the
// kernel that adds them and runs the convolution.
template <int NORM>
int launch_skinny64_conv(const bf16_t* X, const bf16_t* W, bf16_t* Y, int M, int d, int K, float* ws, const FinishExtra& ex,
                         const ConvTail& cv, hipStream_t stream) {
    const int N = 3 * d;
    const SkinnyPlan p = plan_skinny(M, N, K, 16, true);
    if (!ws) return -4;
    const int mt = ceil_div(M, 16);
    dim3 grid(p.tiles, p.slices), block(SK_NT);
#define GO(MT) hipLaunchKernelGGL((gemm_bf16_skinny64_kernel<MT, OUT_BF16, NORM_NONE>), grid, block, 0, stream, X, W, (void*)nullptr, \
                                  M, N, K, p.chunks_per_slice, ws, true, (const float*)nullptr, 0, 0.f)
    if (mt == 2) GO(2); else if (mt == 3) GO(3); else GO(4);
#undef GO
    int rc = launch_status();
    if (rc) return rc;
    hipLaunchKernelGGL((splitk_finish_conv_kernel<NORM>), dim3(ceil_div(d, 64), ceil_div(M, FC_ROWS)), dim3(FC_ROWS * 16), 0, stream,
                       (const float*)ws, Y, M, d, mt * 16, p.slices, ex, cv);
    return launch_status();
}

template <int NORM>
int launch_skinny64_mode(const bf16_t* X, const bf16_t* W, void* Y, int M, int N, int K, int mode, float* ws,
                         const FinishExtra& ex, hipStream_t stream) {
    if (mode == OUT_BF16) return launch_skinny64<OUT_BF16, NORM, false>(X, W, Y, M, N, K, ws, ex, stream);
    if (mode == OUT_F32) return launch_skinny64<OUT_F32, NORM, false>(X, W, Y, M, N, K, ws, ex, stream);
    if (mode == OUT_F32_ACCUM) return launch_skinny64<OUT_F32_ACCUM, NORM, false>(X, W, Y, M, N, K, ws, ex, stream);
    if (mode == OUT_SWIGLU) {
        if (N % 2) return -2;
        return launch_skinny64<OUT_SWIGLU, NORM, false>(X, W, Y, M, N, K, ws, ex, stream);
    }
    return -3;
}

// How the sums of squares of a tiled product with the emitting epilogue are grouped: columns a group, or 0
// where this product cannot emit (K no multiple of 64, K cut into slices, N no whole number of blocks).
int tiled_emit_group(int M, int N, int K) {
    const TiledPlan t = plan_tiled(M, N, K);
    if (t.slices > 1) return 64;                        // the kernel that adds the slices emits, 64 columns a workgroup
    if (K % TBK != 0) return 0;
    const int bn = t.shape == 0 ? 256 : t.shape == 4 ? 192 : t.shape == 3 ? 64 : 128;
    if (N % bn != 0) return 0;
    return bn;                                          // a workgroup's columns
}

bool tiled_scaled_ok(int M, int N, int K) { return K % TBK == 0 || plan_tiled(M, N, K).slices > 1; }

template <int MODE, int AROUND = TILED_PLAIN>
int launch_mode(const bf16_t* X, const bf16_t* W, void* Y, int M, int N, int K, float* ws, hipStream_t stream,
                const TiledExtra& ex = TiledExtra()) {
    if constexpr (AROUND == TILED_PLAIN) {
        if (few_rows_kernel(M, N, K)) return launch_skinny16<MODE, NORM_NONE, false>(X, W, Y, M, N, K, Skinny16Extra(), stream);
        if (M <= 64 && !rows64_tiled(M, N, K)) return launch_skinny64<MODE, NORM_NONE, false>(X, W, Y, M, N, K, ws, FinishExtra(), stream);
    }
    {
        // Large blocks where they give most CUs one.  Of the small ones a CU holds two if there are
        // enough; if not, a block is alone on its CU and hides the memory's latency by itself, with
        // the operands of four steps under way.  Where even the small blocks are fewer than half the
        // CUs (few rows, narrow output), blocks of 64 x 64 take over if K is short, else K is cut into
        // slices, a block a slice.
        TiledPlan t = plan_tiled(M, N, K);
        if (rows64_tiled(M, N, K)) { t.shape = 3; t.slices = 1; t.steps_per_slice = ceil_div(K, TBK); t.ws_floats = 0; }
        if (t.slices > 1 && !ws) return -4;
#define TILED(TM, TN, WM, WN, AHEAD) do { \
            auto kern = gemm_bf16_tiled_kernel<TM, TN, WM, WN, AHEAD, MODE>; \
            constexpr int bm = 16 * TM * WM, bn = 16 * TN * WN, lds = 2 * (bm + bn) * TBK * 2; \
            static bool set = false; \
            if (!set) { \
                if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -1; \
                set = true; \
            } \
            hipLaunchKernelGGL(kern, dim3(ceil_div(N, bn), ceil_div(M, bm), t.slices), dim3(64 * WM * WN), lds, stream, \
                               X, W, Y, M, N, K, t.steps_per_slice, ws); \
        } while (0)
#define TILED_DMA(TM, TN, WM, WN, STAGES) do { \
            auto kern = gemm_bf16_dma_kernel<TM, TN, WM, WN, STAGES, MODE, AROUND>; \
            constexpr int bm = 16 * TM * WM, bn = 16 * TN * WN, lds = STAGES * (bm + bn) * TBK * 2; \
            static bool set = false; \
            if (!set) { \
                if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -1; \
                set = true; \
            } \
            hipLaunchKernelGGL(kern, dim3(ceil_div(N, bn), ceil_div(M, bm), t.slices), dim3(64 * WM * WN), lds, stream, \
                               X, W, Y, M, N, K, t.steps_per_slice, ws, ex); \
        } while (0)
        if constexpr (AROUND != TILED_PLAIN) {
            if (K % TBK != 0 && t.slices == 1) return -2;            // a product in slices is finished by the kernel that adds them
        }
        if (K % TBK == 0) {
            if (t.shape == 3) TILED_DMA(2, 2, 2, 2, 4);
            else if (t.shape == 4) TILED_DMA(8, 3, 2, 4, 2);
            else if (t.shape == 0) TILED_DMA(8, 4, 2, 4, 2);
            else if (t.shape == 1) TILED_DMA(4, 2, 2, 4, 2);
            else TILED_DMA(4, 2, 2, 4, 4);
        }
        else if (t.shape == 0) TILED(8, 4, 2, 4, 1);
        else if (t.shape == 1) TILED(4, 2, 2, 4, 1);
        else TILED(4, 2, 2, 4, 4);
#undef TILED_DMA
#undef TILED
        if (t.slices > 1) {
            int rc = launch_status();
            if (rc) return rc;
            FinishExtra fx;
            fx.ss_rows = M;
            fx.ss_in = ex.ss_in; fx.n_ss = ex.n_ss; fx.eps = ex.eps; fx.K = K;
            fx.emit_nw = ex.emit_nw; fx.emit_xw = ex.emit_xw; fx.emit_ss = ex.emit_ss;
            constexpr int FN = AROUND == TILED_SCALED ? NORM_SCALED : NORM_NONE;
            hipLaunchKernelGGL((splitk_finish_kernel<MODE, FN, AROUND == TILED_EMIT>), dim3(ceil_div(N, 64), ceil_div(M, 16)),
                               dim3(256), 0, stream, (const float*)ws, Y, M, N, M, t.slices, fx);
        }
    }
    return launch_status();
}
}  // namespace

// For measurements: for how many columns and from how many rows on a product of at most 64 rows with a short K
// takes blocks of 64 x 64 instead of slices of K.  Returns the least number of columns before.
TUFF_EXPORT int tuff_gemm_bf16_wide64(int min_n, int max_n, int min_m) {
    const int old = wide64_min_n;
    if (min_n > 0) wide64_min_n = min_n;
    if (max_n > 0) wide64_max_n = max_n;
    if (min_m > 0) wide64_min_m = min_m;
    return old;
}

// For measurements: forces the block shape of every product of more than 64 rows whose K is a multiple
// of 64 (0: 256 x 256, 1: 128 x 128 two a CU, 2: 128 x 128 one a CU, 3: 64 x 64, 4: 256 x 192; -1: by size).
// Returns the value before.
TUFF_EXPORT int tuff_gemm_bf16_force_tiled_shape(int shape) {
    const int old = tiled_shape_forced;
    tiled_shape_forced = shape;
    return old;
}

// How the sums of squares of tuff_gemm_bf16_accum_emit are laid out for a product of M rows:
// *tiles tiles of columns, *rows rows each (16 for M <= 16, 64 for M <= 64).
TUFF_EXPORT int tuff_gemm_bf16_emit_layout(int M, int N, int K, int* tiles, int* rows) {
    if (M > 64) {
        // the tiled product: a group of columns a wave, M rows each; *tiles = 0 where it cannot emit
        const int group = tiled_emit_group(M, N, K);
        *tiles = group ? ceil_div(N, group) : 0;        // (a product in slices may end in a partial group of columns)
        *rows = M;
        return 0;
    }
    *tiles = plan_skinny(M, N, K, 16, true).tiles;
    *rows = M <= 16 ? 16 : 64;                          // (17 to 32 rows: the kernel for few rows, with tiles of 64 rows)
    return 0;
}

// 1 if tuff_gemm_bf16_scaled takes a product of these sizes (always for M <= 64; for more rows where the
// tiled product runs it in one piece), else 0.
TUFF_EXPORT int tuff_gemm_bf16_scaled_supported(int M, int N, int K) {
    if (K % 8 != 0 || M <= 0 || N <= 0) return 0;
    return M <= 64 || tiled_scaled_ok(M, N, K) ? 1 : 0;
}

// Work space a product of this shape needs: *ws_floats float32 for partial tiles (0: none).
// emit: for tuff_gemm_bf16_accum_emit.
TUFF_EXPORT int tuff_gemm_bf16_workspace(int M, int N, int K, int emit, long long* ws_floats) {
    *ws_floats = 0;
    if (N <= 0 || few_rows_kernel(M, N, K)) return 0;
    // (a wide product of few rows that the tiled kernel takes needs none, but only some of its epilogues go that way)
    *ws_floats = M <= 64 ? plan_skinny(M, N, K, 16, emit != 0).ws_floats : plan_tiled(M, N, K).ws_floats;
    return 0;
}

// W: tile-major, as described at the head of this file (ceil(N/16) * ceil(K/32) blocks of 1 KB).
// K must be a multiple of 8 (16-byte operand loads); the host wrapper refuses other K.
TUFF_EXPORT int tuff_gemm_bf16(const void* X, const void* W, void* Y, int M, int N, int K, int mode,
                               float* ws, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 != 0) return -2;
    const bf16_t* x = (const bf16_t*)X;
    const bf16_t* w = (const bf16_t*)W;
    if (mode == OUT_BF16) return launch_mode<OUT_BF16>(x, w, Y, M, N, K, ws, stream);
    if (mode == OUT_F32) return launch_mode<OUT_F32>(x, w, Y, M, N, K, ws, stream);
    if (mode == OUT_F32_ACCUM) return launch_mode<OUT_F32_ACCUM>(x, w, Y, M, N, K, ws, stream);
    if (mode == OUT_SWIGLU) {
        if (N % 2) return -2;
        return launch_mode<OUT_SWIGLU>(x, w, Y, M, N, K, ws, stream);
    }
    return -3;
}

// Y (=|+=) RMSNorm(X[rows]) * W^T for M <= 16 rows: X float32 [*, K], norm_w float32 [K], rows
// optional int32 [M].  K must be a multiple of 8 and at most 8192 (the norm weight sits in LDS).
TUFF_EXPORT int tuff_gemm_bf16_normed(const float* X, const int* rows, const float* norm_w, float eps, const void* W,
                                      void* Y, int M, int N, int K, int mode, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 != 0 || K > 8192 || M > 16) return -2;
    Skinny16Extra x;
    x.norm_w = norm_w; x.eps = eps; x.rows = rows;
    return launch_skinny16_mode<NORM_INSIDE>(X, (const bf16_t*)W, Y, M, N, K, mode, x, stream);
}

// Y += X W^T, and from the new Y (the residual stream, float32 [M, N]) the
// operand of the RMSNorm that follows: xw = bf16(Y * next_norm_w) [M, N] and ss [tiles][rows] (as
// tuff_gemm_bf16_emit_layout says; 0 tiles: this product cannot, -2), the sums of squares of each row
// over each tile of columns.
// ws: for M > 16, the work space tuff_gemm_bf16_workspace(M, N, K, 1) asks for.
TUFF_EXPORT int tuff_gemm_bf16_accum_emit(const void* X, const void* W, float* Y, int M, int N, int K,
                                          const float* next_norm_w, void* xw, float* ss, float* ws, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 != 0) return -2;
    if (M > 64) {
        if (!tiled_emit_group(M, N, K)) return -2;
        TiledExtra t;
        t.emit_nw = next_norm_w; t.emit_xw = (bf16_t*)xw; t.emit_ss = ss;
        return launch_mode<OUT_F32_ACCUM, TILED_EMIT>((const bf16_t*)X, (const bf16_t*)W, Y, M, N, K, ws, stream, t);
    }
    if (few_rows_kernel(M, N, K)) {
        Skinny16Extra x;
        x.emit_nw = next_norm_w; x.emit_xw = (bf16_t*)xw; x.emit_ss = ss;
        return launch_skinny16<OUT_F32_ACCUM, NORM_NONE, true>(X, (const bf16_t*)W, Y, M, N, K, x, stream);
    }
    FinishExtra x;
    x.emit_nw = next_norm_w; x.emit_xw = (bf16_t*)xw; x.emit_ss = ss;
    return launch_skinny64<OUT_F32_ACCUM, NORM_NONE, true>((const bf16_t*)X, (const bf16_t*)W, Y, M, N, K, ws, x, stream);
}

// Y (=|+=) (XW W^T) scaled per row by 1 / sqrt(sum_t ss[t][row] / K + eps), with
// XW and ss as tuff_gemm_bf16_accum_emit leaves them for the same M (n_ss tiles); see
// tuff_gemm_bf16_scaled_supported for M > 64.
// ws: for M > 16, the work space tuff_gemm_bf16_workspace(M, N, K, 0) asks for.
TUFF_EXPORT int tuff_gemm_bf16_scaled(const void* XW, const float* ss, int n_ss, float eps, const void* W, void* Y,
                                      int M, int N, int K, int mode, float* ws, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 != 0 || n_ss < 1) return -2;
    if (M > 64 || (rows64_tiled(M, N, K) && (mode == OUT_BF16 || mode == OUT_SWIGLU))) {
        // ss [n_ss][M] ([n_ss][64] from a product of at most 64 rows); bfloat16 and SwiGLU outputs (what reads a norm in a layer)
        if (!tiled_scaled_ok(M, N, K)) return -2;
        TiledExtra t;
        t.ss_in = ss; t.n_ss = n_ss; t.eps = eps; t.ss_rows = M > 64 ? 0 : 64;
        const bf16_t* x = (const bf16_t*)XW;
        const bf16_t* w = (const bf16_t*)W;
        if (mode == OUT_BF16) return launch_mode<OUT_BF16, TILED_SCALED>(x, w, Y, M, N, K, ws, stream, t);
        if (mode == OUT_SWIGLU) {
            if (N % 2) return -2;
            return launch_mode<OUT_SWIGLU, TILED_SCALED>(x, w, Y, M, N, K, ws, stream, t);
        }
        return -3;
    }
    if (few_rows_kernel(M, N, K)) {
        Skinny16Extra x;
        x.ss_in = ss; x.n_ss = n_ss; x.eps = eps;
        return launch_skinny16_mode<NORM_SCALED>(XW, (const bf16_t*)W, Y, M, N, K, mode, x, stream);
    }
    FinishExtra x;
    x.ss_in = ss; x.n_ss = n_ss; x.eps = eps; x.K = K;
    return launch_skinny64_mode<NORM_SCALED>((const bf16_t*)XW, (const bf16_t*)W, Y, M, N, K, mode, ws, x, stream);
}

// For M <= 16 rows, one token a row: the input projection of a gated short convolution and the
// convolution itself in one kernel.  W: the projection [3 d, K] with its rows regrouped (sixteen
// channels a group: B, C, X of the group), tile-major; d must be a multiple of 16.  Y: bfloat16 [M, d]
// = C * conv(B * X).  taps [d][n_taps] (taps_dt), state float32 [slots][n_taps - 1][d], state_slot [M].
// norm_kind 0: X is bfloat16 [M, K];  1: X is the float32 residual stream and the RMSNorm (norm_w,
// eps; K <= 8192) runs inside;  2: X is bf16(x * norm weight) and ss [n_ss][16] the sums of squares
// that tuff_gemm_bf16_accum_emit left.
// The same for 17 to 64 rows, in two kernels (the projection's partial tiles, then the kernel that adds
// them and runs the convolution), from the projection as the checkpoint has it: W [3 d, K] tile-major,
// rows B | C | X.  X: bfloat16 [M, K], or with ss [n_ss][64] (and eps) bf16(x * norm weight) and the sums of
// squares that tuff_gemm_bf16_accum_emit left for these M rows.  ws: tuff_gemm_bf16_workspace(M, 3 d, K, 1).
TUFF_EXPORT int tuff_gemm_bf16_conv64(const void* X, const float* ss, int n_ss, float eps, const void* W, void* Y,
                                      int M, int d, int K, const void* taps, int taps_dt, int n_taps, float* state,
                                      const int* state_slot, float* ws, hipStream_t stream) {
    if (M <= 0 || d <= 0) return 0;
    if (K % 8 != 0 || M <= SKINNY_ROWS || M > 64 || d % 16 != 0 || n_taps < 2 || n_taps - 1 > CONV_MAX_TAPS) return -2;
    ConvTail cv;
    cv.taps_w = taps; cv.taps_dt = taps_dt; cv.taps = n_taps; cv.state = state; cv.state_slot = state_slot;
    FinishExtra x;
    if (ss) {
        if (n_ss < 1) return -2;
        x.ss_in = ss; x.n_ss = n_ss; x.eps = eps; x.K = K;
        return launch_skinny64_conv<NORM_SCALED>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, d, K, ws, x, cv, stream);
    }
    return launch_skinny64_conv<NORM_NONE>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, d, K, ws, x, cv, stream);
}

TUFF_EXPORT int tuff_gemm_bf16_conv(const void* X, int norm_kind, const float* norm_w, float eps, const float* ss, int n_ss,
                                    const void* W, void* Y, int M, int d, int K,
                                    const void* taps, int taps_dt, int n_taps, float* state, const int* state_slot,
                                    hipStream_t stream) {
    if (M <= 0 || d <= 0) return 0;
    if (K % 8 != 0 || M > SKINNY_ROWS || d % 16 != 0 || n_taps < 2 || n_taps - 1 > CONV_MAX_TAPS) return -2;
    if (norm_kind == 1 && M > 16) return -2;
    Skinny16Extra x;
    x.conv.taps_w = taps; x.conv.taps_dt = taps_dt; x.conv.taps = n_taps; x.conv.state = state; x.conv.state_slot = state_slot;
    const bf16_t* w = (const bf16_t*)W;
    if (norm_kind == 0) return launch_skinny16<OUT_CONV, NORM_NONE, false>(X, w, Y, M, 3 * d, K, x, stream);
    if (norm_kind == 1) {
        if (K > 8192) return -2;
        x.norm_w = norm_w; x.eps = eps;
        return launch_skinny16<OUT_CONV, NORM_INSIDE, false>(X, w, Y, M, 3 * d, K, x, stream);
    }
    if (norm_kind == 2) {
        if (n_ss < 1) return -2;
        x.ss_in = ss; x.n_ss = n_ss; x.eps = eps;
        return launch_skinny16<OUT_CONV, NORM_SCALED, false>(X, w, Y, M, 3 * d, K, x, stream);
    }
    return -3;
}
