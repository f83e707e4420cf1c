// After the q/k/v projection: per-head RMSNorm of q and k, rotary position encoding,
// and the write of k and v into the paged cache, in one pass over the projected row.
//
// Reference: src/lfm25_gpu.cu:420-485 (norm over the head with a shared [hd] weight,
// then half-split rotation with theta_j = base^(-2j/hd), K cached after both) and
// :487-501 (V cached as projected).  Here theta_j comes in as a float32 table and the
// angle pos * theta_j, its cosine and sine are float32.
//
// Cache layout, slot = page * page_size + offset:
//   K [page][kv_head][offset][hd]      a key's channels are contiguous (q.k runs over hd)
//   V [page][kv_head][hd][offset]      a channel's positions are contiguous (p.v runs over keys)
#include "common.h"

namespace {
constexpr int MAX_PER_LANE = 4;            // head sizes up to 256

// Four neighbouring elements as float32, and back (8 bytes of bfloat16 or 16 of float32 at once).
__device__ __forceinline__ void load4(const bf16_t* p, float (&v)[4]) {
    const bf16x4 t = *(const bf16x4*)p;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = (float)t[e];
}
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
    const f32x4 t = *(const f32x4*)p;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = t[e];
}
__device__ __forceinline__ void store4(bf16_t* p, const float (&v)[4]) {
    bf16x4 t = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *(bf16x4*)p = t;
}
__device__ __forceinline__ void store4(float* p, const float (&v)[4]) {
    *(f32x4*)p = f32x4{v[0], v[1], v[2], v[3]};
}

// A workgroup of four waves takes one token; wave w the heads_per_wave heads from
// (blockIdx.y * 4 + w) * heads_per_wave on (q heads, then k heads, then v heads).  The angles of a
// token are the same for all its heads and are computed once a wave.
constexpr int POST_WAVES = 4;

template <typename T, typename TW>
__global__ __launch_bounds__(POST_WAVES * WAVE) void qkv_post_kernel(
    const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache,
    const TW* __restrict__ q_norm_w, const TW* __restrict__ k_norm_w, float eps,
    const float* __restrict__ inv_freq, int rotary_dim, int interleaved,
    const int* __restrict__ positions, const int* __restrict__ slot_mapping,
    int H, int Hkv, int hd, int page_size, int heads, int heads_per_wave,
    const float* __restrict__ angles, int n_angles) {
    __shared__ float vals_all[POST_WAVES][MAX_PER_LANE * WAVE];
    const int t = blockIdx.x, lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    float* vals = vals_all[wave];
    const int head_begin = (blockIdx.y * POST_WAVES + wave) * heads_per_wave;
    const int head_end = min(heads, head_begin + heads_per_wave);
    if (head_begin >= head_end) return;
    const int row_width = (H + 2 * Hkv) * hd;
    const int half = rotary_dim / 2;

    // rotation of element j = lane + 64 i: which frequency, which partner, cosine and sine
    float rc[MAX_PER_LANE], rs[MAX_PER_LANE];
    int partner[MAX_PER_LANE];
    bool first[MAX_PER_LANE], turns[MAX_PER_LANE];
    if (inv_freq != nullptr && head_begin < H + Hkv) {
        const int p = positions[t];
        const float pos = (float)p;
#pragma unroll
        for (int i = 0; i < MAX_PER_LANE; ++i) {
            const int j = lane + i * WAVE;
            turns[i] = j < rotary_dim && j < hd;
            int f = 0;
            if (interleaved) { f = j / 2; first[i] = (j % 2) == 0; partner[i] = first[i] ? j + 1 : j - 1; }
            else { first[i] = j < half; f = first[i] ? j : j - half; partner[i] = first[i] ? j + half : j - half; }
            rc[i] = 1.f; rs[i] = 0.f;
            if (turns[i]) {
                if (p < n_angles) {                      // from the table: the same bits, without the two functions
                    rc[i] = angles[((long long)p * 2) * half + f];
                    rs[i] = angles[((long long)p * 2 + 1) * half + f];
                } else {
                    const float a = pos * inv_freq[f];
                    rc[i] = cosf(a);
                    rs[i] = sinf(a);
                }
            }
        }
    }
    long long slot = -1;
    if (k_cache) slot = slot_mapping[t];

    for (int head = head_begin; head < head_end; ++head) {
        const T* src = qkv + (long long)t * row_width + (long long)head * hd;
        const bool is_q = head < H, is_k = !is_q && head < H + Hkv;
        const int kvh = is_q ? 0 : (is_k ? head - H : head - H - Hkv);

        float v[MAX_PER_LANE];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < MAX_PER_LANE; ++i) {
            const int j = lane + i * WAVE;
            v[i] = (j < hd) ? to_f32(src[j]) : 0.f;
            ss += v[i] * v[i];
        }
        const TW* nw = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
        if (nw) {
            const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)hd + eps);
#pragma unroll
            for (int i = 0; i < MAX_PER_LANE; ++i) {
                const int j = lane + i * WAVE;
                if (j < hd) v[i] = v[i] * inv * to_f32(nw[j]);
            }
        }
        if (inv_freq != nullptr && (is_q || is_k)) {
            // the wave's own LDS row; its reads follow its writes in program order
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int i = 0; i < MAX_PER_LANE; ++i) vals[lane + i * WAVE] = v[i];
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int i = 0; i < MAX_PER_LANE; ++i) {
                if (!turns[i]) continue;
                const float other = vals[partner[i]];
                const float x0 = first[i] ? v[i] : other;
                const float x1 = first[i] ? other : v[i];
                v[i] = first[i] ? (x0 * rc[i] - x1 * rs[i]) : (x0 * rs[i] + x1 * rc[i]);
            }
        }
        T* dst = nullptr;
        T* dst2 = nullptr;
        long long dst_stride = 1;
        if (is_q) dst = q_out + ((long long)t * H + head) * hd;
        else {
            if (is_k && k_out) dst2 = k_out + ((long long)t * Hkv + kvh) * hd;
            if (k_cache && slot >= 0) {
                const long long page = slot / page_size, off = slot % page_size;
                const long long head_base = (page * Hkv + kvh) * page_size * hd;
                if (is_k) dst = k_cache + head_base + off * hd;
                else { dst = v_cache + head_base + off; dst_stride = page_size; }
            }
        }
#pragma unroll
        for (int i = 0; i < MAX_PER_LANE; ++i) {
            const int j = lane + i * WAVE;
            if (j < hd) {
                const T o = from_f32<T>(v[i]);
                if (dst) dst[j * dst_stride] = o;
                if (dst2) dst2[j] = o;
            }
        }
    }
}

// The same for heads of 64 channels with the half-split rotation over the whole head, laid out for
// many tokens.  Two kinds of workgroups in one launch:
//  * q and k: sixteen lanes take one token and walk a share of its heads; lane l holds the channels
//    4l .. 4l+3 of a head (one 8-byte load for bfloat16), the norm's sum of squares is a butterfly over
//    the sixteen lanes, the rotation's partner channel j +- 32 sits in lane l ^ 8, and the token's
//    cosines and sines are computed once for all its heads.
//  * v: a workgroup takes sixteen consecutive tokens and one kv head, brings the rows into LDS and
//    writes, for every channel, the sixteen positions in one run where the tokens fill a run of sixteen
//    slots from a multiple of sixteen (the usual case in a prompt), else one by one: V is kept with a
//    channel's positions contiguous, and a token alone can only write it two bytes at a time.
// Whatever the number of tokens in the step, a token's values go through the same arithmetic.
constexpr int P64_GROUPS = 16;                       // sixteen-lane groups a workgroup
constexpr int P64_TOKENS = 16;                       // tokens a v workgroup

template <typename T, typename TW>
__global__ __launch_bounds__(256) void qkv_post64_kernel(
    const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const TW* __restrict__ q_norm_w, const TW* __restrict__ k_norm_w, float eps, const float* __restrict__ inv_freq,
    const int* __restrict__ positions, const int* __restrict__ slot_mapping,
    int n_tokens, int H, int Hkv, int page_size, int shares, int qk_blocks,
    const float* __restrict__ angles, int n_angles) {
    constexpr int HD = 64;
    const int tid = threadIdx.x;
    const int row_width = (H + 2 * Hkv) * HD;
    if ((int)blockIdx.x < qk_blocks) {
        const int l = tid % 16, grp = tid / 16;
        const long long item = (long long)blockIdx.x * P64_GROUPS + grp;      // (token, share of its heads)
        const int t = (int)(item / shares), share = (int)(item % shares);
        if (t >= n_tokens) return;
        const int n_heads = k_cache ? H + Hkv : H;
        const int per = (n_heads + shares - 1) / shares;
        const int head_begin = share * per, head_end = min(n_heads, head_begin + per);
        const int p = positions[t];
        const float pos = (float)p;
        const bool first = l < 8;
        float rc[4], rs[4], wq[4], wk[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int f = (4 * l + e) & 31;
            if (p < n_angles) {                          // from the table: the same bits, without the two functions
                rc[e] = angles[((long long)p * 2) * 32 + f];
                rs[e] = angles[((long long)p * 2 + 1) * 32 + f];
            } else {
                const float a = pos * inv_freq[f];
                rc[e] = cosf(a);
                rs[e] = sinf(a);
            }
            wq[e] = q_norm_w ? to_f32(q_norm_w[4 * l + e]) : 1.f;
            wk[e] = k_norm_w ? to_f32(k_norm_w[4 * l + e]) : 1.f;
        }
        long long slot = -1;
        if (k_cache) slot = slot_mapping[t];
        const T* row = qkv + (long long)t * row_width + 4 * l;
        for (int head = head_begin; head < head_end; ++head) {
            const bool is_q = head < H;
            float v[4];
            load4(row + (long long)head * HD, v);
            float ss = v[0] * v[0];
            ss = fmaf(v[1], v[1], ss);
            ss = fmaf(v[2], v[2], ss);
            ss = fmaf(v[3], v[3], ss);
            ss += __shfl_xor(ss, 8, WAVE);
            ss += __shfl_xor(ss, 4, WAVE);
            ss += __shfl_xor(ss, 2, WAVE);
            ss += __shfl_xor(ss, 1, WAVE);
            if (is_q ? q_norm_w != nullptr : k_norm_w != nullptr) {
                const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * inv * (is_q ? wq[e] : wk[e]);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float other = __shfl_xor(v[e], 8, WAVE);
                const float x0 = first ? v[e] : other, x1 = first ? other : v[e];
                v[e] = first ? (x0 * rc[e] - x1 * rs[e]) : (x0 * rs[e] + x1 * rc[e]);
            }
            if (is_q) store4(q_out + ((long long)t * H + head) * HD + 4 * l, v);
            else if (slot >= 0) {
                const long long page = slot / page_size, off = slot % page_size;
                store4(k_cache + ((page * Hkv + (head - H)) * page_size + off) * HD + 4 * l, v);
            }
        }
        return;
    }
    // v: tokens t0 .. t0 + 15 of one kv head
    __shared__ __attribute__((aligned(16))) T vt[P64_TOKENS][HD];
    __shared__ int slots[P64_TOKENS];
    const int vb = (int)blockIdx.x - qk_blocks;
    const int t0 = (vb / Hkv) * P64_TOKENS, kvh = vb % Hkv;
    const int n_here = min(P64_TOKENS, n_tokens - t0);
    {
        const int i = tid / 16, c = (tid % 16) * 4;          // 16 tokens x 16 pieces of four channels
        if (i < n_here) {
            float x[4];
            load4(qkv + (long long)(t0 + i) * row_width + (long long)(H + Hkv + kvh) * HD + c, x);
            store4(&vt[i][c], x);
        }
    }
    if (tid < P64_TOKENS) slots[tid] = tid < n_here ? slot_mapping[t0 + tid] : -1;
    __syncthreads();
    const int s0 = slots[0];
    bool run = n_here == P64_TOKENS && s0 >= 0 && s0 % 16 == 0;
#pragma unroll
    for (int i = 1; i < P64_TOKENS; ++i) run = run && slots[i] == s0 + i;
    if (run) {
        if (tid < HD) {                                      // a channel a thread: its sixteen positions in one run
            const long long page = s0 / page_size, off = s0 % page_size;
            T* dst = v_cache + ((page * Hkv + kvh) * HD + tid) * page_size + off;
            T vals[P64_TOKENS];
#pragma unroll
            for (int i = 0; i < P64_TOKENS; ++i) vals[i] = vt[i][tid];
            constexpr int PIECES = P64_TOKENS * (int)sizeof(T) / 16;
#pragma unroll
            for (int q = 0; q < PIECES; ++q) ((uint4*)dst)[q] = ((const uint4*)vals)[q];
        }
    } else {
        const int ch = tid % HD;
        for (int i = tid / HD; i < n_here; i += 256 / HD) {
            const long long slot = slots[i];
            if (slot < 0) continue;
            const long long page = slot / page_size, off = slot % page_size;
            v_cache[((page * Hkv + kvh) * HD + ch) * page_size + off] = vt[i][ch];
        }
    }
}

// Cosines and sines of pos * inv_freq[j] for pos = 0 .. n_pos - 1, as the kernels above compute them
// (the same float32 product and the same cosf and sinf): out [n_pos][2][n_freq], cosines then sines.
// A kernel that takes its angles from this table gives the bits of one that computes them.
__global__ void rope_table_kernel(const float* __restrict__ inv_freq, int n_freq, int n_pos, float* __restrict__ out) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long long)n_pos * n_freq) return;
    const int p = (int)(i / n_freq), j = (int)(i % n_freq);
    const float pos = (float)p;
    const float a = pos * inv_freq[j];
    out[((long long)p * 2) * n_freq + j] = cosf(a);
    out[((long long)p * 2 + 1) * n_freq + j] = sinf(a);
}

// Copies already encoded k and v rows [T, Hkv, hd] into the paged cache.
template <typename T>
__global__ __launch_bounds__(WAVE) void kv_write_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                                        T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                        const int* __restrict__ slot_mapping, int Hkv, int hd, int page_size) {
    const int t = blockIdx.x, kvh = blockIdx.y;
    const long long slot = slot_mapping[t];
    if (slot < 0) return;
    const long long page = slot / page_size, off = slot % page_size;
    const long long head_base = (page * Hkv + kvh) * page_size * hd;
    const long long src = ((long long)t * Hkv + kvh) * hd;
    for (int j = threadIdx.x; j < hd; j += WAVE) {
        k_cache[head_base + off * hd + j] = k[src + j];
        v_cache[head_base + (long long)j * page_size + off] = v[src + j];
    }
}
}  // namespace

// dt: element type of qkv, q_out, k_out and the caches.  norm_dt: element type of the
// norm weights.  Null q_norm_w / k_norm_w: no norm.  Null inv_freq: no rotation.
// Null k_cache: nothing is written to the cache (then only the H query heads and, if
// k_out is given, the key heads are processed).
// How many (token, share of its heads) items the kernel for heads of 64 wants at least: a token's heads
// are dealt to more sixteen-lane groups until there are that many.  For measurements; no result depends on it.
static int post64_items = 8192;
TUFF_EXPORT int tuff_qkv_post64_items(int n) {
    const int old = post64_items;
    if (n > 0) post64_items = n;
    return old;
}

TUFF_EXPORT int tuff_qkv_post(const void* qkv, void* q_out, void* k_out, void* k_cache, void* v_cache, int dt,
                              const void* q_norm_w, const void* k_norm_w, int norm_dt, float eps,
                              const float* inv_freq, int rotary_dim, int interleaved,
                              const int* positions, const int* slot_mapping,
                              int n_tokens, int H, int Hkv, int hd, int page_size,
                              const float* angles, int n_angles, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (hd > MAX_PER_LANE * WAVE || rotary_dim > hd || (rotary_dim % 2) != 0) return -2;
    if (!angles || !inv_freq) n_angles = 0;              // [n_angles][2][rotary_dim / 2] as tuff_rope_table makes it
    if (hd == 64 && inv_freq && rotary_dim == 64 && !interleaved && !k_out && page_size % 16 == 0) {
        // shares of a token's heads: enough sixteen-lane groups for the chip, whole heads each
        const int n_heads = k_cache ? H + Hkv : H;
        int shares = 1;
        const long long items = n_tokens >= 1024 ? 2ll * post64_items : post64_items;   // measured: 2,048 tokens 12.1 -> 10.5 us
        while (shares < n_heads && (long long)n_tokens * shares < items) shares *= 2;
        shares = min(shares, n_heads);
        const int qk_blocks = (int)ceil_div_ll((long long)n_tokens * shares, P64_GROUPS);
        const int v_blocks = k_cache ? ceil_div(n_tokens, P64_TOKENS) * Hkv : 0;
#define LAUNCH64(T, TW) hipLaunchKernelGGL((qkv_post64_kernel<T, TW>), dim3(qk_blocks + v_blocks), dim3(256), 0, stream, \
        (const T*)qkv, (T*)q_out, (T*)k_cache, (T*)v_cache, (const TW*)q_norm_w, (const TW*)k_norm_w, eps, inv_freq, \
        positions, slot_mapping, n_tokens, H, Hkv, page_size, shares, qk_blocks, angles, n_angles)
        if (dt == DT_F32 && norm_dt == DT_F32) LAUNCH64(float, float);
        else if (dt == DT_F32) LAUNCH64(float, bf16_t);
        else if (norm_dt == DT_F32) LAUNCH64(bf16_t, float);
        else LAUNCH64(bf16_t, bf16_t);
#undef LAUNCH64
        return launch_status();
    }
    const int heads = k_cache ? H + 2 * Hkv : (k_out ? H + Hkv : H);
    // few tokens: a wave a head; many: several heads a wave, so that workgroups stay in the thousands
    const long long waves = (long long)n_tokens * heads;
    int heads_per_wave = (int)min((long long)heads, max(1LL, waves / 16384));
    dim3 grid(n_tokens, ceil_div(heads, POST_WAVES * heads_per_wave)), block(POST_WAVES * WAVE);
#define LAUNCH(T, TW) hipLaunchKernelGGL((qkv_post_kernel<T, TW>), grid, block, 0, stream, (const T*)qkv, (T*)q_out, (T*)k_out, \
        (T*)k_cache, (T*)v_cache, (const TW*)q_norm_w, (const TW*)k_norm_w, eps, inv_freq, rotary_dim, interleaved, \
        positions, slot_mapping, H, Hkv, hd, page_size, heads, heads_per_wave, angles, n_angles)
    if (dt == DT_F32 && norm_dt == DT_F32) LAUNCH(float, float);
    else if (dt == DT_F32) LAUNCH(float, bf16_t);
    else if (norm_dt == DT_F32) LAUNCH(bf16_t, float);
    else LAUNCH(bf16_t, bf16_t);
#undef LAUNCH
    return launch_status();
}

TUFF_EXPORT int tuff_kv_write(const void* k, const void* v, void* k_cache, void* v_cache, int dt,
                              const int* slot_mapping, int n_tokens, int Hkv, int hd, int page_size,
                              hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens, Hkv), block(WAVE);
    if (dt == DT_F32) hipLaunchKernelGGL(kv_write_kernel<float>, grid, block, 0, stream, (const float*)k, (const float*)v, (float*)k_cache, (float*)v_cache, slot_mapping, Hkv, hd, page_size);
    else hipLaunchKernelGGL(kv_write_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)k, (const bf16_t*)v, (bf16_t*)k_cache, (bf16_t*)v_cache, slot_mapping, Hkv, hd, page_size);
    return launch_status();
}

TUFF_EXPORT int tuff_rope_table(const float* inv_freq, int n_freq, int n_pos, float* out, hipStream_t stream) {
    if (n_pos <= 0 || n_freq <= 0) return 0;
    const long long n = (long long)n_pos * n_freq;
    hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)ceil_div_ll(n, 256)), dim3(256), 0, stream, inv_freq, n_freq, n_pos, out);
    return launch_status();
}
