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
    int H, int Hkv, int hd, int page_size, int heads, int heads_per_wave) {
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
        const float pos = (float)positions[t];
#pragma unroll
        for (int i = 0; i < MAX_PER_LANE; ++i) {
            const int j = lane + i * WAVE;
            turns[i] = j < rotary_dim && j < hd;
            int f = 0;
            if (interleaved) { f = j / 2; first[i] = (j % 2) == 0; partner[i] = first[i] ? j + 1 : j - 1; }
            else { first[i] = j < half; f = first[i] ? j : j - half; partner[i] = first[i] ? j + half : j - half; }
            rc[i] = 1.f; rs[i] = 0.f;
            if (turns[i]) {
                const float a = pos * inv_freq[f];
                rc[i] = cosf(a);
                rs[i] = sinf(a);
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
TUFF_EXPORT int tuff_qkv_post(const void* qkv, void* q_out, void* k_out, void* k_cache, void* v_cache, int dt,
                              const void* q_norm_w, const void* k_norm_w, int norm_dt, float eps,
                              const float* inv_freq, int rotary_dim, int interleaved,
                              const int* positions, const int* slot_mapping,
                              int n_tokens, int H, int Hkv, int hd, int page_size, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (hd > MAX_PER_LANE * WAVE || rotary_dim > hd || (rotary_dim % 2) != 0) return -2;
    const int heads = k_cache ? H + 2 * Hkv : (k_out ? H + Hkv : H);
    // few tokens: a wave a head; many: several heads a wave, so that workgroups stay in the thousands
    const long long waves = (long long)n_tokens * heads;
    int heads_per_wave = (int)min((long long)heads, max(1LL, waves / 16384));
    dim3 grid(n_tokens, ceil_div(heads, POST_WAVES * heads_per_wave)), block(POST_WAVES * WAVE);
#define LAUNCH(T, TW) hipLaunchKernelGGL((qkv_post_kernel<T, TW>), grid, block, 0, stream, (const T*)qkv, (T*)q_out, (T*)k_out, \
        (T*)k_cache, (T*)v_cache, (const TW*)q_norm_w, (const TW*)k_norm_w, eps, inv_freq, rotary_dim, interleaved, \
        positions, slot_mapping, H, Hkv, hd, page_size, heads, heads_per_wave)
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
