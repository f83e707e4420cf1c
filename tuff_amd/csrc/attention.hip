// Attention of a mixed batch over the paged cache: every token of the step, prompt
// portion or decoded token alike, attends to the keys of its own request at positions
// lo..pos, lo = 0 or pos - window + 1, read from the pages its block table names.  The
// step's own keys were written to the cache before this runs, so nothing but the cache
// is read (cf. src/lfm25_engine.c:552-568: all K/V of a batch are written before any
// attention, and token j is bounded by its own position).
//
// Scores are scaled by 1/sqrt(hd); softmax is the running-max form of
// src/lfm25_gpu.cu:531-555 over key tiles of 64; query head h reads kv head
// h / (H / Hkv).  Scores, softmax and the weighted sum are float32.  The key tiles are
// aligned to absolute positions (0, 64, 128, ...), so the order of every sum depends
// only on the token's position, not on how the sequence was cut into steps.
//
// Cache layout: K [page][kv_head][offset][hd], V [page][kv_head][hd][offset].
//
// This is the general kernel: any head size up to 256, any page size, float32 or
// bfloat16 cache.  One wave per (token, head): lanes are keys for q.k, lanes are
// channels for p.v.
#include "common.h"
#include <math.h>

namespace {
constexpr int MAX_PER_LANE = 4;

template <typename T>
__global__ __launch_bounds__(WAVE) void attention_general_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ out,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ req_of_token,
    const int* __restrict__ positions, int H, int Hkv, int hd, int page_size, int window, float scale) {
    __shared__ float qs[MAX_PER_LANE * WAVE];
    __shared__ float ps[WAVE];
    __shared__ long long voff[WAVE];
    const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int kvh = head / (H / Hkv);
    const int pos = positions[t];
    const int lo = (window > 0) ? max(0, pos - window + 1) : 0;
    const int* table = block_table + (long long)req_of_token[t] * max_blocks;
    const T* qrow = q + ((long long)t * H + head) * hd;
    for (int j = lane; j < hd; j += WAVE) qs[j] = to_f32(qrow[j]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[MAX_PER_LANE];
#pragma unroll
    for (int i = 0; i < MAX_PER_LANE; ++i) acc[i] = 0.f;

    for (int t0 = (lo / WAVE) * WAVE; t0 <= pos; t0 += WAVE) {
        const int kt = t0 + lane;
        const bool valid = kt >= lo && kt <= pos;
        float s = -INFINITY;
        long long base = 0;
        if (valid) {
            const long long page = table[kt / page_size];
            const long long head_base = (page * Hkv + kvh) * page_size * (long long)hd;
            base = head_base + (kt % page_size);          // V: [hd][page_size], this key's column
            const T* krow = k_cache + head_base + (long long)(kt % page_size) * hd;
            float d = 0.f;
            for (int j = 0; j < hd; ++j) d = fmaf(qs[j], to_f32(krow[j]), d);
            s = d * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);          // 0 on the first tile (m = -inf)
        l = l * corr + wave_sum(p);
        m = m_new;
        __syncthreads();                             // previous tile's ps/voff fully consumed
        ps[lane] = p;
        voff[lane] = base;
        __syncthreads();
        const int n_keys = min(WAVE, pos - t0 + 1);
#pragma unroll
        for (int i = 0; i < MAX_PER_LANE; ++i) acc[i] *= corr;
        for (int jj = 0; jj < n_keys; ++jj) {
            const float pj = ps[jj];
            if (pj == 0.f) continue;                 // masked (below the window) or underflowed
            const T* vcol = v_cache + voff[jj];
#pragma unroll
            for (int i = 0; i < MAX_PER_LANE; ++i) {
                const int j = lane + i * WAVE;
                if (j < hd) acc[i] = fmaf(pj, to_f32(vcol[(long long)j * page_size]), acc[i]);
            }
        }
    }
    T* o = out + ((long long)t * H + head) * hd;
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < MAX_PER_LANE; ++i) {
        const int j = lane + i * WAVE;
        if (j < hd) o[j] = from_f32<T>(acc[i] * inv);
    }
}
}  // namespace

TUFF_EXPORT int tuff_attention_general(const void* q, const void* k_cache, const void* v_cache, void* out, int dt,
                                       const int* block_table, int max_blocks, const int* req_of_token,
                                       const int* positions, int n_tokens, int H, int Hkv, int hd, int page_size,
                                       int window, float scale, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (hd > MAX_PER_LANE * WAVE || Hkv <= 0 || H % Hkv != 0) return -2;
    dim3 grid(n_tokens, H), block(WAVE);
    if (dt == DT_F32)
        hipLaunchKernelGGL(attention_general_kernel<float>, grid, block, 0, stream, (const float*)q, (const float*)k_cache,
                           (const float*)v_cache, (float*)out, block_table, max_blocks, req_of_token, positions, H, Hkv, hd,
                           page_size, window, scale);
    else
        hipLaunchKernelGGL(attention_general_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)q, (const bf16_t*)k_cache,
                           (const bf16_t*)v_cache, (bf16_t*)out, block_table, max_blocks, req_of_token, positions, H, Hkv, hd,
                           page_size, window, scale);
    return launch_status();
}
