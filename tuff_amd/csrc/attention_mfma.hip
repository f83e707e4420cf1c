// Paged attention on the gfx950 matrix cores, bfloat16 cache, for prompt portions and decoded
// tokens alike.
//
// Work is cut the same way whatever the batch: the keys of a request are split into partitions
// of 256 positions (0..255, 256..511, ...), each of four units of 64.  A workgroup takes one
// partition, one kv head and one block of query columns (a column = one query head of one token;
// all columns of a block share the request and the kv head): one wave that walks the four units, or,
// where that would leave the chip idle, four waves with a unit each.  Either way a unit starts from
// a fresh state and the units' results (running maximum m, sum l, unnormalised output o, float32)
// are merged in ascending order through one chain of operations, so both give the same bits.  A
// second kernel merges a token's partitions in ascending order.  Since the columns of a matrix product do not influence each
// other, a token's result does not depend on how the sequence was cut into steps or on what
// else was in the batch.
//
// Inside a wave (S^T = K Q^T, O^T = V^T P^T, all with v_mfma_f32_16x16x32_bf16):
//  * 32 keys a step, in two products of 16.  A operand of S^T: K rows [key][hd], 16 bytes a lane;
//    B operand: Q [column][hd], loaded once.  Row m of product kb is key 8 (m/4) + 4 kb + m % 4.
//  * A result tile gives lane (column = l % 16, group g = l / 16) rows 4g..4g+3, so over both
//    products the lane holds the scores of keys 8g..8g+7 in order.  After masking, running max
//    and exp these eight values are, as they lie, the lane's part of the B operand P^T of the
//    second product (k = 8g + i), and the A operand V^T is one 16-byte load of eight consecutive
//    positions of a channel from the transposed V page.
//  * No LDS, no transposes, no barriers; K rows and V columns of the next step are loaded
//    while the current step computes, with streaming (non-temporal) loads: a step of single tokens
//    reads every key once.
//
// Cache layout: K [page][kv_head][offset][hd], V [page][kv_head][hd][offset]; the page size
// must be a multiple of 16 and the head size a multiple of 8 (the host falls back to the
// general kernel otherwise).
#include "common.h"
#include <math.h>
#include <mutex>

namespace {
constexpr int PART = 256;

__device__ __forceinline__ f32x4 mfma32(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// What the kernel does itself, for heads of 64 channels, when it is handed the projected rows
// [q heads | k heads | v heads] of a step of single tokens instead of finished queries: the per-head
// RMSNorm of q and k, the half-split rotation, and the write of the token's key and value into the
// cache (by the workgroup whose partition holds the token's position, before it reads its keys).
// The arithmetic is that of the kernel that does this for prompt portions (qkv_post64_kernel), sum
// for sum, so a key in the cache does not tell which of the two wrote it.
struct FusedQKV {
    const void* q_norm_w = nullptr;        // [64] each, float32 or bfloat16 (norm_dt); null: no norm
    const void* k_norm_w = nullptr;
    int norm_dt = DT_F32;
    float eps = 0.f;
    const float* inv_freq = nullptr;       // [32]
    const float* angles = nullptr;         // [n_angles][2][32]: cosines and sines of pos * inv_freq, or null
    int n_angles = 0;
    const int* slot_mapping = nullptr;     // [tokens]; null: the cache is only read
};

// cosine and sine of pos * inv_freq[j]: from the table where it reaches, else computed (the same bits)
__device__ __forceinline__ void angle(const FusedQKV& fq, int pos, int j, float& rc, float& rs) {
    if (pos < fq.n_angles) {
        rc = fq.angles[((long long)pos * 2) * 32 + j];
        rs = fq.angles[((long long)pos * 2 + 1) * 32 + j];
    } else {
        const float a = (float)pos * fq.inv_freq[j];
        rc = cosf(a);
        rs = sinf(a);
    }
}

__device__ __forceinline__ float norm_weight(const void* w, int dt, int i) {
    return dt == DT_F32 ? ((const float*)w)[i] : (float)((const bf16_t*)w)[i];
}

// One partial result (m, l, o) merged into a running one, element by element:
//   m' = max(m, mu);  l' = l e^(m - m') + lu e^(mu - m');  o' likewise.
// Both forms of the kernel (one wave or four a partition) merge a partition's four units of 64 keys
// through this, in ascending order, so they give the same bits.
__device__ __forceinline__ void merge_weights(float m, float mu, float& m_new, float& ca, float& cb) {
    m_new = fmaxf(m, mu);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    ca = __expf(m - m_safe);               // 0 while nothing was seen
    cb = __expf(mu - m_safe);
}

// a ca + b cb as one product and one fused multiply-add, spelled out: left to the compiler, two
// instantiations of the kernel may fuse the other product and differ in the last bit
__device__ __forceinline__ float merged(float a, float ca, float b, float cb) { return fmaf(b, cb, a * ca); }

constexpr int UNIT = 64;                   // keys a unit: two steps of 32
constexpr int UNITS = PART / UNIT;

// How many pages the partition that starts at key_begin (a multiple of PART) touches: one lane of the
// wave fetches each page's number.  A partition that starts inside a page (page sizes that do not divide
// PART) touches one page more than PART / page_size rounded up.
__host__ __device__ inline int partition_pages(int key_begin, int page_size) {
    return (key_begin + PART - 1) / page_size - key_begin / page_size + 1;
}

// NW: waves a workgroup (1: the wave walks the partition's four units; 4: a unit a wave, merged through LDS).
template <int HDP, int NB, int NW, bool FUSED, bool STREAM_V, bool STAGE_K = false>
__global__ __launch_bounds__(NW * WAVE) void attn_partition_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
    float* __restrict__ ws_o, float* __restrict__ ws_ml,
    const int* __restrict__ block_table, int max_blocks,
    const int2* __restrict__ blk, const int4* __restrict__ req_info,
    int H, int Hkv, int hd, int page_size, int window, float scale, int n_parts, FusedQKV fq, int kv_fast) {
    static_assert(NW == 1 || NW == UNITS, "one wave a partition or one a unit");
    static_assert(!FUSED || (HDP == 64 && NB == 1), "the fused form is for heads of 64 and one column block");
    constexpr int KC = HDP / 32;          // 32-wide chunks of the head dimension
    constexpr int DB = HDP / 16;          // 16-wide blocks of output channels
    // Workgroups that run side by side read neighbouring memory when the kv head is what changes fastest
    // from one to the next (a page holds its kv heads one after the other): that order for launches of
    // several rounds of waves, partitions first for the others.
    const int part = kv_fast ? blockIdx.x / Hkv : blockIdx.x, qb = blockIdx.y, kvh = kv_fast ? blockIdx.x % Hkv : blockIdx.z;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n16 = lane % 16, g = lane / 16;
    const int G = H / Hkv;
    // Every load that depends on another costs a trip to memory, so the chain is kept short:
    // block -> request record (start, length, first position: a portion's positions are
    // consecutive) -> the partition's page numbers, all at once -> keys and values.
    int r = qb, col0 = 0;                  // without a block list every request is one block
    if (blk) { const int2 b = blk[qb]; r = b.x; col0 = b.y; }
    const int4 info = req_info[r];         // (first token of the request in the step, tokens, first position, -)
    const int t0 = info.x, ncols = info.y * G, pos0 = info.z;
    const int* table = block_table + (long long)r * max_blocks;
    const int key_begin = part * PART;
    const int first_page = key_begin / page_size;
    int my_page = -1;                      // lane i: the page of the partition's i-th block of page_size keys
    if (lane < partition_pages(key_begin, page_size) && first_page + lane < max_blocks) my_page = table[first_page + lane];

    // the block's range of keys
    const int last_col = min(ncols, col0 + NB * 16) - 1;
    const int pos_max = pos0 + last_col / G;
    const int lo_min = window > 0 ? max(0, pos0 + col0 / G - window + 1) : 0;
    if (key_begin > pos_max || key_begin + PART <= lo_min) return;
    const int key_end = min(key_begin + PART, pos_max + 1);

    if constexpr (FUSED) {
        // the token's key and value go into the cache before anybody reads the partition that holds them
        if (fq.slot_mapping != nullptr && pos0 / PART == part) {
            if (wave == 0) {
                const long long slot = fq.slot_mapping[t0];
                if (slot >= 0) {
                    const long long page = slot / page_size, off = slot % page_size;
                    const int row_width = (H + 2 * Hkv) * 64;
                    const bf16_t* row = q + (long long)t0 * row_width;
                    // value: lane = channel, as projected
                    v_cache[((page * Hkv + kvh) * 64 + lane) * page_size + off] = row[(H + Hkv + kvh) * 64 + lane];
                    // key: sixteen lanes hold four channels each (the other lanes do the same work again)
                    const int l = lane % 16;
                    const bf16x4 raw = *(const bf16x4*)(row + (H + kvh) * 64 + 4 * l);
                    float v[4] = {(float)raw[0], (float)raw[1], (float)raw[2], (float)raw[3]};
                    float ss = v[0] * v[0];
                    ss = fmaf(v[1], v[1], ss);
                    ss = fmaf(v[2], v[2], ss);
                    ss = fmaf(v[3], v[3], ss);
                    ss += __shfl_xor(ss, 8, WAVE);
                    ss += __shfl_xor(ss, 4, WAVE);
                    ss += __shfl_xor(ss, 2, WAVE);
                    ss += __shfl_xor(ss, 1, WAVE);
                    if (fq.k_norm_w != nullptr) {
                        const float inv = 1.0f / sqrtf(ss / 64.0f + fq.eps);
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = v[e] * inv * norm_weight(fq.k_norm_w, fq.norm_dt, 4 * l + e);
                    }
                    const bool first = l < 8;
                    bf16x4 o4;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float rc, rs;
                        angle(fq, pos0, (4 * l + e) & 31, rc, rs);
                        const float other = __shfl_xor(v[e], 8, WAVE);
                        const float x0 = first ? v[e] : other, x1 = first ? other : v[e];
                        o4[e] = (bf16_t)(first ? (x0 * rc - x1 * rs) : (x0 * rs + x1 * rc));
                    }
                    if (lane < 16) *(bf16x4*)(k_cache + ((page * Hkv + kvh) * page_size + off) * 64 + 4 * l) = o4;
                }
            }
            __syncthreads();               // the stores have landed before a wave of this workgroup loads the keys
        }
    }

    // the unit under way, and the partition's result so far
    float m_run[NB], l_run[NB];
    f32x4 o[DB][NB];
    float m_acc[NB], l_acc[NB];
    f32x4 o_acc[DB][NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        m_acc[nb] = -INFINITY;
        l_acc[nb] = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db) o_acc[db][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // One step covers 32 keys, two halves of 16 that each lie in one page.  The two S^T products
    // of a step do not take the keys in order: row m of product kb is key 8 (m / 4) + 4 kb + m % 4
    // of the step, so that lane group g ends up with the scores of keys 8g .. 8g+7, which is what
    // the second product's operands hold for k = 8g + i.  A step's K rows and V columns are loaded
    // into registers a step ahead of their use (where the head size leaves room for it); large
    // tiles (head size x columns) load as they go.
    constexpr bool AHEAD = HDP * NB <= 256;
    // STAGE_K (heads of up to 64 channels): a step's keys are asked for as they lie in memory, 1 KB an instruction (the
    // 16 keys of a half are one run of 16 hd elements), and go through LDS into the order of the matrix operands.  Asked
    // for in that order at once, an instruction touches half of each of sixteen lines and every line is asked for twice:
    // with several rounds of waves on the chip the memory side is what bounds the kernel, and whole lines are 3 to 7 %
    // faster (16,384 workgroups; nothing at 6,144); with one round the trip through LDS only adds to each wave's chain
    // (3 to 7 % slower), so the launch chooses.
    static_assert(!STAGE_K || (HDP == 64 && HDP * NB <= 256 && NW == 1), "staged keys: heads of up to 64, one wave a partition");
    constexpr bool STAGE = STAGE_K;
    __shared__ __attribute__((aligned(16))) bf16_t k_stage[STAGE ? NW : 1][STAGE ? 32 * 64 : 8];
    // where the 16-byte piece `chunk` of key `key` of the step lies in the wave's 4 KB: rows of 128 bytes, the pieces of
    // a row exchanged so that the sixteen rows an operand read takes its pieces from fall into different banks
    auto stage_at = [&](int key, int chunk) { return key * 64 + ((chunk ^ (((key >> 1) & 1) | (((key >> 3) & 3) << 1))) * 8); };
    const int row_pieces = hd / 8;                                   // 16-byte pieces of a key
    int stage_to[2][2];                                              // where this lane's four pieces of a step go (-1: no piece)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int piece = 64 * i + lane;
            stage_to[h][i] = (STAGE && piece < 16 * row_pieces) ? stage_at(16 * h + piece / row_pieces, piece % row_pieces) : -1;
        }
    struct Tile {
        bf16x8 kf[2][AHEAD ? KC : 1];
        bf16x8 vx[AHEAD ? DB : 1];
        long long base[2];                 // per half: (page, kv head) start in both caches
        int off0[2];                       // per half: offset of its first key in the page
        bool live[2];                      // per half: holds keys some column may see
    };
    const int k_half = n16 / 8;                                    // half of this lane's K rows
    const int k_off = 8 * ((n16 / 4) % 2) + n16 % 4;               // + 4 kb: offset of the row's key in its half
    auto k_frag = [&](const Tile& t, int kb, int kc) {
        const int k = kc * 32 + g * 8;
        bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        // selects, not indexing by a lane-dependent value (that would put the arrays in scratch memory)
        const bool live = k_half ? t.live[1] : t.live[0];
        const long long base = k_half ? t.base[1] : t.base[0];
        const int off0 = k_half ? t.off0[1] : t.off0[0];
        if (!live || k >= hd) return z;
        return __builtin_nontemporal_load((const bf16x8*)(k_cache + base + (long long)(off0 + k_off + 4 * kb) * hd + k));
    };
    // A page's V^T rows are 2 * page_size bytes: with pages of 16 positions a step of 32 keys reads whole rows and
    // never comes back to them; with larger pages it reads a part of each row's cache lines and the steps after it
    // read the rest, so those loads are ordinary ones (a line asked for as streaming does not wait for them):
    // STREAM_V is page_size <= 16.
    auto v_frag = [&](const Tile& t, int db) {
        const int dim = db * 16 + n16;
        bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        const bool live = (g / 2) ? t.live[1] : t.live[0];
        const long long base = (g / 2) ? t.base[1] : t.base[0];
        const int off0 = (g / 2) ? t.off0[1] : t.off0[0];
        if (!live || dim >= hd) return z;
        const bf16x8* at = (const bf16x8*)(v_cache + base + (long long)dim * page_size + off0 + (g % 2) * 8);
        if constexpr (STREAM_V) return __builtin_nontemporal_load(at); else return *at;
    };
    auto load_tile = [&](int key0, Tile& t) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int hs = key0 + h * 16;
            t.live[h] = hs <= pos_max && hs + 15 >= lo_min;
            const long long page = t.live[h] ? __shfl(my_page, hs / page_size - first_page, WAVE) : 0;
            t.off0[h] = hs % page_size;
            t.base[h] = (page * Hkv + kvh) * (long long)page_size * hd;
        }
        if constexpr (STAGE) {
            // kf[h][i]: pieces 64 i + lane of half h, as they lie in memory
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int piece = 64 * i + lane;
                    bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
                    t.kf[h][i] = (t.live[h] && stage_to[h][i] >= 0)
                        ? __builtin_nontemporal_load((const bf16x8*)(k_cache + t.base[h] + (long long)t.off0[h] * hd + piece * 8)) : z;
                }
#pragma unroll
            for (int db = 0; db < DB; ++db) t.vx[db] = v_frag(t, db);
        } else if constexpr (AHEAD) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int kc = 0; kc < KC; ++kc) t.kf[kb][kc] = k_frag(t, kb, kc);
#pragma unroll
            for (int db = 0; db < DB; ++db) t.vx[db] = v_frag(t, db);
        }
    };
    // The first keys and values are asked for before the queries are prepared: they depend on the page
    // numbers alone, and the queries' loads (and, in the fused form, their norm and rotation) then run
    // while the keys are on their way.
    Tile ta, tb;
    const int key_first = NW == 1 ? key_begin : key_begin + wave * UNIT;
    if constexpr (AHEAD) {
        if (key_first < key_end) load_tile(key_first, ta);
        if (NW > 1 && key_first + 32 < key_end) load_tile(key_first + 32, tb);
    }

    // this lane's columns
    int pos_c[NB], lo_c[NB];
    long long qrow[NB];                    // row of the column in the work space; -1: no column
    bf16x8 qf[NB][KC];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int c = col0 + nb * 16 + n16;
        const bool valid = c < ncols;
        const int tok = t0 + (valid ? c / G : 0);
        const int head = kvh * G + (valid ? c % G : 0);
        pos_c[nb] = valid ? pos0 + c / G : -1;
        lo_c[nb] = (valid && window > 0) ? max(0, pos_c[nb] - window + 1) : 0;
        qrow[nb] = valid ? (long long)tok * H + head : -1;
        if constexpr (FUSED) {
            // channels 8g .. 8g+7 and 32 + 8g .. 32 + 8g+7 of the head: partners of the rotation sit in one lane
            const bf16_t* src = q + (long long)tok * ((H + 2 * Hkv) * 64) + head * 64 + g * 8;
            bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
            const bf16x8 r0 = valid ? *(const bf16x8*)src : z, r1 = valid ? *(const bf16x8*)(src + 32) : z;
            float v0[8], v1[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) { v0[e] = (float)r0[e]; v1[e] = (float)r1[e]; }
            // sums of squares of four channels each, then the butterfly of sixteen such sums in the order
            // of the kernel for portions (partners 32, 16, 8 and 4 channels away)
            float p[2][2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float a = v0[4 * h] * v0[4 * h], b = v1[4 * h] * v1[4 * h];
#pragma unroll
                for (int e = 1; e < 4; ++e) { a = fmaf(v0[4 * h + e], v0[4 * h + e], a); b = fmaf(v1[4 * h + e], v1[4 * h + e], b); }
                p[0][h] = a; p[1][h] = b;
            }
            float s0 = p[0][0] + p[1][0], s1 = p[0][1] + p[1][1];
            s0 += __shfl_xor(s0, 32, WAVE); s1 += __shfl_xor(s1, 32, WAVE);
            s0 += __shfl_xor(s0, 16, WAVE); s1 += __shfl_xor(s1, 16, WAVE);
            const float ss = s0 + s1;
            if (fq.q_norm_w != nullptr) {
                const float inv = 1.0f / sqrtf(ss / 64.0f + fq.eps);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    v0[e] = v0[e] * inv * norm_weight(fq.q_norm_w, fq.norm_dt, g * 8 + e);
                    v1[e] = v1[e] * inv * norm_weight(fq.q_norm_w, fq.norm_dt, 32 + g * 8 + e);
                }
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float rc, rs;
                angle(fq, max(pos_c[nb], 0), g * 8 + e, rc, rs);
                const float x0 = v0[e], x1 = v1[e];
                qf[nb][0][e] = (bf16_t)(x0 * rc - x1 * rs);
                qf[nb][1][e] = (bf16_t)(x0 * rs + x1 * rc);
            }
        } else {
#pragma unroll
            for (int kc = 0; kc < KC; ++kc) {
                const int k = kc * 32 + g * 8;
                bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
                qf[nb][kc] = (valid && k < hd) ? *(const bf16x8*)(q + qrow[nb] * hd + k) : z;
            }
        }
    }

    auto compute = [&](int key0, const Tile& t) {
        // ---- S^T = K Q^T, twice 16 keys
        f32x4 s[2][NB];
        bf16_t* stage = k_stage[STAGE ? wave : 0];
        if constexpr (STAGE) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    if (stage_to[h][i] >= 0) *(bf16x8*)(stage + stage_to[h][i]) = t.kf[h][i];
                }
            __builtin_amdgcn_wave_barrier();       // the wave's LDS accesses run in the order of the program
        }
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) s[kb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kc = 0; kc < KC; ++kc) {
                bf16x8 kf;
                if constexpr (STAGE) {
                    bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
                    const int chunk = kc * 4 + g;
                    kf = chunk < row_pieces ? *(const bf16x8*)(stage + stage_at(8 * (n16 / 4) + 4 * kb + n16 % 4, chunk)) : z;
                } else if constexpr (AHEAD) kf = t.kf[kb][kc]; else kf = k_frag(t, kb, kc);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) s[kb][nb] = mfma32(kf, qf[nb][kc], s[kb][nb]);
            }
        }
        // ---- mask, running maximum, exp; P^T stays in registers as the next B operand
        const bool my_live = (g / 2) ? t.live[1] : t.live[0];   // this lane's eight keys lie in half g / 2
        bf16x8 pf[NB];
        float corr[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            float v[8];
            float mx = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int key = key0 + 8 * g + 4 * kb + e;
                    const bool ok = my_live && key <= pos_c[nb] && key >= lo_c[nb];
                    const float x = ok ? s[kb][nb][e] * scale : -INFINITY;
                    v[kb * 4 + e] = x;
                    mx = fmaxf(mx, x);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
            const float m_new = fmaxf(m_run[nb], mx);
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            corr[nb] = __expf(m_run[nb] - m_safe);          // 0 while nothing was seen yet
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float p = __expf(v[i] - m_safe);
                sum += p;
                pf[nb][i] = (bf16_t)p;
            }
            l_run[nb] = fmaf(l_run[nb], corr[nb], sum);
            m_run[nb] = m_new;
        }
        // ---- O^T = O^T * corr + V^T P^T
        const bool tail = key0 + 31 > pos_max;             // keys beyond pos_max were never written
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            bf16x8 vf;
            if constexpr (AHEAD) vf = t.vx[db]; else vf = v_frag(t, db);
            if (tail) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (key0 + 8 * g + i > pos_max) vf[i] = (bf16_t)0.f;
            }
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                f32x4 acc = o[db][nb];
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] *= corr[nb];
                o[db][nb] = mfma32(vf, pf[nb], acc);
            }
        }
    };
    auto begin_unit = [&]() {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            m_run[nb] = -INFINITY;
            l_run[nb] = 0.f;
#pragma unroll
            for (int db = 0; db < DB; ++db) o[db][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    };
    // the unit's sum of a column is spread over the four lane groups until here
    auto unit_sums = [&]() {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            l_run[nb] += __shfl_xor(l_run[nb], 16, WAVE);
            l_run[nb] += __shfl_xor(l_run[nb], 32, WAVE);
        }
    };

    if constexpr (NW == 1) {
        // units in ascending order, each from a fresh state, merged into the partition's result as they end
        for (int key0 = key_begin; key0 < key_end; key0 += UNIT) {
            begin_unit();
            if constexpr (AHEAD) {
                const bool more = key0 + 32 < key_end;
                if (more) load_tile(key0 + 32, tb);
                compute(key0, ta);
                if (more) {
                    if (key0 + UNIT < key_end) load_tile(key0 + UNIT, ta);
                    compute(key0 + 32, tb);
                }
            } else {
                for (int k2 = key0; k2 < min(key0 + UNIT, key_end); k2 += 32) {
                    load_tile(k2, ta);
                    compute(k2, ta);
                }
            }
            unit_sums();
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                float m_new, ca, cb;
                merge_weights(m_acc[nb], m_run[nb], m_new, ca, cb);
                l_acc[nb] = merged(l_acc[nb], ca, l_run[nb], cb);
                m_acc[nb] = m_new;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int e = 0; e < 4; ++e) o_acc[db][nb][e] = merged(o_acc[db][nb][e], ca, o[db][nb][e], cb);
            }
        }
    } else {
        // a unit a wave; the waves' results go through LDS and every wave merges a share of the elements,
        // each element through the same chain as above
        __shared__ float u_ml[UNITS][NB][16][2];
        __shared__ __attribute__((aligned(16))) float u_o[UNITS][NB][DB][WAVE][4];
        const int key0 = key_begin + wave * UNIT;
        begin_unit();
        if (key0 < key_end) {
            if constexpr (AHEAD) {
                compute(key0, ta);
                if (key0 + 32 < key_end) compute(key0 + 32, tb);
            } else {
                for (int k2 = key0; k2 < min(key0 + UNIT, key_end); k2 += 32) {
                    load_tile(k2, ta);
                    compute(k2, ta);
                }
            }
        }
        unit_sums();
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            if (g == 0) { u_ml[wave][nb][n16][0] = m_run[nb]; u_ml[wave][nb][n16][1] = l_run[nb]; }
#pragma unroll
            for (int db = 0; db < DB; ++db) *(f32x4*)u_o[wave][nb][db][lane] = o[db][nb];
        }
        __syncthreads();
        // wave w finishes the channel blocks db = w, w + 4, ... of every column block
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int u = 0; u < UNITS; ++u) {
                const float mu = u_ml[u][nb][n16][0], lu = u_ml[u][nb][n16][1];
                float m_new, ca, cb;
                merge_weights(m_acc[nb], mu, m_new, ca, cb);
                l_acc[nb] = merged(l_acc[nb], ca, lu, cb);
                m_acc[nb] = m_new;
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    if (db % NW != wave) continue;
                    const f32x4 ou = *(const f32x4*)u_o[u][nb][db][lane];
#pragma unroll
                    for (int e = 0; e < 4; ++e) o_acc[db][nb][e] = merged(o_acc[db][nb][e], ca, ou[e], cb);
                }
            }
        }
    }

    // ---- the partition's result per column
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        if (qrow[nb] < 0) continue;
        const long long slot = qrow[nb] * n_parts + part;
        if (g == 0 && wave == 0) { ws_ml[slot * 2] = m_acc[nb]; ws_ml[slot * 2 + 1] = l_acc[nb]; }
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            if (NW > 1 && db % NW != wave) continue;
            const int dim = db * 16 + 4 * g;
            if (dim < hd) *(f32x4*)(ws_o + slot * hd + dim) = o_acc[db][nb];
        }
    }
}

// Merges the partitions of one (token, head) and writes the bfloat16 row:
//   M = max_p m_p;  w_p = exp(m_p - M);  out = (sum_p w_p o_p) / (sum_p w_p l_p),
// both sums over p in ascending order, so the result depends on the token's position only.
constexpr int COMBINE_MAX_PARTS = 2048;

// Up to 64 partitions: lane p keeps (m_p, l_p) in registers, weights travel by shuffle; no LDS.
// Same arithmetic as the general kernel below.  PER: channels a lane (head size / 64, rounded up);
// the partial outputs of BATCH partitions are asked for at once, so that a context of 8192 positions
// with heads of 64 is one trip to memory.
template <int PER, int BATCH>
__global__ __launch_bounds__(WAVE) void attn_combine64_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
                                                              bf16_t* __restrict__ out, const int* __restrict__ positions,
                                                              int H, int hd, int window, int n_parts, int part_keys) {
    const long long row = blockIdx.x;                      // token * H + head
    const int lane = threadIdx.x;
    float m_l = -INFINITY, l_l = 0.f;
    if (lane < n_parts) {                                  // read before the position is known: rows exist for all partitions
        const float* ml = ws_ml + (row * n_parts + lane) * 2;
        m_l = ml[0];
        l_l = ml[1];
    }
    const int pos = positions[row / H];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int p_lo = lo / part_keys, p_hi = pos / part_keys;
    const bool valid = lane >= p_lo && lane <= p_hi && l_l > 0.f;
    const float M = wave_max(valid ? m_l : -INFINITY);
    const float w_l = valid ? __expf(m_l - M) : 0.f;
    const float wl_l = w_l * (valid ? l_l : 0.f);
    const float* o = ws_o + row * n_parts * hd;
    float acc[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) acc[j] = 0.f;
    float L = 0.f;                                         // both sums run over p in ascending order
    // The loads below do not wait for the position: rows of partitions the token does not have
    // exist too (unwritten); their weight is zero and they are skipped by a select, not a product.
    for (int i0 = 0; i0 < n_parts; i0 += BATCH) {
        float ov[BATCH][PER];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                const int d = lane + j * WAVE;
                ov[u][j] = (i0 + u < n_parts && d < hd) ? o[(long long)(i0 + u) * hd + d] : 0.f;
            }
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const float w = __shfl(w_l, i0 + u, WAVE);
            L += __shfl(wl_l, i0 + u, WAVE);
            if (w > 0.f) {
#pragma unroll
                for (int j = 0; j < PER; ++j) acc[j] = fmaf(w, ov[u][j], acc[j]);
            }
        }
    }
    const float inv = 1.0f / L;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int d = lane + j * WAVE;
        if (d < hd) out[row * hd + d] = (bf16_t)(acc[j] * inv);
    }
}

// More than 64 partitions (contexts beyond 16,384 keys): the partitions are taken in groups of 64 by
// their absolute numbers (0..63, 64..127, ...); a wave sums a group in ascending order as above, the
// waves of the workgroup take the groups in turn, and the groups' sums are added in ascending order.
// The grouping is by absolute partition number, so the result still depends on the token's position only.
constexpr int COMBINE_WAVES = 8;
constexpr int COMBINE_GROUP = 64;
constexpr int COMBINE_MAX_GROUPS = COMBINE_MAX_PARTS / COMBINE_GROUP;

__global__ __launch_bounds__(COMBINE_WAVES * WAVE) void attn_combine_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
                                                                            bf16_t* __restrict__ out, const int* __restrict__ positions,
                                                                            int H, int hd, int window, int n_parts, int part_keys) {
    __shared__ float wts[COMBINE_MAX_PARTS], wls[COMBINE_MAX_PARTS];
    __shared__ float grp_acc[COMBINE_MAX_GROUPS][256], grp_l[COMBINE_MAX_GROUPS];
    __shared__ float red[COMBINE_WAVES];
    const long long row = blockIdx.x;                      // token * H + head
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int pos = positions[row / H];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int p_lo = lo / part_keys, p_hi = pos / part_keys;          // the token's partitions, absolute numbers
    const float* ml = ws_ml + row * n_parts * 2;
    float M = -INFINITY;
    for (int p = p_lo + tid; p <= p_hi; p += COMBINE_WAVES * WAVE) M = fmaxf(M, ml[p * 2 + 1] > 0.f ? ml[p * 2] : -INFINITY);
    M = wave_max(M);
    if (lane == 0) red[wave] = M;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < COMBINE_WAVES; ++w) M = fmaxf(M, red[w]);
    for (int p = p_lo + tid; p <= p_hi; p += COMBINE_WAVES * WAVE) {
        const float l = ml[p * 2 + 1];
        const float w = l > 0.f ? __expf(ml[p * 2] - M) : 0.f;
        wts[p] = w;
        wls[p] = w * (l > 0.f ? l : 0.f);
    }
    __syncthreads();
    const int g_lo = p_lo / COMBINE_GROUP, g_hi = p_hi / COMBINE_GROUP;
    const int per = (hd + WAVE - 1) / WAVE;                // channels a lane
    const float* o = ws_o + row * n_parts * hd;
    for (int grp = g_lo + wave; grp <= g_hi; grp += COMBINE_WAVES) {
        const int a = max(p_lo, grp * COMBINE_GROUP), b = min(p_hi, grp * COMBINE_GROUP + COMBINE_GROUP - 1);
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        float L = 0.f;
        // the partial outputs of sixteen partitions are asked for together; the sums run in ascending order
        for (int i0 = a; i0 <= b; i0 += 16) {
            float ov[16][4];
#pragma unroll
            for (int u = 0; u < 16; ++u)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int d = lane + j * WAVE;
                    ov[u][j] = (j < per && i0 + u <= b && d < hd) ? o[(long long)(i0 + u) * hd + d] : 0.f;
                }
#pragma unroll
            for (int u = 0; u < 16; ++u)
                if (i0 + u <= b) {
                    const float w = wts[i0 + u];
                    L += wls[i0 + u];
                    if (w > 0.f) {                         // a partition without weight may hold anything
#pragma unroll
                        for (int j = 0; j < 4; ++j) acc[j] = fmaf(w, ov[u][j], acc[j]);
                    }
                }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = lane + j * WAVE;
            if (d < hd) grp_acc[grp][d] = acc[j];
        }
        if (lane == 0) grp_l[grp] = L;
    }
    __syncthreads();
    if (wave == 0) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        float L = 0.f;
        for (int grp = g_lo; grp <= g_hi; ++grp) {
            L += grp_l[grp];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int d = lane + j * WAVE;
                if (d < hd) acc[j] += grp_acc[grp][d];
            }
        }
        const float inv = 1.0f / L;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = lane + j * WAVE;
            if (d < hd) out[row * hd + d] = (bf16_t)(acc[j] * inv);
        }
    }
}

// Workgroups of four waves where one wave a partition would leave most of the chip idle (a step of a
// few single tokens); the result is the same bit for bit.
int few_waves = 2048;
// From how many workgroups on the kv head is the fastest-changing part of a workgroup's number: with
// several rounds of waves on the chip (it holds about 3,000 of them) that is 7 to 11 % faster, with one
// round it is not.
int kv_fast_waves = 6144;
// From how many workgroups on the keys of heads of up to 64 channels go through LDS (STAGE_K of the kernel).
int stage_k_waves = 8192;

template <int HDP, int NB, bool FUSED, bool STREAM_V = true>
void launch_partition(dim3 grid, hipStream_t stream, const bf16_t* q, bf16_t* kc, bf16_t* vc, float* ws_o,
                      float* ws_ml, const int* bt, int max_blocks, const int2* blk, const int4* req_info,
                      int H, int Hkv, int hd, int ps, int window, float scale, int n_parts, const FusedQKV& fq) {
    if constexpr (STREAM_V) {
        if (ps > 16) {
            launch_partition<HDP, NB, FUSED, false>(grid, stream, q, kc, vc, ws_o, ws_ml, bt, max_blocks, blk, req_info, H, Hkv, hd,
                                                    ps, window, scale, n_parts, fq);
            return;
        }
    }
    const long long waves = (long long)grid.x * grid.y * grid.z;
    const int kv_fast = waves >= kv_fast_waves ? 1 : 0;
    if (kv_fast) grid = dim3(grid.x * grid.z, grid.y, 1);
    if constexpr (HDP * NB <= 128) {
        // the fused form prepares its queries in every wave: four waves pay for that four times
        if (waves < (FUSED ? few_waves / 2 : few_waves)) {
            hipLaunchKernelGGL((attn_partition_kernel<HDP, NB, UNITS, FUSED, STREAM_V>), grid, dim3(UNITS * WAVE), 0, stream, q, kc, vc, ws_o,
                               ws_ml, bt, max_blocks, blk, req_info, H, Hkv, hd, ps, window, scale, n_parts, fq, kv_fast);
            return;
        }
    }
    if constexpr (HDP == 64 && HDP * NB <= 256) {
        if (waves >= stage_k_waves) {
            hipLaunchKernelGGL((attn_partition_kernel<HDP, NB, 1, FUSED, STREAM_V, true>), grid, dim3(WAVE), 0, stream, q, kc, vc, ws_o,
                               ws_ml, bt, max_blocks, blk, req_info, H, Hkv, hd, ps, window, scale, n_parts, fq, kv_fast);
            return;
        }
    }
    hipLaunchKernelGGL((attn_partition_kernel<HDP, NB, 1, FUSED, STREAM_V>), grid, dim3(WAVE), 0, stream, q, kc, vc, ws_o, ws_ml, bt,
                       max_blocks, blk, req_info, H, Hkv, hd, ps, window, scale, n_parts, fq, kv_fast);
}
}  // namespace

// Merges, for every (token, head) of n_tokens tokens, the partial results of its partitions of
// part_keys keys each.
static int launch_merge(const float* ws_o, const float* ws_ml, bf16_t* out, const int* positions, int n_tokens, int H, int hd,
                 int window, int n_parts, int part_keys, hipStream_t stream) {
    const dim3 grid((unsigned)((long long)n_tokens * H));
    if (n_parts <= WAVE) {
#define COMBINE(PER, BATCH) hipLaunchKernelGGL((attn_combine64_kernel<PER, BATCH>), grid, dim3(WAVE), 0, stream, ws_o, ws_ml, out, \
                                               positions, H, hd, window, n_parts, part_keys)
        if (hd <= 64) { if (n_parts <= 8) COMBINE(1, 8); else if (n_parts <= 16) COMBINE(1, 16); else COMBINE(1, 32); }
        else if (hd <= 128) { if (n_parts <= 8) COMBINE(2, 8); else COMBINE(2, 16); }
        else COMBINE(4, 8);
#undef COMBINE
    } else {
        hipLaunchKernelGGL(attn_combine_kernel, grid, dim3(COMBINE_WAVES * WAVE), 0, stream, ws_o, ws_ml, out, positions, H, hd,
                           window, n_parts, part_keys);
    }
    return launch_status();
}

// Query blocks are listed by the host: block b holds the columns blk[b].y .. +16*nb-1 of request
// blk[b].x (a request's columns are numbered (token - its first token) * G + head within the kv
// group); blk == null: block b is request b from column 0 (every request fits one block).
// req_info [R]: (first token of the request in the step, its tokens, position of the first, -).
// positions [n_tokens]: every token's position (read by the merge).
// ws_o: float32 [n_tokens * H * n_parts * hd], ws_ml: float32 [n_tokens * H * n_parts * 2].
// n_parts >= ceil((largest position + 1) / 256).  nb: 1, 2 or 4 column blocks a wave.
static int launch_attention(const void* q, const void* k_cache, const void* v_cache, void* out,
                            float* ws_o, float* ws_ml, const int* block_table, int max_blocks,
                            const int* blk, int n_qblocks, int nb, const int* req_info, const int* positions,
                            int n_tokens, int H, int Hkv, int hd, int page_size, int window, float scale,
                            int n_parts, hipStream_t stream) {
    if (n_tokens <= 0 || n_qblocks <= 0) return 0;
    if (hd > 256 || hd % 8 != 0 || page_size % 16 != 0 || Hkv <= 0 || H % Hkv != 0 || n_parts < 1) return -2;
    if (Hkv > 65535 || n_qblocks > 65535 || n_parts > COMBINE_MAX_PARTS) return -2;
    const bf16_t* Q = (const bf16_t*)q;
    bf16_t* K = (bf16_t*)k_cache;                                        // read only without the fused form
    bf16_t* V = (bf16_t*)v_cache;
    dim3 grid(n_parts, n_qblocks, Hkv);
#define GO(HDP, NB) launch_partition<HDP, NB, false>(grid, stream, Q, K, V, ws_o, ws_ml, block_table, max_blocks, (const int2*)blk, \
                                                     (const int4*)req_info, H, Hkv, hd, page_size, window, scale, n_parts, FusedQKV())
#define BY_NB(HDP) do { if (nb == 1) GO(HDP, 1); else if (nb == 2) GO(HDP, 2); else if (nb == 4) GO(HDP, 4); else return -2; } while (0)
    if (hd <= 32) BY_NB(32);
    else if (hd <= 64) BY_NB(64);
    else if (hd <= 96) BY_NB(96);
    else if (hd <= 128) BY_NB(128);
    else { if (nb == 1) GO(256, 1); else if (nb == 2) GO(256, 2); else return -2; }
#undef BY_NB
#undef GO
    int rc = launch_status();
    if (rc) return rc;
    return launch_merge((const float*)ws_o, (const float*)ws_ml, (bf16_t*)out, positions, n_tokens, H, hd, window, n_parts, PART,
                        stream);
}

// The number of lanes of a wave that fetch page numbers for partition `part` with pages of page_size
// positions (what the kernel computes; host arithmetic, for checks).
TUFF_EXPORT int tuff_attention_partition_pages(int part, int page_size) {
    if (part < 0 || page_size <= 0 || (long long)part * PART + PART > 0x7fffffffll) return -2;
    return partition_pages(part * PART, page_size);
}

// Below how many workgroups a step's partitions get four waves each (0: never).  For measurements and
// tests; the result of the attention does not depend on it.  Returns the value before.
TUFF_EXPORT int tuff_attention_few_waves(int n) {
    const int old = few_waves;
    if (n >= 0) few_waves = n;
    return old;
}

// From how many workgroups on the kv head changes fastest in the order of the workgroups.  For
// measurements and tests; the result does not depend on it.  Returns the value before.
// From how many workgroups on keys are asked for in whole lines and go through LDS.  For measurements and tests; the
// result does not depend on it.  Returns the value before.
TUFF_EXPORT int tuff_attention_stage_k_waves(int n) {
    const int old = stage_k_waves;
    if (n >= 0) stage_k_waves = n;
    return old;
}

TUFF_EXPORT int tuff_attention_kv_fast_waves(int n) {
    const int old = kv_fast_waves;
    if (n >= 0) kv_fast_waves = n;
    return old;
}

TUFF_EXPORT int tuff_attention_mfma(const void* q, const void* k_cache, const void* v_cache, void* out,
                                    float* ws_o, float* ws_ml, const int* block_table, int max_blocks,
                                    const int* blk, int n_qblocks, int nb, const int* req_info, const int* positions,
                                    int n_tokens, int H, int Hkv, int hd, int page_size, int window, float scale,
                                    int n_parts, hipStream_t stream) {
    return launch_attention(q, k_cache, v_cache, out, ws_o, ws_ml, block_table, max_blocks, blk, n_qblocks, nb, req_info,
                            positions, n_tokens, H, Hkv, hd, page_size, window, scale, n_parts, stream);
}

// A step of single tokens (request r's token is row r) over heads of 64 channels, from the projected
// rows qkv [n_tokens, (H + 2 Hkv) * 64]: per-head RMSNorm of q and k (weights [64] of type norm_dt, or
// null), half-split rotation over the whole head by inv_freq [32] (angles [n_angles][2][32]: the
// cosines and sines of the first n_angles positions as tuff_rope_table makes them, or null), the token's key and value written
// to the cache at slot_mapping[r] (null: the cache is only read), attention, merge.  The query heads
// of a kv head must fit one block of sixteen columns (H / Hkv <= 16).
TUFF_EXPORT int tuff_attention_decode_fused(const void* qkv, void* k_cache, void* v_cache, void* out,
                                            float* ws_o, float* ws_ml, const int* block_table, int max_blocks,
                                            const int* req_info, const int* positions, const int* slot_mapping,
                                            const void* q_norm_w, const void* k_norm_w, int norm_dt, float eps,
                                            const float* inv_freq, const float* angles, int n_angles,
                                            int n_tokens, int H, int Hkv, int page_size,
                                            int window, float scale, int n_parts, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (page_size % 16 != 0 || Hkv <= 0 || H % Hkv != 0 || H / Hkv > 16 || n_parts < 1 || !inv_freq) return -2;
    if ((q_norm_w == nullptr) != (k_norm_w == nullptr)) return -2;
    if (Hkv > 65535 || n_tokens > 65535 || n_parts > COMBINE_MAX_PARTS) return -2;
    FusedQKV fq;
    fq.q_norm_w = q_norm_w; fq.k_norm_w = k_norm_w; fq.norm_dt = norm_dt; fq.eps = eps;
    fq.inv_freq = inv_freq; fq.slot_mapping = slot_mapping;
    fq.angles = angles; fq.n_angles = angles ? n_angles : 0;
    launch_partition<64, 1, true>(dim3(n_parts, n_tokens, Hkv), stream, (const bf16_t*)qkv, (bf16_t*)k_cache, (bf16_t*)v_cache,
                                  ws_o, ws_ml, block_table, max_blocks, nullptr, (const int4*)req_info, H, Hkv, 64, page_size,
                                  window, scale, n_parts, fq);
    int rc = launch_status();
    if (rc) return rc;
    return launch_merge((const float*)ws_o, (const float*)ws_ml, (bf16_t*)out, positions, n_tokens, H, 64, window, n_parts, PART,
                        stream);
}

// The merge alone, for partial results that another kernel left in the same layout (ws_o
// [tokens * H * n_parts * hd], ws_ml [tokens * H * n_parts * 2] = (reference exponent, sum); partition
// p of a row holds the keys p * part_keys .. (p + 1) * part_keys - 1).
TUFF_EXPORT int tuff_attention_merge(const float* ws_o, const float* ws_ml, void* out, const int* positions, int n_tokens,
                                     int H, int hd, int window, int n_parts, int part_keys, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (hd > 256 || n_parts < 1 || n_parts > COMBINE_MAX_PARTS || part_keys < 1) return -2;
    return launch_merge(ws_o, ws_ml, (bf16_t*)out, positions, n_tokens, H, hd, window, n_parts, part_keys, stream);
}

// ------------------------------------------------- the same attention without an allocation
// tuff_attention_mfma_static: tuff_attention_mfma with the partitions' partial results kept in an
// array of this library instead of a work space the caller brings, for callers that cannot
// allocate (a HIP graph under capture, a serving loop that must not call the allocator).  It calls
// no hipMalloc, hipFree or allocating library routine.
//
// The array is STATIC_SCRATCH_FLOATS floats (16 MiB) of device memory on every GPU the library is
// loaded on, held until the process ends.  A call needs n_tokens * H * n_parts * (hd + 2) floats
// (rounded up to 64 for the first of its two parts) and is refused with TUFF_STATIC_TOO_LARGE
// beyond that.  All calls on one GPU share that GPU's array: it keeps the last call's contents
// (nothing has to start at zero: a row of a partition that a token does not have is never used),
// and two calls that overlap on one GPU, on different streams or from different threads, race.
//
// In host code the array's name stands for the symbol, not for device memory; the address on the
// current device comes from hipGetSymbolAddress, once per device, and only that pointer is handed
// to the kernels.
constexpr long long STATIC_SCRATCH_FLOATS = 4ll << 20;
constexpr int STATIC_MAX_DEVICES = 64;
enum : int { TUFF_STATIC_TOO_LARGE = -7, TUFF_STATIC_NO_DEVICE = -8 };

static __device__ __align__(256) float static_scratch[STATIC_SCRATCH_FLOATS];
static float* static_scratch_ptr[STATIC_MAX_DEVICES];      // per device; written once, under the lock

static std::mutex static_scratch_lock;

// The array's address on the current device; looked up at the first call on that device.
static int static_scratch_of_current_device(float** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) return TUFF_STATIC_NO_DEVICE;
    std::lock_guard<std::mutex> guard(static_scratch_lock);
    if (!static_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return TUFF_STATIC_NO_DEVICE;
        static_scratch_ptr[dev] = (float*)p;
    }
    *ptr = static_scratch_ptr[dev];
    return 0;
}

// Looks the array up on the current device, so that the first attention call there does nothing
// but launch.  Returns 0, or a HIP error code.
TUFF_EXPORT int tuff_attention_static_setup(void) {
    float* p = nullptr;
    return static_scratch_of_current_device(&p);
}

// Floats of the static array a call of these sizes needs, and (*capacity) how many there are.
TUFF_EXPORT long long tuff_attention_static_floats(int n_tokens, int H, int hd, int n_parts, long long* capacity) {
    if (capacity) *capacity = STATIC_SCRATCH_FLOATS;
    const long long rows = (long long)n_tokens * H * n_parts;
    return (rows * hd + 63) / 64 * 64 + rows * 2;
}

TUFF_EXPORT int tuff_attention_mfma_static(const void* q, const void* k_cache, const void* v_cache, void* out,
                                           const int* block_table, int max_blocks,
                                           const int* blk, int n_qblocks, int nb, const int* req_info, const int* positions,
                                           int n_tokens, int H, int Hkv, int hd, int page_size, int window, float scale,
                                           int n_parts, hipStream_t stream) {
    if (n_tokens <= 0 || n_qblocks <= 0) return 0;
    if (H <= 0 || hd <= 0 || n_parts < 1) return -2;
    if (tuff_attention_static_floats(n_tokens, H, hd, n_parts, nullptr) > STATIC_SCRATCH_FLOATS) return TUFF_STATIC_TOO_LARGE;
    float* base = nullptr;
    const int rc = static_scratch_of_current_device(&base);
    if (rc) return rc;
    const long long rows = (long long)n_tokens * H * n_parts;
    float* ws_o = base;
    float* ws_ml = base + (rows * hd + 63) / 64 * 64;
    return launch_attention(q, k_cache, v_cache, out, ws_o, ws_ml, block_table, max_blocks, blk, n_qblocks, nb, req_info,
                            positions, n_tokens, H, Hkv, hd, page_size, window, scale, n_parts, stream);
}
