// Paged attention for steps that carry prompt portions: bfloat16 cache, matrix cores, keys and
// values shared by a workgroup through LDS.
//
// A workgroup of four waves takes one kv head and one block of 64 * NBW query columns of one
// request (a column = one query head of one token; NBW * 16 columns a wave) and walks over all
// keys these columns may see, 64 at a time, from key 0 (or the first 64 the window still
// reaches).  The K rows and V columns of a step are copied from the pages into LDS once, by all
// threads, one step ahead of their use; every wave reads its MFMA operands from there.  Each
// column carries a running maximum, sum and output (online softmax) and is written normalised at
// the end: no work space and no second kernel.
//
// A column's arithmetic depends only on its own position: steps start at multiples of 64, and
// the columns of a matrix product do not influence each other.  So a token's result does not
// depend on how the prompt was cut into portions or on what else is in the batch.
//
// Products (v_mfma_f32_16x16x32_bf16), per half step of 32 keys, as in the decode kernel:
// S^T = K Q^T in two products of 16 keys whose rows are ordered so that lane group g ends up with
// the scores of keys 8g..8g+7; after mask, maximum and exp these are, as they lie, the lane's
// part of P^T for O^T += V^T P^T.
//
// Cache layout: K [page][kv_head][offset][hd], V [page][kv_head][hd][offset]; page size a
// multiple of 16, head size a multiple of 8.
#include "common.h"
#include <math.h>

namespace {
constexpr int STEP = 64;            // keys a step
constexpr int NT = 256;             // threads a workgroup
constexpr int VROW = STEP + 8;      // bf16 a row of V^T in LDS: 64 keys and 16 bytes that keep rows off each other's banks

__device__ __forceinline__ f32x4 mfma32(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// LDS row of a key of a step.  Product kb of half `sub` takes as row m the key
// 32 sub + 16 (m / 8) + 8 ((m / 4) % 2) + 4 kb + m % 4; its sixteen rows lie next to each other.
__device__ __forceinline__ int k_row_of_key(int key) {
    const int sub = key / 32, h = (key / 16) % 2, q = (key / 8) % 2, kb = (key / 4) % 2, m = key % 4;
    return sub * 32 + kb * 16 + h * 8 + q * 4 + m;
}

template <int HDP, int NBW>
__global__ __launch_bounds__(NT) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int* __restrict__ block_table, int max_blocks,
    const int2* __restrict__ blk, const int4* __restrict__ req_info,
    int H, int Hkv, int hd, int page_size, int window, float scale_log2e) {
    constexpr int KC = HDP / 32;          // 32-wide chunks of the head dimension
    constexpr int DB = HDP / 16;          // 16-wide blocks of output channels
    constexpr int HC = HDP / 8;           // 16-byte chunks of a K row
    constexpr int KROW = HDP + 8;         // bf16 a K row in LDS (padded like V^T rows)
    constexpr int KBUF = STEP * KROW, VBUF = HDP * VROW;
    constexpr int KPT = STEP * HC / NT;   // 16-byte pieces of K a thread copies a step
    constexpr int VPT = HDP * 8 / NT;     // and of V^T
    constexpr int CB = 4 * NBW * 16;      // columns of a workgroup
    extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
    bf16_t* Ks = lds;                     // [2][KBUF]
    bf16_t* Vs = lds + 2 * KBUF;          // [2][VBUF]

    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE, n16 = lane % 16, g = lane / 16;
    const int qb = gridDim.x - 1 - blockIdx.x;      // late blocks have the most keys: start them first
    const int kvh = blockIdx.y;
    const int G = H / Hkv;
    int r = qb, col0 = 0;
    if (blk) { const int2 b = blk[qb]; r = b.x; col0 = b.y; }
    const int4 info = req_info[r];         // (first token of the request in the step, tokens, first position, -)
    const int t0 = info.x, ncols = info.y * G, pos0 = info.z;
    const int* table = block_table + (long long)r * max_blocks;

    const int last_col = min(ncols, col0 + CB) - 1;
    const int pos_max = pos0 + last_col / G;
    const int lo_min = window > 0 ? max(0, pos0 + col0 / G - window + 1) : 0;
    const int key_start = lo_min / STEP * STEP;
    const int nsteps = (pos_max - key_start) / STEP + 1;

    // ---- this wave's columns
    const int wcol0 = col0 + wave * NBW * 16;
    int pos_c[NBW], lo_c[NBW];
    long long qrow[NBW];                   // row of the column in q and out; -1: no column
    bf16x8 qf[NBW][KC];
    int wave_pos_max = -1, wave_pos_min = 0x7fffffff, wave_lo_max = 0;
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) {
        const int c = wcol0 + nb * 16 + n16;
        const bool valid = c < ncols;
        const int tok = t0 + (valid ? c / G : 0);
        const int head = kvh * G + (valid ? c % G : 0);
        pos_c[nb] = valid ? pos0 + c / G : -1;
        lo_c[nb] = (valid && window > 0) ? max(0, pos_c[nb] - window + 1) : 0;
        qrow[nb] = valid ? (long long)tok * H + head : -1;
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) {
            const int k = kc * 32 + g * 8;
            bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
            qf[nb][kc] = (valid && k < hd) ? *(const bf16x8*)(q + qrow[nb] * hd + k) : z;
        }
        // wave-wide: the range of positions of its columns (first and last column of the wave)
        const int cf = wcol0 + nb * 16, cl = min(ncols - 1, wcol0 + nb * 16 + 15);
        if (cf < ncols) {
            wave_pos_max = max(wave_pos_max, pos0 + cl / G);
            wave_pos_min = min(wave_pos_min, pos0 + cf / G);
            if (window > 0) wave_lo_max = max(wave_lo_max, max(0, pos0 + cl / G - window + 1));
        }
    }

    float m_run[NBW], l_run[NBW];
    f32x4 o[DB][NBW];
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) {
        m_run[nb] = -INFINITY;
        l_run[nb] = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db) o[db][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // ---- page numbers: lane i holds the page of granule (16 keys) gran_base + i; 64 granules = 16 steps
    const int gran0 = key_start / 16;
    auto pages_of = [&](int batch) {
        const long long idx = ((long long)(gran0 + batch * 64 + lane) * 16) / page_size;
        return idx < max_blocks ? table[idx] : -1;
    };
    int pages_cur = pages_of(0), pages_next = -1;

    // ---- copies: what this thread moves each step
    bf16x8 kreg[KPT], vreg[VPT];
    auto load_step = [&](int s) {                       // step s of the block -> registers
        const int key0 = key_start + s * STEP;
        const int gslot0 = (s % 16) * 4;                // granule of the step's first key within pages_cur
        const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const int id = tid + i * NT;
            const int key = id / HC, c = id % HC;
            const int page = __shfl(pages_cur, gslot0 + key / 16, WAVE);
            const int kabs = key0 + key;
            const bool live = page >= 0 && kabs <= pos_max && c * 8 < hd;
            kreg[i] = live ? *(const bf16x8*)(k_cache + (((long long)page * Hkv + kvh) * page_size + kabs % page_size) * hd + c * 8) : z;
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int id = tid + i * NT;
            const int dim = id / 8, c8 = id % 8;
            const int page = __shfl(pages_cur, gslot0 + c8 / 2, WAVE);
            const int kabs = key0 + c8 * 8;
            const bool live = page >= 0 && kabs <= pos_max && dim < hd;
            bf16x8 v = live ? *(const bf16x8*)(v_cache + (((long long)page * Hkv + kvh) * hd + dim) * page_size + kabs % page_size) : z;
            if (kabs + 7 > pos_max) {                   // positions beyond the last were never written
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (kabs + e > pos_max) v[e] = (bf16_t)0.f;
            }
            vreg[i] = v;
        }
    };
    auto store_step = [&](int buf) {
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const int id = tid + i * NT;
            *(bf16x8*)(Ks + buf * KBUF + k_row_of_key(id / HC) * KROW + (id % HC) * 8) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int id = tid + i * NT;
            *(bf16x8*)(Vs + buf * VBUF + (id / 8) * VROW + (id % 8) * 8) = vreg[i];
        }
    };

    // ---- one half step (32 keys) of this wave out of LDS
    auto half_step = [&](int buf, int sub, int key0) {
        const bf16_t* Kb = Ks + buf * KBUF + (sub * 32 + n16) * KROW + g * 8;
        const bf16_t* Vb = Vs + buf * VBUF + n16 * VROW + sub * 32 + g * 8;
        f32x4 s[2][NBW];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) s[kb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kc = 0; kc < KC; ++kc) {
                const bf16x8 kf = *(const bf16x8*)(Kb + kb * 16 * KROW + kc * 32);
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb) s[kb][nb] = mfma32(kf, qf[nb][kc], s[kb][nb]);
            }
        }
        // every key of the half is visible to every column of the wave: no mask
        const bool open = key0 + 31 <= wave_pos_min && key0 >= wave_lo_max;
        bf16x8 pf[NBW];
        float corr[NBW];
        bool same = true;
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            float v[8];
            float mx = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int key = key0 + 8 * g + 4 * kb + e;
                    const bool ok = open || (key <= pos_c[nb] && key >= lo_c[nb]);
                    const float x = ok ? s[kb][nb][e] * scale_log2e : -INFINITY;
                    v[kb * 4 + e] = x;
                    mx = fmaxf(mx, x);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
            const float m_new = fmaxf(m_run[nb], mx);
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            corr[nb] = __builtin_amdgcn_exp2f(m_run[nb] - m_safe);           // 0 while nothing was seen yet
            same = same && (m_new == m_run[nb]);
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float p = __builtin_amdgcn_exp2f(v[i] - m_safe);
                sum += p;
                pf[nb][i] = (bf16_t)p;
            }
            l_run[nb] = l_run[nb] * corr[nb] + sum;
            m_run[nb] = m_new;
        }
        const bool rescale = !__all(same);                   // corr is exactly 1 where the maximum stayed
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const bf16x8 vf = *(const bf16x8*)(Vb + db * 16 * VROW);
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) {
                f32x4 acc = o[db][nb];
                if (rescale) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] *= corr[nb];
                }
                o[db][nb] = mfma32(vf, pf[nb], acc);
            }
        }
    };

    load_step(0);
    store_step(0);
    __syncthreads();
    for (int s = 0; s < nsteps; ++s) {
        const int buf = s & 1;
        const int key0 = key_start + s * STEP;
        const bool more = s + 1 < nsteps;
        if (s % 16 == 0) pages_next = pages_of(s / 16 + 1);
        if (more) {
            if ((s + 1) % 16 == 0) pages_cur = pages_next;
            load_step(s + 1);
        }
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            const int k0 = key0 + sub * 32;
            if (k0 <= wave_pos_max && k0 + 31 >= (window > 0 ? max(0, wave_pos_min - window + 1) : 0)) half_step(buf, sub, k0);
        }
        if (more) store_step(buf ^ 1);
        __syncthreads();
    }

    // ---- normalise and write
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) {
        float l = l_run[nb];
        l += __shfl_xor(l, 16, WAVE);
        l += __shfl_xor(l, 32, WAVE);
        if (qrow[nb] < 0) continue;
        const float inv = 1.0f / l;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const int dim = db * 16 + 4 * g;
            if (dim < hd) {
                const f32x4 v = o[db][nb];
                bf16x4 w = {(bf16_t)(v[0] * inv), (bf16_t)(v[1] * inv), (bf16_t)(v[2] * inv), (bf16_t)(v[3] * inv)};
                *(bf16x4*)(out + qrow[nb] * hd + dim) = w;
            }
        }
    }
}

template <int HDP, int NBW>
int launch(dim3 grid, hipStream_t stream, const bf16_t* q, const bf16_t* kc, const bf16_t* vc, bf16_t* out,
           const int* bt, int max_blocks, const int2* blk, const int4* req_info,
           int H, int Hkv, int hd, int ps, int window, float scale_log2e) {
    auto kern = attn_prefill_kernel<HDP, NBW>;
    constexpr int lds = 2 * (STEP * (HDP + 8) + HDP * VROW) * 2;
    static bool set = false;
    if (!set) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -1;
        set = true;
    }
    hipLaunchKernelGGL(kern, grid, dim3(NT), lds, stream, q, kc, vc, out, bt, max_blocks, blk, req_info,
                       H, Hkv, hd, ps, window, scale_log2e);
    return launch_status();
}
}  // namespace

// Columns a block of the list must hold for this head size.
TUFF_EXPORT int tuff_attention_prefill_block_columns(int hd) { return hd <= 128 ? 128 : 64; }

// Query blocks are listed by the host: block b holds the columns blk[b].y .. + block_columns - 1
// of request blk[b].x (a request's columns are numbered (token - its first token) * G + head
// within the kv group); blk == null: block b is request b from column 0.
// req_info [R]: (first token of the request in the step, its tokens, position of the first, -).
TUFF_EXPORT int tuff_attention_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                                       const int* block_table, int max_blocks, const int* blk, int n_qblocks,
                                       const int* req_info, int H, int Hkv, int hd, int page_size, int window,
                                       float scale, hipStream_t stream) {
    if (n_qblocks <= 0) return 0;
    if (hd > 256 || hd % 8 != 0 || page_size % 16 != 0 || Hkv <= 0 || H % Hkv != 0) return -2;
    if (Hkv > 65535) return -2;
    const bf16_t* Q = (const bf16_t*)q;
    const bf16_t* K = (const bf16_t*)k_cache;
    const bf16_t* V = (const bf16_t*)v_cache;
    dim3 grid(n_qblocks, Hkv);
    const float sl = scale * 1.4426950408889634f;
#define GO(HDP, NBW) return launch<HDP, NBW>(grid, stream, Q, K, V, (bf16_t*)out, block_table, max_blocks, (const int2*)blk, \
                                             (const int4*)req_info, H, Hkv, hd, page_size, window, sl)
    if (hd <= 32) GO(32, 2);
    else if (hd <= 64) GO(64, 2);
    else if (hd <= 96) GO(96, 2);
    else if (hd <= 128) GO(128, 2);
    else GO(256, 1);
#undef GO
}
