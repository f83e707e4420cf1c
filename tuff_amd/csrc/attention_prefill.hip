// Paged attention for steps that carry prompt portions: bfloat16 cache, matrix cores, keys and
// values shared by a workgroup through LDS.
//
// A workgroup of four waves takes one kv head and one block of 64 * NBW query columns of one
// request (a column = one query head of one token; NBW * 16 columns a wave) and walks over all
// keys these columns may see, 64 at a time, from key 0 (or the first 64 the window still
// reaches).  The K rows and V columns of a step are copied from the pages into LDS once, by all
// threads, a few steps ahead of their use; every wave reads its MFMA operands from there.  Each
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
// part of P^T for O^T += V^T P^T.  The scores of both halves of a step are taken first and the
// reference point of the exponents is moved once a step of 64 keys, for every step alike, masked
// or not.
//
// Cache layout: K [page][kv_head][offset][hd], V [page][kv_head][hd][offset]; page size a
// multiple of 16, head size a multiple of 8.
#include "common.h"
#include <math.h>

namespace {
constexpr int STEP = 64;            // keys a step
constexpr int NT = 256;             // threads a workgroup
constexpr float SLACK = 8.f;        // see whole_step
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

template <int HDP, int NBW, int AHEAD>
__global__ __launch_bounds__(NT) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int* __restrict__ block_table, int max_blocks,
    const int2* __restrict__ blk, const int4* __restrict__ req_info,
    int H, int Hkv, int hd, int page_size, int window, float scale_log2e,
    int seg_keys, float* __restrict__ ws_o, float* __restrict__ ws_ml) {
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
    // Workgroups are numbered with the kv head changing fastest: the eight XCDs take the numbers in
    // turn, so with eight kv heads an XCD's L2 holds one head's keys and values.  The host lists the
    // blocks with the most keys first, so that the long ones start first and the short ones fill in.
    const int qb = blockIdx.x / Hkv;
    const int kvh = blockIdx.x % Hkv;
    const int G = H / Hkv;
    int r = qb, col0 = 0;
    if (blk) { const int2 b = blk[qb]; r = b.x; col0 = b.y; }
    const int4 info = req_info[r];         // (first token of the request in the step, tokens, first position, -)
    const int t0 = info.x, ncols = info.y * G, pos0 = info.z;
    const int* table = block_table + (long long)r * max_blocks;

    const int last_col = min(ncols, col0 + CB) - 1;
    const int pos_max = pos0 + last_col / G;
    const int lo_min = window > 0 ? max(0, pos0 + col0 / G - window + 1) : 0;
    // gridDim.z > 1: the keys are cut into segments of seg_keys (a multiple of STEP), a workgroup a
    // segment; it leaves what it has summed, unnormalised, with its reference exponent and sum in
    // the work space, for the kernel that merges the partitions of single-token steps.
    const int seg = blockIdx.z, n_segs = gridDim.z;
    const int seg_begin = n_segs > 1 ? seg * seg_keys : 0;
    const int key_last = n_segs > 1 ? min(pos_max, seg_begin + seg_keys - 1) : pos_max;
    const int key_start = max(lo_min / STEP * STEP, seg_begin);
    const int nsteps = key_last >= key_start ? (key_last - key_start) / STEP + 1 : 0;

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

    // The sums of the weights come out of the matrix cores too: V^T is given one more block of rows
    // whose first row is all ones, so row 0 of that block of O^T is the sum of a column's weights (as
    // they are multiplied: rounded to bfloat16, summed in float32), in the lanes of group 0.
    float m_run[NBW];
    f32x4 l_acc[NBW];
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = (bf16_t)(n16 == 0 ? 1.f : 0.f);
    f32x4 o[DB][NBW];
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) {
        m_run[nb] = -INFINITY;
        l_acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int db = 0; db < DB; ++db) o[db][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    if (nsteps == 0) {                     // a segment beyond the block's keys: nothing summed
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb)
            if (qrow[nb] >= 0 && g == 0) {
                const long long slot = qrow[nb] * n_segs + seg;
                ws_ml[slot * 2] = -INFINITY;
                ws_ml[slot * 2 + 1] = 0.f;
            }
        return;
    }

    // ---- page numbers: lane i holds the page of granule (16 keys) gran_base + i; 64 granules = 16 steps
    const int gran0 = key_start / 16;
    auto pages_of = [&](int batch) {
        const long long idx = ((long long)(gran0 + batch * 64 + lane) * 16) / page_size;
        return idx < max_blocks ? table[idx] : -1;
    };
    int pages_cur = pages_of(0), pages_next = pages_of(1);

    // ---- copies: what this thread moves each step.  Memory answers later than a step lasts, so
    // the keys and values of AHEAD steps are on their way at any time, each in a register set.
    // Per piece the thread keeps what does not change from step to step: the granule (16 keys, one
    // page) it lies in, its offset inside the granule's rows, and where it goes in LDS.  The pieces
    // are dealt so that the 64 of a wave lie in one granule: where the granule's rows start in the
    // caches is then scalar arithmetic, once a piece and wave, not a choice among four addresses in
    // every lane.
    bf16x8 kreg[AHEAD][KPT], vreg[AHEAD][VPT];
    int k_gran[KPT], k_key[KPT], k_off[KPT], k_lds[KPT], v_gran[VPT], v_key[VPT], v_off[VPT], v_lds[VPT];
    bool k_ok[KPT], v_ok[VPT];
    static_assert((16 * HC) % WAVE == 0 && (2 * HDP) % WAVE == 0 && NT % WAVE == 0, "a wave's pieces lie in one granule");
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
        const int id = tid + i * NT, key = id / HC, c = id % HC;
        k_gran[i] = __builtin_amdgcn_readfirstlane(key / 16);
        k_key[i] = key;
        k_off[i] = (key % 16) * hd + c * 8;
        k_ok[i] = c * 8 < hd;
        k_lds[i] = k_row_of_key(key) * KROW + c * 8;
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int id = tid + i * NT, c8 = id / HDP, dim = id % HDP;      // lanes run over the channels
        v_gran[i] = __builtin_amdgcn_readfirstlane(c8 / 2);
        v_key[i] = c8 * 8;
        v_off[i] = dim * page_size + (c8 % 2) * 8;
        v_ok[i] = dim < hd;
        v_lds[i] = dim * VROW + c8 * 8;
    }
    const bool whole_rows = hd == HDP;
    const unsigned page_stride = (unsigned)(Hkv * page_size * hd);       // elements of a page in either cache (the host checks that it fits)
    const unsigned head_off = (unsigned)(kvh * page_size * hd);          // this kv head's share of it
    const int ps_mask = (page_size & (page_size - 1)) == 0 ? page_size - 1 : 0;   // a power of two: offsets wrap by a mask
    int ld_off = key_start % page_size;                 // offset in its page of the first key of the next step to load
    auto load_step = [&](int set, int s, int pages) {   // step s of the block -> register set; zeros beyond pos_max
        const int key0 = key_start + s * STEP;
        const int gslot0 = (s % 16) * 4;                // granule of the step's first key within `pages`
        // per piece, the same for the lanes of a wave: where its granule's rows start (-1: no such page)
        auto granule = [&](int g4, long long& base, int& go) {
            const int page = __builtin_amdgcn_readlane(pages, gslot0 + g4);
            go = ld_off + 16 * g4;
            if (ps_mask) go &= ps_mask;
            else {
#pragma unroll
                for (int w = 0; w < 3; ++w)
                    if (go >= page_size) go -= page_size;
            }
            base = page >= 0 ? (long long)((unsigned long long)(unsigned)page * page_stride + head_off) : -1;
        };
        long long bk[KPT], bv[VPT];
        bool all_live = key0 + STEP - 1 <= pos_max;
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            int go;
            granule(k_gran[i], bk[i], go);
            all_live = all_live && bk[i] >= 0;
            bk[i] += (long long)go * hd;                // (-1 stays negative: go * hd < page_stride)
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            int go;
            granule(v_gran[i], bv[i], go);
            all_live = all_live && bv[i] >= 0;
            bv[i] += go;
        }
        if (ps_mask) ld_off = (ld_off + STEP) & ps_mask;
        else {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                ld_off += 16;
                if (ld_off >= page_size) ld_off -= page_size;
            }
        }
        if (all_live && whole_rows) {
#pragma unroll
            for (int i = 0; i < KPT; ++i) kreg[set][i] = *(const bf16x8*)(k_cache + bk[i] + k_off[i]);
#pragma unroll
            for (int i = 0; i < VPT; ++i) vreg[set][i] = *(const bf16x8*)(v_cache + bv[i] + v_off[i]);
            return;
        }
        // first steps under a window, the last step, narrow heads: pieces that do not exist read as zero
        const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const bool live = bk[i] >= 0 && key0 + k_key[i] <= pos_max && k_ok[i];
            const bf16x8 v = *(const bf16x8*)(k_cache + (live ? bk[i] + k_off[i] : 0));
            kreg[set][i] = live ? v : z;
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int kabs = key0 + v_key[i];
            const bool live = bv[i] >= 0 && kabs <= pos_max && v_ok[i];
            bf16x8 v = *(const bf16x8*)(v_cache + (live ? bv[i] + v_off[i] : 0));
            v = live ? v : z;
#pragma unroll
            for (int e = 0; e < 8; ++e)                  // positions beyond the last were never written
                if (kabs + e > pos_max) v[e] = (bf16_t)0.f;
            vreg[set][i] = v;
        }
    };
    auto store_step = [&](int set, int buf) {
#pragma unroll
        for (int i = 0; i < KPT; ++i) *(bf16x8*)(Ks + buf * KBUF + k_lds[i]) = kreg[set][i];
#pragma unroll
        for (int i = 0; i < VPT; ++i) *(bf16x8*)(Vs + buf * VBUF + v_lds[i]) = vreg[set][i];
    };

    // ---- the scores of one half step (32 keys) of this wave, out of LDS
    struct Scores { f32x4 v[2][NBW]; };
    auto scores = [&](int buf, int sub) {
        const bf16_t* Kb = Ks + buf * KBUF + (sub * 32 + n16) * KROW + g * 8;
        Scores sc;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) sc.v[kb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kc = 0; kc < KC; ++kc) {
                const bf16x8 kf = *(const bf16x8*)(Kb + kb * 16 * KROW + kc * 32);
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb) sc.v[kb][nb] = mfma32(kf, qf[nb][kc], sc.v[kb][nb]);
            }
        }
        return sc;
    };
    // One step of 64 keys: the scores of both halves, then, per column, one reference point for the
    // exponents of all 64 (so that the products of one half run while the other's exponentials are
    // computed, and the bookkeeping is done once), then the weighted sums.  open: every key of the step
    // is visible to every column of the wave, no mask.  Otherwise live0/live1 say which halves hold a
    // key that some column sees; a column's masked keys weigh nothing, so what a column sums does not
    // depend on which columns share its wave.
    auto whole_step = [&](int buf, int key0, bool live0, bool live1, auto open_tag) {
        constexpr bool open = decltype(open_tag)::value;
        const bf16_t* Vb = Vs + buf * VBUF + n16 * VROW + g * 8;
        Scores sc[2];
        if (open || live0) sc[0] = scores(buf, 0);
        if (open || live1) sc[1] = scores(buf, 1);
        bf16x8 pf[2][NBW];
        float corr[NBW];
        bool same = true;
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            // The maximum is taken over the raw scores and scaled afterwards (scale > 0, rounding is
            // monotonic), so that score * scale - maximum is one fused operation: written as fmaf,
            // it is the same instruction with and without the mask.
            float mx = -INFINITY;
            bool ok[2][8];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int key = key0 + 32 * sub + 8 * g + 4 * kb + e;
                        const bool v = open || ((sub ? live1 : live0) && key <= pos_c[nb] && key >= lo_c[nb]);
                        ok[sub][kb * 4 + e] = v;
                        mx = fmaxf(mx, v ? sc[sub].v[kb][nb][e] : -INFINITY);
                    }
            mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
            // The reference point of the exponents moves only when a score exceeds it by more than
            // 2^SLACK: until then the weights may reach 2^SLACK instead of 1, which float32 sums and
            // bfloat16 weights hold as well, and the output so far need not be rescaled.
            const float m_cand = mx * scale_log2e;
            const float m_new = (m_cand > m_run[nb] + SLACK) ? m_cand : m_run[nb];
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            corr[nb] = __builtin_amdgcn_exp2f(m_run[nb] - m_safe);           // 0 while nothing was seen yet
            same = same && (m_new == m_run[nb]);
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float p = ok[sub][i] ? __builtin_amdgcn_exp2f(fmaf(sc[sub].v[i / 4][nb][i % 4], scale_log2e, -m_safe)) : 0.f;
                    pf[sub][nb][i] = (bf16_t)p;
                }
            m_run[nb] = m_new;
        }
        if (!__all(same)) {                                  // rare; corr is exactly 1 where the reference stayed
            asm volatile("" ::: "memory");                   // a branch, not a select over every accumulator
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[db][nb][e] *= corr[nb];
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) l_acc[nb][0] *= corr[nb];
        }
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            if (!(open || (sub ? live1 : live0))) continue;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const bf16x8 vf = *(const bf16x8*)(Vb + db * 16 * VROW + sub * 32);
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb) o[db][nb] = mfma32(vf, pf[sub][nb], o[db][nb]);
            }
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) l_acc[nb] = mfma32(ones, pf[sub][nb], l_acc[nb]);
        }
    };

    // set u holds step u, later step u + AHEAD, ...; step s + 1 goes into LDS while step s is computed.
    // (Loops over sets are unrolled, so a set's registers are named at compile time.)
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) load_step(u, u, pages_cur);
    store_step(0, 0);
    __syncthreads();
    for (int s0 = 0; s0 < nsteps; s0 += AHEAD) {
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const int s = s0 + u;
            if (s >= nsteps) break;
            const int buf = s & 1;
            const int key0 = key_start + s * STEP;
            const int ls = s + AHEAD;                   // the step whose loads start now
            if (ls % 16 == 0) pages_cur = pages_next;
            if (ls % 16 == 1) pages_next = pages_of(ls / 16 + 1);
            load_step(u, ls, pages_cur);
            const int lo_any = window > 0 ? max(0, wave_pos_min - window + 1) : 0;
            const bool live0 = key0 <= wave_pos_max && key0 + 31 >= lo_any;
            const bool live1 = key0 + 32 <= wave_pos_max && key0 + 63 >= lo_any;
            if (key0 + 63 <= wave_pos_min && key0 >= wave_lo_max) whole_step(buf, key0, true, true, std::true_type());
            else if (live0 || live1) whole_step(buf, key0, live0, live1, std::false_type());
            store_step((u + 1) % AHEAD, buf ^ 1);
            __syncthreads();
        }
    }

    // ---- normalise and write
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) {
        const float l = __shfl(l_acc[nb][0], n16, WAVE);       // from the lane of group 0 that holds the column's sum
        if (qrow[nb] < 0) continue;
        if (n_segs > 1) {
            const long long slot = qrow[nb] * n_segs + seg;
            // the merge works with natural exponents: reference 2^m = e^(m ln 2)
            if (g == 0) { ws_ml[slot * 2] = m_run[nb] * 0.6931471805599453f; ws_ml[slot * 2 + 1] = l; }
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int dim = db * 16 + 4 * g;
                if (dim < hd) *(f32x4*)(ws_o + slot * hd + dim) = o[db][nb];
            }
            continue;
        }
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

template <int HDP, int NBW, int AHEAD>
int launch(dim3 grid, hipStream_t stream, const bf16_t* q, const bf16_t* kc, const bf16_t* vc, bf16_t* out,
           const int* bt, int max_blocks, const int2* blk, const int4* req_info,
           int H, int Hkv, int hd, int ps, int window, float scale_log2e, int seg_keys, float* ws_o, float* ws_ml) {
    auto kern = attn_prefill_kernel<HDP, NBW, AHEAD>;
    constexpr int lds = 2 * (STEP * (HDP + 8) + HDP * VROW) * 2;
    static bool set = false;
    if (!set) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -1;
        set = true;
    }
    hipLaunchKernelGGL(kern, grid, dim3(NT), lds, stream, q, kc, vc, out, bt, max_blocks, blk, req_info,
                       H, Hkv, hd, ps, window, scale_log2e, seg_keys, ws_o, ws_ml);
    return launch_status();
}
}  // namespace

// Columns a block of the list must hold for this head size.
TUFF_EXPORT int tuff_attention_prefill_block_columns(int hd) { return hd <= 128 ? 128 : 64; }

// Query blocks are listed by the host, best those with the most keys first: block b holds the columns
// blk[b].y .. + block_columns - 1 of request blk[b].x (a request's columns are numbered (token - its first token) * G + head
// within the kv group); blk == null: block b is request b from column 0.
// req_info [R]: (first token of the request in the step, its tokens, position of the first, -).
// n_segs > 1: the keys are cut into segments of seg_keys (a multiple of 64) and `out` is not written:
// the partial results go to ws_o [tokens * H * n_segs * hd] and ws_ml [tokens * H * n_segs * 2] in the
// layout of the single-token kernel's partitions, to be merged by tuff_attention_merge with
// part_keys = seg_keys.
TUFF_EXPORT int tuff_attention_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                                       const int* block_table, int max_blocks, const int* blk, int n_qblocks,
                                       const int* req_info, int H, int Hkv, int hd, int page_size, int window,
                                       float scale, int n_segs, int seg_keys, float* ws_o, float* ws_ml,
                                       hipStream_t stream) {
    if (n_qblocks <= 0) return 0;
    if (hd > 256 || hd % 8 != 0 || page_size % 16 != 0 || Hkv <= 0 || H % Hkv != 0) return -2;
    if (Hkv > 65535 || !(scale > 0.f)) return -2;
    if (n_segs < 1 || n_segs > 65535) return -2;
    if ((long long)Hkv * page_size * hd > 0x7fffffffll) return -2;
    if (n_segs > 1 && (seg_keys <= 0 || seg_keys % STEP != 0 || !ws_o || !ws_ml)) return -2;
    const bf16_t* Q = (const bf16_t*)q;
    const bf16_t* K = (const bf16_t*)k_cache;
    const bf16_t* V = (const bf16_t*)v_cache;
    if ((long long)n_qblocks * Hkv > 0x7fffffffll) return -2;
    dim3 grid(n_qblocks * Hkv, 1, n_segs);
    const float sl = scale * 1.4426950408889634f;
#define GO(HDP, NBW, AHEAD) return launch<HDP, NBW, AHEAD>(grid, stream, Q, K, V, (bf16_t*)out, block_table, max_blocks, (const int2*)blk, \
                                             (const int4*)req_info, H, Hkv, hd, page_size, window, sl, seg_keys, ws_o, ws_ml)
    if (hd <= 32) GO(32, 2, 3);
    else if (hd <= 64) GO(64, 2, 2);
    else if (hd <= 96) GO(96, 2, 2);
    else if (hd <= 128) GO(128, 2, 2);
    else GO(256, 1, 1);
#undef GO
}
