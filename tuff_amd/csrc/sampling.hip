// Picking the next token on the GPU, one workgroup per request row.
//
// Greedy: the first maximum wins (src/sampler.c:103-113, src/lfm25_gpu.cu:691-692).
// Stochastic (temp > 0), the order of src/sampler.c:115-230: repetition penalty (its own
// kernel below) -> maximum -> min-p filter on (l - max)/T >= ln(min_p) -> candidates in
// descending order -> top-k -> softmax -> top-p (smallest prefix with cumulative
// probability >= top_p, renormalised) -> the first candidate whose cumulative probability
// reaches the uniform draw r.
//
// Nothing is sorted.  Candidates are ordered by (value descending, index ascending); every
// "first prefix whose weight reaches X" is found by a radix descent over the bits of an
// order-preserving integer image of the value: 4 levels of 256-bucket histograms, then the
// n-th equal value by index.  Probabilities are exp((l - max)/T) held as 40-bit fixed point
// integers, so sums are exact and do not depend on the order of addition; thresholds
// top_p * S and r * S are formed in float64.  The uniform draw comes from the host (one
// generator per request), so a row's result does not depend on what else is in the batch.
#include "common.h"
#include <math.h>

namespace {
constexpr int SNT = 1024;
typedef unsigned long long u64;

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __float_as_uint(f);
    if (u == 0x80000000u) return 0x80000000u;          // -0 and +0 compare equal: one key, so that the index decides
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct Cut { uint32_t key; int idx; };            // last element kept, in (key desc, idx asc) order

__device__ __forceinline__ bool within(uint32_t key, int i, Cut c) {
    return key > c.key || (key == c.key && i <= c.idx);
}

struct RowView {
    const float* l; int V; float mx, inv_t, lo;
    __device__ __forceinline__ float scaled(int i) const { return (l[i] - mx) * inv_t; }
    __device__ __forceinline__ u64 mass(float s) const { return (u64)(expf(s) * 1099511627776.0f); }
};

struct Shared {
    u64 hist[256];
    int scan[SNT];
    u64 cum; u64 acc; int chosen; int found; int count;
    float redf[SNT / WAVE]; int redi[SNT / WAVE];
};

// Finds the first element e, in (key desc, idx asc) order among the candidates within `cut`,
// at which the running weight reaches `target` (1 <= target <= total weight).  Weight is the
// fixed-point probability (BY_MASS) or 1.  Returns e as a Cut and the running weight
// through e in *through.
template <bool BY_MASS>
__device__ Cut descend(const RowView& row, Cut cut, u64 target, Shared& sh, u64* through) {
    const int tid = threadIdx.x;
    uint32_t prefix = 0;
    u64 cum = 0;
    for (int level = 0; level < 4; ++level) {
        const int shift = 24 - 8 * level;
        if (tid < 256) sh.hist[tid] = 0;
        __syncthreads();
        for (int i = tid; i < row.V; i += SNT) {
            const float s = row.scaled(i);
            if (!(s >= row.lo)) continue;
            const uint32_t key = order_key(s);
            if (!within(key, i, cut)) continue;
            if (level > 0 && (key >> (shift + 8)) != prefix) continue;
            atomicAdd(&sh.hist[(key >> shift) & 255u], BY_MASS ? row.mass(s) : (u64)1);
        }
        __syncthreads();
        if (tid == 0) {
            int chosen = -1, lowest = 0;
            u64 c = cum;
            for (int b = 255; b >= 0; --b) {
                const u64 h = sh.hist[b];
                if (h == 0) continue;
                lowest = b;
                if (c + h >= target) { chosen = b; break; }
                c += h;
            }
            if (chosen < 0) { chosen = lowest; c -= sh.hist[lowest]; }   // target beyond the total: last bucket
            sh.chosen = chosen;
            sh.cum = c;
        }
        __syncthreads();
        prefix = (prefix << 8) | (uint32_t)sh.chosen;
        cum = sh.cum;
        __syncthreads();
    }
    // All elements with this key have the same weight.  Take the n-th of them by index.
    const int per = (row.V + SNT - 1) / SNT;
    const int lo_i = tid * per, hi_i = min(row.V, lo_i + per);
    int cnt = 0;
    u64 w_eq = 0;
    for (int i = lo_i; i < hi_i; ++i) {
        const float s = row.scaled(i);
        if (!(s >= row.lo)) continue;
        const uint32_t key = order_key(s);
        if (key == prefix && within(key, i, cut)) { ++cnt; w_eq = BY_MASS ? row.mass(s) : (u64)1; }
    }
    sh.scan[tid] = cnt;
    if (tid == 0) { sh.acc = 0; sh.found = -1; sh.count = 0; }
    __syncthreads();
    if (cnt > 0) atomicMax(&sh.acc, w_eq);            // identical for all of them
    __syncthreads();
    if (tid == 0) {                                    // exclusive prefix over 1024 counts
        int run = 0;
        for (int t = 0; t < SNT; ++t) { const int c = sh.scan[t]; sh.scan[t] = run; run += c; }
        sh.count = run;
    }
    __syncthreads();
    const u64 w = sh.acc;
    const int total_eq = sh.count;
    u64 need = (w == 0) ? 1 : (target > cum ? (target - cum + w - 1) / w : 1);
    if (need > (u64)total_eq) need = (u64)total_eq;
    if (need < 1) need = 1;
    const int before = sh.scan[tid];
    if (cnt > 0 && (u64)before < need && need <= (u64)(before + cnt)) {
        int seen = before;
        for (int i = lo_i; i < hi_i; ++i) {
            const float s = row.scaled(i);
            if (!(s >= row.lo)) continue;
            const uint32_t key = order_key(s);
            if (key == prefix && within(key, i, cut)) { if ((u64)(++seen) == need) { sh.found = i; break; } }
        }
    }
    __syncthreads();
    Cut e; e.key = prefix; e.idx = sh.found;
    *through = cum + need * w;
    __syncthreads();
    return e;
}

// A thread's part of the search for the largest value of a row and its first index: pieces of four
// values, several loads under way.  The thread sees its indices in ascending order, so a strict
// comparison keeps the first of equal values.
template <int NT>
__device__ __forceinline__ void scan_max(const float* __restrict__ l, int V, int tid, float& best, int& best_i) {
    const bool vec = (V % 4 == 0) && ((reinterpret_cast<uintptr_t>(l) & 15) == 0);
    if (vec) {
        const f32x4* l4 = (const f32x4*)l;
        const int n4 = V / 4;
#pragma unroll 4
        for (int i = tid; i < n4; i += NT) {
            const f32x4 v = l4[i];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (v[e] > best) { best = v[e]; best_i = i * 4 + e; }
        }
    } else {
        for (int i = tid; i < V; i += NT) { const float v = l[i]; if (v > best) { best = v; best_i = i; } }
    }
}

__global__ __launch_bounds__(SNT) void sample_kernel(const float* __restrict__ logits, const float* __restrict__ temps,
                                                     const int* __restrict__ top_ks, const float* __restrict__ top_ps,
                                                     const float* __restrict__ min_ps, const float* __restrict__ uniforms,
                                                     int* __restrict__ out, int V) {
    __shared__ Shared sh;
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* l = logits + (long long)r * V;

    // maximum and its first index
    float best = -INFINITY; int best_i = 0x7fffffff;
    scan_max<SNT>(l, V, tid, best, best_i);
#pragma unroll
    for (int m = WAVE / 2; m > 0; m >>= 1) {
        const float ov = __shfl_xor(best, m, WAVE); const int oi = __shfl_xor(best_i, m, WAVE);
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    if (tid % WAVE == 0) { sh.redf[tid / WAVE] = best; sh.redi[tid / WAVE] = best_i; }
    __syncthreads();
    best = sh.redf[0]; best_i = sh.redi[0];
    for (int w = 1; w < SNT / WAVE; ++w)
        if (sh.redf[w] > best || (sh.redf[w] == best && sh.redi[w] < best_i)) { best = sh.redf[w]; best_i = sh.redi[w]; }
    __syncthreads();

    const float temp = temps ? temps[r] : 0.f;
    if (!(temp > 0.f)) { if (tid == 0) out[r] = best_i == 0x7fffffff ? 0 : best_i; return; }

    RowView row; row.l = l; row.V = V; row.mx = best; row.inv_t = 1.0f / temp;
    const float min_p = min_ps ? min_ps[r] : 0.f;
    row.lo = (min_p > 0.f && min_p < 1.f) ? logf(min_p) : -1e30f;
    const int top_k = top_ks ? top_ks[r] : 0;
    const float top_p = top_ps ? top_ps[r] : 1.f;

    Cut cut; cut.key = 0u; cut.idx = 0x7fffffff;

    // number of candidates and their total weight
    auto totals = [&](Cut c, u64* n_out, u64* s_out) {
        if (tid == 0) { sh.hist[0] = 0; sh.hist[1] = 0; }
        __syncthreads();
        u64 n = 0, s_sum = 0;
        for (int i = tid; i < V; i += SNT) {
            const float s = row.scaled(i);
            if (!(s >= row.lo)) continue;
            if (!within(order_key(s), i, c)) continue;
            ++n; s_sum += row.mass(s);
        }
        atomicAdd(&sh.hist[0], n);
        atomicAdd(&sh.hist[1], s_sum);
        __syncthreads();
        *n_out = sh.hist[0]; *s_out = sh.hist[1];
        __syncthreads();
    };

    u64 n_cand, S;
    totals(cut, &n_cand, &S);
    if (top_k > 0 && n_cand > (u64)top_k) {
        u64 through;
        cut = descend<false>(row, cut, (u64)top_k, sh, &through);
        totals(cut, &n_cand, &S);
    }
    if (top_p > 0.f && top_p < 1.f) {
        u64 target = (u64)ceil((double)top_p * (double)S);
        if (target < 1) target = 1;
        if (target > S) target = S;
        u64 through;
        cut = descend<true>(row, cut, target, sh, &through);
        S = through;
    }
    u64 target = (u64)ceil((double)uniforms[r] * (double)S);
    if (target < 1) target = 1;
    if (target > S) target = S;
    u64 through;
    const Cut pick = descend<true>(row, cut, target, sh, &through);
    if (tid == 0) out[r] = pick.idx >= 0 ? pick.idx : best_i;
}

// l <- l / penalty if l > 0 else l * penalty, once per entry of the request's ring of recent
// tokens (src/sampler.c:135-143: a token that occurs twice in the ring is penalised twice).
__global__ void repeat_penalty_kernel(float* __restrict__ logits, const int* __restrict__ recent,
                                      const int* __restrict__ counts, const float* __restrict__ penalties,
                                      int cap, int V) {
    const int r = blockIdx.x;
    if (threadIdx.x != 0) return;
    const float p = penalties[r];
    if (!(p > 1.0f)) return;
    float* l = logits + (long long)r * V;
    const int n = min(counts[r], cap);
    for (int k = 0; k < n; ++k) {
        const int t = recent[(long long)r * cap + k];
        if (t >= 0 && t < V) { const float v = l[t]; l[t] = (v > 0.f) ? v / p : v * p; }
    }
}

__global__ __launch_bounds__(256) void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int V) {
    __shared__ float redf[4];
    __shared__ int redi[4];
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* l = logits + (long long)r * V;
    float best = -INFINITY; int best_i = 0x7fffffff;
    scan_max<256>(l, V, tid, best, best_i);
#pragma unroll
    for (int m = WAVE / 2; m > 0; m >>= 1) {
        const float ov = __shfl_xor(best, m, WAVE); const int oi = __shfl_xor(best_i, m, WAVE);
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    if (tid % WAVE == 0) { redf[tid / WAVE] = best; redi[tid / WAVE] = best_i; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 4; ++w)
            if (redf[w] > best || (redf[w] == best && redi[w] < best_i)) { best = redf[w]; best_i = redi[w]; }
        out[r] = best_i == 0x7fffffff ? 0 : best_i;
    }
}
}  // namespace

TUFF_EXPORT int tuff_argmax(const float* logits, int* out, int n_rows, int V, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    hipLaunchKernelGGL(argmax_kernel, dim3(n_rows), dim3(256), 0, stream, logits, out, V);
    return launch_status();
}

// temps[r] <= 0 (or temps == null): greedy for that row.  top_ks, top_ps, min_ps may be null (off).
TUFF_EXPORT int tuff_sample(const float* logits, const float* temps, const int* top_ks, const float* top_ps,
                            const float* min_ps, const float* uniforms, int* out, int n_rows, int V,
                            hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (V <= 0 || V >= (1 << 24)) return -2;
    hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(SNT), 0, stream, logits, temps, top_ks, top_ps, min_ps,
                       uniforms, out, V);
    return launch_status();
}

TUFF_EXPORT int tuff_repeat_penalty(float* logits, const int* recent, const int* counts, const float* penalties,
                                    int n_rows, int cap, int V, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    hipLaunchKernelGGL(repeat_penalty_kernel, dim3(n_rows), dim3(64), 0, stream, logits, recent, counts, penalties, cap, V);
    return launch_status();
}
