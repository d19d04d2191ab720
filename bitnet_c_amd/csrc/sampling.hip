// Sampling from logits on the device, one workgroup per row.
//
// Reference (src/sampler.c:137-172): repetition penalty on each distinct recent token
// (logit > 0 ? /p : *p), then argmax at temperature 0 (first index of the maximum,
// src/sampler_backend.c:129-134; ties to the lower index as src/gpu_cuda.cu:9013-9018),
// else logits / T, softmax with a float32 sum, and either the plain cdf walk
// (`r < cdf`) or top-p: drop p < (1-topp)/(n-1), order by probability descending, cut
// where the cumulative sum first exceeds topp, walk r * cumulative.
//
// The uniform number r of a row comes from the host (the per-sequence xorshift64* of
// src/sampler.c:6-15), so what a sequence samples does not depend on its batch.
// Top-p needs no sort here: the place where a descending cumulative sum first exceeds
// a bound is found by a radix descent over the probabilities' bit patterns, with the
// sums kept in 40-bit fixed point so that the order of the atomic adds cannot matter.
// Equal probabilities are ordered by index.
#include "common.h"
#include <math.h>

#define SMP_THREADS 1024

struct ArgMax { float v; int i; };

__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
    if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
    return a;
}

__device__ ArgMax block_argmax(const float* __restrict__ x, int n, ArgMax* scratch) {
    ArgMax best = {-INFINITY, 0x7fffffff};
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        ArgMax c = {x[i], i};
        best = better(best, c);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        ArgMax c = {__shfl_xor(best.v, o, BN_WAVE), __shfl_xor(best.i, o, BN_WAVE)};
        best = better(best, c);
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) scratch[w] = best;
    __syncthreads();
    ArgMax r = scratch[0];
    for (int k = 1; k < nw; ++k) r = better(r, scratch[k]);
    if (r.i == 0x7fffffff) r.i = 0;          // a row of NaNs or -inf: index 0, as a first-max scan gives
    return r;
}

__global__ __launch_bounds__(SMP_THREADS) void argmax_kernel(const float* __restrict__ logits, int ld, int n,
                                                             int* __restrict__ out) {
    __shared__ ArgMax scratch[16];
    const ArgMax r = block_argmax(logits + (size_t)blockIdx.x * ld, n, scratch);
    if (threadIdx.x == 0) out[blockIdx.x] = r.i;
}

// Two stages for few rows of a large vocabulary (src/gpu_cuda.cu:9068, :9125 does the same): stage 1,
// grid (rows, parts), the best of each contiguous part; stage 2, one wave per row, the best of the parts.
// `better` prefers the lower index among equals at both stages, so the result is the first maximum.
#define ARGMAX_PARTS 64
__global__ __launch_bounds__(256) void argmax_part_kernel(const float* __restrict__ logits, int ld, int n,
                                                          float* __restrict__ pv, int* __restrict__ pi) {
    __shared__ ArgMax scratch[16];
    const int part = blockIdx.y, per = (n + ARGMAX_PARTS - 1) / ARGMAX_PARTS;
    const int lo = min(n, part * per), hi = min(n, lo + per);
    const float* x = logits + (size_t)blockIdx.x * ld;
    ArgMax best = {-INFINITY, 0x7fffffff};
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        ArgMax c = {x[i], i};
        best = better(best, c);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        ArgMax c = {__shfl_xor(best.v, o, BN_WAVE), __shfl_xor(best.i, o, BN_WAVE)};
        best = better(best, c);
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) scratch[w] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        ArgMax r = scratch[0];
        for (int k = 1; k < (int)(blockDim.x >> 6); ++k) r = better(r, scratch[k]);
        pv[blockIdx.x * ARGMAX_PARTS + part] = r.v;
        pi[blockIdx.x * ARGMAX_PARTS + part] = r.i;
    }
}
__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi,
                                                          int* __restrict__ out) {
    ArgMax best = {pv[blockIdx.x * ARGMAX_PARTS + threadIdx.x], pi[blockIdx.x * ARGMAX_PARTS + threadIdx.x]};
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        ArgMax c = {__shfl_xor(best.v, o, BN_WAVE), __shfl_xor(best.i, o, BN_WAVE)};
        best = better(best, c);
    }
    if (threadIdx.x == 0) out[blockIdx.x] = best.i == 0x7fffffff ? 0 : best.i;
}

// recent: [rows, window] token ids, -1 = empty.  Each distinct token is penalised once.
__global__ void repeat_penalty_kernel(float* __restrict__ logits, int ld, int n, const int* __restrict__ recent,
                                      int window, float penalty) {
    float* x = logits + (size_t)blockIdx.x * ld;
    const int* rc = recent + (size_t)blockIdx.x * window;
    for (int j = threadIdx.x; j < window; j += blockDim.x) {
        const int tok = rc[j];
        if (tok < 0 || tok >= n) continue;
        bool seen = false;
        for (int k = 0; k < j; ++k) seen = seen || (rc[k] == tok);
        if (seen) continue;
        const float v = x[tok];
        x[tok] = v > 0.f ? v / penalty : v * penalty;
    }
}

#define FIX_ONE 1099511627776.0      // 2^40

__device__ __forceinline__ unsigned long long to_fixed(float p) { return (unsigned long long)((double)p * FIX_ONE); }

#define SMP_WAVES (SMP_THREADS / 64)

// Every wave owns a contiguous range of the row and walks it 64 consecutive elements a time (lane l
// takes element l of each group): loads are coalesced, and (wave, group, lane) order is index order.
__device__ __forceinline__ void wave_range(int n, int& lo, int& hi) {
    const int per = ((n + SMP_WAVES - 1) / SMP_WAVES + 63) / 64 * 64;
    lo = min(n, (int)(threadIdx.x >> 6) * per);
    hi = min(n, lo + per);
}

__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned lo = __shfl_xor((unsigned)v, o, BN_WAVE), hi = __shfl_xor((unsigned)(v >> 32), o, BN_WAVE);
        v += ((unsigned long long)hi << 32) | lo;
    }
    return v;
}

// Descending cumulative sum over {p_i >= cutoff}: finds the element at which the sum first
// exceeds `bound` (fixed point).  Returns its index; *cum_out = the sum including it.  When the
// sum never exceeds the bound the last (smallest) candidate and the whole sum are returned.
__device__ int descend(const float* __restrict__ p, int n, float cutoff, unsigned long long bound,
                       unsigned long long* cum_out, unsigned long long* hist, int* ibuf) {
    // ibuf: [SMP_THREADS + 8] ints of shared memory; hist: [258]
    uint32_t prefix = 0, mask = 0;
    unsigned long long above = 0;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int lo, hi;
    wave_range(n, lo, hi);
    for (int level = 0; level < 4; ++level) {
        const int shift = 24 - 8 * level;
        for (int b = threadIdx.x; b < 256; b += blockDim.x) hist[b] = 0;
        __syncthreads();
        for (int g0 = lo; g0 < hi; g0 += 64) {
            const int i = g0 + lane;
            const float v = i < hi ? p[i] : 0.f;
            const uint32_t bits = __float_as_uint(v);
            const bool cand = i < hi && v >= cutoff && (bits & mask) == prefix;
            const int bin = (bits >> shift) & 255u;
            const unsigned long long any = __ballot(cand);
            if (any == 0) continue;
            // neighbours mostly fall into one bucket at the upper levels: then one add for the wave
            const int first_bin = __shfl(bin, __ffsll((long long)any) - 1, BN_WAVE);
            if (__all(!cand || bin == first_bin)) {
                const unsigned long long sum = wave_sum_u64(cand ? to_fixed(v) : 0ull);
                if (lane == 0) atomicAdd(&hist[first_bin], sum);
            } else if (cand) {
                atomicAdd(&hist[bin], to_fixed(v));
            }
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            int chosen = -1, lowest = -1;
            unsigned long long acc = above;
            for (int b = 255; b >= 0; --b) {
                if (hist[b] == 0) continue;
                lowest = b;
                if (acc + hist[b] > bound) { chosen = b; break; }
                acc += hist[b];
            }
            if (chosen < 0) {                     // never exceeded: stay in the lowest bucket that has elements
                chosen = lowest < 0 ? 0 : lowest;
                acc -= (lowest < 0 ? 0 : hist[chosen]);
            }
            ibuf[SMP_THREADS] = chosen;
            hist[256] = acc;
        }
        __syncthreads();
        prefix |= ((uint32_t)ibuf[SMP_THREADS]) << shift;
        mask |= 255u << shift;
        above = hist[256];
        __syncthreads();
    }
    // the group of elements whose probability has exactly the bit pattern `prefix`, in index order
    const float v = __uint_as_float(prefix);
    const unsigned long long qv = to_fixed(v);
    int cnt = 0;
    for (int g0 = lo; g0 < hi; g0 += 64) {
        const int i = g0 + lane;
        const bool hit = i < hi && p[i] >= cutoff && __float_as_uint(p[i]) == prefix;
        cnt += __popcll(__ballot(hit));
    }
    if (lane == 0) ibuf[wave] = cnt;
    __syncthreads();
    if (threadIdx.x == 0) {
        int total = 0;
        for (int t = 0; t < SMP_WAVES; ++t) total += ibuf[t];
        long long k = 1;
        if (qv > 0 && bound >= above) k = (long long)((bound - above) / qv) + 1;
        if (k > total) k = total;
        if (k < 1) k = 1;
        // wave that holds the k-th element of the group
        int seen = 0, owner = 0, rank = (int)k;
        for (int t = 0; t < SMP_WAVES; ++t) {
            if (seen + ibuf[t] >= (int)k) { owner = t; rank = (int)k - seen; break; }
            seen += ibuf[t];
        }
        ibuf[SMP_THREADS + 1] = owner;
        ibuf[SMP_THREADS + 2] = rank;
        ibuf[SMP_THREADS + 3] = total;
        hist[257] = above + (unsigned long long)k * qv;
    }
    __syncthreads();
    const int owner = ibuf[SMP_THREADS + 1], rank = ibuf[SMP_THREADS + 2], total = ibuf[SMP_THREADS + 3];
    if (wave == owner) {
        int seen = 0, found = n - 1;
        for (int g0 = lo; g0 < hi; g0 += 64) {
            const int i = g0 + lane;
            const bool hit = i < hi && p[i] >= cutoff && __float_as_uint(p[i]) == prefix;
            unsigned long long m = __ballot(hit);
            const int c = __popcll(m);
            if (seen + c >= rank) {
                for (int skip = rank - seen - 1; skip > 0; --skip) m &= m - 1;       // drop the lower set bits
                found = g0 + __ffsll((long long)m) - 1;
                break;
            }
            seen += c;
        }
        if (lane == 0) ibuf[SMP_THREADS + 4] = total > 0 ? found : n - 1;
    }
    __syncthreads();
    *cum_out = hist[257];
    const int res = ibuf[SMP_THREADS + 4];
    __syncthreads();
    return res;
}

// probs: [rows, n] scratch.  r: [rows] uniform numbers in [0, 1).
__global__ __launch_bounds__(SMP_THREADS) void sample_kernel(const float* __restrict__ logits, int ld, int n,
                                                             float* __restrict__ probs, const float* __restrict__ r,
                                                             float temperature, float top_p, int* __restrict__ out) {
    __shared__ ArgMax am[16];
    __shared__ float fs[16];
    __shared__ unsigned long long hist[258];
    __shared__ int ibuf[SMP_THREADS + 8];
    __shared__ float wtot[SMP_WAVES];
    const float* x = logits + (size_t)blockIdx.x * ld;
    float* p = probs + (size_t)blockIdx.x * n;
    if (temperature == 0.0f) {
        const ArgMax a = block_argmax(x, n, am);
        if (threadIdx.x == 0) out[blockIdx.x] = a.i;
        return;
    }
    // softmax(x / T): the assignment of elements to lanes is fixed, so the sums have a fixed order
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int lo, hi;
    wave_range(n, lo, hi);
    float mx = -INFINITY;
    for (int i = lo + lane; i < hi; i += 64) mx = fmaxf(mx, x[i] / temperature);
    mx = block_max(mx, fs);
    float part = 0.f;
    for (int i = lo + lane; i < hi; i += 64) {
        const float e = expf(x[i] / temperature - mx);
        p[i] = e;
        part += e;
    }
    const float total = block_sum(part, fs);
    part = 0.f;
    for (int i = lo + lane; i < hi; i += 64) {
        const float q = p[i] / total;
        p[i] = q;
        part += q;
    }
    part = wave_sum(part);
    if (lane == 0) wtot[wave] = part;
    __syncthreads();                        // also: every lane's p[] is visible to the whole workgroup
    const float rr = r[blockIdx.x];
    if (n == 1) { if (threadIdx.x == 0) out[blockIdx.x] = 0; return; }
    if (top_p <= 0.0f || top_p >= 1.0f) {
        // cdf walk: first i with rr < cdf_i (src/sampler.c:65-74); n-1 if none.  First the wave whose
        // range holds it, then that wave walks its range with a prefix sum over each 64 elements.
        if (threadIdx.x == 0) {
            float c = 0.f;
            int owner = -1;
            for (int t = 0; t < SMP_WAVES; ++t) {
                const float s = wtot[t];
                if (owner < 0 && rr < c + s) { owner = t; fs[0] = c; }
                c += s;
            }
            ibuf[0] = owner;
        }
        __syncthreads();
        const int owner = ibuf[0];
        if (owner < 0) { if (threadIdx.x == 0) out[blockIdx.x] = n - 1; return; }
        if (wave == owner) {
            float c = fs[0];
            int found = hi - 1;
            for (int g0 = lo; g0 < hi; g0 += 64) {
                const int i = g0 + lane;
                float sc = i < hi ? p[i] : 0.f;
#pragma unroll
                for (int o = 1; o < 64; o <<= 1) {
                    const float t = __shfl_up(sc, o, BN_WAVE);
                    if (lane >= o) sc += t;
                }
                const unsigned long long m = __ballot(i < hi && rr < c + sc);
                if (m) { found = g0 + __ffsll((long long)m) - 1; break; }
                c += __shfl(sc, 63, BN_WAVE);
            }
            if (lane == 0) out[blockIdx.x] = found;
        }
        return;
    }
    const float cutoff = (1.0f - top_p) / (float)(n - 1);
    unsigned long long cum = 0;
    (void)descend(p, n, cutoff, to_fixed(top_p), &cum, hist, ibuf);
    const unsigned long long target = (unsigned long long)((double)rr * (double)cum);
    unsigned long long cum2 = 0;
    const int tok = descend(p, n, cutoff, target, &cum2, hist, ibuf);
    if (threadIdx.x == 0) out[blockIdx.x] = tok;
}

// ---------------------------------------------------------------------------------------
// The same sampling with a row spread over many workgroups, for large vocabularies: one workgroup
// walks a row of 128k logits 17 times (half a millisecond); here every pass is a launch of
// rows x WIDE_PARTS workgroups that read a part each, and what one workgroup decided alone
// (the maximum, the sum, each level's bucket of the radix descent) is recomputed by every
// workgroup from small per-row tables in a work buffer: per-part maxima and sums, the 2 x 4
// histograms of the two descents (added up with 64-bit atomics in fixed point, so the order cannot
// matter), per-part counts of the final bit pattern.  Probabilities are never stored: every pass
// computes q_i = expf(x_i / T - max) / sum again, the same value each time.
// ---------------------------------------------------------------------------------------
#define WIDE_PARTS 32
#define WIDE_THREADS 256
#define WIDE_HIST (2 * 4 * 256)                      // 64-bit words of histograms per row
#define WIDE_ROW_WORDS (WIDE_HIST + 3 * WIDE_PARTS)  // + maxima, sums, cdf sums (floats) and counts (2 x parts ints)

struct WideArgs {
    const float* logits;
    int ld, n, part_len;
    unsigned long long* ws;      // [rows][WIDE_ROW_WORDS], zero when the first kernel starts
    const float* r;
    float temperature, top_p;
    int* out;
};

struct WideRow {
    unsigned long long* hist;    // [2][4][256]
    float *pmax, *psum, *pcdf;   // [WIDE_PARTS] each
    int* cnt;                    // [2][WIDE_PARTS]
};

__device__ __forceinline__ WideRow wide_row(const WideArgs& a, int row) {
    WideRow w;
    w.hist = a.ws + (size_t)row * WIDE_ROW_WORDS;
    w.pmax = reinterpret_cast<float*>(w.hist + WIDE_HIST);
    w.psum = w.pmax + WIDE_PARTS;
    w.pcdf = w.psum + WIDE_PARTS;
    w.cnt = reinterpret_cast<int*>(w.pcdf + WIDE_PARTS);
    return w;
}

// The row's maximum and sum from the per-part tables, in part order (every thread computes them: 64 loads).
__device__ __forceinline__ void wide_stats(const WideRow& w, float& mx, float& total) {
    mx = -INFINITY;
    for (int p = 0; p < WIDE_PARTS; ++p) mx = fmaxf(mx, w.pmax[p]);
    total = 0.f;
    for (int p = 0; p < WIDE_PARTS; ++p) total += w.psum[p];
}

// One level of the descent, decided by a whole wave from the level's 256 sums (lane l holds the bins
// 4l .. 4l+3): the highest bin b with a non-zero sum for which above + sum(bins >= b) exceeds the bound,
// else the lowest non-zero bin (bin 0 when all are empty); `above` becomes the sum over the bins above it.
// The same choice as the loop over the bins from 255 down in descend().
__device__ __forceinline__ int wide_choose(const unsigned long long h[4], unsigned long long& above,
                                           unsigned long long bound, int lane) {
    unsigned long long own = h[0] + h[1] + h[2] + h[3];
    unsigned long long suf = own;                      // inclusive suffix sum over the lanes (lane 63 first)
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const unsigned lo32 = __shfl_down((unsigned)suf, o, BN_WAVE), hi32 = __shfl_down((unsigned)(suf >> 32), o, BN_WAVE);
        if (lane + o < 64) suf += ((unsigned long long)hi32 << 32) | lo32;
    }
    const unsigned long long higher = above + suf - own;       // above + sum over the bins of higher lanes
    int best = -1, lowest = -1;
    unsigned long long acc_best = 0, acc_low = 0, acc = higher;
#pragma unroll
    for (int j = 3; j >= 0; --j) {
        if (h[j] != 0) {
            lowest = 4 * lane + j; acc_low = acc;
            if (best < 0 && acc + h[j] > bound) { best = 4 * lane + j; acc_best = acc; }
        }
        acc += h[j];
    }
    // the highest lane that found one wins
    const unsigned long long found = __ballot(best >= 0);
    if (found) {
        const int src = 63 - __clzll((long long)found);
        above = ((unsigned long long)__shfl((unsigned)(acc_best >> 32), src, BN_WAVE) << 32) | __shfl((unsigned)acc_best, src, BN_WAVE);
        return __shfl(best, src, BN_WAVE);
    }
    const unsigned long long any = __ballot(lowest >= 0);
    if (any) {
        const int src = __ffsll((long long)any) - 1;   // the lowest lane that has a non-zero bin
        above = ((unsigned long long)__shfl((unsigned)(acc_low >> 32), src, BN_WAVE) << 32) | __shfl((unsigned)acc_low, src, BN_WAVE);
        return __shfl(lowest, src, BN_WAVE);
    }
    return 0;                                          // nothing there: bin 0, `above` as it was
}

struct WideState {            // what a descent has decided so far
    uint32_t prefix, mask;
    unsigned long long above;
};

// Wave 0 replays `levels` levels of descent d from the stored histograms.
__device__ __forceinline__ WideState wide_replay(const WideRow& w, int d, int levels, unsigned long long bound, int lane) {
    WideState st = {0u, 0u, 0ull};
    unsigned long long h[4][4];
#pragma unroll
    for (int l = 0; l < 4; ++l)
#pragma unroll
        for (int j = 0; j < 4; ++j) h[l][j] = l < levels ? w.hist[(d * 4 + l) * 256 + 4 * lane + j] : 0ull;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        if (l < levels) {
            const int shift = 24 - 8 * l;
            const int chosen = wide_choose(h[l], st.above, bound, lane);
            st.prefix |= ((uint32_t)chosen) << shift;
            st.mask |= 255u << shift;
        }
    }
    return st;
}

// The end of a descent: how many elements of the final bit pattern are taken (k) and the sum including them.
__device__ __forceinline__ long long wide_take(const WideState& st, unsigned long long bound, int total,
                                               unsigned long long& cum) {
    const unsigned long long qv = to_fixed(__uint_as_float(st.prefix));
    long long k = 1;
    if (qv > 0 && bound >= st.above) k = (long long)((bound - st.above) / qv) + 1;
    if (k > total) k = total;
    if (k < 1) k = 1;
    cum = st.above + (unsigned long long)k * qv;
    return k;
}

__device__ __forceinline__ int wide_total(const WideRow& w, int d) {
    int t = 0;
    for (int p = 0; p < WIDE_PARTS; ++p) t += w.cnt[d * WIDE_PARTS + p];
    return t;
}

// The bound of descent d: top_p itself for the first, r times the first descent's sum for the second.
__device__ __forceinline__ unsigned long long wide_bound(const WideArgs& a, const WideRow& w, int d, int row, int lane) {
    const unsigned long long b0 = to_fixed(a.top_p);
    if (d == 0) return b0;
    const WideState s0 = wide_replay(w, 0, 4, b0, lane);
    unsigned long long cum0 = 0;
    (void)wide_take(s0, b0, wide_total(w, 0), cum0);
    return (unsigned long long)((double)a.r[row] * (double)cum0);
}

// The probability of one element; every kernel computes it with this one function, so that an element has the
// same bit pattern in every pass.
__device__ __forceinline__ float wide_q(float x, float temperature, float mx, float total) {
    return expf(x / temperature - mx) / total;
}

__device__ __forceinline__ void wide_part(const WideArgs& a, int& lo, int& hi) {
    lo = min(a.n, (int)blockIdx.x * a.part_len);
    hi = min(a.n, lo + a.part_len);
}

__global__ __launch_bounds__(WIDE_THREADS) void wide_max_kernel(WideArgs a) {
    __shared__ float fs[16];
    const int row = blockIdx.y;
    const float* x = a.logits + (size_t)row * a.ld;
    int lo, hi;
    wide_part(a, lo, hi);
    float mx = -INFINITY;
    for (int i = lo + threadIdx.x; i < hi; i += WIDE_THREADS) mx = fmaxf(mx, x[i] / a.temperature);
    mx = block_max(mx, fs);
    if (threadIdx.x == 0) wide_row(a, row).pmax[blockIdx.x] = mx;
}

// CDF != 0: the part's sum of the probabilities (for the plain cdf walk) instead of the exponentials
template <bool CDF>
__global__ __launch_bounds__(WIDE_THREADS) void wide_sum_kernel(WideArgs a) {
    __shared__ float fs[16];
    const int row = blockIdx.y;
    const WideRow w = wide_row(a, row);
    const float* x = a.logits + (size_t)row * a.ld;
    int lo, hi;
    wide_part(a, lo, hi);
    float mx, total = 1.f;
    if (CDF) {
        wide_stats(w, mx, total);
    } else {
        mx = -INFINITY;
        for (int p = 0; p < WIDE_PARTS; ++p) mx = fmaxf(mx, w.pmax[p]);
    }
    float part = 0.f;
    for (int i = lo + threadIdx.x; i < hi; i += WIDE_THREADS) {
        part += CDF ? wide_q(x[i], a.temperature, mx, total) : expf(x[i] / a.temperature - mx);
    }
    part = block_sum(part, fs);
    if (threadIdx.x == 0) (CDF ? w.pcdf : w.psum)[blockIdx.x] = part;
}

// The plain cdf walk: first i with r < cdf_i (src/sampler.c:65-74), n - 1 if none.  The part that holds it is
// found from the parts' sums; one wave of that part's workgroup walks it with a prefix sum over each 64 elements.
__global__ __launch_bounds__(64) void wide_walk_kernel(WideArgs a) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const WideRow w = wide_row(a, row);
    const float rr = a.r[row];
    float c = 0.f, c0 = 0.f;
    int owner = -1;
    for (int p = 0; p < WIDE_PARTS; ++p) {
        const float s = w.pcdf[p];
        if (owner < 0 && rr < c + s) { owner = p; c0 = c; }
        c += s;
    }
    if (owner < 0) { if (blockIdx.x == 0 && lane == 0) a.out[row] = a.n - 1; return; }
    if ((int)blockIdx.x != owner) return;
    float mx, total;
    wide_stats(w, mx, total);
    const float* x = a.logits + (size_t)row * a.ld;
    int lo, hi;
    wide_part(a, lo, hi);
    c = c0;
    int found = hi - 1;
    for (int g0 = lo; g0 < hi; g0 += 64) {
        const int i = g0 + lane;
        float sc = i < hi ? wide_q(x[i], a.temperature, mx, total) : 0.f;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float t = __shfl_up(sc, o, BN_WAVE);
            if (lane >= o) sc += t;
        }
        const unsigned long long m = __ballot(i < hi && rr < c + sc);
        if (m) { found = g0 + __ffsll((long long)m) - 1; break; }
        c += __shfl(sc, 63, BN_WAVE);
    }
    if (lane == 0) a.out[row] = found;
}

// One level of a descent: the sums of the candidates' probabilities by the next 8 bits of their bit pattern.
__global__ __launch_bounds__(WIDE_THREADS) void wide_hist_kernel(WideArgs a, int d, int level) {
    __shared__ unsigned long long hist[256];
    __shared__ uint32_t st_s[2];
    const int row = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const WideRow w = wide_row(a, row);
    hist[threadIdx.x] = 0;                              // 256 threads, 256 bins
    if (wave == 0) {
        const unsigned long long bound = wide_bound(a, w, d, row, lane);
        const WideState st = wide_replay(w, d, level, bound, lane);
        if (lane == 0) { st_s[0] = st.prefix; st_s[1] = st.mask; }
    }
    __syncthreads();
    const uint32_t prefix = st_s[0], mask = st_s[1];
    float mx, total;
    wide_stats(w, mx, total);
    const float cutoff = (1.0f - a.top_p) / (float)(a.n - 1);
    const int shift = 24 - 8 * level;
    const float* x = a.logits + (size_t)row * a.ld;
    int lo, hi;
    wide_part(a, lo, hi);
    for (int i = lo + threadIdx.x; i < hi; i += WIDE_THREADS) {
        const float v = wide_q(x[i], a.temperature, mx, total);
        const uint32_t bits = __float_as_uint(v);
        if (v >= cutoff && (bits & mask) == prefix) atomicAdd(&hist[(bits >> shift) & 255u], to_fixed(v));
    }
    __syncthreads();
    const unsigned long long mine = hist[threadIdx.x];
    if (mine) atomicAdd(&w.hist[(d * 4 + level) * 256 + threadIdx.x], mine);
}

// After the four levels the bit pattern is complete: how many elements of this part have it.
__global__ __launch_bounds__(WIDE_THREADS) void wide_count_kernel(WideArgs a, int d) {
    __shared__ uint32_t st_s[1];
    __shared__ int cs[WIDE_THREADS / 64];
    const int row = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const WideRow w = wide_row(a, row);
    if (wave == 0) {
        const unsigned long long bound = wide_bound(a, w, d, row, lane);
        const WideState st = wide_replay(w, d, 4, bound, lane);
        if (lane == 0) st_s[0] = st.prefix;
    }
    __syncthreads();
    const uint32_t prefix = st_s[0];
    float mx, total;
    wide_stats(w, mx, total);
    const float cutoff = (1.0f - a.top_p) / (float)(a.n - 1);
    const float* x = a.logits + (size_t)row * a.ld;
    int lo, hi;
    wide_part(a, lo, hi);
    int c = 0;
    for (int i = lo + threadIdx.x; i < hi; i += WIDE_THREADS) {
        const float v = wide_q(x[i], a.temperature, mx, total);
        c += (v >= cutoff && __float_as_uint(v) == prefix) ? 1 : 0;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, BN_WAVE);
    if (lane == 0) cs[wave] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int k = 0; k < WIDE_THREADS / 64; ++k) t += cs[k];
        w.cnt[d * WIDE_PARTS + blockIdx.x] = t;
    }
}

// The token: the k-th element, in index order, of those with the second descent's bit pattern.
__global__ __launch_bounds__(64) void wide_pick_kernel(WideArgs a) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const WideRow w = wide_row(a, row);
    const unsigned long long bound = wide_bound(a, w, 1, row, lane);
    const WideState st = wide_replay(w, 1, 4, bound, lane);
    const int total_hits = wide_total(w, 1);
    unsigned long long cum = 0;
    const long long k = wide_take(st, bound, total_hits, cum);
    if (total_hits <= 0) { if (blockIdx.x == 0 && lane == 0) a.out[row] = a.n - 1; return; }
    int seen = 0, owner = WIDE_PARTS - 1, rank = 1;
    for (int p = 0; p < WIDE_PARTS; ++p) {
        const int c = w.cnt[WIDE_PARTS + p];
        if (seen + c >= (int)k) { owner = p; rank = (int)k - seen; break; }
        seen += c;
    }
    if ((int)blockIdx.x != owner) return;
    float mx, total;
    wide_stats(w, mx, total);
    const float cutoff = (1.0f - a.top_p) / (float)(a.n - 1);
    const float* x = a.logits + (size_t)row * a.ld;
    int lo, hi;
    wide_part(a, lo, hi);
    int found = a.n - 1;
    seen = 0;
    for (int g0 = lo; g0 < hi; g0 += 64) {
        const int i = g0 + lane;
        const float v = i < hi ? wide_q(x[i], a.temperature, mx, total) : 0.f;
        unsigned long long m = __ballot(i < hi && v >= cutoff && __float_as_uint(v) == st.prefix);
        const int c = __popcll(m);
        if (seen + c >= rank) {
            for (int skip = rank - seen - 1; skip > 0; --skip) m &= m - 1;       // drop the lower set bits
            found = g0 + __ffsll((long long)m) - 1;
            break;
        }
        seen += c;
    }
    if (lane == 0) a.out[row] = found;
}

// 64-bit words of zeroed work memory that bn_sample_wide needs for `rows` rows.
extern "C" long long bn_sample_wide_words(int rows) { return (long long)rows * WIDE_ROW_WORDS; }

// As bn_sample for temperature > 0, a row spread over WIDE_PARTS workgroups.  ws: bn_sample_wide_words(rows)
// 64-bit words, all zero.
extern "C" int bn_sample_wide(const float* logits, int ld, int rows, int n, unsigned long long* ws, const float* r,
                              float temperature, float top_p, int* out, hipStream_t s) {
    if (rows <= 0 || rows > 65535 || n < 2 || ld < n || !(temperature > 0.f) || !ws || !r || !out) return BN_ERR_ARG;
    WideArgs a;
    a.logits = logits; a.ld = ld; a.n = n; a.ws = ws; a.r = r; a.temperature = temperature; a.top_p = top_p; a.out = out;
    a.part_len = ((n + WIDE_PARTS - 1) / WIDE_PARTS + 63) / 64 * 64;
    const dim3 grid(WIDE_PARTS, rows);
    hipLaunchKernelGGL(wide_max_kernel, grid, dim3(WIDE_THREADS), 0, s, a);
    hipLaunchKernelGGL(wide_sum_kernel<false>, grid, dim3(WIDE_THREADS), 0, s, a);
    if (top_p <= 0.0f || top_p >= 1.0f) {
        hipLaunchKernelGGL(wide_sum_kernel<true>, grid, dim3(WIDE_THREADS), 0, s, a);
        hipLaunchKernelGGL(wide_walk_kernel, grid, dim3(64), 0, s, a);
        return bn_launch_status();
    }
    for (int d = 0; d < 2; ++d) {
        for (int level = 0; level < 4; ++level)
            hipLaunchKernelGGL(wide_hist_kernel, grid, dim3(WIDE_THREADS), 0, s, a, d, level);
        hipLaunchKernelGGL(wide_count_kernel, grid, dim3(WIDE_THREADS), 0, s, a, d);
    }
    hipLaunchKernelGGL(wide_pick_kernel, grid, dim3(64), 0, s, a);
    return bn_launch_status();
}

// work: rows * 64 floats and rows * 64 ints for the two-stage form (may be null: one stage)
extern "C" int bn_argmax(const float* logits, int ld, int rows, int n, int* out, float* work_v, int* work_i,
                         hipStream_t s) {
    if (rows <= 0 || n <= 0 || ld < n) return BN_ERR_ARG;
    if (work_v && work_i && rows <= 256 && n >= 16384 && rows <= 65535) {
        hipLaunchKernelGGL(argmax_part_kernel, dim3(rows, ARGMAX_PARTS), dim3(256), 0, s, logits, ld, n, work_v, work_i);
        hipLaunchKernelGGL(argmax_final_kernel, dim3(rows), dim3(64), 0, s, work_v, work_i, out);
        return bn_launch_status();
    }
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(SMP_THREADS), 0, s, logits, ld, n, out);
    return bn_launch_status();
}

extern "C" int bn_repeat_penalty(float* logits, int ld, int rows, int n, const int* recent, int window,
                                 float penalty, hipStream_t s) {
    if (rows <= 0 || n <= 0 || ld < n || window <= 0 || !(penalty > 0.f)) return BN_ERR_ARG;
    hipLaunchKernelGGL(repeat_penalty_kernel, dim3(rows), dim3(64), 0, s, logits, ld, n, recent, window, penalty);
    return bn_launch_status();
}

extern "C" int bn_sample(const float* logits, int ld, int rows, int n, float* probs, const float* r,
                         float temperature, float top_p, int* out, hipStream_t s) {
    if (rows <= 0 || n <= 0 || ld < n || temperature < 0.f) return BN_ERR_ARG;
    if (temperature != 0.f && (!probs || !r)) return BN_ERR_ARG;
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SMP_THREADS), 0, s, logits, ld, n, probs, r, temperature,
                       top_p, out);
    return bn_launch_status();
}
