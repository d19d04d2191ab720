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
