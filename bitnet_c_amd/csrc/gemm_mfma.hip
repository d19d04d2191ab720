// Prompt-phase matrix product for bf16 on the matrix cores: Y[M, N] = X[M, K] . W[N, K]^T for many
// rows of activations, with float32 accumulation and a bf16 or float32 result.  It is the
// library-free form of the reference's batched products (src/gpu_cuda.cu:11571 hands them to a
// library; its own tiled kernels are src/gpu_cuda.cu:4012-4170), written for 64-wide waves and
// v_mfma_f32_16x16x32_bf16.
//
// A workgroup of eight waves (2 x 4, two waves on every SIMD so that one multiplies while the other
// waits for shared memory) owns a tile of 256 rows of X by BN (256, 192 or 128) rows of W and
// walks K in steps of 64.  Both operands are K-contiguous, so a lane's MFMA operand is 16
// contiguous bytes of one row.  A step's two tiles are fetched with 16-byte loads (eight threads
// cover the 128 bytes of a row) into registers while earlier steps are multiplied, then parked
// in the other half of shared memory: one barrier a step.  The narrower tiles have registers for
// a second set of loads and fetch two steps ahead.  The loop's body has no branch (rows past the
// end are clamped, a K tail is peeled off), and scheduling barriers keep the loads ahead of the
// products and the stores behind them: left alone, the compiler moves the loads down to their
// stores and every step waits out the memory latency.  A wave raises its priority while it
// multiplies, so that the matrix instructions of one wave are not held up by the loads and
// stores that the other wave of its SIMD issues (+3 to 6 %).  Rows are stored without padding and
// their 16-byte chunks swizzled (chunk c of row r at c ^ swizzle(r)) so that the sixteen lanes
// which shared memory serves together never meet in a bank.
//
// W is the A operand and X the B operand of the instruction: a lane then holds four consecutive
// columns n of one row m of the result, which it stores as one 8- or 16-byte word.  With gate and
// up rows interleaved in blocks of 8 (GLU8, see skinny_gemm.hip) the two halves of eight result
// columns sit in lanes 32 apart of the same tile, and the epilogue writes silu(gate) * up
// (src/transformer/cpu_backend.c:385-391) instead of the product.
//
// Workgroups are numbered so that the eight XCDs (consecutive workgroup ids go to consecutive
// XCDs, each with an L2 of its own) each take a band of W and run through all row tiles of X for
// it: a tile of W comes from HBM once.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define GM_BM 256             // rows of X per workgroup
#define GM_BK 64              // K elements per step: a tile row is 128 bytes, 8 chunks of 16 bytes
#define GM_XCDS 8
#ifndef GM_WGM
#define GM_WGM 2              // waves of a workgroup along the rows of X ...
#endif
#ifndef GM_WGN
#define GM_WGN 4              // ... and along the rows of W
#endif
#define GM_THREADS (64 * GM_WGM * GM_WGN)

__device__ __forceinline__ bf16x8 gm_as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

// Shared memory serves a 16-byte read in four turns of 16 lanes; in the operand layout
// (lane = i + 16 g reads chunk c0 + g of row i) a turn holds two values of g and, for each, two
// values of i / 4.  Two 128-byte rows share the 256 bytes that the banks span: the row's lowest
// bit separates them, bit 1 goes into bit 2 of the chunk, and (-(i / 4)) & 3 makes g ^ h distinct
// over a turn.
__device__ __forceinline__ int gm_swizzle(int row) {
    return ((-(row >> 2)) & 3) | (((row >> 1) & 1) << 2);
}

template <int BN, bool GLU8, typename TO>
__global__ __launch_bounds__(GM_THREADS) void gemm_mfma_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W,
                                                               TO* __restrict__ Y, int M, int N, int K, int ldx, int ldw,
                                                               int ldy, int tiles_m, int tiles_n, int vec, int act) {
    constexpr int WM = GM_BM / GM_WGM, WN = BN / GM_WGN;      // a wave's part of the tile
    constexpr int MT = WM / 16, NT = WN / 16;         // 16 x 16 result tiles of a wave: MT x NT
    constexpr int PASS = GM_THREADS / 8;              // rows staged by one pass of the workgroup
    constexpr int XL = GM_BM / PASS, WL = BN / PASS;  // staging loads per thread and step
    extern __shared__ __align__(16) unsigned char smem[];     // [2][(GM_BM + BN) rows][128 bytes]
    constexpr int STAGE = (GM_BM + BN) * 128;

    // workgroup -> tile: XCD x takes the column tiles x, x + 8, ...; inside an XCD the row tiles run fastest
    const int xcd = blockIdx.x % GM_XCDS, local = blockIdx.x / GM_XCDS;
    const int tn = xcd + GM_XCDS * (local / tiles_m), tm = local % tiles_m;
    if (tn >= tiles_n) return;                        // the grid is padded to a multiple of 8 column tiles
    const int m0 = tm * GM_BM, n0 = tn * BN;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int wm = (wave / GM_WGN) * WM, wn = (wave % GM_WGN) * WN;
    const int srow = t >> 3, schunk = t & 7;          // staging: 8 threads a row

    f32x4 acc[NT][MT];
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
        for (int b = 0; b < MT; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

    struct Regs { uint4 x[XL]; uint4 w[WL]; };
    // rows past the end are clamped (their results are dropped), so that a full step's loads carry no predicate
    const bf16* xbase = X + (size_t)min(m0 + srow, M - 1) * ldx + schunk * 8;
    const bf16* wbase = W + (size_t)min(n0 + srow, N - 1) * ldw + schunk * 8;
    const int xrows_left = M - 1 - (m0 + srow), wrows_left = N - 1 - (n0 + srow);
    auto fetch_full = [&](Regs& r, int k0) {
#pragma unroll
        for (int j = 0; j < XL; ++j)
            r.x[j] = *reinterpret_cast<const uint4*>(xbase + (size_t)max(0, min(PASS * j, xrows_left)) * ldx + k0);
#pragma unroll
        for (int j = 0; j < WL; ++j)
            r.w[j] = *reinterpret_cast<const uint4*>(wbase + (size_t)max(0, min(PASS * j, wrows_left)) * ldw + k0);
    };
    auto fetch_tail = [&](Regs& r, int k0) {
        const bool in = k0 + schunk * 8 < K;
#pragma unroll
        for (int j = 0; j < XL; ++j)
            r.x[j] = in ? *reinterpret_cast<const uint4*>(xbase + (size_t)max(0, min(PASS * j, xrows_left)) * ldx + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < WL; ++j)
            r.w[j] = in ? *reinterpret_cast<const uint4*>(wbase + (size_t)max(0, min(PASS * j, wrows_left)) * ldw + k0) : make_uint4(0, 0, 0, 0);
    };
    auto park = [&](const Regs& r, int buf) {
        unsigned char* xs = smem + (size_t)buf * STAGE;
        unsigned char* ws = xs + GM_BM * 128;
#pragma unroll
        for (int j = 0; j < XL; ++j) {
            const int row = srow + PASS * j;
            *reinterpret_cast<uint4*>(xs + row * 128 + ((schunk ^ gm_swizzle(row & 15)) << 4)) = r.x[j];
        }
#pragma unroll
        for (int j = 0; j < WL; ++j) {
            const int row = srow + PASS * j;
            *reinterpret_cast<uint4*>(ws + row * 128 + ((schunk ^ gm_swizzle(row & 15)) << 4)) = r.w[j];
        }
    };
    const int swz = gm_swizzle(i);
    auto multiply = [&](int buf) {
        const unsigned char* xs = smem + (size_t)buf * STAGE;
        const unsigned char* ws = xs + GM_BM * 128;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const int coff = ((kk * 4 + g) ^ swz) << 4;
            uint4 xf[MT], wf[NT];
#pragma unroll
            for (int b = 0; b < MT; ++b) xf[b] = *reinterpret_cast<const uint4*>(xs + (wm + b * 16 + i) * 128 + coff);
#pragma unroll
            for (int a = 0; a < NT; ++a) wf[a] = *reinterpret_cast<const uint4*>(ws + (wn + a * 16 + i) * 128 + coff);
#pragma unroll
            for (int a = 0; a < NT; ++a)
#pragma unroll
                for (int b = 0; b < MT; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gm_as_bf16x8(wf[a]), gm_as_bf16x8(xf[b]), acc[a][b], 0, 0, 0);
        }
    };

    const int n_steps = (K + GM_BK - 1) / GM_BK;
    const int full = K / GM_BK;                       // steps that need no K guard
    constexpr bool TWO = BN < 256;                    // a second set of staging registers: loads two steps ahead
    Regs r0, r1;
    int s = 0;
    if (TWO) {
        fetch_tail(r0, 0);
        if (n_steps > 1) fetch_tail(r1, GM_BK);
        park(r0, 0);
        __syncthreads();
        // even s: buffer 0 holds step s, r1 step s + 1 (on its way), r0 is free
        for (; s + 3 < full; s += 2) {
            fetch_full(r0, (s + 2) * GM_BK);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(1);
            multiply(0);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            park(r1, 1);
            __syncthreads();
            fetch_full(r1, (s + 3) * GM_BK);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(1);
            multiply(1);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            park(r0, 0);
            __syncthreads();
        }
        // the rest one step ahead: the step on its way is parked first, then r0 alone carries on
        if (s < n_steps) {
            __builtin_amdgcn_s_setprio(1);
            multiply(0);
            __builtin_amdgcn_s_setprio(0);
            if (s + 1 < n_steps) park(r1, 1);
            __syncthreads();
            ++s;
        }
        for (; s < n_steps; ++s) {
            const bool more = s + 1 < n_steps;
            if (more) fetch_tail(r0, (s + 1) * GM_BK);
            __builtin_amdgcn_s_setprio(1);
            multiply(s & 1);
            __builtin_amdgcn_s_setprio(0);
            if (more) park(r0, (s + 1) & 1);
            __syncthreads();
        }
    } else {
        if (full > 0) fetch_full(r0, 0); else fetch_tail(r0, 0);
        park(r0, 0);
        __syncthreads();
        for (; s + 1 < full; ++s) {                   // the next step is a full one: no branch in the body
            fetch_full(r0, (s + 1) * GM_BK);
            __builtin_amdgcn_sched_barrier(0);        // the loads stay ahead of the products ...
            __builtin_amdgcn_s_setprio(1);
            multiply(s & 1);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);        // ... and the stores of their data behind them
            park(r0, (s + 1) & 1);
            __syncthreads();
        }
        for (; s < n_steps; ++s) {
            const bool more = s + 1 < n_steps;
            if (more) fetch_tail(r0, (s + 1) * GM_BK);
            __builtin_amdgcn_s_setprio(1);
            multiply(s & 1);
            __builtin_amdgcn_s_setprio(0);
            if (more) park(r0, (s + 1) & 1);
            __syncthreads();
        }
    }

    // acc[a][b]: lane (i, g) holds columns n = 4g..4g+3 of row m = i of the result tile (a, b); vec: rows of Y
    // are aligned so that the four go out as one word
    auto store4 = [&](TO* dst, f32x4 v, int valid) {
        if (vec && valid >= 4) {
            if (sizeof(TO) == 4) {
                *reinterpret_cast<f32x4*>(dst) = v;
            } else {
                uint2 p;
                p.x = (uint32_t)__builtin_bit_cast(uint16_t, __float2bfloat16(v[0])) |
                      ((uint32_t)__builtin_bit_cast(uint16_t, __float2bfloat16(v[1])) << 16);
                p.y = (uint32_t)__builtin_bit_cast(uint16_t, __float2bfloat16(v[2])) |
                      ((uint32_t)__builtin_bit_cast(uint16_t, __float2bfloat16(v[3])) << 16);
                *reinterpret_cast<uint2*>(dst) = p;
            }
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (r < valid) dst[r] = from_f32<TO>(v[r]);
        }
    };
#pragma unroll
    for (int a = 0; a < NT; ++a) {
        const int n = n0 + wn + a * 16 + 4 * g;
#pragma unroll
        for (int b = 0; b < MT; ++b) {
            const int m = m0 + wm + b * 16 + i;
            f32x4 v = acc[a][b];
            if (GLU8) {
                // rows 16t..16t+7 of W are gates, 16t+8..16t+15 the ups of the same result columns:
                // lanes with g >= 2 hold the ups of what lanes g - 2 hold the gates of
                f32x4 up;
#pragma unroll
                for (int r = 0; r < 4; ++r) up[r] = __shfl_xor(v[r], 32, BN_WAVE);
                if (g < 2 && m < M) {
                    const int f = ((n0 + wn + a * 16) >> 1) + 4 * g;      // result column of v[0]
#pragma unroll
                    // silu(g) * u with the hardware's exp2 and reciprocal (an ulp each, far below the result's
                    // rounding): expf and a division cost 25 vector instructions a value, a tenth of this kernel's time
                    for (int r = 0; r < 4; ++r)
                        v[r] = (act == BN_ACT_SILU ? v[r] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * v[r]))
                                                   : bn_gate_act(v[r], act)) * up[r];
                    store4(Y + (size_t)m * ldy + f, v, (N >> 1) - f);
                }
            } else if (m < M) {
                store4(Y + (size_t)m * ldy + n, v, N - n);
            }
        }
    }
}

template <int BN, bool GLU8, typename TO>
static int gm_launch(const void* X, const void* W, void* Y, int M, int N, int K, int ldx, int ldw, int ldy, int act,
                     hipStream_t s) {
    auto kernel = gemm_mfma_kernel<BN, GLU8, TO>;
    const size_t smem = (size_t)2 * (GM_BM + BN) * 128;
    static bool raised = false;                       // per instantiation
    if (!raised) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return (int)e;
        raised = true;
    }
    const int tiles_m = (M + GM_BM - 1) / GM_BM, tiles_n = (N + BN - 1) / BN;
    const int bands = (tiles_n + GM_XCDS - 1) / GM_XCDS;           // column tiles per XCD
    const long long grid = (long long)bands * GM_XCDS * tiles_m;
    if (grid > 0x7fffffffLL) return BN_ERR_ARG;
    const int vec = (ldy % 4 == 0 && ((uintptr_t)Y % (4 * sizeof(TO))) == 0) ? 1 : 0;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(GM_THREADS), smem, s, (const bf16*)X, (const bf16*)W, (TO*)Y,
                       M, N, K, ldx, ldw, ldy, tiles_m, tiles_n, vec, act);
    return bn_launch_status();
}

static int gm_compute_units() {
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) cus = p.multiProcessorCount;
        if (cus <= 0) cus = 256;
    }
    return cus;
}

static int gm_pick_bn(int M, int N, int cus) {
    const int widths[3] = {256, 192, 128};
    const int weight[3] = {100, 104, 112};            // cost of a result column, relative
    const long long tiles_m = (M + GM_BM - 1) / GM_BM;
    long long best = -1;
    int pick = 128;
    for (int c = 0; c < 3; ++c) {
        const long long wgs = tiles_m * ((N + widths[c] - 1) / widths[c]);
        const long long cost = ((wgs + cus - 1) / cus) * widths[c] * weight[c];
        if (best < 0 || cost < best) { best = cost; pick = widths[c]; }
    }
    return pick;
}

// 1 if the kernel takes the shape.
extern "C" int bn_gemm_mfma_supports(int M, int N, int K, int ldx, int ldw) {
    return (M >= 1 && N >= 1 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldx >= K && ldw >= K) ? 1 : 0;
}

// out_dtype: type of Y (bf16 or float32).  glu8 != 0: W has 2N rows, gate and up interleaved in
// blocks of 8 (N a multiple of 8), and Y[M, N] = act(gate) * up, act one of BN_ACT_*.  width: the tile's rows of W
// (256, 192 or 128), or 0 for the one that suits the shape.
extern "C" int bn_gemm_mfma(int out_dtype, const void* X, const void* W, void* Y, int M, int N, int K, int ldx, int ldw,
                            int ldy, int glu8, int act, int width, hipStream_t s) {
    if (!bn_gemm_mfma_supports(M, N, K, ldx, ldw) || ldy < N || act < 0 || act >= BN_ACT_KINDS) return BN_ERR_ARG;
    if (width != 0 && width != 256 && width != 192 && width != 128) return BN_ERR_ARG;
    if (((uintptr_t)X | (uintptr_t)W) & 15) return BN_ERR_ARG;
    if (out_dtype != BN_DT_BF16 && out_dtype != BN_DT_F32) return BN_ERR_DTYPE;
    if (glu8) {
        if (N % 8) return BN_ERR_ARG;
        N *= 2;                                       // rows of W
    }
    // The tile width: the one with the least work on the busiest CU (rounds of workgroups over the
    // CUs times the width), a wider tile counting a little less than its width because it reads
    // less of X per result.
    const int bn = width ? width : gm_pick_bn(M, N, gm_compute_units());
    const bool f32 = out_dtype == BN_DT_F32;
#define GM_GO(BN_, GLU_)                                                                          \
    return f32 ? gm_launch<BN_, GLU_, float>(X, W, Y, M, N, K, ldx, ldw, ldy, act, s)             \
               : gm_launch<BN_, GLU_, bf16>(X, W, Y, M, N, K, ldx, ldw, ldy, act, s)
    if (glu8) {
        if (bn == 256) { GM_GO(256, true); }
        if (bn == 192) { GM_GO(192, true); }
        GM_GO(128, true);
    }
    if (bn == 256) { GM_GO(256, false); }
    if (bn == 192) { GM_GO(192, false); }
    GM_GO(128, false);
#undef GM_GO
}
