// Products of up to 128 activation rows whose result is added to the residual stream (the last product of a
// feed-forward, the output projection of a mixer): P[s, M, N] = X[M, k-range s] . W[N, k-range s]^T,
// float32 partial sums, one slab per k-range; the kernel of the next norm adds the slabs to the stream in
// slab order (elementwise.hip), so no pass of its own forms the sum and the product is never rounded to bf16.
// Same formula as every matrix product here (src/transformer/cpu.c:933-939, :1301-1303).
//
// At these row counts the product is bound by reading W once.  A workgroup of 8 waves owns 128 columns of W
// (16 a wave, loaded straight into the A-operand layout of v_mfma_f32_16x16x32_bf16, the next 256 of K in
// flight while the current ones are multiplied) and one k-range; X is staged once per workgroup and step
// through shared memory (double-buffered, one barrier a step) and read by all 8 waves.  K is split over
// workgroups so that columns/128 x splits is about the number of CUs: a CU pulls its bytes no faster when
// others idle, and a long chain of steps in few workgroups leaves most of the chip waiting.
//
// The same loop with four waves (64 columns a workgroup), K unsplit and a SwiGLU epilogue is the gate/up product of a
// feed-forward at these row counts: W holds gate and up rows interleaved in blocks of 8, a wave's 16 columns are 8 gate
// and 8 up columns of the same 8 outputs, out = silu(gate) * up in bf16 (src/transformer/cpu.c:1164-1304).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

#define SG_WAVES 8                    // waves per workgroup of the partial-sum form
#define SG_COLS (SG_WAVES * 16)       // its columns of W per workgroup
#define SG_GLU_WAVES 4                // waves per workgroup of the SwiGLU form
#define SG_STEP 256                   // K per step
#define SG_XROW 528                   // bytes of a staged row of X: 512 + 16, so that the 16 rows a read touches spread over the banks
#define SG_MAX_ROWS 128

// GLU: P is unused and Y [M, N / 2] (row stride ldy) takes act(gate) * up (bn_gate_act); else Y is unused and P takes
// the partial sums.
template <int MT, int NWV, bool GLU>
__global__ __launch_bounds__(NWV * 64) void splitk_gemm_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W,
                                                               float* __restrict__ P, bf16* __restrict__ Y, int M, int N, int K,
                                                               int ldx, int ldw, int ldy, int k_per_split, int act) {
    extern __shared__ __align__(16) unsigned char xs[];       // [2][MT * 16][SG_XROW]
    constexpr int ROWS = MT * 16;
    constexpr int RP = NWV * 2;                               // rows staged per pass of the workgroup (32 threads a row)
    constexpr int XL = (ROWS + RP - 1) / RP;                  // staging loads per thread and step
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * (NWV * 16) + wave * 16;
    const bf16* wrow = W + (size_t)min(n0 + i, N - 1) * ldw;
    const int k_begin = blockIdx.y * k_per_split;
    const int k_end = min(K, k_begin + k_per_split);
    const int n_steps = (k_end - k_begin + SG_STEP - 1) / SG_STEP;
    const int srow = t >> 5, scol = t & 31;

    f32x4 acc[MT];
#pragma unroll
    for (int a = 0; a < MT; ++a) acc[a] = (f32x4){0.f, 0.f, 0.f, 0.f};
    uint4 wv[8], wn[8], xd[XL];

    // K is a multiple of 8 and so are k_begin and every k below: a 16-byte load at k < k_end stays inside the row
    auto load_x = [&](int k0) {
        const int k = k0 + scol * 8;
#pragma unroll
        for (int j = 0; j < XL; ++j) {
            const int row = srow + RP * j;
            xd[j] = (row < M && k < k_end) ? *reinterpret_cast<const uint4*>(X + (size_t)row * ldx + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto load_w = [&](uint4* dst, int k0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int k = k0 + g * 8 + j * 32;
            dst[j] = (k < k_end) ? *reinterpret_cast<const uint4*>(wrow + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto store_x = [&](int buf) {
        unsigned char* b = xs + (size_t)buf * ROWS * SG_XROW;
#pragma unroll
        for (int j = 0; j < XL; ++j)
            if (srow + RP * j < ROWS) *reinterpret_cast<uint4*>(b + (srow + RP * j) * SG_XROW + scol * 16) = xd[j];
    };

    load_x(k_begin);
    load_w(wv, k_begin);
    store_x(0);
    __syncthreads();
    for (int s = 0; s < n_steps; ++s) {
        const bool more = s + 1 < n_steps;
        if (more) {
            load_x(k_begin + (s + 1) * SG_STEP);
            load_w(wn, k_begin + (s + 1) * SG_STEP);
        }
        const unsigned char* b = xs + (size_t)(s & 1) * ROWS * SG_XROW;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            uint4 xv[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) xv[j] = *reinterpret_cast<const uint4*>(b + (mt * 16 + i) * SG_XROW + j * 64 + g * 16);
#pragma unroll
            for (int j = 0; j < 8; ++j)
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xv[j]), as_bf16x8(wv[j]), acc[mt], 0, 0, 0);
        }
        if (more) {
            store_x((s + 1) & 1);                 // the buffer that the step before this one read: a barrier lies between
#pragma unroll
            for (int j = 0; j < 8; ++j) wv[j] = wn[j];
        }
        __syncthreads();
    }
    // result layout: lane (i, g) holds rows 4g..4g+3 of every 16-row tile at column n0 + i
    if (GLU) {
        // columns n0..n0+7 are gate, n0+8..n0+15 up of outputs n0/2..n0/2+7: lane i < 8 gets its up value from lane i + 8
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float v = acc[mt][r];
                const float up = __shfl_xor(v, 8, BN_WAVE);
                const int m = mt * 16 + 4 * g + r;
                if ((i & 8) == 0 && m < M && n0 + i < N)
                    Y[(size_t)m * ldy + (n0 >> 1) + i] = __float2bfloat16(bn_gate_act(v, act) * up);
            }
        return;
    }
    float* out = P + (size_t)blockIdx.y * M * N;
    if (n0 + i < N) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = mt * 16 + 4 * g + r;
                if (m < M) out[(size_t)m * N + n0 + i] = acc[mt][r];
            }
    }
}

static int sg_compute_units() {
    static int cus = 0;
    if (!cus) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
        else cus = 256;
    }
    return cus;
}

// K per k-range for a product of N columns over K: as many ranges as make column groups x ranges about the
// number of CUs, each a multiple of the step and at least two steps long.
static int sg_k_per_split(int N, int K) {
    const int groups = (N + SG_COLS - 1) / SG_COLS;
    int want = (sg_compute_units() + groups / 2) / groups;
    want = max(1, min(want, K / (2 * SG_STEP)));
    int kps = (K + want - 1) / want;
    return (kps + SG_STEP - 1) / SG_STEP * SG_STEP;
}

// 1 when the kernel takes this product
extern "C" int bn_splitk_gemm_supports(int M, int N, int K, int ldx, int ldw) {
    return (M >= 1 && M <= SG_MAX_ROWS && N >= 1 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldx >= K &&
            ldw >= K) ? 1 : 0;
}

// number of k-ranges (= slabs of the result) for a product of N columns over K
extern "C" int bn_splitk_gemm_splits(int N, int K) {
    if (N < 1 || K < 1) return 0;
    const int kps = sg_k_per_split(N, K);
    return (K + kps - 1) / kps;
}

// P[splits, M, N] (float32, contiguous) = the partial products of X[M, K] (bf16, row stride ldx) and W[N, K] (bf16,
// row stride ldw) over bn_splitk_gemm_splits(N, K) ranges of K.  X and W 16-byte aligned.
extern "C" int bn_splitk_gemm(const void* X, const void* W, float* P, int M, int N, int K, int ldx, int ldw, int splits,
                              hipStream_t s) {
    if (!bn_splitk_gemm_supports(M, N, K, ldx, ldw) || !X || !W || !P) return BN_ERR_ARG;
    if ((((uintptr_t)X | (uintptr_t)W | (uintptr_t)P) & 15) || splits != bn_splitk_gemm_splits(N, K)) return BN_ERR_ARG;
    const int kps = sg_k_per_split(N, K);
    const int MT = (M + 15) / 16;
    const dim3 grid((N + SG_COLS - 1) / SG_COLS, splits), block(SG_WAVES * 64);
    const size_t smem = (size_t)2 * MT * 16 * SG_XROW;
    auto go = [&](auto kernel) {
        // Every instantiation decays to the same pointer type, so this lambda exists once: the flags are kept per MT.
        static bool raised[SG_MAX_ROWS / 16 + 1] = {false};
        if (smem > 64 * 1024 && !raised[MT]) {    // more than the default limit of dynamic shared memory
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            raised[MT] = true;
        }
        hipLaunchKernelGGL(kernel, grid, block, smem, s, (const bf16*)X, (const bf16*)W, P, (bf16*)nullptr, M, N, K, ldx, ldw, 0,
                           kps, 0);
        return bn_launch_status();
    };
    switch (MT) {
        case 1: return go(splitk_gemm_kernel<1, SG_WAVES, false>);
        case 2: return go(splitk_gemm_kernel<2, SG_WAVES, false>);
        case 3: return go(splitk_gemm_kernel<3, SG_WAVES, false>);
        case 4: return go(splitk_gemm_kernel<4, SG_WAVES, false>);
        case 5: return go(splitk_gemm_kernel<5, SG_WAVES, false>);
        case 6: return go(splitk_gemm_kernel<6, SG_WAVES, false>);
        case 7: return go(splitk_gemm_kernel<7, SG_WAVES, false>);
        case 8: return go(splitk_gemm_kernel<8, SG_WAVES, false>);
    }
    return BN_ERR_ARG;
}

// Y[M, F] (bf16, row stride ldy) = act(X . Wg^T) * (X . Wu^T) for W [2F, K] with gate and up rows interleaved in blocks
// of 8 (F a multiple of 8); X, W as above; act one of BN_ACT_*.
extern "C" int bn_splitk_gemm_swiglu(const void* X, const void* W, void* Y, int M, int F, int K, int ldx, int ldw, int ldy,
                                     int act, hipStream_t s) {
    if (act < 0 || act >= BN_ACT_KINDS) return BN_ERR_ARG;
    if (F < 8 || F % 8 || F > (1 << 29) || !bn_splitk_gemm_supports(M, 2 * F, K, ldx, ldw) || !X || !W || !Y || ldy < F)
        return BN_ERR_ARG;
    if (((uintptr_t)X | (uintptr_t)W) & 15) return BN_ERR_ARG;
    const int N = 2 * F, MT = (M + 15) / 16;
    const int kps = (K + SG_STEP - 1) / SG_STEP * SG_STEP;
    const dim3 grid((N + SG_GLU_WAVES * 16 - 1) / (SG_GLU_WAVES * 16), 1), block(SG_GLU_WAVES * 64);
    const size_t smem = (size_t)2 * MT * 16 * SG_XROW;
    auto go = [&](auto kernel) {
        static bool raised[SG_MAX_ROWS / 16 + 1] = {false};       // per MT, as above
        if (smem > 64 * 1024 && !raised[MT]) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            raised[MT] = true;
        }
        hipLaunchKernelGGL(kernel, grid, block, smem, s, (const bf16*)X, (const bf16*)W, (float*)nullptr, (bf16*)Y, M, N, K, ldx,
                           ldw, ldy, kps, act);
        return bn_launch_status();
    };
    switch (MT) {
        case 1: return go(splitk_gemm_kernel<1, SG_GLU_WAVES, true>);
        case 2: return go(splitk_gemm_kernel<2, SG_GLU_WAVES, true>);
        case 3: return go(splitk_gemm_kernel<3, SG_GLU_WAVES, true>);
        case 4: return go(splitk_gemm_kernel<4, SG_GLU_WAVES, true>);
        case 5: return go(splitk_gemm_kernel<5, SG_GLU_WAVES, true>);
        case 6: return go(splitk_gemm_kernel<6, SG_GLU_WAVES, true>);
        case 7: return go(splitk_gemm_kernel<7, SG_GLU_WAVES, true>);
        case 8: return go(splitk_gemm_kernel<8, SG_GLU_WAVES, true>);
    }
    return BN_ERR_ARG;
}
