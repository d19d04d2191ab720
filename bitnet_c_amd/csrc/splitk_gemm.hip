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
// The staged rows are swizzled: shared memory serves a 16-byte read of a wave in four turns of 16 lanes (the
// quads of lanes {0, 3, 5, 6} or {1, 2, 4, 7} of each half of the wave), and with lane = row + 16 g of the
// operand layout a turn mixes two values of g; chunk c of row r at c ^ (r & 15) keeps the sixteen lanes of every
// turn in sixteen different groups of banks, for the fragments' reads and for the staging stores alike (with rows
// padded to 528 bytes instead, four reads in ten met a conflict).  Steps that lie wholly inside the k-range load
// without a test per load, and the two sets of weight registers swap roles from step to step instead of being
// copied: a fifth of the vector instructions of the loop's first form.
// Up to 64 rows the loop runs further ahead: three sets of weight registers take the weights of the step after the next
// while the current ones are multiplied, and a step parks the activations that the step before it asked for.  Its loads
// and stores are straight-line code for that (every thread loads, rows past M a second time, and stores, rows past the tile
// into a spare row): with a load or a store under a branch the compiler waits for every load in flight at the next use of
// any, which ended each step with the weights it had just asked for.  (8B shape, 64 rows: gate/up 50.1 -> 47.2 us, the
// partial-sum products 20.0 -> 18.3.  With more rows the three sets do not fit into the registers.)
//
// TILED: W is a copy laid out for this way of reading it (the streamed copy of common.h): tiles of tile_rows <= 16 rows x
// 32 columns in the lanes' order, the tiles of one block of rows one after another along K.  A load of a wave is then
// one run of 64 tile_rows bytes and a wave's whole stream one run of memory, where the row-major matrix gives 64 bytes
// in each of 16 rows: measured 5 to 15 % faster at every shape tried (8B down product, 64 rows: 29.2 -> 26.8 us; 70B
// gate/up, 17 rows: 192 -> 165).  ldw is then the number of tiles along K, and a wave owns tile_rows columns.
//
// The same loop with K unsplit and a SwiGLU epilogue is the gate/up product of a feed-forward, from one row on: W holds
// gate and up rows interleaved in blocks of 8, a wave's 16 columns are 8 gate and 8 up columns of the same 8 outputs,
// out = silu(gate) * up in bf16 (src/transformer/cpu.c:1164-1304).  Its workgroups have four waves, or seven over a tiled W where that
// leaves the busiest CU fewer columns (1,792 column tiles over 256 CUs: 256 workgroups of seven waves, one a CU, where
// 448 of four waves give every other CU two; over a row-major W four waves were fastest at every shape).  Where the activations are the copy that a deferred norm
// leaves (the stream times the norm's weights), the rows' 1/sqrt(mean(x^2) + eps) (src/transformer/rmsnorm_scalar.c:4-13)
// multiplies gate and up in the epilogue: the sums of squares arrive in parts, which every workgroup adds up in a fixed
// order while its first weights are on their way.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

#define SG_WAVES 8                    // waves per workgroup of the partial-sum form
#define SG_COLS (SG_WAVES * 16)       // its columns of W per workgroup
#define SG_GLU_WAVES 4                // waves per workgroup of the SwiGLU form
#define SG_GLU_WIDE_WAVES 7           // or, over a tiled W, where it spreads the columns more evenly
#define SG_STEP 256                   // K per step
#define SG_XROW 512                   // bytes of a staged row of X: its 32 chunks of 16 bytes lie swizzled, chunk c of row r at c ^ (r & 15)
#define SG_MAX_ROWS 128

// A deferred norm's sums of squares: slots [M, n_slots], null for none.
struct SgNorm {
    const float* slots;
    int n_slots;
    float inv_width, eps;             // 1 / columns of the stream, the norm's eps
    int per_row;                      // lanes that share a row's parts: the power of two >= min(n_slots, 64)
};
#define SG_NORM_PASSES 4              // a wave adds up the parts of at most this many groups of 64 / per_row rows,
#define SG_NORM_LOADS 8               // each lane at most this many parts of a row

// GLU: P is unused and Y [M, N / 2] (row stride ldy) takes act(gate) * up (bn_gate_act), both scaled by the row's factor
// if nrm brings one; else Y and nrm are unused and P takes the partial sums.
template <int MT, int NWV, bool GLU, bool TILED>
__global__ __launch_bounds__(NWV * 64) void splitk_gemm_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W,
                                                               float* __restrict__ P, bf16* __restrict__ Y, int M, int N, int K,
                                                               int ldx, int ldw, int ldy, int k_per_split, int act, SgNorm nrm,
                                                               int tile_rows) {
    extern __shared__ __align__(16) unsigned char xs[];       // [2][MT * 16][SG_XROW], GLU: then MT * 16 row factors
    constexpr int ROWS = MT * 16;
    constexpr int RP = NWV * 2;                               // rows staged per pass of the workgroup (32 threads a row)
    constexpr int XL = (ROWS + RP - 1) / RP;                  // staging loads per thread and step
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int CW = TILED ? tile_rows : 16;                    // columns of the result that a wave owns
    const int n0 = (blockIdx.x * NWV + wave) * CW;
    const bool col = i < CW;
    // row-major: this lane's row (rows past N are computed and dropped); tiled: this lane's 16 bytes of the wave's first
    // tile (the last block of rows stands in for a wave past the end)
    const int TS = CW * BN_STREAM_TILE_COLS;                  // elements of a tile
    // (the wave's row of tiles is a base in scalar registers, the lane adds its 16 bytes' place at the load)
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const bf16* wrow = TILED ? W + (size_t)min((int)(blockIdx.x * NWV + wave_u), (N - 1) / CW) * ldw * TS
                             : W + (size_t)min(n0 + i, N - 1) * ldw;
    const unsigned lane_at = TILED ? (g * CW + i) * 8 : 0;
    const int k_begin = blockIdx.y * k_per_split;
    const int k_end = min(K, k_begin + k_per_split);
    const int n_steps = (k_end - k_begin + SG_STEP - 1) / SG_STEP;
    const int srow = t >> 5, scol = t & 31;

    f32x4 acc[MT];
#pragma unroll
    for (int a = 0; a < MT; ++a) acc[a] = (f32x4){0.f, 0.f, 0.f, 0.f};
    uint4 wa[8], wb[8], xd[XL];

    // K is a multiple of 8 and so are k_begin and every k below: a 16-byte load at k < k_end stays inside the row.
    // A step that lies wholly inside [k_begin, k_end) needs no test per load.
    auto load_x = [&](int k0) {
        const int k = k0 + scol * 8;
        const bool whole = k0 + SG_STEP <= k_end;
#pragma unroll
        for (int j = 0; j < XL; ++j) {
            const int row = srow + RP * j;
            xd[j] = (row < M && (whole || k < k_end)) ? *reinterpret_cast<const uint4*>(X + (size_t)row * ldx + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto load_w = [&](uint4* dst, int k0) {
        // load j: columns k0 + 32 j + 8 g .. + 7 of the lane's row; in the tiled copy that is tile k0 / 32 + j (whose
        // columns past K hold zeros, so a tile that begins below k_end is read whole)
        const int JS = TILED ? TS : 32;
        const bf16* p = TILED ? wrow + (size_t)(k0 >> 5) * TS + lane_at : wrow + k0 + g * 8;
        const int kl = TILED ? k0 : k0 + g * 8;
        if (col && k0 + SG_STEP <= k_end) {
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[j] = *reinterpret_cast<const uint4*>(p + j * JS);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                dst[j] = (col && kl + j * 32 < k_end) ? *reinterpret_cast<const uint4*>(p + j * JS) : make_uint4(0, 0, 0, 0);
        }
    };
    auto store_x = [&](int buf) {
        unsigned char* b = xs + (size_t)buf * ROWS * SG_XROW;
#pragma unroll
        for (int j = 0; j < XL; ++j) {
            const int row = srow + RP * j;
            if (row < ROWS) *reinterpret_cast<uint4*>(b + row * SG_XROW + ((scol ^ (row & 15)) << 4)) = xd[j];
        }
    };
    auto multiply = [&](const uint4* w, int buf) {
        const unsigned char* b = xs + (size_t)buf * ROWS * SG_XROW;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            uint4 xv[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)            // chunk 4 j + g of row mt * 16 + i, whose swizzle is i
                xv[j] = *reinterpret_cast<const uint4*>(b + (mt * 16 + i) * SG_XROW + (((4 * j + g) ^ i) << 4));
#pragma unroll
            for (int j = 0; j < 8; ++j)
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xv[j]), as_bf16x8(w[j]), acc[mt], 0, 0, 0);
        }
    };
    // one step: the next step's activations and weights are asked for (the weights into the other set of registers),
    // this step is multiplied, the activations are parked in the buffer that the step before this one read
    auto step = [&](const uint4* cur, uint4* next, int st) {
        const bool more = st + 1 < n_steps;
        if (more) {
            load_x(k_begin + (st + 1) * SG_STEP);
            load_w(next, k_begin + (st + 1) * SG_STEP);
        }
        multiply(cur, st & 1);
        if (more) store_x((st + 1) & 1);
        __syncthreads();
    };

    // The same for steps that lie wholly inside the range, in straight-line code: every thread loads (a row past M is
    // row M - 1 again, a lane without a column its neighbour's weights: what comes of them is never stored) and every
    // thread stores (a row past the tile goes to a spare row), so that the compiler can tell the loads apart when it
    // waits and leaves the weights of later steps in flight.
    unsigned char* spare = xs + (size_t)2 * ROWS * SG_XROW + ROWS * sizeof(float);
    const unsigned lane_at_w = TILED ? (g * CW + min(i, CW - 1)) * 8 : 0;
    auto load_x_whole = [&](uint4* dst, int k0) {
#pragma unroll
        for (int j = 0; j < XL; ++j)
            dst[j] = *reinterpret_cast<const uint4*>(X + (size_t)min(srow + RP * j, M - 1) * ldx + k0 + scol * 8);
    };
    auto load_w_whole = [&](uint4* dst, int k0) {
        const int JS = TILED ? TS : 32;
        const bf16* p = TILED ? wrow + (size_t)(k0 >> 5) * TS + lane_at_w : wrow + k0 + g * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[j] = *reinterpret_cast<const uint4*>(p + j * JS);
    };
    auto store_x_all = [&](const uint4* src, int buf) {
        unsigned char* b = xs + (size_t)buf * ROWS * SG_XROW;
#pragma unroll
        for (int j = 0; j < XL; ++j) {
            const int row = srow + RP * j;
            unsigned char* at = row < ROWS ? b + row * SG_XROW + ((scol ^ (row & 15)) << 4) : spare + (scol << 4);
            *reinterpret_cast<uint4*>(at) = src[j];
        }
    };
    const int n_whole = (k_end - k_begin) / SG_STEP;
    const bool piped = MT <= 4 && n_whole >= 5;            // (with more row tiles the three sets of weights do not fit into the registers)
    uint4 wc[8];

    if (piped) {
        load_x_whole(xd, k_begin);
        load_w_whole(wa, k_begin);
    } else {
        load_x(k_begin);
        load_w(wa, k_begin);
    }
    float* scale_s = reinterpret_cast<float*>(xs + (size_t)2 * ROWS * SG_XROW);
    if (GLU && nrm.slots) {
        // A row's parts go to `per` lanes (the power of two that holds them, at most the wave), 64 / per rows to a wave and
        // pass; every load of every pass is asked for before the first sum, the lanes add their parts in order and a tree
        // adds the lanes: a fixed order.  The host has checked that SG_NORM_PASSES passes of SG_NORM_LOADS loads do.
        const int per = nrm.per_row, part = lane & (per - 1), rows_a_pass = NWV * (64 / per);
        const int first = wave * (64 / per) + lane / per;
        float sv[SG_NORM_PASSES][SG_NORM_LOADS];
#pragma unroll
        for (int a = 0; a < SG_NORM_PASSES; ++a)
#pragma unroll
            for (int q = 0; q < SG_NORM_LOADS; ++q) {
                const int m = first + a * rows_a_pass, p2 = part + q * per;
                sv[a][q] = (m < M && p2 < nrm.n_slots) ? nrm.slots[(size_t)m * nrm.n_slots + p2] : 0.f;
            }
#pragma unroll
        for (int a = 0; a < SG_NORM_PASSES; ++a) {
            const int m = first + a * rows_a_pass;
            float v = 0.f;
#pragma unroll
            for (int q = 0; q < SG_NORM_LOADS; ++q) v += sv[a][q];
            for (int o = per >> 1; o >= 1; o >>= 1) v += __shfl_xor(v, o, BN_WAVE);
            if (part == 0 && m < M) scale_s[m] = 1.0f / sqrtf(v * nrm.inv_width + nrm.eps);
        }
    }
    if (piped) {
        store_x_all(xd, 0);
        load_x_whole(xd, k_begin + SG_STEP);
        load_w_whole(wb, k_begin + SG_STEP);
    } else {
        store_x(0);
    }
    __syncthreads();
    int st = 0;
    if (piped) {
        // Weights two steps ahead, activations one and a half: a step parks the next step's activations, which the step
        // before it asked for (parked in the step that asks for them, they make every step wait out the way to the L2 and
        // back), asks for the activations and the weights of the step after the next and multiplies its own.  Three sets
        // of registers take the weights in turn, in triples of steps while five whole steps are left; the rest is done
        // below, one step ahead.
        auto ahead = [&](const uint4* cur, uint4* far, int at) {
            store_x_all(xd, (at + 1) & 1);
            load_x_whole(xd, k_begin + (at + 2) * SG_STEP);
            load_w_whole(far, k_begin + (at + 2) * SG_STEP);
            multiply(cur, at & 1);
            __syncthreads();
        };
        for (; st + 5 <= n_whole; st += 3) {
            ahead(wa, wc, st);
            ahead(wb, wa, st + 1);
            ahead(wc, wb, st + 2);
        }
        // step st: its weights are in wa, the next step's in wb and its activations in xd
        store_x_all(xd, (st + 1) & 1);
        multiply(wa, st & 1);
        __syncthreads();
        ++st;
        for (; st < n_steps; st += 2) {
            step(wb, wc, st);
            if (st + 1 < n_steps) step(wc, wb, st + 1);
        }
    } else {
        for (; st < n_steps; st += 2) {
            step(wa, wb, st);
            if (st + 1 < n_steps) step(wb, wa, st + 1);
        }
    }
    // result layout: lane (i, g) holds rows 4g..4g+3 of every 16-row tile at column n0 + i
    if (GLU) {
        // columns n0..n0+7 are gate, n0+8..n0+15 up of outputs n0/2..n0/2+7: lane i < 8 gets its up value from lane i + 8
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = mt * 16 + 4 * g + r;
                const float v = acc[mt][r] * ((nrm.slots && m < M) ? scale_s[m] : 1.0f);
                const float up = __shfl_xor(v, 8, BN_WAVE);
                if ((i & 8) == 0 && m < M && n0 + i < N)
                    Y[(size_t)m * ldy + (n0 >> 1) + i] = __float2bfloat16(bn_gate_act(v, act) * up);
            }
        return;
    }
    float* out = P + (size_t)blockIdx.y * M * N;
    if (col && n0 + i < N) {
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

// K per k-range for a product whose columns fall into `groups` workgroups: as many ranges as make groups x ranges about
// the number of CUs, each a multiple of the step and at least two steps long.
static int sg_k_per_split(int groups, int K) {
    int want = (sg_compute_units() + groups / 2) / groups;
    want = max(1, min(want, K / (2 * SG_STEP)));
    int kps = (K + want - 1) / want;
    return (kps + SG_STEP - 1) / SG_STEP * SG_STEP;
}
// workgroups along the columns: SG_WAVES waves of 16 columns each, or of tile_rows over a streamed copy
static int sg_groups(int N, int tile_rows) {
    const int cw = tile_rows > 0 ? tile_rows : 16;
    return ((N + cw - 1) / cw + SG_WAVES - 1) / SG_WAVES;
}
static bool sg_tile_rows_ok(int tile_rows) { return tile_rows == 0 || (tile_rows >= 1 && tile_rows <= BN_STREAM_TILE_ROWS); }

// 1 when the kernel takes this product.  tile_rows > 0: W is the streamed copy (common.h) with that many rows a tile and
// ldw its tiles along K; 0: W is row-major with row stride ldw.
extern "C" int bn_splitk_gemm_supports(int M, int N, int K, int ldx, int ldw, int tile_rows) {
    if (!(M >= 1 && M <= SG_MAX_ROWS && N >= 1 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldx >= K)) return 0;
    if (!sg_tile_rows_ok(tile_rows)) return 0;
    return (tile_rows ? ldw == (K + BN_STREAM_TILE_COLS - 1) / BN_STREAM_TILE_COLS : (ldw % 8 == 0 && ldw >= K)) ? 1 : 0;
}

// number of k-ranges (= slabs of the result) for a product of N columns over K (tile_rows as above)
extern "C" int bn_splitk_gemm_splits(int N, int K, int tile_rows) {
    if (N < 1 || K < 1 || !sg_tile_rows_ok(tile_rows)) return 0;
    const int kps = sg_k_per_split(sg_groups(N, tile_rows), K);
    return (K + kps - 1) / kps;
}

// Launches kernel<MT> for the M at hand; smem and the attribute that more than 64 KB of it need are looked after here.
template <int NWV, bool GLU, bool TILED, typename... Args>
static int sg_launch(int M, dim3 grid, hipStream_t s, Args... args) {
    const int MT = (M + 15) / 16;
    const size_t smem = (size_t)2 * MT * 16 * SG_XROW + (size_t)MT * 16 * sizeof(float) + SG_XROW;    // two stages, row factors, a spare row
    auto go = [&](auto kernel) {
        static bool raised[SG_MAX_ROWS / 16 + 1] = {false};       // per MT: this function exists once per NWV, GLU, TILED
        if (smem > 64 * 1024 && !raised[MT]) {                    // more than the default limit of dynamic shared memory
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            raised[MT] = true;
        }
        hipLaunchKernelGGL(kernel, grid, dim3(NWV * 64), smem, s, args...);
        return bn_launch_status();
    };
    switch (MT) {
        case 1: return go(splitk_gemm_kernel<1, NWV, GLU, TILED>);
        case 2: return go(splitk_gemm_kernel<2, NWV, GLU, TILED>);
        case 3: return go(splitk_gemm_kernel<3, NWV, GLU, TILED>);
        case 4: return go(splitk_gemm_kernel<4, NWV, GLU, TILED>);
        case 5: return go(splitk_gemm_kernel<5, NWV, GLU, TILED>);
        case 6: return go(splitk_gemm_kernel<6, NWV, GLU, TILED>);
        case 7: return go(splitk_gemm_kernel<7, NWV, GLU, TILED>);
        case 8: return go(splitk_gemm_kernel<8, NWV, GLU, TILED>);
    }
    return BN_ERR_ARG;
}

// P[splits, M, N] (float32, contiguous) = the partial products of X[M, K] (bf16, row stride ldx) and W[N, K] (bf16,
// row stride ldw; tile_rows > 0: the streamed copy, ldw its tiles along K) over bn_splitk_gemm_splits(N, K, tile_rows)
// ranges of K.  X and W 16-byte aligned.
extern "C" int bn_splitk_gemm(const void* X, const void* W, float* P, int M, int N, int K, int ldx, int ldw, int splits,
                              int tile_rows, hipStream_t s) {
    if (!bn_splitk_gemm_supports(M, N, K, ldx, ldw, tile_rows) || !X || !W || !P) return BN_ERR_ARG;
    if ((((uintptr_t)X | (uintptr_t)W | (uintptr_t)P) & 15) || splits != bn_splitk_gemm_splits(N, K, tile_rows)) return BN_ERR_ARG;
    const int groups = sg_groups(N, tile_rows);
    const int kps = sg_k_per_split(groups, K);
    const dim3 grid(groups, splits);
    const SgNorm none{nullptr, 0, 0.f, 0.f, 1};
    if (tile_rows)
        return sg_launch<SG_WAVES, false, true>(M, grid, s, (const bf16*)X, (const bf16*)W, P, (bf16*)nullptr, M, N, K, ldx, ldw,
                                                0, kps, 0, none, tile_rows);
    return sg_launch<SG_WAVES, false, false>(M, grid, s, (const bf16*)X, (const bf16*)W, P, (bf16*)nullptr, M, N, K, ldx, ldw, 0,
                                             kps, 0, none, 0);
}

// Whether workgroups of SG_GLU_WIDE_WAVES waves leave the busiest CU fewer of the N / 16 column tiles than workgroups of
// SG_GLU_WAVES (a CU pulls its bytes no faster when others idle).
static bool sg_glu_wide(int N) {
    const int tiles = (N + 15) / 16, cus = sg_compute_units();
    auto busiest = [&](int w) { return (long long)(((tiles + w - 1) / w + cus - 1) / cus) * w; };
    return busiest(SG_GLU_WIDE_WAVES) < busiest(SG_GLU_WAVES);
}

// Y[M, F] (bf16, row stride ldy) = act(c X . Wg^T) * (c X . Wu^T) for W [2F, K] with gate and up rows interleaved in blocks
// of 8 (F a multiple of 8); X, W as above; tiled: W is the streamed copy with 16 rows a tile (a tile then holds both halves
// of 8 outputs) and ldw its tiles along K; act one of BN_ACT_*.  c is 1 with slots == null; else X is the copy of a
// stream of stream_width columns that a deferred norm leaves, slots [M, n_slots] (contiguous) the parts of its rows' sums
// of squares, and c the row's 1 / sqrt(sum / stream_width + eps).
extern "C" int bn_splitk_gemm_swiglu(const void* X, const void* W, void* Y, int M, int F, int K, int ldx, int ldw, int ldy,
                                     int act, const float* slots, int n_slots, int stream_width, float eps, int tiled,
                                     hipStream_t s) {
    if (act < 0 || act >= BN_ACT_KINDS) return BN_ERR_ARG;
    const int tile_rows = tiled ? 16 : 0;
    if (F < 8 || F % 8 || F > (1 << 29) || !bn_splitk_gemm_supports(M, 2 * F, K, ldx, ldw, tile_rows) || !X || !W || !Y || ldy < F)
        return BN_ERR_ARG;
    if (((uintptr_t)X | (uintptr_t)W) & 15) return BN_ERR_ARG;
    if (slots && (n_slots < 1 || stream_width < 1)) return BN_ERR_ARG;
    int per = 1;
    while (per < 64 && per < n_slots) per <<= 1;
    const SgNorm nrm{slots, n_slots, slots ? 1.0f / (float)stream_width : 0.f, eps, per};
    const int N = 2 * F;
    // the fewest waves a workgroup may have decide whether the passes suffice
    if (slots && ((M + SG_GLU_WAVES * (64 / per) - 1) / (SG_GLU_WAVES * (64 / per)) > SG_NORM_PASSES ||
                  (n_slots + per - 1) / per > SG_NORM_LOADS))
        return BN_ERR_ARG;
    const int kps = (K + SG_STEP - 1) / SG_STEP * SG_STEP;
    auto grid = [&](int waves) { return dim3((N + waves * 16 - 1) / (waves * 16), 1); };
    if (!tiled)
        return sg_launch<SG_GLU_WAVES, true, false>(M, grid(SG_GLU_WAVES), s, (const bf16*)X, (const bf16*)W, (float*)nullptr,
                                                    (bf16*)Y, M, N, K, ldx, ldw, ldy, kps, act, nrm, 0);
    if (sg_glu_wide(N))
        return sg_launch<SG_GLU_WIDE_WAVES, true, true>(M, grid(SG_GLU_WIDE_WAVES), s, (const bf16*)X, (const bf16*)W,
                                                        (float*)nullptr, (bf16*)Y, M, N, K, ldx, ldw, ldy, kps, act, nrm, 16);
    return sg_launch<SG_GLU_WAVES, true, true>(M, grid(SG_GLU_WAVES), s, (const bf16*)X, (const bf16*)W, (float*)nullptr,
                                               (bf16*)Y, M, N, K, ldx, ldw, ldy, kps, act, nrm, 16);
}
