// Decode-phase matrix product for bf16: Y[M, N] = X[M, K] . W[N, K]^T with M <= 64 rows
// of activations, on the matrix cores (v_mfma_f32_16x16x32_bf16).  The weights are
// streamed once from HBM with 16-byte loads, four lanes covering 64 contiguous bytes of
// one weight row per load and a wave 512 bytes of 16 rows per 256-element K chunk; K is split over the waves of a workgroup and
// the partial sums are added through shared memory in wave order, so the result does
// not depend on timing.  It plays the part of the reference's matvec kernels
// (src/gpu_cuda.cu:3976-4010, one warp per output row) and of its stacked gate/up
// matvec followed by the activation (src/gpu_cuda.cu:4176, :8971), written for 64-wide
// waves and MFMA instead.
//
// DUAL: W holds two row blocks (gate rows n, up rows up_off + n); the epilogue writes
// act(gate) * up, act one of the kinds of bn_gate_act (silu(g) = g / (1 + exp(-g)) for this
// architecture, src/transformer/cpu_backend.c:385-391).
// GLU8: the same product with gate and up rows interleaved in blocks of 8 (rows 16t..16t+7 are
// gate rows 8t..8t+7, rows 16t+8..16t+15 the up rows of the same columns): every 16-row tile holds
// both halves of 8 result columns, so the plain kernel does it with half the loads in flight.
//
// The activations: all workgroups read the same X, and a load in the operand layout (one row per
// lane, 64 bytes of it per load) costs a full load instruction however few rows there are.  With
// up to 16 rows (XS) a wave therefore fetches its K chunk of X with dense loads (32 lanes x 16 bytes
// a row), parks it in a region of shared memory of its own (no workgroup barrier) and reads the
// operand fragments from there; the vector memory pipe is left to the weights.
//
// TILED: W is the streamed copy of the matrix (common.h: tiles of up to 16 rows x 32 columns in the lanes' order); a
// load of a wave is then one tile, up to 1 KB of consecutive bytes, ldw the number of tiles along K, and a workgroup
// owns the columns of one row of tiles.  Measured against
// the row-major matrix at 8 rows of an 8B shape: QKV 14.3 -> 13.2 us, output projection 10.7 -> 9.3, gate/up 49.5 ->
// 43.9, down 28.0 -> 24.0.
//
// Needs K % 8 == 0 and 16-byte aligned rows; other shapes go to the tiled kernel.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define SK_CHUNK 256          // K elements per wave iteration

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

#define SK_XROW 528           // bytes between rows of a wave's staged X chunk (512 + 16: conflict-free 16-byte reads)

template <int MT, bool DUAL, typename TO, bool GLU8 = false, bool XS = false, bool TILED = false>
__global__ __launch_bounds__((DUAL && MT >= 3) ? 512 : 1024) void skinny_gemm_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W,
                                                           TO* __restrict__ Y, int M, int N, int K, int ldx,
                                                           int ldw, int ldy, int up_off, int act) {
    constexpr int NA = DUAL ? 2 * MT : MT;            // accumulator tiles per wave
    extern __shared__ __align__(16) float red[];      // [n_waves][NA][64][4]
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);      // a scalar
    const int n_waves = blockDim.x >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int CW = TILED ? up_off : 16;               // columns a workgroup owns; TILED: up_off carries the copy's rows per tile
    const int n0 = blockIdx.x * CW;
    const int n = min(n0 + i, N - 1);                 // clamp: rows past N are computed and dropped
    const int TS = CW * BN_STREAM_TILE_COLS;          // elements of a tile
    // tiled: the row of tiles is the same for all lanes (a base in scalar registers), the lane adds its 16 bytes' place
    const bf16* wrow = TILED ? W + (size_t)blockIdx.x * ldw * TS : W + (size_t)n * ldw;
    const unsigned lane_at = (g * CW + i) * 8;
    const bf16* urow = DUAL ? W + (size_t)(up_off + n) * ldw : nullptr;

    f32x4 acc[NA];
#pragma unroll
    for (int a = 0; a < NA; ++a) acc[a] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // XS: this wave's staging region, after the partial sums
    unsigned char* xs = reinterpret_cast<unsigned char*>(red + (size_t)n_waves * NA * 256) + (size_t)wave * M * SK_XROW;

    for (int kc = wave * SK_CHUNK; kc < K; kc += n_waves * SK_CHUNK) {
        const int kb = kc + g * 8;                    // lane group g: 8 elements of every 32 (64 contiguous bytes per row and load)
        uint4 wv[8], uv[8];
        uint4 xd[8];
        if (XS) {                                     // issued before the weights: loads return in order
            const int xk = kc + (lane & 31) * 8;
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const int row = 2 * r + (lane >> 5);
                if (2 * r < M)
                    xd[r] = (row < M && xk < K) ? *reinterpret_cast<const uint4*>(X + (size_t)row * ldx + xk)
                                                : make_uint4(0, 0, 0, 0);
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int k = kb + j * 32;
            if (TILED)          // tile kc / 32 + j of this block of rows; its columns past K hold zeros
                wv[j] = (i < CW && kc + j * 32 < K) ? *reinterpret_cast<const uint4*>(wrow + (size_t)((kc >> 5) + j) * TS + lane_at)
                                                    : make_uint4(0, 0, 0, 0);
            else
                wv[j] = (k < K) ? *reinterpret_cast<const uint4*>(wrow + k) : make_uint4(0, 0, 0, 0);
            if (DUAL) uv[j] = (k < K) ? *reinterpret_cast<const uint4*>(urow + k) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + i;
            const bf16* xrow = X + (size_t)m * ldx;
            uint4 xv[8];
            if (XS) {
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    const int row = 2 * r + (lane >> 5);
                    if (2 * r < M && row < M)
                        *reinterpret_cast<uint4*>(xs + row * SK_XROW + (lane & 31) * 16) = xd[r];
                }
                __builtin_amdgcn_wave_barrier();      // one wave: its shared-memory operations run in order
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    xv[j] = (m < M) ? *reinterpret_cast<const uint4*>(xs + m * SK_XROW + j * 64 + g * 16)
                                    : make_uint4(0, 0, 0, 0);
                __builtin_amdgcn_wave_barrier();
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int k = kb + j * 32;
                    xv[j] = (m < M && k < K) ? *reinterpret_cast<const uint4*>(xrow + k) : make_uint4(0, 0, 0, 0);
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xv[j]), as_bf16x8(wv[j]), acc[mt], 0, 0, 0);
                if (DUAL)
                    acc[MT + mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xv[j]), as_bf16x8(uv[j]),
                                                                          acc[MT + mt], 0, 0, 0);
            }
        }
    }
    // partial sums of every wave -> shared memory
#pragma unroll
    for (int a = 0; a < NA; ++a)
        *reinterpret_cast<f32x4*>(red + (((size_t)wave * NA + a) * 64 + lane) * 4) = acc[a];
    __syncthreads();
    // thread (l, r): C row 4*(l/16)+r of each tile, column l%16; sums over waves in wave order
    for (int idx = threadIdx.x; idx < MT * 256; idx += blockDim.x) {
        const int mt = idx >> 8, rem = idx & 255;
        const int l = rem & 63, r = rem >> 6;
        float v = 0.f, u = 0.f;
        for (int w = 0; w < n_waves; ++w) {
            v += red[(((size_t)w * NA + mt) * 64 + l) * 4 + r];
            if (DUAL) u += red[(((size_t)w * NA + MT + mt) * 64 + l) * 4 + r];
        }
        const int m = mt * 16 + 4 * (l >> 4) + r;
        const int nn = (l & 15) < CW ? n0 + (l & 15) : N;          // a column past the workgroup's own is nobody's
        if (GLU8) {
            // columns 0..7 of the tile are gates, 8..15 the ups of the same result columns
            const float up = __shfl_xor(v, 8, BN_WAVE);
            if ((l & 8) == 0 && m < M && nn < N)
                Y[(size_t)m * ldy + (n0 >> 1) + (l & 7)] = from_f32<TO>(bn_gate_act(v, act) * up);
        } else if (m < M && nn < N) {
            const float y = DUAL ? bn_gate_act(v, act) * u : v;
            Y[(size_t)m * ldy + nn] = from_f32<TO>(y);
        }
    }
}

// ---------------------------------------------------------------------------------------
// The same product for up to 16 rows with the neighbouring norm folded in, so that a decode layer
// needs no kernel for its two norms:
//   RES: the product is a part's output.  The epilogue adds it to the float32 residual stream in
//        place (its 16 columns), writes a bf16 copy of the new stream multiplied by the next norm's
//        weights, and the sum of the squares of its 16 columns of every row into a slot of its own.
//   PRE: the activations are such a copy.  1/sqrt(mean(x^2) + eps) (src/transformer/rmsnorm_scalar.c:4-13)
//        multiplies a whole row of the result, so it is applied in the epilogue: every wave fetches the
//        slots of two rows before its K loop and adds them up behind it (lane-strided sums, a tree over
//        the lanes: a fixed order); the staged activations need no work at all.  (Asked for later, before
//        the wave's last chunk, the same loads cost three times as much.)
// GLU8 as above.  bf16 result (RES: no result of its own).
#define SK_SLOT_LOADS 8       // slots per row and lane: at most 512 column tiles (a stream of 8,192 columns)

struct SkinnyFused {
    const float* slots_in;    // [M, n_slots] sums of squares, PRE
    int n_slots;
    float inv_width, eps;     // 1 / columns of the stream, the norm's eps, PRE
    float* resid;             // [M, ld_resid] float32 stream, RES
    bf16* resid_bf16;         // [M, ld_rb] its bf16 copy times next_weight, RES
    const float* next_weight; // [N] weights of the norm that reads the copy, RES
    float* slots_out;         // [M, gridDim.x], RES
    int ld_resid, ld_rb;
};

template <bool GLU8, bool PRE, bool RES, int SL, bool TILED>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4)))
void skinny_gemm_fused_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W, bf16* __restrict__ Y, int M, int N,
                              int K, int ldx, int ldw, int ldy, int tile_cols, int act, SkinnyFused f) {
    constexpr int NW = 8;                              // always eight waves: wave w owns rows w and w + 8 of the norm
    extern __shared__ __align__(16) float red[];       // [NW][64][4], then 16 row scales, then the staging
    // the wave's number as a scalar: what depends on it alone (its chunks of K, a tile's address) stays in scalar registers
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, g = lane >> 4;
    // A workgroup owns tile_cols <= 16 columns (the rest of its MFMA tile is not loaded and not stored): the
    // host picks the width that spreads the column tiles evenly over the CUs.
    const int n0 = blockIdx.x * tile_cols;
    const bool col = i < tile_cols;
    const int n = min(n0 + i, N - 1);
    // tiled: tile_cols is the copy's rows per tile and the workgroup's rows are one row of tiles
    const int TS = tile_cols * BN_STREAM_TILE_COLS;
    // (the row of tiles is the same for all lanes, a base in scalar registers; the lane adds its 16 bytes' place)
    const bf16* wrow = TILED ? W + (size_t)blockIdx.x * ldw * TS : W + (size_t)n * ldw;
    const unsigned lane_at = (g * tile_cols + i) * 8;
    float* scale_s = red + NW * 256;
    unsigned char* xs = reinterpret_cast<unsigned char*>(red + NW * 256 + 16) + (size_t)wave * M * SK_XROW;

    f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
    auto fetch = [&](int kc, uint4* wv, uint4* xd) {
        const int kb = kc + g * 8;
        const int xk = kc + (lane & 31) * 8;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int row = 2 * r + (lane >> 5);
            if (2 * r < M)
                xd[r] = (row < M && xk < K) ? *reinterpret_cast<const uint4*>(X + (size_t)row * ldx + xk) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int k = kb + j * 32;
            if (TILED)
                wv[j] = (col && kc + j * 32 < K) ? *reinterpret_cast<const uint4*>(wrow + (size_t)((kc >> 5) + j) * TS + lane_at)
                                                 : make_uint4(0, 0, 0, 0);
            else
                wv[j] = (col && k < K) ? *reinterpret_cast<const uint4*>(wrow + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto multiply = [&](const uint4* wv, const uint4* xd) {
        uint4 xv[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int row = 2 * r + (lane >> 5);
            if (2 * r < M && row < M) *reinterpret_cast<uint4*>(xs + row * SK_XROW + (lane & 31) * 16) = xd[r];
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 8; ++j)
            xv[j] = (i < M) ? *reinterpret_cast<const uint4*>(xs + i * SK_XROW + j * 64 + g * 16) : make_uint4(0, 0, 0, 0);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 8; ++j)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xv[j]), as_bf16x8(wv[j]), acc, 0, 0, 0);
    };
    auto step = [&](int kc) {
        uint4 wv[8], xd[8];
        fetch(kc, wv, xd);
        multiply(wv, xd);
    };
    // the slots of the norm are asked for first: they arrive while the wave waits for its first weights
    float sv[2][SL];                                   // PRE: this lane's slots of rows wave and wave + 8
    if (PRE) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int m = wave + NW * h;
#pragma unroll
            for (int j = 0; j < SL; ++j) {
                const int t = lane + 64 * j;
                sv[h][j] = (m < M && t < f.n_slots) ? f.slots_in[(size_t)m * f.n_slots + t] : 0.f;
            }
        }
    }
    for (int kc = wave * SK_CHUNK; kc < K; kc += NW * SK_CHUNK) step(kc);
    if (PRE) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float v = 0.f;
#pragma unroll
            for (int j = 0; j < SL; ++j) v += sv[h][j];
            v = wave_sum(v);
            if (lane == 0 && wave + NW * h < 16) scale_s[wave + NW * h] = 1.0f / sqrtf(v * f.inv_width + f.eps);
        }
    }
    *reinterpret_cast<f32x4*>(red + ((size_t)wave * 64 + lane) * 4) = acc;
    __syncthreads();
    // waves 0..3: thread (l, r = wave): C row 4*(l/16)+r, column l%16; sums over waves in wave order
    if (wave < 4) {
        const int l = lane, r = wave;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) v += red[((size_t)w * 64 + l) * 4 + r];
        const int m = 4 * (l >> 4) + r;
        const int nn = n0 + (l & 15);
        const bool mine = (l & 15) < tile_cols && nn < N;                 // a column this workgroup owns
        if (PRE) v *= scale_s[m];
        if (GLU8) {
            const float up = __shfl_xor(v, 8, BN_WAVE);
            if ((l & 8) == 0 && m < M && nn < N)                          // GLU8: tile_cols is 16
                Y[(size_t)m * ldy + (n0 >> 1) + (l & 7)] = __float2bfloat16(bn_gate_act(v, act) * up);
        } else if (RES) {
            float xn = 0.f;
            if (m < M && mine) {
                xn = f.resid[(size_t)m * f.ld_resid + nn] + v;
                f.resid[(size_t)m * f.ld_resid + nn] = xn;
                f.resid_bf16[(size_t)m * f.ld_rb + nn] = __float2bfloat16(xn * f.next_weight[nn]);
            }
            float sq = xn * xn;                                   // the tile's columns of row m: lanes 16 (l / 16) + 0..15
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) sq += __shfl_xor(sq, o, BN_WAVE);
            if ((l & 15) == 0 && m < M) f.slots_out[(size_t)m * gridDim.x + blockIdx.x] = sq;
        } else if (m < M && mine) {
            Y[(size_t)m * ldy + nn] = __float2bfloat16(v);
        }
    }
}

extern "C" int bn_skinny_gemm_supports(int M, int N, int K, int ldx, int ldw);
static bool sk_tiled_ok(int K, int ldw) { return ldw == (K + BN_STREAM_TILE_COLS - 1) / BN_STREAM_TILE_COLS; }

static int sk_compute_units() {
    static int cus = 0;
    if (!cus) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
        else cus = 256;
    }
    return cus;
}

// Columns per workgroup of the fused kernel for a product of N columns (not GLU8): 16, or fewer when that spreads
// the column tiles so much more evenly over the CUs that the busiest CU has at least 15 % fewer columns
// (6,144 columns: 384 tiles of 16 are one and a half rounds over 256 CUs, 512 tiles of 12 are two even ones).
// A CU pulls its bytes no faster when others idle, so the busiest CU's columns are the kernel's time.
static int sk_fused_tile_cols(int N) {
    const int cus = sk_compute_units();
    auto busiest = [&](int tc) { const int tiles = (N + tc - 1) / tc; return (long long)((tiles + cus - 1) / cus) * tc; };
    int pick = 16;
    long long best = busiest(16);
    for (int tc = 14; tc >= 8; tc -= 2) {
        const int tiles = (N + tc - 1) / tc;
        if (tiles > 64 * SK_SLOT_LOADS) continue;                 // a consumer adds up at most that many slots
        const long long c = busiest(tc);
        if (c * 100 <= best * 85 && c < busiest(pick)) pick = tc;
    }
    return pick;
}

// Columns per workgroup that the fused kernel picks for a product of N columns over a row-major W: the rows per tile
// that a streamed copy of W is best made with.
extern "C" int bn_skinny_gemm_fused_tile_cols(int N) { return N < 1 ? 0 : sk_fused_tile_cols(N); }

// Column tiles (= slots per row that a RES call writes) of the fused kernel for N columns; over a streamed copy of W
// (tile_rows > 0) they are its rows of tiles.
extern "C" int bn_skinny_gemm_fused_tiles(int N, int tile_rows) {
    if (N < 1 || tile_rows < 0 || tile_rows > BN_STREAM_TILE_ROWS) return 0;
    const int tc = tile_rows ? tile_rows : sk_fused_tile_cols(N);
    return (N + tc - 1) / tc;
}

// X, W, Y as bn_skinny_gemm with a bf16 result and M <= 16; glu8 as dual == 2 there, act the gate's activation.
// slots_in != null (PRE): X is a stream's bf16 copy as a RES call leaves it, slots_in [M, n_slots] its rows'
// sums of squares in parts, stream_width its number of columns; the result's rows are scaled by
// 1/sqrt(sum / stream_width + eps).
// resid != null (RES): the product is added to resid [M, N] in place; resid_bf16 [M, N] becomes the new stream
// times next_weight [N], slots_out [M, bn_skinny_gemm_fused_tiles(N)] the sums of squares of its column tiles
// (glu8 == 0, no Y).
// tile_rows > 0: W is the streamed copy (common.h) of the matrix (of its 2N interleaved rows with glu8, then with 16 rows
// a tile) with that many rows a tile and ldw its tiles along K; a RES call then writes a slot per row of tiles.
extern "C" int bn_skinny_gemm_fused(const void* X, const void* W, void* Y, int M, int N, int K, int ldx, int ldw, int ldy,
                                    int glu8, int act, const float* slots_in, int n_slots, int stream_width, float eps,
                                    float* resid, int ld_resid, void* resid_bf16, int ld_rb, const float* next_weight,
                                    float* slots_out, int tile_rows, hipStream_t s) {
    const bool tiled = tile_rows != 0;
    if (!bn_skinny_gemm_supports(M, N, K, ldx, tiled ? 8 : ldw) || M > 16 || act < 0 || act >= BN_ACT_KINDS) return BN_ERR_ARG;
    if (tiled && (!sk_tiled_ok(K, ldw) || tile_rows < 1 || tile_rows > BN_STREAM_TILE_ROWS || (glu8 && tile_rows != 16)))
        return BN_ERR_ARG;
    if (((uintptr_t)X | (uintptr_t)W) & 15) return BN_ERR_ARG;
    const bool pre = slots_in != nullptr, res = resid != nullptr;
    if (!pre && !res) return BN_ERR_ARG;
    if (pre && (n_slots < 1 || n_slots > 64 * SK_SLOT_LOADS || stream_width < 1)) return BN_ERR_ARG;
    if (res && (glu8 || !resid_bf16 || !next_weight || !slots_out || ld_resid < N || ld_rb < N)) return BN_ERR_ARG;
    if (!res && (!Y || ldy < N)) return BN_ERR_ARG;
    if (glu8) {
        if (N % 8) return BN_ERR_ARG;
        N *= 2;
    }
    SkinnyFused f;
    f.slots_in = slots_in; f.n_slots = n_slots; f.inv_width = pre ? 1.0f / (float)stream_width : 0.f; f.eps = eps;
    f.resid = resid; f.resid_bf16 = (bf16*)resid_bf16; f.next_weight = next_weight; f.slots_out = slots_out;
    f.ld_resid = ld_resid; f.ld_rb = ld_rb;
    const size_t smem = (size_t)(8 * 256 + 16) * sizeof(float) + (size_t)8 * M * SK_XROW;
    const int tile_cols = tiled ? tile_rows : (glu8 ? 16 : sk_fused_tile_cols(N));
    const dim3 grid((N + tile_cols - 1) / tile_cols), block(8 * 64);
    auto go = [&](auto kernel) {
        if (smem > 64 * 1024) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
        }
        hipLaunchKernelGGL(kernel, grid, block, smem, s, (const bf16*)X, (const bf16*)W, (bf16*)Y, M, N, K, ldx, ldw, ldy,
                           tile_cols, act, f);
        return bn_launch_status();
    };
    const bool few = n_slots <= 256;                  // four slot loads per row and lane are enough
    if (glu8 && !pre) return BN_ERR_ARG;
#define SK_FUSED(T)                                                                                                      \
    do {                                                                                                                 \
        if (glu8) return few ? go(skinny_gemm_fused_kernel<true, true, false, 4, T>)                                     \
                             : go(skinny_gemm_fused_kernel<true, true, false, 8, T>);                                    \
        if (pre && res) return few ? go(skinny_gemm_fused_kernel<false, true, true, 4, T>)                               \
                                   : go(skinny_gemm_fused_kernel<false, true, true, 8, T>);                              \
        if (pre) return few ? go(skinny_gemm_fused_kernel<false, true, false, 4, T>)                                     \
                            : go(skinny_gemm_fused_kernel<false, true, false, 8, T>);                                    \
        return go(skinny_gemm_fused_kernel<false, false, true, 4, T>);                                                   \
    } while (0)
    if (tiled) SK_FUSED(true);
    SK_FUSED(false);
#undef SK_FUSED
}

template <int MT, bool DUAL, typename TO, bool GLU8 = false, bool TILED = false>
static int launch(const void* X, const void* W, void* Y, int M, int N, int K, int ldx, int ldw, int ldy,
                  int up_off, int act, int n_waves, hipStream_t s) {
    constexpr int NA = DUAL ? 2 * MT : MT;
    constexpr bool XS = MT == 1 && !DUAL;          // the two-block form has no registers to spare for it
    const size_t smem = (size_t)n_waves * NA * 64 * 4 * sizeof(float) + (XS ? (size_t)n_waves * M * SK_XROW : 0);
    auto kernel = skinny_gemm_kernel<MT, DUAL, TO, GLU8, XS, TILED>;
    if (smem > 64 * 1024) {                           // beyond the default limit of dynamic shared memory
        static bool raised = false;                   // per instantiation
        if (!raised) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            raised = true;
        }
    }
    const int cols = TILED ? up_off : 16;             // columns a workgroup owns
    hipLaunchKernelGGL(kernel, dim3((N + cols - 1) / cols), dim3(n_waves * 64), smem, s,
                       (const bf16*)X, (const bf16*)W, (TO*)Y, M, N, K, ldx, ldw, ldy, up_off, act);
    return bn_launch_status();
}

template <typename TO>
static int launch_glu8(int MT, const void* X, const void* W, void* Y, int M, int N, int K, int ldx, int ldw,
                       int ldy, int act, int n_waves, hipStream_t s) {
    switch (MT) {
        case 1: return launch<1, false, TO, true>(X, W, Y, M, N, K, ldx, ldw, ldy, 0, act, n_waves, s);
        case 2: return launch<2, false, TO, true>(X, W, Y, M, N, K, ldx, ldw, ldy, 0, act, n_waves, s);
        case 3: return launch<3, false, TO, true>(X, W, Y, M, N, K, ldx, ldw, ldy, 0, act, n_waves, s);
        case 4: return launch<4, false, TO, true>(X, W, Y, M, N, K, ldx, ldw, ldy, 0, act, n_waves, s);
    }
    return BN_ERR_ARG;
}

template <bool DUAL, typename TO>
static int launch_mt(int MT, const void* X, const void* W, void* Y, int M, int N, int K, int ldx, int ldw,
                     int ldy, int up_off, int act, int n_waves, hipStream_t s) {
    switch (MT) {
        case 1: return launch<1, DUAL, TO>(X, W, Y, M, N, K, ldx, ldw, ldy, up_off, act, n_waves, s);
        case 2: return launch<2, DUAL, TO>(X, W, Y, M, N, K, ldx, ldw, ldy, up_off, act, n_waves, s);
        case 3: return launch<3, DUAL, TO>(X, W, Y, M, N, K, ldx, ldw, ldy, up_off, act, n_waves, s);
        case 4: return launch<4, DUAL, TO>(X, W, Y, M, N, K, ldx, ldw, ldy, up_off, act, n_waves, s);
    }
    return BN_ERR_ARG;
}

// 1 if the kernel takes the shape, 0 if the caller must use the tiled kernel.
extern "C" int bn_skinny_gemm_supports(int M, int N, int K, int ldx, int ldw) {
    return (M >= 1 && M <= 64 && N >= 1 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0) ? 1 : 0;
}

// out_dtype: type of Y (bf16 or float32).  dual == 1: N is the width of the result and W has
// the gate rows at [0, N) and the up rows at [up_off, up_off + N).  dual == 2: W has 2N rows, gate
// and up interleaved in blocks of 8 (N a multiple of 8); the result has N columns.  act: the gate's activation
// (BN_ACT_*), used when dual != 0.
// tile_rows > 0: W is the streamed copy (common.h) with that many rows a tile and ldw its tiles along K; up to 16 rows,
// dual == 0.
extern "C" int bn_skinny_gemm(int out_dtype, const void* X, const void* W, void* Y, int M, int N, int K,
                              int ldx, int ldw, int ldy, int dual, int up_off, int act, int tile_rows, hipStream_t s) {
    const bool tiled = tile_rows != 0;
    if (!bn_skinny_gemm_supports(M, N, K, ldx, tiled ? 8 : ldw) || ldy < N || act < 0 || act >= BN_ACT_KINDS) return BN_ERR_ARG;
    if (((uintptr_t)X | (uintptr_t)W) & 15) return BN_ERR_ARG;
    if (tiled) {
        if (dual || M > 16 || !sk_tiled_ok(K, ldw) || tile_rows < 1 || tile_rows > BN_STREAM_TILE_ROWS) return BN_ERR_ARG;
        int n_waves = 8;                           // as the row-major form with staged activations
        const int k_chunks = (K + SK_CHUNK - 1) / SK_CHUNK;
        while (n_waves > 1 && n_waves / 2 >= k_chunks) n_waves >>= 1;
        // the kernel's up_off carries the rows per tile; its grid is one workgroup per row of tiles
        if (out_dtype == BN_DT_BF16)
            return launch<1, false, bf16, false, true>(X, W, Y, M, N, K, ldx, ldw, ldy, tile_rows, act, n_waves, s);
        if (out_dtype == BN_DT_F32)
            return launch<1, false, float, false, true>(X, W, Y, M, N, K, ldx, ldw, ldy, tile_rows, act, n_waves, s);
        return BN_ERR_DTYPE;
    }
    if (dual == 2) {
        if (N % 8) return BN_ERR_ARG;
        N *= 2;                                   // rows of W; the kernel halves the column index itself
    }
    const int MT = (M + 15) / 16;
    const int NA = dual == 1 ? 2 * MT : MT;
    // waves per workgroup: enough loads in flight when there are few column tiles, bounded by
    // the K chunks there are and by 48 KB of shared memory for the partial sums
    const int tiles = (N + 15) / 16;
    int n_waves = tiles >= 2048 ? 4 : (tiles >= 1024 ? 8 : 16);
    if (MT == 1 && dual != 1) n_waves = 8;        // staged activations: measured best at every size (several workgroups per CU)
    const int k_chunks = (K + SK_CHUNK - 1) / SK_CHUNK;
    while (n_waves > 1 && n_waves / 2 >= k_chunks) n_waves >>= 1;
    while (n_waves > 1 && n_waves * NA > 48) n_waves >>= 1;
    if (dual == 1 && MT >= 3 && n_waves > 8) n_waves = 8;      // that variant is built for 512 threads
    if (dual == 2) {
        if (out_dtype == BN_DT_BF16) return launch_glu8<bf16>(MT, X, W, Y, M, N, K, ldx, ldw, ldy, act, n_waves, s);
        if (out_dtype == BN_DT_F32) return launch_glu8<float>(MT, X, W, Y, M, N, K, ldx, ldw, ldy, act, n_waves, s);
        return BN_ERR_DTYPE;
    }
    if (out_dtype == BN_DT_BF16)
        return dual ? launch_mt<true, bf16>(MT, X, W, Y, M, N, K, ldx, ldw, ldy, up_off, act, n_waves, s)
                    : launch_mt<false, bf16>(MT, X, W, Y, M, N, K, ldx, ldw, ldy, up_off, act, n_waves, s);
    if (out_dtype == BN_DT_F32)
        return dual ? launch_mt<true, float>(MT, X, W, Y, M, N, K, ldx, ldw, ldy, up_off, act, n_waves, s)
                    : launch_mt<false, float>(MT, X, W, Y, M, N, K, ldx, ldw, ldy, up_off, act, n_waves, s);
    return BN_ERR_DTYPE;
}
