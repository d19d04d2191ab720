// Shared device helpers for the gfx950 kernels of this library.
// Wavefronts are 64 lanes wide; every reduction below assumes that.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#define BN_WAVE 64
#define BN_PAGE 64            // tokens per cache page; the Python side reads this line (csrc/build.py: header_constant)
// Decode attention splits a sequence's keys over workgroups in runs of at least this many pages: shorter
// runs cost more in merging than they gain in parallelism (measured at batch 1, 8 and 64 of an 8B shape).
#define BN_SPLIT_MIN_PAGES 2
// A float32 cache's keys are summed in runs of this many positions (whole pages, counted from position 0), each run by
// itself and the runs folded in order: a decode step then spreads a long sequence's runs over workgroups and still forms
// every sum in the order in which a prompt step forms it, so that float32 logits do not depend on how a sequence was cut.
#define BN_F32_FOLD_KEYS 2048
#define BN_MAX_HEAD_DIM 256   // the attention kernels take every even head size up to this; the configuration reads this line too

// The streamed copy of a bf16 weight matrix W[N, K], for the kernels that read W once per call in the operand layout of
// v_mfma_f32_16x16x32_bf16 (lane l = r + 16 g holds columns 8 g .. 8 g + 7 of row r of a 16 x 32 block): tile (a, b) is rows
// R a .. R a + R - 1, columns 32 b .. 32 b + 31, for a number R <= 16 of rows per tile that the copy names (16, or fewer
// where that spreads the tiles more evenly over the CUs); its 32 R elements are stored so that the eight of lane
// r + 16 g (r < R) are the elements 8 (R g + r) .. 8 (R g + r) + 7; tiles in the order [ceil(N / R)][ceil(K / 32)], rows
// past N and columns past K zero.  One load of a wave reads one tile as 64 R consecutive bytes (the lanes r >= R idle).
// The Python side reads these lines too.
#define BN_STREAM_TILE_ROWS 16        // the most rows of a tile
#define BN_STREAM_TILE_COLS 32

// Cache pages in the matrix-core attention kernels' own order ("blocked"; bf16, head sizes that are multiples of 32).  A
// page still holds BN_PAGE positions of hs elements for every kv head, keys and values each, but inside a (page, kv head)
// they lie in blocks of 32 positions, and a block in the order in which a wave of the decode kernel loads it: one load
// instruction takes 1 KB of consecutive bytes where pages that hold a row per position (or a row per dimension) give it
// 64 bytes in each of 16 rows.  With position p = 32 b + r inside the page:
//   keys:   the operand of the first product (S^T = K Q^T) is a tile of 16 positions x 32 dimensions, lane i + 16 g holding
//           dimensions 8 g .. 8 g + 7 of tile row i; a block is two such row sets (tile 0: r = 8 (i / 4) + i % 4, tile 1:
//           4 further) for each of hs / 32 dimension chunks c.  Element (p, d = 32 c + 8 g + e) lies at
//           32 hs b + 8 (64 (2 c + tile) + 16 g + i) + e.
//   values: the operand of the second product is a tile of 16 dimensions x 32 positions, lane i + 16 g holding positions
//           8 g .. 8 g + 7 of dimension 16 t + i.  Element (p = 32 b + 8 g + e, d = 16 t + i) lies at
//           32 hs b + 8 (64 t + 16 g + i) + e.
// Eight consecutive dimensions of a key, and eight consecutive positions (from a multiple of 8) of a value's dimension,
// stay 16 consecutive bytes, which is what the writers store at once.
#define BN_KV_BLOCK 32
// the head sizes that the matrix-core attention kernels are built for (the Python side reads these lines)
#define BN_MFMA_HEAD_DIM_SMALL 64
#define BN_MFMA_HEAD_DIM_LARGE 128
__host__ __device__ __forceinline__ int bn_blocked_k_offset(int p, int d, int hs) {
    const int b = p >> 5, r = p & 31;
    const int tile = (r >> 2) & 1, i = ((r >> 3) << 2) | (r & 3);
    return 32 * hs * b + 8 * (64 * (2 * (d >> 5) + tile) + 16 * ((d >> 3) & 3) + i) + (d & 7);
}
__host__ __device__ __forceinline__ int bn_blocked_v_offset(int p, int d, int hs) {
    const int b = p >> 5;
    return 32 * hs * b + 8 * (64 * (d >> 4) + 16 * ((p >> 3) & 3) + (d & 15)) + (p & 7);
}

// error codes returned by the extern "C" entry points (0 = ok, >0 = hipError_t)
#define BN_ERR_ARG   (-1)     // an argument the kernel cannot take (size, alignment)
#define BN_ERR_DTYPE (-2)

#define BN_DT_F32  0
#define BN_DT_BF16 1

typedef __hip_bfloat16 bf16;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return __bfloat162float(v); }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return __float2bfloat16(v); }

// bf16 bits <-> float without going through the class type (for packed loads)
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
    return __uint_as_float(((uint32_t)b) << 16);
}
__device__ __forceinline__ float bf16lo_to_f32(uint32_t two) { return __uint_as_float(two << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t two) { return __uint_as_float(two & 0xffff0000u); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, BN_WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, BN_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of shared memory.  The order of the additions is
// fixed by the block size alone.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (BN_WAVE - 1), w = threadIdx.x / BN_WAVE;
    const int nw = (blockDim.x + BN_WAVE - 1) / BN_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += scratch[i];
    return t;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & (BN_WAVE - 1), w = threadIdx.x / BN_WAVE;
    const int nw = (blockDim.x + BN_WAVE - 1) / BN_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[w] = v;
    __syncthreads();
    float t = scratch[0];
    for (int i = 1; i < nw; ++i) t = fmaxf(t, scratch[i]);
    return t;
}

// Keys per split of a decode step whose longest sequence holds max_len keys, cut into n_splits runs of whole
// pages (the same rule as ops.decode_splits): the kernels use it when the length arrives in device memory.
__host__ __device__ __forceinline__ int bn_split_chunk(int max_len, int n_splits) {
    const int pages = max_len > 0 ? (max_len + BN_PAGE - 1) / BN_PAGE : 1;
    int per = (pages + n_splits - 1) / n_splits;
    if (per < BN_SPLIT_MIN_PAGES) per = BN_SPLIT_MIN_PAGES;
    return per * BN_PAGE;
}

// The gate's activation in a gated feed-forward, out = act(gate) * up: the kinds the reference knows
// (src/transformer/cpu_backend.c:343-417).  silu(g) = g / (1 + exp(-g)) with the exact exponential (:356);
// gelu in its tanh form 0.5 g (1 + tanh(0.79788456 g (1 + 0.044715 g^2))) (:27-29; the reference's function also
// returns 0 below -10 and g above 10 and rounds g and the result to half precision, :20-30, which this one does not:
// it is no activation of the architecture built here, and its parity with the reference is not pinned by a test);
// relu2(g) = max(g, 0)^2 (:349-350).  Every kernel that ends in a gated unit takes the kind as an argument.
#define BN_ACT_SILU 0
#define BN_ACT_GELU_TANH 1
#define BN_ACT_RELU2 2
#define BN_ACT_KINDS 3
__device__ __forceinline__ float bn_gate_act(float g, int act) {
    if (act == BN_ACT_SILU) return g / (1.0f + expf(-g));
    if (act == BN_ACT_GELU_TANH) return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * g * (1.0f + 0.044715f * g * g)));
    const float p = fmaxf(g, 0.f);
    return p * p;
}

static inline int bn_launch_status() { return (int)hipGetLastError(); }
