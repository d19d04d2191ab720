// Rotary position encoding of Q and K and the write of K, V into the paged cache, one
// launch for all new tokens of a step.
//
// Rotation pairs are split-half: (i, i + rope_dims/2) inside each head
// (src/transformer/cpu_backend.c:283-296).  angle = float(pos) * inv_freq[i], cos/sin
// at full float32 accuracy (src/transformer.c:143-162 uses cosf/sinf).  The cache
// holds rotated keys (src/transformer/cpu.c:893-898 rotates the cached row).
// Cache layout per layer (`layout` below): K [page, kv_head, BN_PAGE, head_dim] and V the same (BN_KV_ROWS), or V
// transposed [page, kv_head, head_dim, BN_PAGE] (BN_KV_TRANSPOSED), or keys and values of a (page, kv head) in the
// matrix-core attention kernels' own order (BN_KV_BLOCKED, common.h).  Adding BN_KV_V_BY_TILES says that the values are
// stored by the page-tile kernel below (a prompt's tokens), not here.
#include "common.h"

#define BN_KV_ROWS 0
#define BN_KV_TRANSPOSED 1
#define BN_KV_BLOCKED 2
#define BN_KV_V_BY_TILES 4

template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, int row_stride,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ seq_index,
                                     const int* __restrict__ block_table, int bt_stride,
                                     T* __restrict__ k_pages, T* __restrict__ v_pages,
                                     const float* __restrict__ inv_freq, int rope_dims,
                                     int H, int Hkv, int hs, int layout) {
    extern __shared__ float cs[];            // cos[half], sin[half]
    const int t = blockIdx.x;
    const int pos = positions[t];
    if (pos < 0) return;                     // a padding row
    const int half = rope_dims / 2;
    const int kind = layout & 3;
    const bool v_elsewhere = (layout & BN_KV_V_BY_TILES) != 0;
    float* cos_s = cs;
    float* sin_s = cs + half;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float s, c;
        sincosf((float)pos * inv_freq[i], &s, &c);
        cos_s[i] = c;
        sin_s[i] = s;
    }
    __syncthreads();
    T* row = qkv + (size_t)t * row_stride;
    // Q in place: one thread per pair
    for (int idx = threadIdx.x; idx < H * half; idx += blockDim.x) {
        const int h = idx / half, i = idx - h * half;
        T* hd = row + h * hs;
        const float v0 = to_f32(hd[i]), v1 = to_f32(hd[i + half]);
        hd[i] = from_f32<T>(v0 * cos_s[i] - v1 * sin_s[i]);
        hd[i + half] = from_f32<T>(v0 * sin_s[i] + v1 * cos_s[i]);
    }
    if (k_pages == nullptr) return;
    const int page = block_table[(size_t)seq_index[t] * bt_stride + pos / BN_PAGE];
    const int off = pos % BN_PAGE;
    const T* krow = row + H * hs;
    const T* vrow = krow + Hkv * hs;
    for (int idx = threadIdx.x; idx < Hkv * hs; idx += blockDim.x) {
        const int kh = idx / hs, d = idx - kh * hs;
        const T* hd = krow + kh * hs;
        float o;
        if (d < half) {
            o = to_f32(hd[d]) * cos_s[d] - to_f32(hd[d + half]) * sin_s[d];
        } else if (d < 2 * half) {
            const int i = d - half;
            o = to_f32(hd[i]) * sin_s[i] + to_f32(hd[d]) * cos_s[i];
        } else {
            o = to_f32(hd[d]);
        }
        const size_t head = ((size_t)page * Hkv + kh) * BN_PAGE * hs;       // this kv head's part of the page
        const size_t dst = head + (size_t)off * hs + d;
        k_pages[kind == BN_KV_BLOCKED ? head + bn_blocked_k_offset(off, d, hs) : dst] = from_f32<T>(o);
        if (v_elsewhere) continue;              // the page-tile kernel below stores V
        if (kind == BN_KV_BLOCKED)
            v_pages[head + bn_blocked_v_offset(off, d, hs)] = vrow[idx];
        else if (kind == BN_KV_TRANSPOSED)      // V pages [page, kv_head, head_dim, BN_PAGE]
            v_pages[head + (size_t)d * BN_PAGE + off] = vrow[idx];
        else
            v_pages[dst] = vrow[idx];
    }
}

// bf16 with 8-element groups: the same work with 16-byte loads and stores (one thread rotates the 8
// pairs of two 16-byte groups).  Needs hs, rope_dims / 2 and row_stride to be multiples of 8 and
// 16-byte aligned buffers.
__device__ __forceinline__ void rotate_groups(uint4& lo, uint4& hi, const float* __restrict__ c,
                                              const float* __restrict__ sn) {
    uint32_t* pl = reinterpret_cast<uint32_t*>(&lo);
    uint32_t* ph = reinterpret_cast<uint32_t*>(&hi);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float a0 = bf16lo_to_f32(pl[k]), a1 = bf16hi_to_f32(pl[k]);
        const float b0 = bf16lo_to_f32(ph[k]), b1 = bf16hi_to_f32(ph[k]);
        const float c0 = c[2 * k], c1 = c[2 * k + 1], s0 = sn[2 * k], s1 = sn[2 * k + 1];
        const bf16 l0 = __float2bfloat16(a0 * c0 - b0 * s0), l1 = __float2bfloat16(a1 * c1 - b1 * s1);
        const bf16 h0 = __float2bfloat16(a0 * s0 + b0 * c0), h1 = __float2bfloat16(a1 * s1 + b1 * c1);
        pl[k] = (uint32_t)__builtin_bit_cast(uint16_t, l0) | ((uint32_t)__builtin_bit_cast(uint16_t, l1) << 16);
        ph[k] = (uint32_t)__builtin_bit_cast(uint16_t, h0) | ((uint32_t)__builtin_bit_cast(uint16_t, h1) << 16);
    }
}

// The work of one workgroup on token row t; cs: shared memory for cos[half], sin[half].
__device__ __forceinline__ void rope_kv_write_bf16x8_row(int t, float* cs, bf16* __restrict__ qkv, int row_stride,
                                                         const int* __restrict__ positions,
                                                         const int* __restrict__ seq_index,
                                                         const int* __restrict__ block_table, int bt_stride,
                                                         bf16* __restrict__ k_pages, bf16* __restrict__ v_pages,
                                                         const float* __restrict__ inv_freq, int rope_dims,
                                                         int H, int Hkv, int hs, int layout) {
    const int pos = positions[t];
    if (pos < 0) return;                     // a padding row
    const int half = rope_dims / 2;
    const int kind = layout & 3;
    const bool v_elsewhere = (layout & BN_KV_V_BY_TILES) != 0;
    float* cos_s = cs;
    float* sin_s = cs + half;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float s, c;
        sincosf((float)pos * inv_freq[i], &s, &c);
        cos_s[i] = c;
        sin_s[i] = s;
    }
    __syncthreads();
    bf16* row = qkv + (size_t)t * row_stride;
    const int hg = half / 8;                 // 16-byte groups in half a rotated head
    // Q in place
    for (int idx = threadIdx.x; idx < H * hg; idx += blockDim.x) {
        const int h = idx / hg, c = idx - h * hg;
        uint4* lo = reinterpret_cast<uint4*>(row + h * hs + c * 8);
        uint4* hi = reinterpret_cast<uint4*>(row + h * hs + half + c * 8);
        uint4 a = *lo, b = *hi;
        rotate_groups(a, b, cos_s + c * 8, sin_s + c * 8);
        *lo = a;
        *hi = b;
    }
    if (k_pages == nullptr) return;
    const int page = block_table[(size_t)seq_index[t] * bt_stride + pos / BN_PAGE];
    const int off = pos % BN_PAGE;
    const bf16* krow = row + H * hs;
    const bf16* vrow = krow + Hkv * hs;
    // K: the rotated pairs, then what lies beyond rope_dims as it is
    for (int idx = threadIdx.x; idx < Hkv * hg; idx += blockDim.x) {
        const int kh = idx / hg, c = idx - kh * hg;
        uint4 a = *reinterpret_cast<const uint4*>(krow + kh * hs + c * 8);
        uint4 b = *reinterpret_cast<const uint4*>(krow + kh * hs + half + c * 8);
        rotate_groups(a, b, cos_s + c * 8, sin_s + c * 8);
        // 8 consecutive dimensions of a key are 16 consecutive bytes in either order of a page
        bf16* head = k_pages + ((size_t)page * Hkv + kh) * BN_PAGE * hs;
        const bool blocked = kind == BN_KV_BLOCKED;
        *reinterpret_cast<uint4*>(head + (blocked ? bn_blocked_k_offset(off, c * 8, hs) : off * hs + c * 8)) = a;
        *reinterpret_cast<uint4*>(head + (blocked ? bn_blocked_k_offset(off, half + c * 8, hs) : off * hs + half + c * 8)) = b;
    }
    const int tail = (hs - rope_dims) / 8;
    for (int idx = threadIdx.x; idx < Hkv * tail; idx += blockDim.x) {
        const int kh = idx / tail, c = idx - kh * tail;
        bf16* head = k_pages + ((size_t)page * Hkv + kh) * BN_PAGE * hs;
        const int d = rope_dims + c * 8;
        *reinterpret_cast<uint4*>(head + (kind == BN_KV_BLOCKED ? bn_blocked_k_offset(off, d, hs) : off * hs + d)) =
            *reinterpret_cast<const uint4*>(krow + kh * hs + d);
    }
    // V (unless the page-tile kernel below stores it)
    const int vg = hs / 8;
    for (int idx = threadIdx.x; !v_elsewhere && idx < Hkv * vg; idx += blockDim.x) {
        const int kh = idx / vg, c = idx - kh * vg;
        const uint4 v = *reinterpret_cast<const uint4*>(vrow + kh * hs + c * 8);
        const uint16_t* e = reinterpret_cast<const uint16_t*>(&v);
        uint16_t* head = reinterpret_cast<uint16_t*>(v_pages) + ((size_t)page * Hkv + kh) * BN_PAGE * hs;
        if (kind == BN_KV_BLOCKED) {
#pragma unroll
            for (int j = 0; j < 8; ++j) head[bn_blocked_v_offset(off, c * 8 + j, hs)] = e[j];
        } else if (kind == BN_KV_TRANSPOSED) {      // V pages [page, kv_head, head_dim, BN_PAGE]
#pragma unroll
            for (int j = 0; j < 8; ++j) head[(size_t)(c * 8 + j) * BN_PAGE + off] = e[j];
        } else {
            *reinterpret_cast<uint4*>(head + (size_t)off * hs + c * 8) = v;
        }
    }
}

__global__ __launch_bounds__(256) void rope_kv_write_bf16x8_kernel(bf16* __restrict__ qkv, int row_stride,
                                                                   const int* __restrict__ positions,
                                                                   const int* __restrict__ seq_index,
                                                                   const int* __restrict__ block_table, int bt_stride,
                                                                   bf16* __restrict__ k_pages, bf16* __restrict__ v_pages,
                                                                   const float* __restrict__ inv_freq, int rope_dims,
                                                                   int H, int Hkv, int hs, int layout) {
    extern __shared__ __align__(16) unsigned char dyn_s[];
    rope_kv_write_bf16x8_row(blockIdx.x, reinterpret_cast<float*>(dyn_s), qkv, row_stride, positions, seq_index, block_table,
                             bt_stride, k_pages, v_pages, inv_freq, rope_dims, H, Hkv, hs, layout);
}

// V into transposed or blocked pages for the tokens of a prompt: a workgroup takes the rows of one sequence
// that fall into one page (tile = sequence, first row, rows, position of the first) and one kv
// head, turns the [rows, hs] block through shared memory and stores runs of 8 positions with
// 16 bytes, instead of 2 bytes a position and dimension (8 positions from a multiple of 8 of one dimension are
// 16 consecutive bytes in either order).
#define VT_PAD 2
// The work of one workgroup on (tile, kv head kh); vt_s: shared memory [hs][BN_PAGE + VT_PAD], column = position inside the page.
__device__ __forceinline__ void v_transposed_write_tile(int tile, int kh, uint16_t* vt_s, const bf16* __restrict__ qkv,
                                                        int row_stride, const int* __restrict__ tiles,
                                                        const int* __restrict__ block_table, int bt_stride,
                                                        bf16* __restrict__ v_pages, int H, int Hkv, int hs, int blocked) {
    const int* tl = tiles + 4 * tile;
    const int seq = tl[0], row0 = tl[1], n = tl[2], pos0 = tl[3];
    const int off = pos0 % BN_PAGE;
    if (n <= 0 || off + n > BN_PAGE) return;
    const int page = block_table[(size_t)seq * bt_stride + pos0 / BN_PAGE];
    const int ld = BN_PAGE + VT_PAD;
    const int groups = hs / 8;
    for (int idx = threadIdx.x; idx < n * groups; idx += blockDim.x) {
        const int r = idx / groups, c = idx - r * groups;
        const uint4 v = *reinterpret_cast<const uint4*>(qkv + (size_t)(row0 + r) * row_stride + (size_t)(H + Hkv + kh) * hs + c * 8);
        const uint16_t* e = reinterpret_cast<const uint16_t*>(&v);
#pragma unroll
        for (int j = 0; j < 8; ++j) vt_s[(c * 8 + j) * ld + off + r] = e[j];
    }
    __syncthreads();
    uint16_t* dst = reinterpret_cast<uint16_t*>(v_pages) + ((size_t)page * Hkv + kh) * hs * BN_PAGE;
    for (int idx = threadIdx.x; idx < hs * (BN_PAGE / 8); idx += blockDim.x) {
        const int d = idx / (BN_PAGE / 8), p8 = (idx - d * (BN_PAGE / 8)) * 8;     // positions p8 .. p8+7 of the page
        if (p8 + 8 <= off || p8 >= off + n) continue;
        const uint16_t* src = vt_s + d * ld + p8;
        uint16_t* run = dst + (blocked ? bn_blocked_v_offset(p8, d, hs) : d * BN_PAGE + p8);
        if (p8 >= off && p8 + 8 <= off + n) {
            uint4 w;
            w.x = src[0] | ((uint32_t)src[1] << 16);
            w.y = src[2] | ((uint32_t)src[3] << 16);
            w.z = src[4] | ((uint32_t)src[5] << 16);
            w.w = src[6] | ((uint32_t)src[7] << 16);
            *reinterpret_cast<uint4*>(run) = w;
        } else {
            for (int j = 0; j < 8; ++j)
                if (p8 + j >= off && p8 + j < off + n) run[j] = src[j];
        }
    }
}

__global__ __launch_bounds__(256) void v_transposed_write_kernel(const bf16* __restrict__ qkv, int row_stride,
                                                                 const int* __restrict__ tiles,
                                                                 const int* __restrict__ block_table, int bt_stride,
                                                                 bf16* __restrict__ v_pages, int H, int Hkv, int hs, int blocked) {
    extern __shared__ __align__(16) unsigned char dyn_s[];
    v_transposed_write_tile(blockIdx.x, blockIdx.y, reinterpret_cast<uint16_t*>(dyn_s), qkv, row_stride, tiles, block_table,
                            bt_stride, v_pages, H, Hkv, hs, blocked);
}

// Both at once: the first n_v_blocks workgroups (the longer ones) store the values of a (tile, kv head) each, the others
// rotate a token row and store its keys.  One launch instead of two that do not depend on each other.
__global__ __launch_bounds__(256) void rope_kv_write_tiles_kernel(bf16* __restrict__ qkv, int row_stride,
                                                                  const int* __restrict__ positions,
                                                                  const int* __restrict__ seq_index,
                                                                  const int* __restrict__ block_table, int bt_stride,
                                                                  bf16* __restrict__ k_pages, bf16* __restrict__ v_pages,
                                                                  const float* __restrict__ inv_freq, int rope_dims,
                                                                  int H, int Hkv, int hs, int layout,
                                                                  const int* __restrict__ tiles, int n_v_blocks) {
    extern __shared__ __align__(16) unsigned char dyn_s[];
    const int b = blockIdx.x;
    if (b < n_v_blocks)
        v_transposed_write_tile(b / Hkv, b % Hkv, reinterpret_cast<uint16_t*>(dyn_s), qkv, row_stride, tiles, block_table,
                                bt_stride, v_pages, H, Hkv, hs, (layout & 3) == BN_KV_BLOCKED);
    else
        rope_kv_write_bf16x8_row(b - n_v_blocks, reinterpret_cast<float*>(dyn_s), qkv, row_stride, positions, seq_index,
                                 block_table, bt_stride, k_pages, v_pages, inv_freq, rope_dims, H, Hkv, hs,
                                 layout | BN_KV_V_BY_TILES);
}

// tiles: [n_tiles, 4] int32 as above; every tile lies inside one page.  V heads are read from qkv.  blocked: the pages
// are in the blocked order (hs a multiple of 32), else transposed.
extern "C" int bn_v_transposed_write(const void* qkv, int row_stride, const int* tiles, int n_tiles,
                                     const int* block_table, int bt_stride, void* v_pages, int H, int Hkv, int hs,
                                     int blocked, hipStream_t s) {
    if (n_tiles <= 0 || H <= 0 || Hkv <= 0 || hs <= 0 || hs % 8 || row_stride % 8 || row_stride < (H + 2 * Hkv) * hs ||
        !tiles || !block_table || !v_pages || n_tiles > 0x7fffffff / 4 || Hkv > 65535 || (blocked && hs % 32))
        return BN_ERR_ARG;
    if (((uintptr_t)qkv | (uintptr_t)v_pages) & 15) return BN_ERR_ARG;
    const size_t smem = (size_t)hs * (BN_PAGE + VT_PAD) * sizeof(uint16_t);
    if (smem > 64 * 1024) return BN_ERR_ARG;
    hipLaunchKernelGGL(v_transposed_write_kernel, dim3(n_tiles, Hkv), dim3(256), smem, s, (const bf16*)qkv, row_stride,
                       tiles, block_table, bt_stride, (bf16*)v_pages, H, Hkv, hs, blocked);
    return bn_launch_status();
}

// qkv: [n_tokens, row_stride] with Q heads first, then K heads, then V heads.
// k_pages == null: rotate Q only (a layer that reads another layer's cache).
// rope_dims == 0: no rotation, the write alone.
// layout: BN_KV_ROWS (0) = V pages like K pages, BN_KV_TRANSPOSED (1) = transposed V pages, BN_KV_BLOCKED (2) = keys and
// values in the blocked order (hs a multiple of 32); + BN_KV_V_BY_TILES (4): bn_v_transposed_write fills the values (V is
// left alone here).
extern "C" int bn_rope_kv_write(int dtype, void* qkv, int row_stride, const int* positions,
                                const int* seq_index, const int* block_table, int bt_stride,
                                void* k_pages, void* v_pages, const float* inv_freq, int rope_dims,
                                int n_tokens, int H, int Hkv, int hs, int layout, hipStream_t s) {
    if (n_tokens <= 0 || H <= 0 || Hkv < 0 || hs <= 0 || rope_dims < 0 || rope_dims > hs ||
        (rope_dims & 1) || row_stride < (H + 2 * Hkv) * hs)
        return BN_ERR_ARG;
    if (layout < 0 || (layout & 3) > BN_KV_BLOCKED || (layout & ~7) || ((layout & 3) == BN_KV_BLOCKED && hs % 32))
        return BN_ERR_ARG;
    const int v_transposed = layout;
    if (rope_dims > 0 && inv_freq == nullptr) return BN_ERR_ARG;
    if (k_pages && (!v_pages || !block_table || !seq_index)) return BN_ERR_ARG;
    const size_t smem = (size_t)(rope_dims > 0 ? rope_dims : 2) * sizeof(float);
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(rope_kv_write_kernel<float>, dim3(n_tokens), dim3(256), smem, s,
                           (float*)qkv, row_stride, positions, seq_index, block_table, bt_stride,
                           (float*)k_pages, (float*)v_pages, inv_freq, rope_dims, H, Hkv, hs, v_transposed);
    else if (dtype == BN_DT_BF16 && rope_dims > 0 && hs % 8 == 0 && rope_dims % 16 == 0 && row_stride % 8 == 0 &&
             !(((uintptr_t)qkv | (uintptr_t)k_pages | (uintptr_t)v_pages) & 15))
        hipLaunchKernelGGL(rope_kv_write_bf16x8_kernel, dim3(n_tokens), dim3(256), smem, s,
                           (bf16*)qkv, row_stride, positions, seq_index, block_table, bt_stride,
                           (bf16*)k_pages, (bf16*)v_pages, inv_freq, rope_dims, H, Hkv, hs, v_transposed);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(rope_kv_write_kernel<bf16>, dim3(n_tokens), dim3(256), smem, s,
                           (bf16*)qkv, row_stride, positions, seq_index, block_table, bt_stride,
                           (bf16*)k_pages, (bf16*)v_pages, inv_freq, rope_dims, H, Hkv, hs, v_transposed);
    else
        return BN_ERR_DTYPE;
    return bn_launch_status();
}

// bn_rope_kv_write and bn_v_transposed_write in one launch, for bf16 rows that the 16-byte kernel takes (rope_dims a
// positive multiple of 16, hs and row_stride multiples of 8, 16-byte aligned pointers) and transposed or blocked pages.
// Returns BN_ERR_ARG for anything else: the caller then makes the two calls.
extern "C" int bn_rope_kv_write_tiles(void* qkv, int row_stride, const int* positions, const int* seq_index,
                                      const int* block_table, int bt_stride, void* k_pages, void* v_pages,
                                      const float* inv_freq, int rope_dims, int n_tokens, int H, int Hkv, int hs, int layout,
                                      const int* tiles, int n_tiles, hipStream_t s) {
    if (n_tokens <= 0 || n_tiles <= 0 || H <= 0 || Hkv <= 0 || Hkv > 65535 || hs <= 0 || hs % 8 || rope_dims <= 0 ||
        rope_dims > hs || rope_dims % 16 || row_stride % 8 || row_stride < (H + 2 * Hkv) * hs)
        return BN_ERR_ARG;
    const int kind = layout & 3;
    if ((layout & ~7) || (kind != BN_KV_TRANSPOSED && kind != BN_KV_BLOCKED) || (kind == BN_KV_BLOCKED && hs % 32)) return BN_ERR_ARG;
    if (!qkv || !positions || !seq_index || !block_table || !k_pages || !v_pages || !inv_freq || !tiles) return BN_ERR_ARG;
    if (((uintptr_t)qkv | (uintptr_t)k_pages | (uintptr_t)v_pages) & 15) return BN_ERR_ARG;
    const long long n_v_blocks = (long long)n_tiles * Hkv;
    if (n_v_blocks + n_tokens > 0x7fffffff) return BN_ERR_ARG;
    const size_t smem_v = (size_t)hs * (BN_PAGE + VT_PAD) * sizeof(uint16_t), smem_r = (size_t)rope_dims * sizeof(float);
    const size_t smem = smem_v > smem_r ? smem_v : smem_r;
    if (smem > 64 * 1024) return BN_ERR_ARG;
    hipLaunchKernelGGL(rope_kv_write_tiles_kernel, dim3((unsigned)(n_v_blocks + n_tokens)), dim3(256), smem, s, (bf16*)qkv,
                       row_stride, positions, seq_index, block_table, bt_stride, (bf16*)k_pages, (bf16*)v_pages, inv_freq,
                       rope_dims, H, Hkv, hs, layout, tiles, (int)n_v_blocks);
    return bn_launch_status();
}
