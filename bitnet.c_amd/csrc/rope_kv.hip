// Rotary position encoding of Q and K and the write of K, V into the paged cache, one
// launch for all new tokens of a step.
//
// Rotation pairs are split-half: (i, i + rope_dims/2) inside each head
// (src/transformer/cpu_backend.c:283-296).  angle = float(pos) * inv_freq[i], cos/sin
// at full float32 accuracy (src/transformer.c:143-162 uses cosf/sinf).  The cache
// holds rotated keys (src/transformer/cpu.c:893-898 rotates the cached row).
// Cache layout per layer: K [page, kv_head, BN_PAGE, head_dim]; V the same, or transposed
// [page, kv_head, head_dim, BN_PAGE] (v_transposed) for the matrix-core attention kernels.
#include "common.h"

template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, int row_stride,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ seq_index,
                                     const int* __restrict__ block_table, int bt_stride,
                                     T* __restrict__ k_pages, T* __restrict__ v_pages,
                                     const float* __restrict__ inv_freq, int rope_dims,
                                     int H, int Hkv, int hs, int v_transposed) {
    extern __shared__ float cs[];            // cos[half], sin[half]
    const int t = blockIdx.x;
    const int pos = positions[t];
    if (pos < 0) return;                     // a padding row
    const int half = rope_dims / 2;
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
        const size_t dst = (((size_t)page * Hkv + kh) * BN_PAGE + off) * hs + d;
        k_pages[dst] = from_f32<T>(o);
        if (v_transposed)       // V pages [page, kv_head, head_dim, BN_PAGE]
            v_pages[(((size_t)page * Hkv + kh) * hs + d) * BN_PAGE + off] = vrow[idx];
        else
            v_pages[dst] = vrow[idx];
    }
}

// qkv: [n_tokens, row_stride] with Q heads first, then K heads, then V heads.
// k_pages == null: rotate Q only (a layer that reads another layer's cache).
// rope_dims == 0: no rotation, the write alone.
extern "C" int bn_rope_kv_write(int dtype, void* qkv, int row_stride, const int* positions,
                                const int* seq_index, const int* block_table, int bt_stride,
                                void* k_pages, void* v_pages, const float* inv_freq, int rope_dims,
                                int n_tokens, int H, int Hkv, int hs, int v_transposed, hipStream_t s) {
    if (n_tokens <= 0 || H <= 0 || Hkv < 0 || hs <= 0 || rope_dims < 0 || rope_dims > hs ||
        (rope_dims & 1) || row_stride < (H + 2 * Hkv) * hs)
        return BN_ERR_ARG;
    if (rope_dims > 0 && inv_freq == nullptr) return BN_ERR_ARG;
    if (k_pages && (!v_pages || !block_table || !seq_index)) return BN_ERR_ARG;
    const size_t smem = (size_t)(rope_dims > 0 ? rope_dims : 2) * sizeof(float);
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(rope_kv_write_kernel<float>, dim3(n_tokens), dim3(256), smem, s,
                           (float*)qkv, row_stride, positions, seq_index, block_table, bt_stride,
                           (float*)k_pages, (float*)v_pages, inv_freq, rope_dims, H, Hkv, hs, v_transposed);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(rope_kv_write_kernel<bf16>, dim3(n_tokens), dim3(256), smem, s,
                           (bf16*)qkv, row_stride, positions, seq_index, block_table, bt_stride,
                           (bf16*)k_pages, (bf16*)v_pages, inv_freq, rope_dims, H, Hkv, hs, v_transposed);
    else
        return BN_ERR_DTYPE;
    return bn_launch_status();
}
