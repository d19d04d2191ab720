// Row-wise kernels around the matrix products: embedding gather, residual add fused with
// RMSNorm, SwiGLU, bias add, row gather.  The residual stream is float32; `T` is the
// activation type (float or bf16) that the matrix products read and write.
#include "common.h"

// x[t, :] = float(E[token[t], :]) * scale.  A token outside [0, vocab) gives a zero row, as the
// reference's embedding does (src/model_embed.c:6-28, test/test_safety.c:278-315); the
// step function rejects such tokens before it launches anything.  scale is the architecture's
// embedding multiplier (src/model_embed.c:23-27 scales by sqrt(dim) under one of its policies;
// 1 for this architecture, which changes no bit).
template <typename T>
__global__ void embed_gather_kernel(float* __restrict__ x, const T* __restrict__ table,
                                    const int* __restrict__ tokens, int dim, int vocab, float scale) {
    const int t = blockIdx.x;
    const int tok = tokens[t];
    float* row = x + (size_t)t * dim;
    if (tok < 0 || tok >= vocab) {
        for (int i = threadIdx.x; i < dim; i += blockDim.x) row[i] = 0.f;
        return;
    }
    const T* src = table + (size_t)tok * dim;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) row[i] = to_f32(src[i]) * scale;
}

// logits = cap * tanh(logits / cap), in place (src/transformer/logits.c:325-333)
__global__ void softcap_kernel(float* __restrict__ x, size_t n, float cap, float inv) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = tanhf(x[i] * inv) * cap;
}

// One block per output row r.  src row = rows ? rows[r] : r.
//   s = x[src] (+ delta[src])          float32; written back to x[src] when delta && !rows
//   out[r] = s * rsqrt(mean(s^2) + eps) * w     (src/transformer/rmsnorm_scalar.c:4-13;
//   the fused add is the reference's residual_rmsnorm, src/gpu_cuda.cu:5077)
// The sum of squares is float32: per thread in index order, then a fixed tree.
// delta may come as n_parts slabs (part_stride elements apart) that are added in slab order: the partial sums of
// a product whose K was split over workgroups (splitk_gemm.hip); TD is the slabs' type.
template <typename T, typename TD>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const TD* __restrict__ delta, int n_parts, size_t part_stride,
                                   const float* __restrict__ w, T* __restrict__ out,
                                   const int* __restrict__ rows, int dim, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    float* xr = x + (size_t)src * dim;
    const TD* dr = delta ? delta + (size_t)src * dim : nullptr;
    const bool write_back = (dr != nullptr) && (rows == nullptr);
    float ss = 0.f;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) {
        float v = xr[i];
        if (dr)
            for (int p = 0; p < n_parts; ++p) v += to_f32(dr[p * part_stride + i]);
        if (write_back) xr[i] = v;
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
    T* o = out + (size_t)r * dim;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) {
        float v = xr[i];
        if (dr && !write_back)
            for (int p = 0; p < n_parts; ++p) v += to_f32(dr[p * part_stride + i]);
        o[i] = from_f32<T>(v * scale * w[i]);
    }
}

// The same for rows of up to 256*4*NV elements (a multiple of 4): every load of the row is
// issued before anything waits, the row stays in registers, one block reduction, one store.
// Each thread's partial sum runs over its elements in index order; the tree is the same as above.
template <typename T, typename TD, int NV>
__global__ __launch_bounds__(256) void add_rmsnorm_row_kernel(float* __restrict__ x, const TD* __restrict__ delta,
                                                              int n_parts, size_t part_stride,
                                                              const float* __restrict__ w, T* __restrict__ out,
                                                              const int* __restrict__ rows, int dim, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    float* xr = x + (size_t)src * dim;
    const TD* dr = delta ? delta + (size_t)src * dim : nullptr;
    const bool write_back = (dr != nullptr) && (rows == nullptr);
    float4 v[NV], wv[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int i = (k * 256 + threadIdx.x) * 4;
        v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
        wv[k] = v[k];
        if (i < dim) {
            v[k] = *reinterpret_cast<const float4*>(xr + i);
            wv[k] = *reinterpret_cast<const float4*>(w + i);
        }
    }
    if (dr) {
#pragma unroll 4
        for (int p = 0; p < n_parts; ++p, dr += part_stride) {       // several slabs' loads in flight at once
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const int i = (k * 256 + threadIdx.x) * 4;
                if (i < dim) {
                    float d[4];
                    if (sizeof(TD) == 2) {
                        const uint2 t = *reinterpret_cast<const uint2*>(dr + i);
                        d[0] = bf16lo_to_f32(t.x); d[1] = bf16hi_to_f32(t.x); d[2] = bf16lo_to_f32(t.y); d[3] = bf16hi_to_f32(t.y);
                    } else {
                        const float4 t = *reinterpret_cast<const float4*>(dr + i);
                        d[0] = t.x; d[1] = t.y; d[2] = t.z; d[3] = t.w;
                    }
                    v[k].x += d[0]; v[k].y += d[1]; v[k].z += d[2]; v[k].w += d[3];
                }
            }
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int i = (k * 256 + threadIdx.x) * 4;
        if (i < dim) {
            if (write_back) *reinterpret_cast<float4*>(xr + i) = v[k];
            ss += v[k].x * v[k].x; ss += v[k].y * v[k].y; ss += v[k].z * v[k].z; ss += v[k].w * v[k].w;
        }
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
    T* o = out + (size_t)r * dim;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int i = (k * 256 + threadIdx.x) * 4;
        if (i < dim) {
            const float a = v[k].x * scale * wv[k].x, b = v[k].y * scale * wv[k].y;
            const float c = v[k].z * scale * wv[k].z, d = v[k].w * scale * wv[k].w;
            if (sizeof(T) == 2) {
                bf16 t[4] = {from_f32<bf16>(a), from_f32<bf16>(b), from_f32<bf16>(c), from_f32<bf16>(d)};
                *reinterpret_cast<uint2*>(o + i) = *reinterpret_cast<const uint2*>(t);
            } else {
                *reinterpret_cast<float4*>(o + i) = make_float4(a, b, c, d);
            }
        }
    }
}

// The same sum and norm for many slabs in two launches that use the whole chip (one workgroup a row, as above, has a
// CU pull all slabs of its row alone): first x += the slabs in slab order, 1,024 columns of a row per workgroup, and
// the sum of squares of each such piece to ssq[row][piece]; then the norm from those sums (pieces added in order).
#define SP_PIECE 1024
__global__ __launch_bounds__(256) void sum_parts_kernel(float* __restrict__ x, const float* __restrict__ parts, int n_parts,
                                                        size_t part_stride, float* __restrict__ ssq, int dim) {
    __shared__ float scratch[16];
    const int row = blockIdx.y, i = blockIdx.x * SP_PIECE + threadIdx.x * 4;
    const bool in = i < dim;                                  // dim is a multiple of 4
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (in) {
        float* xr = x + (size_t)row * dim + i;
        const float* pr = parts + (size_t)row * dim + i;
        v = *reinterpret_cast<const float4*>(xr);
#pragma unroll 8
        for (int p = 0; p < n_parts; ++p) {
            const float4 d = *reinterpret_cast<const float4*>(pr + (size_t)p * part_stride);
            v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        }
        *reinterpret_cast<float4*>(xr) = v;
    }
    float ss = 0.f;
    ss += v.x * v.x; ss += v.y * v.y; ss += v.z * v.z; ss += v.w * v.w;
    ss = block_sum(ss, scratch);
    if (threadIdx.x == 0) ssq[(size_t)row * gridDim.x + blockIdx.x] = ss;
}

// The sum for a norm that its consumer applies itself: x += delta (n_parts float32 slabs in slab order, or one tensor of
// type TD when n_parts is 1; none when delta is null), the bf16 copy of the new x times the next norm's weights, and the
// piece's sum of squares to ssq[row][piece].  The consumer multiplies its result's rows by 1/sqrt(sum / dim + eps)
// (src/transformer/rmsnorm_scalar.c:4-13: the factor is the same for a whole row, so it commutes with the product).
template <typename TD>
__global__ __launch_bounds__(256) void sum_deferred_kernel(float* __restrict__ x, const TD* __restrict__ delta, int n_parts,
                                                           size_t part_stride, const float* __restrict__ w,
                                                           bf16* __restrict__ scaled, float* __restrict__ ssq, int dim) {
    __shared__ float scratch[16];
    const int row = blockIdx.y, i = blockIdx.x * SP_PIECE + threadIdx.x * 4;
    const bool in = i < dim;                                  // dim is a multiple of 4
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (in) {
        float* xr = x + (size_t)row * dim + i;
        v = *reinterpret_cast<const float4*>(xr);
        if (delta) {
            const TD* pr = delta + (size_t)row * dim + i;
            if (sizeof(TD) == 4) {
#pragma unroll 8
                for (int p = 0; p < n_parts; ++p) {
                    const float4 d = *reinterpret_cast<const float4*>(pr + (size_t)p * part_stride);
                    v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
                }
            } else {
                const uint2 d = *reinterpret_cast<const uint2*>(pr);
                v.x += bf16lo_to_f32(d.x); v.y += bf16hi_to_f32(d.x); v.z += bf16lo_to_f32(d.y); v.w += bf16hi_to_f32(d.y);
            }
            *reinterpret_cast<float4*>(xr) = v;
        }
        const float4 wv = *reinterpret_cast<const float4*>(w + i);
        bf16 t[4] = {from_f32<bf16>(v.x * wv.x), from_f32<bf16>(v.y * wv.y), from_f32<bf16>(v.z * wv.z), from_f32<bf16>(v.w * wv.w)};
        *reinterpret_cast<uint2*>(scaled + (size_t)row * dim + i) = *reinterpret_cast<const uint2*>(t);
    }
    float ss = 0.f;
    ss += v.x * v.x; ss += v.y * v.y; ss += v.z * v.z; ss += v.w * v.w;
    ss = block_sum(ss, scratch);
    if (threadIdx.x == 0) ssq[(size_t)row * gridDim.x + blockIdx.x] = ss;
}

template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_ssq_kernel(const float* __restrict__ x, const float* __restrict__ ssq,
                                                          int n_pieces, const float* __restrict__ w, T* __restrict__ out,
                                                          int dim, float eps) {
    const int row = blockIdx.x;
    float ss = 0.f;
    for (int p = 0; p < n_pieces; ++p) ss += ssq[(size_t)row * n_pieces + p];
    const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
    const float* xr = x + (size_t)row * dim;
    T* o = out + (size_t)row * dim;
    for (int i = threadIdx.x * 4; i < dim; i += 1024) {
        const float4 v = *reinterpret_cast<const float4*>(xr + i), wv = *reinterpret_cast<const float4*>(w + i);
        const float a = v.x * scale * wv.x, b = v.y * scale * wv.y, c = v.z * scale * wv.z, d = v.w * scale * wv.w;
        if (sizeof(T) == 2) {
            bf16 t[4] = {from_f32<bf16>(a), from_f32<bf16>(b), from_f32<bf16>(c), from_f32<bf16>(d)};
            *reinterpret_cast<uint2*>(o + i) = *reinterpret_cast<const uint2*>(t);
        } else {
            *reinterpret_cast<float4*>(o + i) = make_float4(a, b, c, d);
        }
    }
}

// out[r, :] = x[rows[r], :] in type T: the wanted rows of the stream for an output matrix that no norm precedes
template <typename T>
__global__ void gather_rows_kernel(T* __restrict__ out, const float* __restrict__ x, const int* __restrict__ rows, int dim) {
    const float* xr = x + (size_t)rows[blockIdx.x] * dim;
    T* o = out + (size_t)blockIdx.x * dim;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) o[i] = from_f32<T>(xr[i]);
}

// x[t, :] += delta[t, :]   (src/transformer/cpu_backend.c:252-256)
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ x, const T* __restrict__ delta, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] += to_f32(delta[i]);
}

// x += the n_parts float32 slabs of n elements each, in slab order
__global__ void residual_add_parts_kernel(float* __restrict__ x, const float* __restrict__ parts, int n_parts, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = x[i];
    for (int p = 0; p < n_parts; ++p) v += parts[(size_t)p * n + i];
    x[i] = v;
}

// out[t, f] = act(gu[t, f]) * gu[t, F + f], act one of bn_gate_act's kinds: silu(g) = g / (1 + exp(-g))
// (src/transformer/cpu_backend.c:385-391, exact exponential), gelu, relu2
// il8: gate and up interleaved in blocks of 8 columns (gate f at 16*(f/8) + f%8, up 8 further)
template <typename T>
__global__ void swiglu_kernel(T* __restrict__ out, const T* __restrict__ gu, int F, size_t n, int il8, int act) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    size_t t = i / F;
    int f = (int)(i - t * F);
    const size_t gi = il8 ? t * 2 * F + 16 * (f / 8) + (f % 8) : t * 2 * F + f;
    float g = to_f32(gu[gi]);
    float u = to_f32(gu[il8 ? gi + 8 : gi + F]);
    out[i] = from_f32<T>(bn_gate_act(g, act) * u);
}

// the same, 8 bf16 values a thread (F a multiple of 8, 16-byte aligned rows)
__global__ void swiglu_bf16x8_kernel(bf16* __restrict__ out, const bf16* __restrict__ gu, int F, size_t n8, int il8, int act) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    const int f8 = F / 8;
    const size_t t = i / f8;
    const int f = (int)(i - t * f8) * 8;
    const uint4 g = *reinterpret_cast<const uint4*>(gu + t * 2 * F + (il8 ? 2 * f : f));
    const uint4 u = *reinterpret_cast<const uint4*>(gu + t * 2 * F + (il8 ? 2 * f + 8 : F + f));
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t ow[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float g0 = bf16lo_to_f32(gw[k]), g1 = bf16hi_to_f32(gw[k]);
        const float r0 = bn_gate_act(g0, act) * bf16lo_to_f32(uw[k]);
        const float r1 = bn_gate_act(g1, act) * bf16hi_to_f32(uw[k]);
        const bf16 b0 = __float2bfloat16(r0), b1 = __float2bfloat16(r1);
        ow[k] = (uint32_t)(*reinterpret_cast<const uint16_t*>(&b0)) | ((uint32_t)(*reinterpret_cast<const uint16_t*>(&b1)) << 16);
    }
    *reinterpret_cast<uint4*>(out + t * F + f) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

// The gated unit behind a product whose norm was deferred: gate and up (interleaved in blocks of 8 columns) are both
// multiplied by the row's 1/sqrt(sum of the ssq pieces / width + eps) first, in float32, then act(gate) * up.
__global__ void swiglu_scaled_bf16x8_kernel(bf16* __restrict__ out, const bf16* __restrict__ gu, int F, size_t n8, int il8,
                                            int act, const float* __restrict__ ssq, int n_pieces, float inv_width, float eps) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    const int f8 = F / 8;
    const size_t t = i / f8;
    const int f = (int)(i - t * f8) * 8;
    float ss = 0.f;
    for (int p = 0; p < n_pieces; ++p) ss += ssq[t * n_pieces + p];          // in piece order: the same in every thread
    const float sc = 1.0f / sqrtf(ss * inv_width + eps);
    const uint4 g = *reinterpret_cast<const uint4*>(gu + t * 2 * F + (il8 ? 2 * f : f));
    const uint4 u = *reinterpret_cast<const uint4*>(gu + t * 2 * F + (il8 ? 2 * f + 8 : F + f));
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t ow[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float r0 = bn_gate_act(bf16lo_to_f32(gw[k]) * sc, act) * (bf16lo_to_f32(uw[k]) * sc);
        const float r1 = bn_gate_act(bf16hi_to_f32(gw[k]) * sc, act) * (bf16hi_to_f32(uw[k]) * sc);
        const bf16 b0 = __float2bfloat16(r0), b1 = __float2bfloat16(r1);
        ow[k] = (uint32_t)(*reinterpret_cast<const uint16_t*>(&b0)) | ((uint32_t)(*reinterpret_cast<const uint16_t*>(&b1)) << 16);
    }
    *reinterpret_cast<uint4*>(out + t * F + f) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

// y[t, n] += b[n]   (src/gpu_cuda.cu:5161-5166)
template <typename T>
__global__ void bias_add_kernel(T* __restrict__ y, const float* __restrict__ b, int N, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = from_f32<T>(to_f32(y[i]) + b[i % N]);
}

template <typename T>
static int embed_gather_t(void* x, const void* table, const int* tokens, int n_tokens, int dim,
                          int vocab, float scale, hipStream_t s) {
    hipLaunchKernelGGL(embed_gather_kernel<T>, dim3(n_tokens), dim3(256), 0, s, (float*)x,
                       (const T*)table, tokens, dim, vocab, scale);
    return bn_launch_status();
}

extern "C" int bn_embed_gather(int dtype, void* x, const void* table, const int* tokens, int n_tokens,
                               int dim, int vocab, float scale, hipStream_t s) {
    if (n_tokens <= 0 || dim <= 0 || vocab <= 0) return BN_ERR_ARG;
    if (dtype == BN_DT_F32) return embed_gather_t<float>(x, table, tokens, n_tokens, dim, vocab, scale, s);
    if (dtype == BN_DT_BF16) return embed_gather_t<bf16>(x, table, tokens, n_tokens, dim, vocab, scale, s);
    return BN_ERR_DTYPE;
}

// out [n_rows, dim] (dtype) = the rows `rows` of x [., dim] (float32)
extern "C" int bn_gather_rows(int dtype, void* out, const float* x, const int* rows, int n_rows, int dim, hipStream_t s) {
    if (n_rows <= 0 || dim <= 0 || !out || !x || !rows) return BN_ERR_ARG;
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(gather_rows_kernel<float>, dim3(n_rows), dim3(256), 0, s, (float*)out, x, rows, dim);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(gather_rows_kernel<bf16>, dim3(n_rows), dim3(256), 0, s, (bf16*)out, x, rows, dim);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

extern "C" int bn_softcap(float* x, long long n, float cap, hipStream_t s) {
    if (n <= 0 || !(cap > 0.f)) return BN_ERR_ARG;
    hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, x, (size_t)n, cap, 1.0f / cap);
    return bn_launch_status();
}

template <typename T, typename TD = T>
static void launch_add_rmsnorm(float* x, const void* delta, const float* w, void* out, const int* rows, int n_rows,
                               int dim, float eps, hipStream_t s, int n_parts = 1, size_t part_stride = 0) {
    const bool aligned = dim % 4 == 0 && part_stride % 4 == 0 &&
                         !(((uintptr_t)x | (uintptr_t)w | (uintptr_t)out | (uintptr_t)delta) & 15);
    const int nv = (dim + 1023) / 1024;
    if (aligned && nv <= 8) {
#define ROW_CASE(NV) hipLaunchKernelGGL((add_rmsnorm_row_kernel<T, TD, NV>), dim3(n_rows), dim3(256), 0, s, x, (const TD*)delta, n_parts, part_stride, w, (T*)out, rows, dim, eps)
        switch (nv) {
            case 1: ROW_CASE(1); break;
            case 2: ROW_CASE(2); break;
            case 3: case 4: ROW_CASE(4); break;
            default: ROW_CASE(8); break;
        }
#undef ROW_CASE
        return;
    }
    const int threads = dim >= 2048 ? 512 : 256;
    hipLaunchKernelGGL((add_rmsnorm_kernel<T, TD>), dim3(n_rows), dim3(threads), 0, s, x, (const TD*)delta, n_parts, part_stride,
                       w, (T*)out, rows, dim, eps);
}

extern "C" int bn_add_rmsnorm(int dtype, void* x, const void* delta, const float* w, void* out,
                              const int* rows, int n_rows, int dim, float eps, hipStream_t s) {
    if (n_rows <= 0 || dim <= 0) return BN_ERR_ARG;
    if (dtype == BN_DT_F32) launch_add_rmsnorm<float>((float*)x, delta, w, out, rows, n_rows, dim, eps, s);
    else if (dtype == BN_DT_BF16) launch_add_rmsnorm<bf16>((float*)x, delta, w, out, rows, n_rows, dim, eps, s);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// The same with delta given as n_parts float32 slabs [n_parts][total_rows][dim] that are added in slab order
// (total_rows: the rows of x, which the slabs match).
extern "C" int bn_add_rmsnorm_parts(int dtype, void* x, const float* parts, int n_parts, int total_rows, const float* w,
                                    void* out, const int* rows, int n_rows, int dim, float eps, hipStream_t s) {
    if (n_rows <= 0 || dim <= 0 || n_parts < 1 || total_rows < 1 || !parts) return BN_ERR_ARG;
    const size_t stride = (size_t)total_rows * dim;
    if (dtype == BN_DT_F32) launch_add_rmsnorm<float, float>((float*)x, parts, w, out, rows, n_rows, dim, eps, s, n_parts, stride);
    else if (dtype == BN_DT_BF16) launch_add_rmsnorm<bf16, float>((float*)x, parts, w, out, rows, n_rows, dim, eps, s, n_parts, stride);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// Pieces of a row (= floats of ssq per row) that bn_add_rmsnorm_parts_wide wants for rows of dim elements
extern "C" int bn_add_rmsnorm_parts_pieces(int dim) { return dim > 0 ? (dim + SP_PIECE - 1) / SP_PIECE : 0; }

// x[total_rows, dim] += the n_parts slabs, all rows normed into out (no row selection); ssq: total_rows x pieces floats of
// work space.  dim a multiple of 4, everything 16-byte aligned.
extern "C" int bn_add_rmsnorm_parts_wide(int dtype, void* x, const float* parts, int n_parts, int total_rows, const float* w,
                                         void* out, float* ssq, int dim, float eps, hipStream_t s) {
    if (dim <= 0 || dim % 4 || n_parts < 1 || total_rows < 1 || total_rows > 65535 || !parts || !ssq) return BN_ERR_ARG;
    if (((uintptr_t)x | (uintptr_t)parts | (uintptr_t)w | (uintptr_t)out) & 15) return BN_ERR_ARG;
    if (dtype != BN_DT_F32 && dtype != BN_DT_BF16) return BN_ERR_DTYPE;
    const int pieces = bn_add_rmsnorm_parts_pieces(dim);
    hipLaunchKernelGGL(sum_parts_kernel, dim3(pieces, total_rows), dim3(256), 0, s, (float*)x, parts, n_parts,
                       (size_t)total_rows * dim, ssq, dim);
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(rmsnorm_ssq_kernel<float>, dim3(total_rows), dim3(256), 0, s, (const float*)x, ssq, pieces, w, (float*)out, dim, eps);
    else
        hipLaunchKernelGGL(rmsnorm_ssq_kernel<bf16>, dim3(total_rows), dim3(256), 0, s, (const float*)x, ssq, pieces, w, (bf16*)out, dim, eps);
    return bn_launch_status();
}

// x[total_rows, dim] (float32) += delta, scaled [total_rows, dim] (bf16) = the new x times w, ssq [total_rows, pieces] the
// sums of squares of the pieces of bn_add_rmsnorm_parts_pieces(dim).  delta: null, or n_parts float32 slabs
// [n_parts][total_rows][dim] (delta_dtype float32), or one bf16 tensor (delta_dtype bf16, n_parts 1).
extern "C" int bn_sum_deferred(int delta_dtype, void* x, const void* delta, int n_parts, int total_rows, const float* w,
                               void* scaled, float* ssq, int dim, hipStream_t s) {
    if (dim <= 0 || dim % 4 || total_rows < 1 || total_rows > 65535 || !x || !w || !scaled || !ssq) return BN_ERR_ARG;
    if (delta && (n_parts < 1 || (delta_dtype == BN_DT_BF16 && n_parts != 1))) return BN_ERR_ARG;
    if (((uintptr_t)x | (uintptr_t)delta | (uintptr_t)w | (uintptr_t)scaled) & 15) return BN_ERR_ARG;
    const dim3 grid(bn_add_rmsnorm_parts_pieces(dim), total_rows);
    const size_t stride = (size_t)total_rows * dim;
    if (delta_dtype == BN_DT_F32)
        hipLaunchKernelGGL(sum_deferred_kernel<float>, grid, dim3(256), 0, s, (float*)x, (const float*)delta, n_parts, stride, w,
                           (bf16*)scaled, ssq, dim);
    else if (delta_dtype == BN_DT_BF16)
        hipLaunchKernelGGL(sum_deferred_kernel<bf16>, grid, dim3(256), 0, s, (float*)x, (const bf16*)delta, n_parts, stride, w,
                           (bf16*)scaled, ssq, dim);
    else
        return BN_ERR_DTYPE;
    return bn_launch_status();
}

// bn_swiglu for bf16 with gate and up interleaved in blocks of 8, both multiplied first by the rows' deferred norm factors
// 1/sqrt(sum of ssq[row][0..n_pieces) / width + eps).
extern "C" int bn_swiglu_scaled(void* out, const void* gu, int n_rows, int F, int act, const float* ssq, int n_pieces,
                                int width, float eps, hipStream_t s) {
    if (n_rows <= 0 || F <= 0 || F % 8 || act < 0 || act >= BN_ACT_KINDS || !ssq || n_pieces < 1 || width < 1) return BN_ERR_ARG;
    if (((uintptr_t)out | (uintptr_t)gu) & 15) return BN_ERR_ARG;
    const size_t n8 = (size_t)n_rows * F / 8;
    hipLaunchKernelGGL(swiglu_scaled_bf16x8_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, s, (bf16*)out,
                       (const bf16*)gu, F, n8, 1, act, ssq, n_pieces, 1.0f / (float)width, eps);
    return bn_launch_status();
}

extern "C" int bn_residual_add_parts(void* x, const float* parts, int n_parts, long long n, hipStream_t s) {
    if (n <= 0 || n_parts < 1 || !parts) return BN_ERR_ARG;
    hipLaunchKernelGGL(residual_add_parts_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (float*)x, parts, n_parts,
                       (size_t)n);
    return bn_launch_status();
}

extern "C" int bn_residual_add(int dtype, void* x, const void* delta, long long n, hipStream_t s) {
    if (n <= 0) return BN_ERR_ARG;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(residual_add_kernel<float>, dim3(blocks), dim3(256), 0, s, (float*)x,
                           (const float*)delta, (size_t)n);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(residual_add_kernel<bf16>, dim3(blocks), dim3(256), 0, s, (float*)x,
                           (const bf16*)delta, (size_t)n);
    else
        return BN_ERR_DTYPE;
    return bn_launch_status();
}

extern "C" int bn_swiglu(int dtype, void* out, const void* gu, int n_rows, int F, int il8, int act, hipStream_t s) {
    if (n_rows <= 0 || F <= 0 || (il8 && F % 8) || act < 0 || act >= BN_ACT_KINDS) return BN_ERR_ARG;
    const size_t n = (size_t)n_rows * F;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(swiglu_kernel<float>, dim3(blocks), dim3(256), 0, s, (float*)out,
                           (const float*)gu, F, n, il8, act);
    else if (dtype == BN_DT_BF16 && F % 8 == 0 && !(((uintptr_t)out | (uintptr_t)gu) & 15))
        hipLaunchKernelGGL(swiglu_bf16x8_kernel, dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0, s, (bf16*)out,
                           (const bf16*)gu, F, n / 8, il8, act);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(swiglu_kernel<bf16>, dim3(blocks), dim3(256), 0, s, (bf16*)out,
                           (const bf16*)gu, F, n, il8, act);
    else
        return BN_ERR_DTYPE;
    return bn_launch_status();
}

extern "C" int bn_bias_add(int dtype, void* y, const float* b, int n_rows, int N, hipStream_t s) {
    if (n_rows <= 0 || N <= 0) return BN_ERR_ARG;
    const size_t n = (size_t)n_rows * N;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(bias_add_kernel<float>, dim3(blocks), dim3(256), 0, s, (float*)y, b, N, n);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(bias_add_kernel<bf16>, dim3(blocks), dim3(256), 0, s, (bf16*)y, b, N, n);
    else
        return BN_ERR_DTYPE;
    return bn_launch_status();
}
