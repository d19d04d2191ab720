// Attention over the paged cache for any even head size up to 256, any number of heads and
// kv groups, float32 or bf16 cache, written on the vector ALUs.  Head sizes whose rows are
// not whole 16-byte groups are staged element by element and padded with zeros in shared
// memory to the next multiple of 8, which changes no sum.
// It serves the float32 path, every shape the matrix-core kernels do not take, and
// both phases: a workgroup owns up to RT "rows", a row being one (query token, query
// head) pair that shares one kv head; decode is the case of one query token per
// sequence, where the keys of a long context are split over gridDim.z and merged by
// attn_combine_kernel in a fixed order.
//
// Formulas (reference): kv head of head h is h / (H/Hkv) (src/transformer/gqa_scalar.c:77);
// score = (q.k) * scale, the product first (gqa_scalar.c:92-93); only keys at
// positions <= the query's are visited (gqa_scalar.c:69,80); softmax by max-subtract
// and exp, here as the online form of src/transformer/gqa_scalar.c:127-207 with
// expf; out = sum_t p_t * V_t (gqa_scalar.c:104-119).  All of it in float32.
#include "common.h"
#include <math.h>

#define ATT_THREADS 256

struct AttnArgs {
    const void* q;        // [n_tokens, q_stride], head h at h*hs (already rotated)
    void* out;            // [n_tokens, out_stride], head h at h*hs
    const void* k_pages;  // [n_pages, Hkv, BN_PAGE, hs]
    const void* v_pages;
    const int* block_table;   // [n_seqs, bt_stride] page of each BN_PAGE positions
    const int* seq_lens;      // [n_seqs] keys in the cache after this step (decode mode)
    const int* tiles;         // [n_tiles, 4] = seq, first token row, n tokens, position of the
                              // first; null = decode: tile b is sequence b's one new token
    float* part_o;            // [n_tokens*H, n_splits, hs]   (n_splits > 1)
    float* part_ml;           // [n_tokens*H, n_splits, 2]
    int q_stride, out_stride, bt_stride;
    int H, Hkv, hs;
    int GT;                   // heads of one kv group handled together (power of two <= RT)
    int KT;                   // keys per tile: 16, 32 or 64
    int window;               // 0 = all earlier keys, else the last `window` of them
    int n_splits, chunk;      // keys per split, a multiple of BN_PAGE
    int v_transposed;         // V pages are [page, kv_head, hs, BN_PAGE]
    float scale;
    const int* max_len;       // != null (decode form, n_splits > 1): the longest sequence's key count in device
                              // memory; the keys per split follow from it (bn_split_chunk) instead of from `chunk`
    int fold;                 // > 0: keys are summed in runs of `fold` positions (a multiple of BN_PAGE, counted from
                              // position 0) and the runs folded in order (fold_factors, fold_value below); a split is then one run
};

// The fold of one run of keys into the sums of the runs before it: (M, L, O) <- (M, L, O) + (m, l, o) with both sides
// rescaled to the larger maximum.  Every place that folds calls these two functions, and their operations are written out
// (no contraction left to the compiler), so the same runs give the same bits wherever they are folded.
__device__ __forceinline__ void fold_factors(float M, float m, float& m2, float& fa, float& fb) {
    m2 = fmaxf(M, m);
    fa = expf(M - m2);                                   // 0 when nothing was there before (M = -inf)
    fb = expf(m - m2);
}
__device__ __forceinline__ float fold_value(float O, float fa, float o, float fb) { return __fmaf_rn(O, fa, __fmul_rn(o, fb)); }

template <typename T> struct Vec4;
template <> struct Vec4<float> {
    typedef float4 type;
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        float4 t = *reinterpret_cast<const float4*>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
};
template <> struct Vec4<bf16> {
    typedef uint2 type;
    static __device__ __forceinline__ void load(const bf16* p, float (&v)[4]) {
        uint2 t = *reinterpret_cast<const uint2*>(p);
        v[0] = bf16lo_to_f32(t.x); v[1] = bf16hi_to_f32(t.x);
        v[2] = bf16lo_to_f32(t.y); v[3] = bf16hi_to_f32(t.y);
    }
};

template <typename T, int RT>
__global__ __launch_bounds__(ATT_THREADS) void attn_rows_kernel(AttnArgs a) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int hs = a.hs, KT = a.KT, GT = a.GT;
    const int hsp = (hs + 7) & ~7;                       // the head size padded to whole groups of 8
    const int QT = RT / GT;
    const int G = a.H / a.Hkv;
    const int n_head_tiles = (G + GT - 1) / GT;
    const int kvh = blockIdx.y / n_head_tiles;
    const int ht = blockIdx.y - kvh * n_head_tiles;
    const int split = blockIdx.z;
    const int tid = threadIdx.x;

    int seq, tok0, n_tok, pos0;
    if (a.tiles) {
        const int* tl = a.tiles + 4 * blockIdx.x;
        seq = tl[0]; tok0 = tl[1]; n_tok = tl[2]; pos0 = tl[3];
    } else {
        seq = blockIdx.x; tok0 = blockIdx.x; n_tok = 1; pos0 = a.seq_lens[seq] - 1;
    }
    if (n_tok > QT) n_tok = QT;

    // shared memory
    const int kstride = hsp + 16 / (int)sizeof(T);       // elements; keeps rows 16-byte aligned
    float* q_s = reinterpret_cast<float*>(smem_raw);     // [RT][hsp], zero beyond hs
    float* s_s = q_s + RT * hsp;                         // [RT][KT] scores
    float* p_s = s_s + RT * KT;                          // [KT][RT] probabilities
    float* m_s = p_s + KT * RT;                          // [16] running max
    float* l_s = m_s + 16;                               // [16] running sum
    float* a_s = l_s + 16;                               // [16] rescale of this tile
    float* Mt_s = a_s + 16;                              // [16] fold mode: maximum and sum over the runs folded so far,
    float* Lt_s = Mt_s + 16;                             // [16]
    float* fa_s = Lt_s + 16;                             // [16] and the factors of the fold that is under way
    float* fb_s = fa_s + 16;                             // [16]
    T* k_s = reinterpret_cast<T*>(fb_s + 16);            // [KT][kstride]
    T* v_s = k_s + KT * kstride;

    // rows: r = i*GT + g  ->  token tok0+i, head kvh*G + ht*GT + g
    for (int idx = tid; idx < RT * hsp; idx += ATT_THREADS) {
        const int r = idx / hsp, d = idx - r * hsp;
        const int i = r / GT, g = r - i * GT;
        const int hg = ht * GT + g;
        float v = 0.f;
        if (d < hs && i < n_tok && hg < G && pos0 >= 0) {
            const T* qp = reinterpret_cast<const T*>(a.q) + (size_t)(tok0 + i) * a.q_stride +
                          (size_t)(kvh * G + hg) * hs;
            v = to_f32(qp[d]);
        }
        q_s[idx] = v;
    }
    if (tid < 16) { m_s[tid] = -INFINITY; l_s[tid] = 0.f; a_s[tid] = 1.f; Mt_s[tid] = -INFINITY; Lt_s[tid] = 0.f; }
    const bool whole_groups = (hs * (int)sizeof(T)) % 16 == 0;      // rows of 16-byte groups in the pages
    if (hsp != hs)                                                  // the padding of the staged rows stays zero
        for (int idx = tid; idx < 2 * KT * kstride; idx += ATT_THREADS) k_s[idx] = from_f32<T>(0.f);

    // keys this workgroup visits
    int lo = 0, hi = 0;
    if (pos0 >= 0 && n_tok > 0) {
        hi = pos0 + n_tok;                                        // exclusive
        lo = a.window > 0 ? max(0, pos0 + 1 - a.window) : 0;      // first key of the first row
        const int chunk = a.max_len ? bn_split_chunk(*a.max_len, a.n_splits) : a.chunk;
        lo = max(lo, split * chunk);
        hi = min(hi, (split + 1) * chunk);
    }

    // phase C ownership: thread -> (jp, dp): keys jp, jp+JP, ...; output dims 2dp, 2dp+1
    const int DP = hs / 2;
    int JP = ATT_THREADS / DP; if (JP > 8) JP = 8; if (JP > KT) JP = KT;
    const int jp = tid / DP, dp = tid - jp * DP;
    const bool c_active = jp < JP;
    float acc[RT][2];
#pragma unroll
    for (int r = 0; r < RT; ++r) { acc[r][0] = 0.f; acc[r][1] = 0.f; }

    // fold mode: the sums over the runs folded so far (the threads with jp == 0 hold them)
    float tot[RT][2];
#pragma unroll
    for (int r = 0; r < RT; ++r) { tot[r][0] = 0.f; tot[r][1] = 0.f; }
    // Adds the JP partial accumulators up in a fixed order, through `scratch` ([RT][hs] floats that nobody else uses now);
    // the threads with jp == 0 then hold the sums.
    auto sum_partials = [&](float* scratch) {
        for (int src = 1; src < JP; ++src) {
            if (c_active && jp == src) {
#pragma unroll
                for (int r = 0; r < RT; ++r) { scratch[r * hs + 2 * dp] = acc[r][0]; scratch[r * hs + 2 * dp + 1] = acc[r][1]; }
            }
            __syncthreads();
            if (jp == 0) {
#pragma unroll
                for (int r = 0; r < RT; ++r) { acc[r][0] += scratch[r * hs + 2 * dp]; acc[r][1] += scratch[r * hs + 2 * dp + 1]; }
            }
            __syncthreads();
        }
    };
    // The end of a run of keys: its sums join the sums of the runs before it, and the next run starts from nothing.  The
    // staged keys are not needed any more when this is called (a barrier has passed): their memory is the scratch.
    auto fold_run = [&]() {
        sum_partials(reinterpret_cast<float*>(k_s));
        if (tid < RT) {
            const float m = m_s[tid];
            float fa = 1.f, fb = 0.f;
            if (m != -INFINITY) {                         // a run of which this row saw no key changes nothing
                float m2;
                fold_factors(Mt_s[tid], m, m2, fa, fb);
                Lt_s[tid] = fold_value(Lt_s[tid], fa, l_s[tid], fb);
                Mt_s[tid] = m2;
            }
            fa_s[tid] = fa; fb_s[tid] = fb;
            m_s[tid] = -INFINITY; l_s[tid] = 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            if (jp == 0 && fb_s[r] != 0.f) {
                tot[r][0] = fold_value(tot[r][0], fa_s[r], acc[r][0], fb_s[r]);
                tot[r][1] = fold_value(tot[r][1], fa_s[r], acc[r][1], fb_s[r]);
            }
            acc[r][0] = 0.f; acc[r][1] = 0.f;
        }
        if (hsp != hs)                                    // the scratch lay over the staged rows, whose padding is zero
            for (int idx = tid; idx < 2 * KT * kstride; idx += ATT_THREADS) k_s[idx] = from_f32<T>(0.f);
        __syncthreads();
    };

    const int P = ATT_THREADS / KT;          // threads per key in phase A: 4, 8 or 16
    const int ja = tid / P, pa = tid - ja * P;
    const int n_chunks = hsp / 4;
    const int lane = tid & 63, wave = tid >> 6;
    __syncthreads();

    for (int j0 = (lo / KT) * KT; j0 < hi; j0 += KT) {
        // ---- load the K and V tile (rows j0 .. j0+KT-1 of one page) ----
        {
            const int page = a.block_table[(size_t)seq * a.bt_stride + j0 / BN_PAGE];
            const size_t base = (((size_t)page * a.Hkv + kvh) * BN_PAGE + (j0 % BN_PAGE)) * hs;
            const int vec_per_row = hs * (int)sizeof(T) / 16;
            const uint4* kg = reinterpret_cast<const uint4*>(reinterpret_cast<const T*>(a.k_pages) + base);
            const uint4* vg = reinterpret_cast<const uint4*>(reinterpret_cast<const T*>(a.v_pages) + base);
            for (int idx = tid; whole_groups && idx < KT * vec_per_row; idx += ATT_THREADS) {
                const int j = idx / vec_per_row, c = idx - j * vec_per_row;
                uint4 kv = make_uint4(0, 0, 0, 0), vv = make_uint4(0, 0, 0, 0);
                if (j0 + j < hi) { kv = kg[idx]; if (!a.v_transposed) vv = vg[idx]; }   // rows not yet written stay zero
                *reinterpret_cast<uint4*>(reinterpret_cast<unsigned char*>(k_s + j * kstride) + c * 16) = kv;
                if (!a.v_transposed)
                    *reinterpret_cast<uint4*>(reinterpret_cast<unsigned char*>(v_s + j * kstride) + c * 16) = vv;
            }
            if (!whole_groups) {
                const T* ke = reinterpret_cast<const T*>(a.k_pages) + base;
                const T* ve = reinterpret_cast<const T*>(a.v_pages) + base;
                for (int idx = tid; idx < KT * hs; idx += ATT_THREADS) {
                    const int j = idx / hs, d = idx - j * hs;
                    const bool in = j0 + j < hi;
                    k_s[j * kstride + d] = in ? ke[idx] : from_f32<T>(0.f);
                    if (!a.v_transposed) v_s[j * kstride + d] = in ? ve[idx] : from_f32<T>(0.f);
                }
            }
            if (a.v_transposed) {
                const T* vt = reinterpret_cast<const T*>(a.v_pages) + ((size_t)page * a.Hkv + kvh) * hs * BN_PAGE +
                              (j0 % BN_PAGE);
                for (int idx = tid; idx < KT * hs; idx += ATT_THREADS) {
                    const int d = idx / KT, j = idx - d * KT;
                    v_s[j * kstride + d] = (j0 + j < hi) ? vt[(size_t)d * BN_PAGE + j] : from_f32<T>(0.f);
                }
            }
        }
        __syncthreads();
        // ---- phase A: scores ----
        {
            float dot[RT];
#pragma unroll
            for (int r = 0; r < RT; ++r) dot[r] = 0.f;
            const T* kr = k_s + ja * kstride;
            for (int c = pa; c < n_chunks; c += P) {
                float kv[4];
                Vec4<T>::load(kr + c * 4, kv);
#pragma unroll
                for (int r = 0; r < RT; ++r) {
                    const float4 qv = *reinterpret_cast<const float4*>(q_s + r * hsp + c * 4);
                    dot[r] = fmaf(kv[0], qv.x, dot[r]);
                    dot[r] = fmaf(kv[1], qv.y, dot[r]);
                    dot[r] = fmaf(kv[2], qv.z, dot[r]);
                    dot[r] = fmaf(kv[3], qv.w, dot[r]);
                }
            }
#pragma unroll
            for (int r = 0; r < RT; ++r) {
                float v = dot[r];
                for (int o = 1; o < P; o <<= 1) v += __shfl_xor(v, o, BN_WAVE);
                dot[r] = v;
            }
            const int key = j0 + ja;
#pragma unroll
            for (int r = 0; r < RT; ++r) {
                if ((r % P) == pa) {
                    const int i = r / GT, g = r - i * GT;
                    const int qpos = pos0 + i;
                    bool ok = (i < n_tok) && (ht * GT + g < G) && key <= qpos && key >= lo && key < hi;
                    if (a.window > 0) ok = ok && (key > qpos - a.window);
                    s_s[r * KT + ja] = ok ? dot[r] * a.scale : -INFINITY;
                }
            }
        }
        __syncthreads();
        // ---- phase B: online softmax, one wave per row ----
        for (int r = wave; r < RT; r += ATT_THREADS / 64) {
            const float sv = lane < KT ? s_s[r * KT + lane] : -INFINITY;
            const float tmax = wave_max(sv);
            const float m_old = m_s[r];
            const float m_new = fmaxf(m_old, tmax);
            float p = 0.f, alpha = 1.f;
            if (m_new != -INFINITY) {
                p = expf(sv - m_new);                 // exp(-inf) = 0 for masked keys
                alpha = expf(m_old - m_new);          // 0 when nothing was seen before
            }
            const float psum = wave_sum(p);
            if (lane < KT) p_s[lane * RT + r] = p;
            if (lane == 0) {
                m_s[r] = m_new;
                l_s[r] = l_s[r] * alpha + psum;
                a_s[r] = alpha;
            }
        }
        __syncthreads();
        // ---- phase C: acc = acc*alpha + P.V ----
        if (c_active) {
#pragma unroll
            for (int r = 0; r < RT; ++r) { const float al = a_s[r]; acc[r][0] *= al; acc[r][1] *= al; }
            const int kt_valid = min(KT, hi - j0);
            for (int j = jp; j < kt_valid; j += JP) {
                float v0, v1;
                if (sizeof(T) == 2) {
                    const uint32_t two = *reinterpret_cast<const uint32_t*>(
                        reinterpret_cast<const unsigned char*>(v_s + j * kstride) + dp * 4);
                    v0 = bf16lo_to_f32(two); v1 = bf16hi_to_f32(two);
                } else {
                    const float2 two = *reinterpret_cast<const float2*>(
                        reinterpret_cast<const unsigned char*>(v_s + j * kstride) + dp * 8);
                    v0 = two.x; v1 = two.y;
                }
#pragma unroll
                for (int r = 0; r < RT; ++r) {
                    const float p = p_s[j * RT + r];
                    acc[r][0] = fmaf(p, v0, acc[r][0]);
                    acc[r][1] = fmaf(p, v1, acc[r][1]);
                }
            }
        }
        __syncthreads();
        // a run of keys ends here and more keys follow (one workgroup walks several runs: a prompt step, or a decode step
        // whose keys are not split): fold it
        if (a.fold > 0 && a.n_splits == 1 && (j0 + KT) % a.fold == 0 && j0 + KT < hi) fold_run();
    }

    const bool folded = a.fold > 0 && a.n_splits == 1;
    if (folded) {
        fold_run();                                       // the last run; the result is in tot, Mt_s, Lt_s
    } else {
        // ---- sum the JP partial accumulators in a fixed order (q_s is free now) ----
        sum_partials(q_s);
    }
    if (jp != 0) return;
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const int i = r / GT, g = r - i * GT;
        const int hg = ht * GT + g;
        const bool decode_pad = (a.tiles == nullptr) && pos0 < 0;
        if (!((i < n_tok || (decode_pad && i == 0)) && hg < G)) continue;
        const int head = kvh * G + hg;
        const size_t tok = (size_t)(tok0 + i);
        if (a.n_splits == 1) {
            const float l = folded ? Lt_s[r] : l_s[r];
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            T* o = reinterpret_cast<T*>(a.out) + tok * a.out_stride + (size_t)head * hs + 2 * dp;
            o[0] = from_f32<T>(__fmul_rn(folded ? tot[r][0] : acc[r][0], inv));
            o[1] = from_f32<T>(__fmul_rn(folded ? tot[r][1] : acc[r][1], inv));
        } else {
            const size_t row = (tok * a.H + head) * a.n_splits + split;
            a.part_o[row * hs + 2 * dp] = acc[r][0];
            a.part_o[row * hs + 2 * dp + 1] = acc[r][1];
            if (dp == 0) { a.part_ml[row * 2] = m_s[r]; a.part_ml[row * 2 + 1] = l_s[r]; }
        }
    }
}

// out[row, d] = sum_s e^{m_s - m} o_s[d] / sum_s e^{m_s - m} l_s, splits in index order
template <typename T>
__global__ void attn_combine_kernel(T* __restrict__ out, int out_stride, const float* __restrict__ part_o,
                                    const float* __restrict__ part_ml, int H, int hs, int n_splits) {
    const int row = blockIdx.x;               // token*H + head
    const int tok = row / H, head = row - tok * H;
    const float* ml = part_ml + (size_t)row * n_splits * 2;
    float m = -INFINITY;
    for (int s = 0; s < n_splits; ++s) m = fmaxf(m, ml[2 * s]);
    for (int d = threadIdx.x; d < hs; d += blockDim.x) {
        float num = 0.f, den = 0.f;
        if (m != -INFINITY) {
            for (int s = 0; s < n_splits; ++s) {
                const float w = expf(ml[2 * s] - m);          // 0 for an empty split
                num = fmaf(w, part_o[((size_t)row * n_splits + s) * hs + d], num);
                den = fmaf(w, ml[2 * s + 1], den);
            }
        }
        out[(size_t)tok * out_stride + (size_t)head * hs + d] = from_f32<T>(den > 0.f ? num / den : 0.f);
    }
}

// The merge of a decode step whose keys were split in runs (fold mode): the runs' sums folded in run order with the
// operations of fold_factors and fold_value, which is what a workgroup that walks all runs by itself does; runs without keys are passed over.
template <typename T>
__global__ void attn_fold_kernel(T* __restrict__ out, int out_stride, const float* __restrict__ part_o,
                                 const float* __restrict__ part_ml, int H, int hs, int n_splits) {
    const int row = blockIdx.x;               // token*H + head
    const int tok = row / H, head = row - tok * H;
    const float* ml = part_ml + (size_t)row * n_splits * 2;
    for (int d = threadIdx.x; d < hs; d += blockDim.x) {
        float M = -INFINITY, L = 0.f, O = 0.f;
        for (int s = 0; s < n_splits; ++s) {
            const float m = ml[2 * s];
            if (m == -INFINITY) continue;
            float m2, fa, fb;
            fold_factors(M, m, m2, fa, fb);
            L = fold_value(L, fa, ml[2 * s + 1], fb);
            O = fold_value(O, fa, part_o[((size_t)row * n_splits + s) * hs + d], fb);
            M = m2;
        }
        const float inv = L > 0.f ? 1.0f / L : 0.f;
        out[(size_t)tok * out_stride + (size_t)head * hs + d] = from_f32<T>(__fmul_rn(O, inv));
    }
}

static size_t attn_smem_bytes(int RT, int hs, int KT, int elt) {
    const int hsp = (hs + 7) & ~7;
    return (size_t)(RT * hsp + 2 * RT * KT + 112) * sizeof(float) + (size_t)2 * KT * (hsp * elt + 16);
}

template <typename T, int RT>
static int launch_rows(const AttnArgs& a, int n_tiles, hipStream_t s) {
    const int G = a.H / a.Hkv;
    const int n_head_tiles = (G + a.GT - 1) / a.GT;
    const size_t smem = attn_smem_bytes(RT, a.hs, a.KT, (int)sizeof(T));
    hipLaunchKernelGGL((attn_rows_kernel<T, RT>), dim3(n_tiles, a.Hkv * n_head_tiles, a.n_splits),
                       dim3(ATT_THREADS), smem, s, a);
    return bn_launch_status();
}

template <typename T>
static int launch_rows_rt(const AttnArgs& a, int RT, int n_tiles, hipStream_t s) {
    switch (RT) {
        case 1: return launch_rows<T, 1>(a, n_tiles, s);
        case 2: return launch_rows<T, 2>(a, n_tiles, s);
        case 4: return launch_rows<T, 4>(a, n_tiles, s);
        case 8: return launch_rows<T, 8>(a, n_tiles, s);
        case 16: return launch_rows<T, 16>(a, n_tiles, s);
    }
    return BN_ERR_ARG;
}

// Keys per tile: the largest of 64, 32, 16 whose shared memory stays within 64 KB for the widest
// workgroup (16 rows); 0 if none does.  It is a function of the cache type and the head size alone,
// never of the rows a launch happens to hold: a query's keys are then cut into the same tiles, and
// its sums formed in the same order, whether it arrives alone, in a prompt or in a batch (the
// reference keeps one order per kernel, src/transformer/gqa_scalar.c:61-121).
extern "C" int bn_attn_rows_key_tile(int dtype, int hs) {
    const int elt = dtype == BN_DT_F32 ? 4 : 2;
    for (int kt = 64; kt >= 16; kt >>= 1)
        if (attn_smem_bytes(16, hs, kt, elt) <= 64 * 1024) return kt;
    return 0;
}

// RT rows per workgroup = QT query tokens x GT heads.  tiles == null: decode (one token per
// sequence, n_tiles sequences).  With n_splits > 1 the partial buffers must hold
// n_tokens*H*n_splits rows and the combine kernel runs right after.
extern "C" int bn_attn_rows(int dtype, const void* q, int q_stride, void* out, int out_stride,
                            const void* k_pages, const void* v_pages, const int* block_table,
                            int bt_stride, const int* seq_lens, const int* tiles, int n_tiles,
                            int n_tokens, int H, int Hkv, int hs, int RT, int GT, int window,
                            float scale, int n_splits, int chunk, float* part_o, float* part_ml,
                            int v_transposed, const int* max_len, int fold, hipStream_t s) {
    if (n_tiles <= 0 || n_tokens <= 0 || H <= 0 || Hkv <= 0 || H % Hkv) return BN_ERR_ARG;
    // fold mode: runs of whole pages; a split is one run, and the runs' length does not follow the longest sequence
    if (fold < 0 || fold % BN_PAGE || (fold > 0 && n_splits > 1 && (chunk != fold || max_len))) return BN_ERR_ARG;
    if (hs < 2 || hs > BN_MAX_HEAD_DIM || hs % 2) return BN_ERR_ARG;
    if (GT <= 0 || GT > RT || (GT & (GT - 1)) || RT > 16 || (RT & (RT - 1))) return BN_ERR_ARG;
    if (n_splits < 1 || window < 0) return BN_ERR_ARG;
    if (n_splits > 1 && (!part_o || !part_ml || (!max_len && (chunk <= 0 || chunk % BN_PAGE)))) return BN_ERR_ARG;
    if (!tiles && !seq_lens) return BN_ERR_ARG;
    if (max_len && tiles) return BN_ERR_ARG;
    AttnArgs a;
    a.max_len = n_splits > 1 ? max_len : nullptr;
    a.q = q; a.out = out; a.k_pages = k_pages; a.v_pages = v_pages;
    a.block_table = block_table; a.seq_lens = seq_lens; a.tiles = tiles;
    a.part_o = part_o; a.part_ml = part_ml;
    a.q_stride = q_stride; a.out_stride = out_stride; a.bt_stride = bt_stride;
    a.H = H; a.Hkv = Hkv; a.hs = hs; a.GT = GT; a.window = window;
    a.n_splits = n_splits; a.chunk = n_splits > 1 ? chunk : 0x40000000;
    a.scale = scale;
    a.v_transposed = v_transposed;
    a.fold = fold;
    a.KT = bn_attn_rows_key_tile(dtype, hs);
    if (a.KT == 0) return BN_ERR_ARG;
    int rc;
    if (dtype == BN_DT_F32) rc = launch_rows_rt<float>(a, RT, n_tiles, s);
    else if (dtype == BN_DT_BF16) rc = launch_rows_rt<bf16>(a, RT, n_tiles, s);
    else return BN_ERR_DTYPE;
    if (rc != 0 || n_splits == 1) return rc;
    if (fold > 0) {
        if (dtype == BN_DT_F32)
            hipLaunchKernelGGL(attn_fold_kernel<float>, dim3(n_tokens * H), dim3(64), 0, s, (float*)out, out_stride, part_o,
                               part_ml, H, hs, n_splits);
        else
            hipLaunchKernelGGL(attn_fold_kernel<bf16>, dim3(n_tokens * H), dim3(64), 0, s, (bf16*)out, out_stride, part_o,
                               part_ml, H, hs, n_splits);
        return bn_launch_status();
    }
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(attn_combine_kernel<float>, dim3(n_tokens * H), dim3(64), 0, s, (float*)out,
                           out_stride, part_o, part_ml, H, hs, n_splits);
    else
        hipLaunchKernelGGL(attn_combine_kernel<bf16>, dim3(n_tokens * H), dim3(64), 0, s, (bf16*)out,
                           out_stride, part_o, part_ml, H, hs, n_splits);
    return bn_launch_status();
}
