// Attention over the paged bf16 cache on the matrix cores (v_mfma_f32_16x16x32_bf16), for
// head sizes 64 and 128, both phases.  Formulas as in attn_rows.hip (reference:
// src/transformer/gqa_scalar.c:61-207, src/transformer/batched_attn_scalar.c:97-245):
// kv head of head h is h / (H/Hkv); score = (q.k) * scale over the keys at positions <= the
// query's (and inside the window); online softmax; out = sum_t p_t V_t.  Scores, maxima,
// sums and the output accumulate in float32; p is rounded to bf16 for the second product.
//
// A wave works on "columns": a column is one (query token, query head) pair of one kv head,
// 16 columns per MFMA tile.  Everything stays in registers:
//   S^T[key, col]  = K[key, :] . Q[col, :]          A = 16 key rows of K,   B = Q^T
//   O^T[dim, col] += V^T[dim, keys] . P^T[keys, col]  A = 16 rows of V^T,   B = P^T
// The S^T tile leaves lane (col, g) with 4 keys per 16-key tile; the key rows fed to the two
// tiles of a 32-key block are permuted (row i of tile sb is key 8*(i/4) + 4*sb + i%4) so
// that each lane group g ends up with the 8 consecutive keys 8g..8g+7, which is exactly what
// the B operand of the second product wants and what 16 bytes of 8 consecutive positions of one
// value dimension hold.  The pages are laid out for exactly these operands ("blocked" pages,
// common.h): a (page, kv head) holds its 64 positions in two blocks of 32, and a block its keys and
// its values tile by tile in the lanes' order, so that the decode form loads an operand tile as 1 KB of
// consecutive bytes and the prompt form fetches a stage as one run.
//
// Prompt form: a workgroup of 4 waves owns 64*NT columns = consecutive query tokens x GT heads;
// the keys and values it walks are staged through shared memory once for all four waves.
// Decode form: the 16 columns are the heads of one kv group for the sequence's one new token;
// the 4 waves take 32-key blocks in turn and merge through shared memory; long contexts are
// also split over gridDim.z and merged by attn_mfma_combine_kernel in a fixed order.  What a decode workgroup needs
// before its first block (the query, the frequencies, the new key and value, the length, the first block itself) is
// asked for at once, in straight-line code, with the length and the page numbers through the scalar unit: the first
// block of keys is on its way before the length is known (see the kernel), so that a short launch is two trips to
// memory instead of five.  Every entry of a block table must name a page of the pool for that, also the entries
// behind a sequence's last page.
#include "common.h"
#include "attn_mfma.h"
#include <mutex>

#define PROMPT_BUFFERS 3      // staged key blocks of the prompt form in shared memory

static int compute_units() {
    static int n[64] = {0};                 // per device
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (n[dev] == 0) {
        int v = 0;
        n[dev] = (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) ? v : 256;
    }
    return n[dev];
}
#include <math.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define LOG2E 1.4426950408889634f
#define LN2 0.6931471805599453f

struct MfmaArgs {
    const bf16* q;            // [n_tokens, q_stride], head h at h*HS, rotated
    bf16* out;                // [n_tokens, out_stride]
    const bf16* k_pages;      // [pages, Hkv, 64 * HS]: keys in the blocked order of common.h
    const bf16* vt_pages;     // [pages, Hkv, HS * 64]: values in the blocked order of common.h
    const int* block_table;   // [n_seqs, bt_stride]
    const int* seq_lens;      // decode: keys in the cache, the new one included; 0 = padding row
    const int* tiles;         // prompt: [n, 4] = seq, first token row, tokens, position of the first
    float* part_o;            // [n_tokens*H, n_splits, HS]
    float* part_ml;           // [n_tokens*H, n_splits, 2]   (max in natural-log units, sum)
    int q_stride, out_stride, bt_stride;
    int H, Hkv, GT;           // GT: heads of a kv group per column tile row (power of two <= 16)
    int window;
    int n_splits, chunk;
    float scale;
    // decode form only.  rotate != 0: q (and the new key) arrive unrotated and are rotated here,
    // angle = position * inv_freq[i], pairs (i, i + HS/2).  write_kv != 0: the workgroup whose keys
    // include the new position stores the new key (rotated) and value into the pages first.
    const float* inv_freq;
    int rotate, write_kv;
    // by_length != null: the sequences ordered by length, longest first.  Workgroups are handed out
    // in that order, every other run of `order_period` sequences backwards: when the launch puts
    // two workgroups on every CU, the ones that share a CU are then a long and a short sequence.
    const int* by_length;
    int order_period;
    // row_ssq != null (decode form with rotate): q, the new key and the new value of row b are what a product made of
    // an RMSNorm's input times the norm's weights, without the norm's factor (a deferred norm).  The factor
    // 1/sqrt(sum of row_ssq[b][0..n_pieces) / ssq_width + eps) multiplies the whole row, so it is applied here: folded
    // into the rotation's cosines and sines for q and the key, a multiplication for the value.
    const float* row_ssq;
    int n_pieces;
    float inv_ssq_width, ssq_eps;
    // max_len != null (decode form, n_splits > 1): the longest sequence's key count lives in device memory and
    // the keys per split follow from it (bn_split_chunk) instead of from `chunk`: a captured launch then adapts
    // its splits to the lengths of every replay.
    const int* max_len;
};

__device__ __forceinline__ bf16x8 ld16(const bf16* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
// Combining a value with the ones 16 and 32 lanes away (the four lane groups of a column) without
// going through shared memory: gfx950 swaps 16- and 32-lane halves between two registers.
// The largest of three in one instruction; fmaxf would first bring each operand into canonical form (an instruction
// each), which the scores out of the matrix cores do not need.
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float max_over_lane_groups(float x) {
    const unsigned b = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    const unsigned c = __float_as_uint(fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1])));
    auto t = __builtin_amdgcn_permlane32_swap(c, c, false, false);
    return fmaxf(__uint_as_float(t[0]), __uint_as_float(t[1]));
}
typedef __attribute__((ext_vector_type(8))) float f32x8;
// eight floats to eight bf16, round to nearest even (gfx950 converts two a time in hardware)
__device__ __forceinline__ bf16x8 pack8(const float (&s)[8]) {
    const f32x8 v = {s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7]};
    return __builtin_convertvector(v, bf16x8);
}
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    // round to nearest even, as __float2bfloat16 does
    uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b);
    ua += 0x7fffu + ((ua >> 16) & 1u);
    ub += 0x7fffu + ((ub >> 16) & 1u);
    return (ua >> 16) | (ub & 0xffff0000u);
}

// A barrier of the workgroup that orders its shared memory only.  __syncthreads() also waits for everything that the wave
// has asked from global memory; this one leaves such loads in flight (whoever needs their data waits for it there).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// The float32 value of a bf16 bit pattern, widened where this stands and nowhere else: the compiler moves a plain shift
// up to the load of the pattern, and the load's wait with it.
__device__ __forceinline__ float widen_here(unsigned bits) {
    float f;
    asm volatile("v_lshlrev_b32 %0, 16, %1" : "=v"(f) : "v"(bits));
    return f;
}

// A read of p[idx] for an index that is the same in every lane, through the scalar unit (the
// constant address space makes the compiler pick a scalar load).  Only for memory that no kernel
// writes while this one runs (block tables, lengths).
__device__ __forceinline__ int uniform_load(const int* p, size_t idx) {
    typedef const int __attribute__((address_space(4))) * scalar_ptr;
    return reinterpret_cast<scalar_ptr>(reinterpret_cast<uintptr_t>(p))[idx];
}

// Shared memory serves 16 lanes of a 16-byte read at once, from 64 banks of 4 bytes.  The lanes
// that read a staged key block together hold rows 8a + b (+4 for the second tile), a, b in 0..3, and
// all want the same 16-byte chunk: rows are stored without padding and chunk c of row r lives at
// c ^ f(r), with f distinct for those 16 rows over the 256 bytes that the banks span (head size
// 128: a row is 256 bytes, f = 4a + b; head size 64: two rows share 256 bytes, the row's parity is
// one bit already and f = 2a + b/2 supplies the other three).
template <int HS>
__device__ __forceinline__ int k_swizzle(int row) {
    const int a = (row >> 3) & 3, b = row & 3;
    return HS == 128 ? (a << 2 | b) : (a << 1 | b >> 1);
}

// A 16-byte read serves the lanes in four turns of 16: quads of lanes {0, 3, 5, 6}, {1, 2, 4, 7} and
// the same of the upper 32 lanes (measured with a probe kernel and the bank-conflict counter).  In
// the operand layout lane = i + 16 g, so a turn holds two values of g (0 and 1, or 2 and 3) and, for
// the even one, i/4 in {0, 3}, for the odd one i/4 in {1, 2} (the other turn: the other way round).
// The staged V^T block (rows = dimensions, 16-byte chunks of 8 keys) is stored without padding with
// chunk c of row r at c ^ v_swizzle(r): h(i/4) = (-(i/4)) & 3 makes g ^ h distinct over a turn for
// rows that share their position inside 256 bytes; with 64 keys a row (two rows in 256 bytes, the
// row's lowest bit separates them) bit 1 of the row goes into bit 2 of the chunk as well.
template <int KEYS>
__device__ __forceinline__ int v_swizzle(int row) {
    const int h = (-(row >> 2)) & 3;
    return KEYS == 64 ? (h | ((row >> 1) & 1) << 2) : h;
}

// One 32-key block for NT column tiles, operands straight from the pages (the decode form).  kbase/vbase point at
// the block inside its page (blocked pages, common.h: every load below is 1 KB of consecutive bytes).  qpos/lo: per tile, this lane's column's
// position and first visible key (qpos < 0: no such column).  key_hi: keys >= key_hi do not exist (split end /
// length).  All operands are asked for up front: they come from memory, and the latency is paid once.
// The prompt form below has code of its own on purpose: the decode kernel is sensitive to how the compiler lays
// this code out, and changes made for the staged form must not move it.
// The operands of a block of 32 keys from blocked pages: tile row i of key tile 0 is the block's key 8 (i / 4) + i % 4,
// tile 1 four further; lane i + 16 g of value tile t holds dimension 16 t + i of the block's keys 8 g .. 8 g + 7.
template <int HS>
__device__ __forceinline__ void load_block(const bf16* __restrict__ kbase, const bf16* __restrict__ vbase,
                                           bf16x8 (&ka)[HS / 32][2], bf16x8 (&va)[HS / 16], int lane) {
#pragma unroll
    for (int c = 0; c < HS / 32; ++c) {
        ka[c][0] = ld16(kbase + (2 * c) * 512 + lane * 8);
        ka[c][1] = ld16(kbase + (2 * c + 1) * 512 + lane * 8);
    }
#pragma unroll
    for (int t = 0; t < HS / 16; ++t) va[t] = ld16(vbase + t * 512 + lane * 8);
}

template <int HS, int NT, bool need_mask>
__device__ __forceinline__ void attend_loaded_m(const bf16x8 (&ka)[HS / 32][2], bf16x8 (&va)[HS / 16],
                                               int kb, const bf16x8 (&q)[NT][HS / 32], f32x4 (&acc)[NT][HS / 16],
                                               float (&m)[NT], float (&l)[NT], const int (&qpos)[NT],
                                               const int (&lo)[NT], int key_hi, float scale2, int lane) {
    constexpr int DC = HS / 32, DT = HS / 16;
    const int g = lane >> 4;
    f32x4 st[NT][2];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) { st[nt][0] = (f32x4){0.f, 0.f, 0.f, 0.f}; st[nt][1] = (f32x4){0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
    for (int c = 0; c < DC; ++c) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            st[nt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[c][0], q[nt][c], st[nt][0], 0, 0, 0);
            st[nt][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[c][1], q[nt][c], st[nt][1], 0, 0, 0);
        }
    }
    // keys that do not exist may hold anything, NaN included: they are cleared in V^T (0 * NaN is NaN)
    const int first = kb + 8 * g;                     // this lane's 8 keys are first .. first+7
    auto clear_missing = [&](bf16x8 x) {
        uint4 v = __builtin_bit_cast(uint4, x);
        if (first + 0 >= key_hi) v.x &= 0xffff0000u;
        if (first + 1 >= key_hi) v.x &= 0x0000ffffu;
        if (first + 2 >= key_hi) v.y &= 0xffff0000u;
        if (first + 3 >= key_hi) v.y &= 0x0000ffffu;
        if (first + 4 >= key_hi) v.z &= 0xffff0000u;
        if (first + 5 >= key_hi) v.z &= 0x0000ffffu;
        if (first + 6 >= key_hi) v.w &= 0xffff0000u;
        if (first + 7 >= key_hi) v.w &= 0x0000ffffu;
        return __builtin_bit_cast(bf16x8, v);
    };
    if (need_mask) {
#pragma unroll
        for (int t = 0; t < DT; ++t) va[t] = clear_missing(va[t]);
    }
    bf16x8 pb[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        // raw scores; the scale (with log2 e folded in) is applied inside the exponent's fma
        float s[8];
#pragma unroll
        for (int sb = 0; sb < 2; ++sb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float v = st[nt][sb][r];
                if (need_mask) {
                    const int key = kb + 8 * g + 4 * sb + r;
                    if (key > qpos[nt] || key < lo[nt] || key >= key_hi) v = -INFINITY;
                }
                s[sb * 4 + r] = v;
            }
        float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
        mx = max_over_lane_groups(mx);
        mx *= scale2;                                  // scale2 > 0: the maximum of the scaled scores
        // The reference point of the exponents moves only when the maximum has grown by more than
        // 2^8: until then p = 2^(s - m) may exceed 1 (at most 256), which float32 sums and bf16
        // weights hold as well, and the accumulators need no rescaling.  The result is the same.
        float m_new = m[nt];
        if (mx > m[nt] + 8.0f || m[nt] == -INFINITY) m_new = mx;
        if (m_new == -INFINITY) {
#pragma unroll
            for (int e = 0; e < 8; ++e) s[e] = 0.f;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) s[e] = __builtin_amdgcn_exp2f(fmaf(s[e], scale2, -m_new));
        }
        const bool moved = m_new != m[nt];
        if (__any(moved)) {
            const float alpha = (moved && m[nt] != -INFINITY) ? __builtin_amdgcn_exp2f(m[nt] - m_new) : (moved ? 0.f : 1.f);
            l[nt] *= alpha;
#pragma unroll
            for (int t = 0; t < DT; ++t) acc[nt][t] *= alpha;
        }
        m[nt] = m_new;
        pb[nt] = pack8(s);
    }
    // The sums of the weights come from the matrix cores too: a tile of ones times P gives every lane
    // the sum over the 32 keys for its column (the same bf16 weights that multiply V, so numerator
    // and denominator agree), instead of eight additions and two exchanges between lane groups.
    f32x4 lsum[NT];
    {
        const bf16x8 ones = __builtin_bit_cast(bf16x8, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            lsum[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[nt], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            acc[nt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[t], pb[nt], acc[nt][t], 0, 0, 0);
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) l[nt] += lsum[nt][0];
}

// The prompt form runs a block in two halves, so that a wave can have the first product of the next block on the
// matrix cores while its vector units work on the weights of the current one:
//   block_scores:   S^T = K . Q^T of a staged block of 32 keys (two 16-key tiles per column tile), nothing else;
//   block_weights_values: mask, reference point, exponentials, the sums of the weights and O^T += V^T . P^T.
// Operands come from the staged copies in shared memory (swizzled as k_swizzle / v_swizzle say).
// stage: the staged buffer (the same address in every lane); koff[c]: this lane's byte offset of chunk c of its key row
// of tile 0 (k_read_offsets), the row of tile 1 lies 4 rows further.
template <int HS, int NT, int KSTRIDE>
__device__ __forceinline__ void block_scores(const unsigned char* __restrict__ stage, const int (&koff)[HS / 32],
                                             const bf16x8 (&q)[NT][HS / 32], f32x4 (&st)[NT][2]) {
    constexpr int DC = HS / 32;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) { st[nt][0] = (f32x4){0.f, 0.f, 0.f, 0.f}; st[nt][1] = (f32x4){0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
    for (int c = 0; c < DC; ++c) {
        const bf16x8 k0 = ld16(reinterpret_cast<const bf16*>(stage + koff[c]));
        const bf16x8 k1 = ld16(reinterpret_cast<const bf16*>(stage + koff[c] + 4 * KSTRIDE * 2));
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            st[nt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0, q[nt][c], st[nt][0], 0, 0, 0);
            st[nt][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1, q[nt][c], st[nt][1], 0, 0, 0);
        }
    }
}

// stage as above; voff: this lane's byte offset of its 8 keys of V^T row i (v_read_offset), row t * 16 + i lies t * 16 rows further.
template <int HS, int NT, int VSTRIDE, bool need_mask>
__device__ __forceinline__ void block_weights_values_m(const f32x4 (&st)[NT][2], const unsigned char* __restrict__ stage, int voff,
                                                       int kb, f32x4 (&acc)[NT][HS / 16], float (&m)[NT], float (&l)[NT],
                                                       const int (&qpos)[NT], const int (&lo)[NT], int key_hi, float scale2,
                                                       int lane) {
    constexpr int DT = HS / 16;
    const int g = lane >> 4;
    const int first = kb + 8 * g;                     // this lane's 8 keys are first .. first+7
    // keys that do not exist may hold anything, NaN included: they are cleared in V^T (0 * NaN is NaN)
    auto clear_missing = [&](bf16x8 x) {
        uint4 v = __builtin_bit_cast(uint4, x);
        if (first + 0 >= key_hi) v.x &= 0xffff0000u;
        if (first + 1 >= key_hi) v.x &= 0x0000ffffu;
        if (first + 2 >= key_hi) v.y &= 0xffff0000u;
        if (first + 3 >= key_hi) v.y &= 0x0000ffffu;
        if (first + 4 >= key_hi) v.z &= 0xffff0000u;
        if (first + 5 >= key_hi) v.z &= 0x0000ffffu;
        if (first + 6 >= key_hi) v.w &= 0xffff0000u;
        if (first + 7 >= key_hi) v.w &= 0x0000ffffu;
        return __builtin_bit_cast(bf16x8, v);
    };
    // the first tiles of V^T are asked for now, so that they arrive while the weights are computed; every later
    // tile is asked for when an earlier one has been used
    constexpr int PF = DT < 4 ? DT : 4;
    bf16x8 vpre[PF];
    auto staged_v = [&](int t) { return ld16(reinterpret_cast<const bf16*>(stage + voff + t * 16 * VSTRIDE * 2)); };
#pragma unroll
    for (int t = 0; t < PF; ++t) vpre[t] = staged_v(t);
    bf16x8 pb[NT];
    float s[NT][8];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        // raw scores; the scale (with log2 e folded in) is applied inside the exponent's fma
#pragma unroll
        for (int sb = 0; sb < 2; ++sb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float v = st[nt][sb][r];
                if (need_mask) {
                    const int key = kb + 8 * g + 4 * sb + r;
                    if (key > qpos[nt] || key < lo[nt] || key >= key_hi) v = -INFINITY;
                }
                s[nt][sb * 4 + r] = v;
            }
        // The reference point m of the exponents moves only when some score of the column exceeds it
        // by more than 2^8: until then p = 2^(s - m) may exceed 1 (at most 256), which float32 sums
        // and bf16 weights hold as well, and nothing has to be rescaled.  So the common block only
        // asks whether any lane of the wave sees such a score; the exchange between the four lane
        // groups of a column, the new reference point and the rescaling happen when one does.
        float mx = max3(s[nt][0], s[nt][1], s[nt][2]);
        mx = max3(mx, s[nt][3], s[nt][4]);
        mx = max3(mx, s[nt][5], s[nt][6]);
        mx = max3(mx, s[nt][7], s[nt][7]);
        float m_new = m[nt];
        mx *= scale2;                                  // scale2 > 0: the maximum of the scaled scores
        if (__any(mx > m[nt] + 8.0f)) {                // also true for a column's first visible key (m = -inf)
            mx = max_over_lane_groups(mx);
            if (mx > m[nt] + 8.0f) m_new = mx;
            const bool moved = m_new != m[nt];
            if (__any(moved)) {
                const float alpha = (moved && m[nt] != -INFINITY) ? __builtin_amdgcn_exp2f(m[nt] - m_new) : (moved ? 0.f : 1.f);
                l[nt] *= alpha;
#pragma unroll
                for (int t = 0; t < DT; ++t) acc[nt][t] *= alpha;
            }
        }
        m[nt] = m_new;
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        // a column that has seen no key yet (only behind a mask) has m = -inf and only scores of -inf: 2^(-inf - 0) = 0
        const float ref = (need_mask && m[nt] == -INFINITY) ? 0.f : m[nt];
#pragma unroll
        for (int e = 0; e < 8; ++e) s[nt][e] = __builtin_amdgcn_exp2f(fmaf(s[nt][e], scale2, -ref));
        pb[nt] = pack8(s[nt]);
    }
    // The sums of the weights come from the matrix cores too: a tile of ones times P gives every lane
    // the sum over the 32 keys for its column (the same bf16 weights that multiply V, so numerator
    // and denominator agree), instead of eight additions and two exchanges between lane groups.
    f32x4 lsum[NT];
    {
        const bf16x8 ones = __builtin_bit_cast(bf16x8, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            lsum[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[nt], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        bf16x8 va = vpre[t % PF];
        if (t + PF < DT) vpre[t % PF] = staged_v(t + PF);
        if (need_mask) va = clear_missing(va);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            acc[nt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb[nt], acc[nt][t], 0, 0, 0);
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) l[nt] += lsum[nt][0];
}

// The masked form (a block on the causal diagonal, at a window's edge or at the end of the keys) and
// the plain one are separate instantiations: almost every block is plain, and it carries no mask code.
template <int HS, int NT>
__device__ __forceinline__ void attend_block(const bf16* __restrict__ kbase, const bf16* __restrict__ vbase,
                                             int kb, const bf16x8 (&q)[NT][HS / 32], f32x4 (&acc)[NT][HS / 16],
                                             float (&m)[NT], float (&l)[NT], const int (&qpos)[NT],
                                             const int (&lo)[NT], int key_hi, bool need_mask, float scale2,
                                             int lane) {
    bf16x8 ka[HS / 32][2];
    bf16x8 va[HS / 16];
    load_block<HS>(kbase, vbase, ka, va, lane);
    if (need_mask)
        attend_loaded_m<HS, NT, true>(ka, va, kb, q, acc, m, l, qpos, lo, key_hi, scale2, lane);
    else
        attend_loaded_m<HS, NT, false>(ka, va, kb, q, acc, m, l, qpos, lo, key_hi, scale2, lane);
}
template <int HS, int NT, int VSTRIDE>
__device__ __forceinline__ void block_weights_values(const f32x4 (&st)[NT][2], const unsigned char* __restrict__ stage, int voff, int kb,
                                                     f32x4 (&acc)[NT][HS / 16], float (&m)[NT], float (&l)[NT],
                                                     const int (&qpos)[NT], const int (&lo)[NT], int key_hi, bool need_mask,
                                                     float scale2, int lane) {
    if (need_mask) block_weights_values_m<HS, NT, VSTRIDE, true>(st, stage, voff, kb, acc, m, l, qpos, lo, key_hi, scale2, lane);
    else block_weights_values_m<HS, NT, VSTRIDE, false>(st, stage, voff, kb, acc, m, l, qpos, lo, key_hi, scale2, lane);
}

// ---------------------------------------------------------------------------------------
// prompt form
// ---------------------------------------------------------------------------------------
// The waves of a workgroup need the same keys, so a stage of keys is fetched once per workgroup
// into shared memory, three buffers in turn, one barrier per stage: while stage s is multiplied, stage s + 1
// lies ready, stage s + 2 is stored from registers and the loads of stage s + 3 are in flight.  A wave works on
// two stages at once: it issues the first product of stage s + 1 (S^T = K . Q^T), then turns the scores of
// stage s into weights on the vector units while the last of those matrix instructions finish, and then
// multiplies the weights with the values of stage s.  (The compiler keeps the two in separate basic blocks, so
// inside one wave little more than that tail overlaps; most of the overlap of matrix cores and vector units
// comes from the two waves that share a SIMD.  Measured against one stage at a time: 65 -> 61 us at 2,048
// tokens of the 8B shape, 10.9 -> 9.9 ms at 32,768.)  A workgroup has NG groups of 4 waves; all groups hold the
// same query rows and a stage is NG blocks of 32 keys, one for each group, so the chain of blocks
// that a tile of late positions has to walk is NG times shorter; at the end the groups' partial
// results (reference point, sum, accumulators) are merged through shared memory in group order.  NG is 2 for
// launches of one round over the chip and 1 (with two workgroups a CU) for longer ones; the launch code says why.
//
// A causal tile's work grows with its position, and a launch is as long as its longest workgroup.  A workgroup
// therefore takes two tiles, 2p and 2p + 1 of the list, and the host orders the list so that these are a long and
// a short tile of the same sequence (the first with the last, the second with the last but one, ...): every
// workgroup walks about the same number of key blocks (a prompt of 2,048 tokens: 65 blocks each, half of them
// per wave group, where the last tile alone walks 64), and the workgroups that run at the same time walk the
// keys of one sequence, which its L2 then holds.  Any order gives the same result.  A launch whose tiles all
// fit on the chip at once (paired = 0) gives every workgroup one tile: it is as long as its longest tile either
// way, and a second tile would only add its fixed cost.  The grid is
// one-dimensional with the kv heads running fastest: consecutive workgroups go to consecutive XCDs, so with
// eight kv heads every XCD serves one of them and its keys and values live in one L2 only.
template <int HS, int NT, int NG>
__global__ __launch_bounds__(256 * NG) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_mfma_prompt_kernel(MfmaArgs a, int n_tiles, int paired) {
    constexpr int DC = HS / 32, DT = HS / 16;
    constexpr int KB = 32 * NG;                           // keys per stage
    constexpr int KS = HS, VS = KB;                       // row strides (elements); both blocks swizzled, no padding
    constexpr int KV4 = 32 * HS / 8 / 256;                // uint4 loads per thread for K (and for V^T)
    constexpr int STAGE = (KB * KS + HS * VS) * 2;        // bytes of one buffer
    constexpr int MERGE = NG > 1 ? 4 * 64 * (DT * 4 + 2) * 4 : 0;
    static_assert(PROMPT_BUFFERS * STAGE >= MERGE, "the merge of the wave groups reuses the staging memory");
    extern __shared__ __align__(16) unsigned char smem[];     // prompt_smem_bytes(HS, NG)
    const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) & 3, grp = threadIdx.x >> 8;
    const int n = lane & 15, g = lane >> 4;
    // Where this thread's pieces of a stage come from (bytes from the page's keys of this kv head, and from its
    // V^T rows) and where they go in a staged buffer, and where this lane's operands lie in it: a handful of
    // numbers that depend on the thread alone.  They are made opaque to the compiler, which otherwise works them
    // out again in every stage (some seventy vector instructions of index arithmetic beside thirty-four products).
    static_assert(KV4 == 1 || KV4 == 2, "a thread stages one or two pieces of K and of V^T");
    int k_src[2], v_src[2], k_dst[2], v_dst[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        // A stage is one or two whole blocks of the blocked pages (common.h), and the threads fetch it in the pages' own
        // order, 16 consecutive bytes a thread: piece idx of the keys is lane i + 16 g of tile (c, tile) of block b, which
        // holds dimensions 32 c + 8 g .. + 7 of the block's key 8 (i / 4) + i % 4 + 4 tile; piece idx of the values is lane
        // i + 16 g of tile t of block b: keys 8 g .. 8 g + 7 of dimension 16 t + i.  The staged copies keep their own
        // (swizzled) order, and sixteen neighbouring lanes store the sixteen rows that sixteen lanes later read together.
        const int idx = threadIdx.x + h * 256 * NG;
        const int b = idx / (4 * HS), rem = idx % (4 * HS);
        const int li = rem & 15, lg = (rem >> 4) & 3, tl = rem >> 6;
        k_src[h] = idx * 16;
        const int krow = 32 * b + 8 * (li >> 2) + (li & 3) + 4 * (tl & 1), kchunk = 4 * (tl >> 1) + lg;
        k_dst[h] = (krow * KS + ((kchunk ^ k_swizzle<HS>(krow)) * 8)) * 2;
        const int vrow = 16 * tl + li, vchunk = 4 * b + lg;
        v_src[h] = idx * 16;
        v_dst[h] = (KB * KS + vrow * VS + ((vchunk ^ v_swizzle<KB>(vrow & 15)) * 8)) * 2;
        asm volatile("" : "+v"(k_src[h]), "+v"(v_src[h]), "+v"(k_dst[h]), "+v"(v_dst[h]));
    }
    int k_read[DC], v_read;
    {
        const int krow0 = 32 * grp + 8 * (n >> 2) + (n & 3);          // this group's block, key row of tile 0
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            k_read[c] = (krow0 * KS + (((c * 4 + g) ^ k_swizzle<HS>(krow0)) * 8)) * 2;
            asm volatile("" : "+v"(k_read[c]));
        }
        v_read = (KB * KS + n * VS + (((4 * grp + g) ^ v_swizzle<VS>(n)) * 8)) * 2;
        asm volatile("" : "+v"(v_read));
    }
    const int G = a.H / a.Hkv, GT = a.GT;
    const int n_head_tiles = (G + GT - 1) / GT;
    const int hy = a.Hkv * n_head_tiles;
    const int pair = blockIdx.x / hy, y = blockIdx.x - pair * hy;
    const int kvh = y / n_head_tiles, ht = y - kvh * n_head_tiles;
  for (int turn = 0; turn <= paired; ++turn) {
    const int tile = paired ? 2 * pair + turn : pair;
    if (tile >= n_tiles) break;                           // an odd number of tiles: the last one has no partner
    const int* tl = a.tiles + 4 * tile;
    const int seq = tl[0], tok0 = tl[1], n_tok = tl[2], pos0 = tl[3];
    if (n_tok <= 0) continue;                             // an empty tile (a list padded to a fixed length): the whole workgroup skips it

    bf16x8 q[NT][DC];
    int qpos[NT], lo[NT], head[NT], tok[NT];
    int w_hi = -1, w_lo = 0x7fffffff, all_hi = 0x7fffffff, all_lo = 0;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int c = (wave * NT + nt) * 16 + n;
        const int ti = c / GT, hg = ht * GT + (c - ti * GT);
        const bool ok = ti < n_tok && hg < G;
        head[nt] = kvh * G + hg;
        tok[nt] = tok0 + ti;
        qpos[nt] = ok ? pos0 + ti : -1;
        lo[nt] = (ok && a.window > 0) ? max(0, qpos[nt] + 1 - a.window) : 0;
#pragma unroll
        for (int c2 = 0; c2 < DC; ++c2) {
            uint4 z = make_uint4(0, 0, 0, 0);
            if (ok) z = *reinterpret_cast<const uint4*>(a.q + (size_t)tok[nt] * a.q_stride + (size_t)head[nt] * HS + c2 * 32 + g * 8);
            q[nt][c2] = __builtin_bit_cast(bf16x8, z);
        }
        if (ok) { w_hi = max(w_hi, qpos[nt]); w_lo = min(w_lo, lo[nt]); all_hi = min(all_hi, qpos[nt]); all_lo = max(all_lo, lo[nt]); }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        w_hi = max(w_hi, __shfl_xor(w_hi, o, BN_WAVE));
        w_lo = min(w_lo, __shfl_xor(w_lo, o, BN_WAVE));
        all_hi = min(all_hi, __shfl_xor(all_hi, o, BN_WAVE));
        all_lo = max(all_lo, __shfl_xor(all_lo, o, BN_WAVE));
    }
    f32x4 acc[NT][DT];
    float m[NT], l[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        m[nt] = -INFINITY; l[nt] = 0.f;
#pragma unroll
        for (int t = 0; t < DT; ++t) acc[nt][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    const float scale2 = a.scale * LOG2E;
    // the workgroup's key range: every wave takes part in the staging of all of it
    const int g_hi = pos0 + n_tok - 1;
    const int g_lo = a.window > 0 ? max(0, pos0 + 1 - a.window) : 0;
    const size_t bt_row = (size_t)seq * a.bt_stride;
    // Two stages are in flight: one or two 16-byte pieces of K and of V^T per thread and stage, in named
    // registers (arrays indexed in a loop end up in memory when they have to live across the products).
    struct Stage { uint4 k0, k1, v0, v1; };
    auto fetch = [&](int kb, Stage& st) {                 // a stage never crosses a page: KB divides BN_PAGE
        const int page = uniform_load(a.block_table, bt_row + kb / BN_PAGE);
        const int koff = kb % BN_PAGE;
        // the same addresses in every lane: the first of the stage's blocks of 32 keys in the page's keys of this kv
        // head, and in its values
        const unsigned char* kg = reinterpret_cast<const unsigned char*>(a.k_pages + (((size_t)page * a.Hkv + kvh) * BN_PAGE + koff) * HS);
        const unsigned char* vg = reinterpret_cast<const unsigned char*>(a.vt_pages + (((size_t)page * a.Hkv + kvh) * BN_PAGE + koff) * HS);
        st.k0 = *reinterpret_cast<const uint4*>(kg + (unsigned)k_src[0]);
        st.v0 = *reinterpret_cast<const uint4*>(vg + (unsigned)v_src[0]);
        if (KV4 > 1) {
            st.k1 = *reinterpret_cast<const uint4*>(kg + (unsigned)k_src[1]);
            st.v1 = *reinterpret_cast<const uint4*>(vg + (unsigned)v_src[1]);
        }
    };
    auto stash = [&](int buf, const Stage& st, int zero = 0) {    // zero: 0, in a form the compiler cannot see through
        unsigned char* stage = smem + buf * STAGE + zero;
        *reinterpret_cast<uint4*>(stage + k_dst[0]) = st.k0;
        *reinterpret_cast<uint4*>(stage + v_dst[0]) = st.v0;
        if (KV4 > 1) {
            *reinterpret_cast<uint4*>(stage + k_dst[1]) = st.k1;
            *reinterpret_cast<uint4*>(stage + v_dst[1]) = st.v1;
        }
    };
    // Stage t holds the keys kb0 + t KB ..; its block for this wave group begins at kbb(t).  A wave skips the blocks
    // that none of its columns can see.
    const int kb0 = (g_lo / KB) * KB;
    const int n_stages = (g_hi - kb0) / KB + 1;
    auto kbb = [&](int t) { return kb0 + t * KB + 32 * grp; };
    auto active = [&](int t) { return t < n_stages && w_hi >= 0 && kbb(t) <= w_hi && kbb(t) + 31 >= w_lo; };
    auto scores = [&](int t, f32x4 (&st)[NT][2]) {
        if (active(t)) block_scores<HS, NT, KS>(smem + (t % PROMPT_BUFFERS) * STAGE, k_read, q, st);
    };
    // One stage of the walk.  `cur` holds the scores of stage t (computed a stage ago), `next` takes those of stage
    // t + 1; `have` holds the loads of stage t + 2, `want` takes those of stage t + 3.
    auto step = [&](int t, f32x4 (&cur)[NT][2], f32x4 (&next)[NT][2], Stage& want, const Stage& have) {
        if (t + 3 < n_stages) fetch(kb0 + (t + 3) * KB, want);
        // The scores of the next block go to the matrix cores before the vector units start on the weights of this
        // one.  (Put into one basic block with the exponentials, so that the compiler can interleave them, they cost
        // more registers than a wave has here: 188 spilled.)
        scores(t + 1, next);
        if (active(t)) {
            const bool need_mask = (kbb(t) + 31 > all_hi) || (kbb(t) < all_lo);
            block_weights_values<HS, NT, VS>(cur, smem + (t % PROMPT_BUFFERS) * STAGE, v_read, kbb(t), acc, m, l, qpos, lo, w_hi + 1,
                                             need_mask, scale2, lane);
        }
        // The stores of a later stage must stay behind the products: next to their loads (where the
        // compiler puts them otherwise) they would wait out the memory latency before the block is
        // multiplied, instead of hiding it behind the block.  An empty asm makes the store offset look
        // as if it came out of the last product.
        int after_products = 0;
        asm volatile("" : "+v"(after_products) : "v"(acc[NT - 1][DT - 1][3]));
        if (t + 2 < n_stages) stash((t + 2) % PROMPT_BUFFERS, have, after_products);
        __syncthreads();
    };
    Stage sa = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)}, sb = sa;
    fetch(kb0, sa);
    if (n_stages > 1) fetch(kb0 + KB, sb);
    stash(0, sa);
    if (n_stages > 1) stash(1, sb);
    if (n_stages > 2) fetch(kb0 + 2 * KB, sa);
    __syncthreads();
    f32x4 s_even[NT][2], s_odd[NT][2];
    scores(0, s_even);
    for (int t = 0; t < n_stages; t += 2) {
        step(t, s_even, s_odd, sb, sa);
        if (t + 1 >= n_stages) break;
        step(t + 1, s_odd, s_even, sa, sb);
    }
    if (NG > 1) {
        // the later groups hand their partial results to group 0, one column tile a time; the staging
        // memory is free now (the loop ended with a barrier)
        float* x_s = reinterpret_cast<float*>(smem);      // [wave][slot][lane]
        constexpr int SLOTS = DT * 4 + 2;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            for (int src = 1; src < NG; ++src) {
                float* mine = x_s + ((size_t)wave * SLOTS) * 64 + lane;
                if (grp == src) {
                    mine[0] = m[nt];
                    mine[64] = l[nt];
#pragma unroll
                    for (int t = 0; t < DT; ++t)
#pragma unroll
                        for (int r = 0; r < 4; ++r) mine[(2 + t * 4 + r) * 64] = acc[nt][t][r];
                }
                __syncthreads();
                if (grp == 0) {
                    const float m1 = mine[0], l1 = mine[64];
                    const float M = fmaxf(m[nt], m1);
                    if (M != -INFINITY) {
                        const float a0 = m[nt] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[nt] - M);
                        const float a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - M);
                        l[nt] = l[nt] * a0 + l1 * a1;
#pragma unroll
                        for (int t = 0; t < DT; ++t)
#pragma unroll
                            for (int r = 0; r < 4; ++r) acc[nt][t][r] = acc[nt][t][r] * a0 + mine[(2 + t * 4 + r) * 64] * a1;
                        m[nt] = M;
                    }
                }
                __syncthreads();
            }
        }
    }
    if (grp == 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            if (qpos[nt] < 0) continue;
            const float inv = l[nt] > 0.f ? 1.0f / l[nt] : 0.f;
            bf16* o = a.out + (size_t)tok[nt] * a.out_stride + (size_t)head[nt] * HS + 4 * g;
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                uint2 w;
                w.x = pack2(acc[nt][t][0] * inv, acc[nt][t][1] * inv);
                w.y = pack2(acc[nt][t][2] * inv, acc[nt][t][3] * inv);
                *reinterpret_cast<uint2*>(o + t * 16) = w;
            }
        }
    }
    __syncthreads();                                      // the staging memory is free for the next tile
  }
}

// ---------------------------------------------------------------------------------------
// decode form
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ void rotate8(uint4& lo, uint4& hi, const float* __restrict__ cs, const float* __restrict__ sn) {
    // lo/hi: 8 bf16 each, element e of lo pairs with element e of hi; cs/sn: their 8 cos/sin
    uint32_t* pl = reinterpret_cast<uint32_t*>(&lo);
    uint32_t* ph = reinterpret_cast<uint32_t*>(&hi);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float a0 = bf16lo_to_f32(pl[k]), a1 = bf16hi_to_f32(pl[k]);
        const float b0 = bf16lo_to_f32(ph[k]), b1 = bf16hi_to_f32(ph[k]);
        const float c0 = cs[2 * k], c1 = cs[2 * k + 1], s0 = sn[2 * k], s1 = sn[2 * k + 1];
        pl[k] = pack2(a0 * c0 - b0 * s0, a1 * c1 - b1 * s1);
        ph[k] = pack2(a0 * s0 + b0 * c0, a1 * s1 + b1 * c1);
    }
}

template <int HS>
__global__ __launch_bounds__(256) void attn_mfma_decode_kernel(MfmaArgs a) {
    constexpr int DC = HS / 32, DT = HS / 16, HALF = HS / 2;
    __shared__ float m_s[4][16], l_s[4][16];
    __shared__ float o_s[4][HS][17];                    // [wave][dim][col], padded
    __shared__ float cos_s[HALF], sin_s[HALF];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int G = a.H / a.Hkv, GT = a.GT;
    const int n_head_tiles = (G + GT - 1) / GT;
    // kv heads run fastest in the grid: consecutive workgroups go to different XCDs, so every XCD gets
    // a share of every sequence, however unequal their lengths (with the sequences fastest and a
    // batch that is a multiple of 8, a sequence's heads all landed on one XCD)
    const int kvh = blockIdx.x / n_head_tiles, ht = blockIdx.x - kvh * n_head_tiles;
    int seq = blockIdx.y;
    const int split = blockIdx.z;
    if (a.by_length) {
        int r = seq;
        if (a.order_period > 0) {
            const int run = r / a.order_period;
            if (run & 1) {
                const int first = run * a.order_period, last = min(first + a.order_period, (int)gridDim.y) - 1;
                r = first + (last - r);
            }
        }
        seq = uniform_load(a.by_length, r);
        if ((unsigned)seq >= gridDim.y) return;          // not a permutation: touch nothing
    }
    // Everything that does not depend on the sequence's length is asked for now, in straight-line code with no lane left
    // out of a load (a lane without a head, a thread without an element asks for a neighbour's and drops it), so that
    // nothing waits for anything but its own data: the query's heads, the frequencies, the new key and value, the sums of
    // squares of a deferred norm.  The length and the pages come through the scalar unit, beside those loads.
    const int hg = ht * GT + n;
    const bool q_lane = n < GT && hg < G;
    const int head = kvh * G + (q_lane ? hg : 0);
    const bf16* row = a.q + (size_t)seq * a.q_stride;
    uint4 z[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) z[c] = *reinterpret_cast<const uint4*>(row + (size_t)head * HS + c * 32 + g * 8);
    const int tid = threadIdx.x;
    float freq = 0.f, piece = 0.f;
    if (a.rotate) freq = a.inv_freq[tid & (HALF - 1)];
    if (a.row_ssq) piece = a.row_ssq[(size_t)seq * a.n_pieces + min(lane, a.n_pieces - 1)];
    unsigned new_k0 = 0, new_k1 = 0, new_v = 0;          // bf16 bit patterns, widened where they are used
    if (a.write_kv) {        // threads below HALF hold a pair of the key, the HS behind them an element of the value
        const unsigned short* kn = reinterpret_cast<const unsigned short*>(row + (size_t)(a.H + kvh) * HS);
        const unsigned short* vn = reinterpret_cast<const unsigned short*>(row + (size_t)(a.H + a.Hkv + kvh) * HS);
        new_k0 = kn[tid & (HALF - 1)];
        new_k1 = kn[(tid & (HALF - 1)) + HALF];
        new_v = vn[(tid - HALF) & (HS - 1)];
    }
    const int L = uniform_load(a.seq_lens, seq);
    const int chunk = a.max_len ? bn_split_chunk(uniform_load(a.max_len, 0), a.n_splits) : a.chunk;
    // So is the first block of keys that this wave will take, whose place does not depend on the length when no window
    // cuts the keys: its page and its 16 KB are on their way while the rotation is worked out and the new token is
    // stored, instead of after all that.  If the sequence turns out to end before the block, it is dropped unused (every
    // entry of a block table names a page of the pool, also those behind a sequence's last page); if the block holds
    // the new token's position, it is asked for again behind the store.
    // (With a window, or a table that ends before the block, the loads go to the table's first page and are dropped:
    // loads under a branch would make everything behind it wait for all of them.)
    const int kb_first = split * chunk + 32 * __builtin_amdgcn_readfirstlane(wave);
    const bool ahead = a.window == 0 && kb_first / BN_PAGE < a.bt_stride;
    bf16x8 ka0[DC][2];
    bf16x8 va0[DT];
    const int page0 = uniform_load(a.block_table, (size_t)seq * a.bt_stride + (ahead ? kb_first / BN_PAGE : 0));
    const size_t at0 = (((size_t)page0 * a.Hkv + kvh) * BN_PAGE + kb_first % BN_PAGE) * HS;
    const bf16* kbase0 = a.k_pages + at0;
    const bf16* vbase0 = a.vt_pages + at0;
    load_block<HS>(kbase0, vbase0, ka0, va0, lane);
    const bool ok = q_lane && L > 0;
    const int lo_key = a.window > 0 ? max(0, L - a.window) : 0;
    const int k_lo = max(lo_key, split * chunk), k_hi = min(L, (split + 1) * chunk);       // [k_lo, k_hi)
    if (a.n_splits > 1 && k_lo >= k_hi) {
        // A split without keys (a sequence shorter than the launch's longest, a padding row): it leaves "nothing seen"
        // for the merge, which then does not read its sums, and is gone before it asks for anything else.
        if (threadIdx.x < GT && ht * GT + threadIdx.x < G) {
            const size_t prow = ((size_t)seq * a.H + kvh * G + ht * GT + threadIdx.x) * a.n_splits + split;
            a.part_ml[prow * 2] = -INFINITY;
            a.part_ml[prow * 2 + 1] = 0.f;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // what was asked for has arrived before the wave ends
        return;
    }
    float row_scale = 1.0f;
    if (a.row_ssq) {                                     // the same few floats in every lane, added in piece order
        float ss = 0.f;
        for (int p = 0; p < a.n_pieces; ++p)
            ss += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, piece), p));
        row_scale = 1.0f / sqrtf(ss * a.inv_ssq_width + a.ssq_eps);
    }

    if (a.rotate && L > 0) {
        if (tid < HALF) {                                // HALF <= 64: one frequency a thread
            float sv, cv;
            sincosf((float)(L - 1) * freq, &sv, &cv);
            cos_s[tid] = cv * row_scale; sin_s[tid] = sv * row_scale;
        }
        lds_barrier();                                   // the block that is on its way stays on its way
    }
    // the new token's key and value go into the cache before anyone reads them: the workgroup
    // that owns the new position does it (there is one per kv head: write_kv needs n_head_tiles == 1)
    if (a.write_kv && L > 0 && L - 1 >= k_lo && L - 1 < k_hi) {
        const int pos = L - 1;
        // through the scalar unit (the length is the same in every lane), so that it does not queue behind the block
        // that is on its way
        const int page = uniform_load(a.block_table, (size_t)seq * a.bt_stride + __builtin_amdgcn_readfirstlane(pos / BN_PAGE));
        const int off = pos % BN_PAGE;
        bf16* kdst = const_cast<bf16*>(a.k_pages) + ((size_t)page * a.Hkv + kvh) * BN_PAGE * HS;
        bf16* vdst = const_cast<bf16*>(a.vt_pages) + ((size_t)page * a.Hkv + kvh) * BN_PAGE * HS;
        const int t = threadIdx.x;
        if (t < HALF) {
            float k0 = widen_here(new_k0), k1 = widen_here(new_k1);
            if (a.rotate) {
                const float c = cos_s[t], sv = sin_s[t];
                const float r0 = k0 * c - k1 * sv, r1 = k0 * sv + k1 * c;
                k0 = r0; k1 = r1;
            }
            kdst[bn_blocked_k_offset(off, t, HS)] = __float2bfloat16(k0);
            kdst[bn_blocked_k_offset(off, t + HALF, HS)] = __float2bfloat16(k1);
        } else if (t < HALF + HS) {
            const int d = t - HALF;
            reinterpret_cast<unsigned short*>(vdst)[bn_blocked_v_offset(off, d, HS)] =
                a.row_ssq ? __builtin_bit_cast(unsigned short, __float2bfloat16(widen_here(new_v) * row_scale))
                          : (unsigned short)new_v;
        }
        // only this workgroup reads what it has just stored: a fence of workgroup scope is enough
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
        __syncthreads();
    }

    bf16x8 q[1][DC];
    {
        if (!q_lane) {
#pragma unroll
            for (int c = 0; c < DC; ++c) z[c] = make_uint4(0, 0, 0, 0);
        }
        if (a.rotate && L > 0) {
#pragma unroll
            for (int c = 0; c < DC / 2; ++c)      // chunk c holds pair indices c*32 + g*8 .. +7, its partners are in chunk c + DC/2
                rotate8(z[c], z[c + DC / 2], cos_s + c * 32 + g * 8, sin_s + c * 32 + g * 8);
        }
#pragma unroll
        for (int c = 0; c < DC; ++c) q[0][c] = __builtin_bit_cast(bf16x8, z[c]);
    }
    int qpos[1] = {ok ? L - 1 : -1};
    int lo[1] = {lo_key};

    f32x4 acc[1][DT];
    float m[1] = {-INFINITY}, l[1] = {0.f};
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[0][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const float scale2 = a.scale * LOG2E;
    if (k_lo < k_hi) {
        const size_t bt_row = (size_t)seq * a.bt_stride;
        // (Keeping the next block's operands in a second set of registers while the current block is multiplied was
        // measured and gained nothing: the CU's other waves already cover a wave's wait for its loads.)
        // The waves take the blocks of 32 keys in turn, so that neighbouring waves ask for the two halves of a page at
        // the same time (a wave that takes whole pages by itself was measured 10 to 20 % slower, and so was splitting
        // the sequences of a large batch: the order by length with unsplit sequences keeps the CUs busiest).
        int kb = (k_lo / 32) * 32 + 32 * wave;
        if (ahead && kb == kb_first && kb < k_hi) {        // the block that was asked for at the start
            if (a.write_kv && L - 1 >= kb && L - 1 < kb + 32) load_block<HS>(kbase0, vbase0, ka0, va0, lane);
            if ((kb + 32 > k_hi) || (kb < k_lo))
                attend_loaded_m<HS, 1, true>(ka0, va0, kb, q, acc, m, l, qpos, lo, k_hi, scale2, lane);
            else
                attend_loaded_m<HS, 1, false>(ka0, va0, kb, q, acc, m, l, qpos, lo, k_hi, scale2, lane);
            kb += 128;
        }
        for (; kb < k_hi; kb += 128) {
            // the page index is the same for the whole wave: read through the scalar unit, so that it
            // does not queue behind the vector loads
            const int page = uniform_load(a.block_table, bt_row + __builtin_amdgcn_readfirstlane(kb / BN_PAGE));
            const int koff = kb % BN_PAGE;                 // 0 or 32: the page's first or second block
            const bf16* kbase = a.k_pages + (((size_t)page * a.Hkv + kvh) * BN_PAGE + koff) * HS;
            const bf16* vbase = a.vt_pages + (((size_t)page * a.Hkv + kvh) * BN_PAGE + koff) * HS;
            const bool need_mask = (kb + 32 > k_hi) || (kb < k_lo);
            attend_block<HS, 1>(kbase, vbase, kb, q, acc, m, l, qpos, lo, k_hi, need_mask, scale2, lane);
        }
    }
    // merge the four waves: every wave's (m, l, O^T) through shared memory, in wave order
    if (g == 0) { m_s[wave][n] = m[0]; l_s[wave][n] = l[0]; }
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_s[wave][t * 16 + 4 * g + r][n] = acc[0][t][r];
    __syncthreads();
    for (int idx = threadIdx.x; idx < HS * GT; idx += 256) {
        const int col = idx / HS, dim = idx - col * HS;      // consecutive threads: consecutive dims
        const int hg2 = ht * GT + col;
        if (hg2 >= G) continue;
        float M = fmaxf(fmaxf(m_s[0][col], m_s[1][col]), fmaxf(m_s[2][col], m_s[3][col]));
        float num = 0.f, den = 0.f;
        if (M != -INFINITY) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float e = exp2f(m_s[w][col] - M);
                num = fmaf(e, o_s[w][dim][col], num);
                den = fmaf(e, l_s[w][col], den);
            }
        }
        const int hd = kvh * G + hg2;
        if (a.n_splits == 1) {
            a.out[(size_t)seq * a.out_stride + (size_t)hd * HS + dim] = __float2bfloat16(den > 0.f ? num / den : 0.f);
        } else {
            const size_t prow = ((size_t)seq * a.H + hd) * a.n_splits + split;
            a.part_o[prow * HS + dim] = num;
            if (dim == 0) { a.part_ml[prow * 2] = (M == -INFINITY) ? -INFINITY : M * LN2; a.part_ml[prow * 2 + 1] = den; }
        }
    }
}

// out[row, d] = sum_s e^{m_s - m} o_s[d] / sum_s e^{m_s - m} l_s: one wave per row, the weights
// of all splits computed at once (one lane per split), the sums in split order.
__global__ __launch_bounds__(64) void attn_mfma_combine_kernel(bf16* __restrict__ out, int out_stride,
                                                               const float* __restrict__ part_o,
                                                               const float* __restrict__ part_ml, int H, int hs,
                                                               int n_splits) {
    const int row = blockIdx.x, lane = threadIdx.x;
    const int tok = row / H, head = row - tok * H;
    const float* ml = part_ml + (size_t)row * n_splits * 2;
    float ms = -INFINITY, ls = 0.f;
    if (lane < n_splits) { ms = ml[2 * lane]; ls = ml[2 * lane + 1]; }
    const float M = wave_max(ms);
    const float w = (M == -INFINITY || ms == -INFINITY) ? 0.f : expf(ms - M);
    // splits behind the last one with keys (a table much wider than the sequences are long) add nothing: stop there
    const unsigned long long live = __ballot(w != 0.f);
    const int n_live = live ? 64 - __builtin_clzll(live) : 0;
    float den = 0.f;
    for (int s = 0; s < n_live; ++s) den = fmaf(__shfl(w, s, BN_WAVE), __shfl(ls, s, BN_WAVE), den);
    const float inv = den > 0.f ? 1.0f / den : 0.f;
    // dimensions lane and lane + 64 together, sixteen splits' loads in flight at once (a split without keys is not read)
    const bool two = lane + 64 < hs;
    float num0 = 0.f, num1 = 0.f;
    const float* po = part_o + (size_t)row * n_splits * hs + lane;
    for (int s0 = 0; s0 < n_live; s0 += 16) {
        float v0[16], v1[16], wj[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            wj[j] = __shfl(w, min(s0 + j, 63), BN_WAVE);
            const bool in = s0 + j < n_live && wj[j] != 0.f;
            v0[j] = (in && lane < hs) ? po[(size_t)(s0 + j) * hs] : 0.f;
            v1[j] = (in && two) ? po[(size_t)(s0 + j) * hs + 64] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) {                                     // then the sums, in split order
            num0 = fmaf(wj[j], v0[j], num0);
            num1 = fmaf(wj[j], v1[j], num1);
        }
    }
    bf16* o = out + (size_t)tok * out_stride + (size_t)head * hs;
    if (lane < hs) o[lane] = __float2bfloat16(num0 * inv);
    if (two) o[lane + 64] = __float2bfloat16(num1 * inv);
}

// 1 when the matrix-core kernels take this shape
extern "C" int bn_attn_mfma_supports(int hs) { return (hs == BN_MFMA_HEAD_DIM_SMALL || hs == BN_MFMA_HEAD_DIM_LARGE) ? 1 : 0; }

// query tokens per tile of the prompt form, for GT heads per group
extern "C" int bn_attn_mfma_prompt_tokens(int hs, int GT) { return (hs == 64 ? 256 : 128) / GT; }

static int attn_mfma_launch(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                            const void* vt_pages, const int* block_table, int bt_stride, const int* seq_lens,
                            const int* tiles, int n_tiles, int n_tokens, int H, int Hkv, int hs, int GT,
                            int window, float scale, int n_splits, int chunk, float* part_o, float* part_ml,
                            const float* inv_freq, int rotate, int write_kv, const int* by_length,
                            const int* max_len, const float* row_ssq, int n_pieces, int ssq_width, float ssq_eps,
                            hipStream_t s) {
    if (!bn_attn_mfma_supports(hs) || n_tiles <= 0 || n_tokens <= 0 || H <= 0 || Hkv <= 0 || H % Hkv) return BN_ERR_ARG;
    if (row_ssq && (tiles || !rotate || n_pieces < 1 || n_pieces > 64 || ssq_width < 1)) return BN_ERR_ARG;   // decode form, rotating
    if (GT <= 0 || GT > 16 || (GT & (GT - 1)) || window < 0 || n_splits < 1 || n_splits > 64) return BN_ERR_ARG;
    if (n_splits > 1 && (!part_o || !part_ml || (!max_len && (chunk <= 0 || chunk % BN_PAGE)))) return BN_ERR_ARG;
    if (!tiles && (!seq_lens || bt_stride < 1)) return BN_ERR_ARG;      // the decode form reads a row's first entry unasked
    if (max_len && tiles) return BN_ERR_ARG;                               // decode form only
    if (q_stride % 8 || out_stride % 4 || (((uintptr_t)q | (uintptr_t)k_pages | (uintptr_t)vt_pages) & 15) ||
        ((uintptr_t)out & 7))
        return BN_ERR_ARG;
    const int G = H / Hkv;
    const int n_head_tiles = (G + GT - 1) / GT;
    if ((rotate || write_kv) && tiles) return BN_ERR_ARG;                 // decode form only
    if (rotate && !inv_freq) return BN_ERR_ARG;
    if (write_kv && (n_head_tiles != 1 || q_stride < (H + 2 * Hkv) * hs)) return BN_ERR_ARG;
    MfmaArgs a;
    a.q = (const bf16*)q; a.out = (bf16*)out; a.k_pages = (const bf16*)k_pages; a.vt_pages = (const bf16*)vt_pages;
    a.block_table = block_table; a.seq_lens = seq_lens; a.tiles = tiles; a.part_o = part_o; a.part_ml = part_ml;
    a.q_stride = q_stride; a.out_stride = out_stride; a.bt_stride = bt_stride;
    a.H = H; a.Hkv = Hkv; a.GT = GT; a.window = window; a.scale = scale;
    a.n_splits = n_splits; a.chunk = n_splits > 1 ? chunk : 0x40000000;
    a.inv_freq = inv_freq; a.rotate = rotate; a.write_kv = write_kv;
    a.row_ssq = row_ssq; a.n_pieces = n_pieces; a.inv_ssq_width = row_ssq ? 1.0f / (float)ssq_width : 0.f; a.ssq_eps = ssq_eps;
    a.max_len = n_splits > 1 ? max_len : nullptr;
    // the order matters only when the launch holds more workgroups than CUs and no sequence is split
    const int wgs_per_seq = Hkv * n_head_tiles;
    a.by_length = (!tiles && n_splits == 1 && (long long)n_tiles * wgs_per_seq > compute_units()) ? by_length : nullptr;
    a.order_period = compute_units() / wgs_per_seq;
    if (tiles) {
        // a workgroup takes a pair of tiles when there are more tiles than CUs
        const int paired = (long long)n_tiles * wgs_per_seq > compute_units() ? 1 : 0;
        const long long wgs = (long long)(paired ? (n_tiles + 1) / 2 : n_tiles) * wgs_per_seq;
        if (wgs > 0x7fffffff) return BN_ERR_ARG;
        const dim3 grid((unsigned)wgs);
        // Two groups of waves a workgroup (eight waves, one workgroup a CU) halve the chain of blocks that a tile walks,
        // which is what a launch of one round waits for.  A launch of several rounds is faster with one group a
        // workgroup and two workgroups a CU: they share nothing and drift apart, so that one's matrix instructions
        // meet the other's vector work, where the two groups of one workgroup meet at a barrier in every stage and do
        // the same thing at the same time (8 to 16 % at 8,192 tokens and for eight or 64 prompts of 128 to 2,048).
        // It is taken from four rounds on, and from two when its rounds (of two workgroups a CU) are not much emptier
        // than those of the wide form (6,144 tokens of one sequence are three full rounds of the wide form and one and
        // a half of the other: 410 against 445 us).
        const long long cus = compute_units();
        const double fill1 = (double)wgs / (double)(((wgs + 2 * cus - 1) / (2 * cus)) * 2 * cus);
        const double fill2 = (double)wgs / (double)(((wgs + cus - 1) / cus) * cus);
        const int ng = (wgs >= 4 * cus || (wgs >= 2 * cus && fill1 * 1.1 >= fill2)) ? 1 : 2;
        // three staged blocks of 32 keys a group with their values: up to 96 KB, beyond the default limit of dynamic
        // shared memory
        const size_t smem = (size_t)PROMPT_BUFFERS * (32 * ng * hs + hs * 32 * ng) * 2;
        auto go = [&](auto kernel, int which) {
            static bool raised[4] = {false, false, false, false};
            if (!raised[which]) {
                const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return (int)e;
                raised[which] = true;
            }
            hipLaunchKernelGGL(kernel, grid, dim3(256 * ng), smem, s, a, n_tiles, paired);
            return bn_launch_status();
        };
        if (ng == 1) return hs == 64 ? go(attn_mfma_prompt_kernel<64, 4, 1>, 2) : go(attn_mfma_prompt_kernel<128, 2, 1>, 3);
        return hs == 64 ? go(attn_mfma_prompt_kernel<64, 4, 2>, 0) : go(attn_mfma_prompt_kernel<128, 2, 2>, 1);
    }
    if (n_tiles > 65535) return BN_ERR_ARG;                 // sequences are the grid's y
    const dim3 grid(Hkv * n_head_tiles, n_tiles, n_splits);
    if (hs == 64) hipLaunchKernelGGL(attn_mfma_decode_kernel<64>, grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL(attn_mfma_decode_kernel<128>, grid, dim3(256), 0, s, a);
    int rc = bn_launch_status();
    if (rc != 0 || n_splits == 1) return rc;
    hipLaunchKernelGGL(attn_mfma_combine_kernel, dim3(n_tokens * H), dim3(64), 0, s, (bf16*)out, out_stride, part_o,
                       part_ml, H, hs, n_splits);
    return bn_launch_status();
}

extern "C" int bn_attn_mfma(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                            const void* vt_pages, const int* block_table, int bt_stride, const int* seq_lens,
                            const int* tiles, int n_tiles, int n_tokens, int H, int Hkv, int hs, int GT,
                            int window, float scale, int n_splits, int chunk, float* part_o, float* part_ml,
                            const float* inv_freq, int rotate, int write_kv, const int* by_length,
                            const int* max_len, hipStream_t s) {
    return attn_mfma_launch(q, q_stride, out, out_stride, k_pages, vt_pages, block_table, bt_stride, seq_lens, tiles, n_tiles,
                            n_tokens, H, Hkv, hs, GT, window, scale, n_splits, chunk, part_o, part_ml, inv_freq, rotate,
                            write_kv, by_length, max_len, nullptr, 0, 0, 0.f, s);
}

// The decode form (tiles none, rotate on) over rows whose RMSNorm was left undone: q, the new key and the new value of
// row b still lack the factor 1/sqrt(sum of row_ssq[b][0..n_pieces) / ssq_width + eps), which is applied here.
extern "C" int bn_attn_mfma_scaled(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                                   const void* vt_pages, const int* block_table, int bt_stride, const int* seq_lens,
                                   int n_seqs, int H, int Hkv, int hs, int GT, int window, float scale, int n_splits,
                                   int chunk, float* part_o, float* part_ml, const float* inv_freq, int write_kv,
                                   const int* by_length, const int* max_len, const float* row_ssq, int n_pieces,
                                   int ssq_width, float ssq_eps, hipStream_t s) {
    if (!row_ssq) return BN_ERR_ARG;
    return attn_mfma_launch(q, q_stride, out, out_stride, k_pages, vt_pages, block_table, bt_stride, seq_lens, nullptr, n_seqs,
                            n_seqs, H, Hkv, hs, GT, window, scale, n_splits, chunk, part_o, part_ml, inv_freq, 1, write_kv,
                            by_length, max_len, row_ssq, n_pieces, ssq_width, ssq_eps, s);
}

// ---------------------------------------------------------------------------------------
// decode form for callers that cannot allocate (declared and described in attn_mfma.h)
// ---------------------------------------------------------------------------------------
// The split partials of bn_attn_mfma_decode_static.  In host code this name is a stand-in, not a device
// address: the address on the current GPU comes from hipGetSymbolAddress, once per device, and only that
// pointer is ever handed to a kernel.
static __device__ __align__(256) float scratch[BN_ATTN_STATIC_SCRATCH_FLOATS];

static int static_scratch(float** ptr) {
    static std::mutex lock;
    static float* per_device[64] = {nullptr};         // each GPU holds its own copy of the array at its own address
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return BN_ERR_ARG;
    std::lock_guard<std::mutex> hold(lock);
    if (per_device[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return (int)hipErrorInvalidSymbol;
        per_device[dev] = static_cast<float*>(p);
    }
    *ptr = per_device[dev];
    return 0;
}

extern "C" int bn_attn_mfma_decode_static(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                                          const void* vt_pages, const int* block_table, int bt_stride,
                                          const int* seq_lens, int n_seqs, int H, int Hkv, int hs, int GT, int window,
                                          float scale, int n_splits, int chunk, const float* inv_freq, int rotate,
                                          int write_kv, const int* by_length, hipStream_t s) {
    if (!seq_lens || n_seqs <= 0 || H <= 0 || n_splits < 1 || n_splits > 64 || !bn_attn_mfma_supports(hs)) return BN_ERR_ARG;
    float* part_o = nullptr;
    float* part_ml = nullptr;
    if (n_splits > 1) {
        const unsigned long long rows = (unsigned long long)n_seqs * (unsigned)H * (unsigned)n_splits;
        if (rows * (unsigned)(hs + 2) > BN_ATTN_STATIC_SCRATCH_FLOATS) return BN_ERR_SCRATCH;
        float* base = nullptr;
        const int rc = static_scratch(&base);
        if (rc != 0) return rc;
        part_o = base;                                // [rows, hs]
        part_ml = base + rows * (unsigned)hs;         // [rows, 2]
    }
    return bn_attn_mfma(q, q_stride, out, out_stride, k_pages, vt_pages, block_table, bt_stride, seq_lens, nullptr,
                        n_seqs, n_seqs, H, Hkv, hs, GT, window, scale, n_splits, chunk, part_o, part_ml, inv_freq, rotate,
                        write_kv, by_length, nullptr, s);
}
