// Prompt attention on the matrix cores for the attention mixer's general form: head sizes that are multiples of 32,
// values of a width of their own (a multiple of 32), a logarithmic distance bias, a sink in the softmax, no rotation
// (the queries and keys arrive encoded).  bf16, 16x16x32 MFMA.  Keys lie in pages with a row per position
// ([page, kv head, BN_PAGE, hs]), values transposed ([page, kv head, vd, BN_PAGE]): both operands of both products are
// then 16 consecutive bytes a lane, straight from the pages (no shared memory, no barrier: a wave is on its own).
//
// A wave owns one tile of up to 16 query tokens of one head and walks the keys 0 .. last query in blocks of 32 (with a
// window w > 0 a query at position i sees the keys i - w + 1 .. i only, and the walk begins at the block of the tile's
// first visible key):
//   S^T = K . Q^T      two tiles of 16 keys x 16 queries; tile h holds the block's keys 8 (i / 4) + 4 h + i % 4 in its
//                      row i, so that lane group g ends up with the scores of keys 8 g .. 8 g + 7 of its query column:
//                      what the second product wants from it as its operand, without any exchange
//   s = S scale - a[h] ln(1 + b[h] (i - j)), masked above the diagonal; online softmax in base 2, float32
//   O^T += V^T . P^T   vd / 16 tiles; the weights' sums from the matrix cores as well (a tile of ones times P^T), so that
//                      numerator and denominator see the same bf16 weights
// and at the end the sink (one more term of score 0 without a value) joins the sums, then O / l is stored.
//
// Decode form (attn_general_decode_kernel): the 16 columns of a tile are the query heads that share a kv head (the one new
// token of a sequence), so a block of keys and values is loaded once for all of them: a wave owns (sequence, kv head,
// sixteen of its heads, split of the keys) and either stores the result or, with the keys split over gridDim.z, leaves
// unnormalised sums with their maximum and weight sum for attn_general_combine_kernel, which merges the splits in index
// order.  Splits are runs of whole pages; with a window they are counted from the page of the window's first key.
// Every other shape or type is the vector kernel's (attn_rows.hip).
#include "common.h"
#include <math.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define AG_LOG2E 1.4426950408889634f
#define AG_WAVES 4            // waves (heads) of a workgroup

struct GenArgs {
    const bf16* q;            // [T, q_stride]: head h at h * hs, norms and temperature applied
    bf16* out;                // [T, out_stride]: head h at h * vd
    const bf16* k_pages;      // [pages, Hkv, BN_PAGE, hs]
    const bf16* v_pages;      // [pages, Hkv, vd, BN_PAGE]
    const int* block_table;   // [seqs, bt_stride]
    const int* tiles;         // [n, 4]: sequence, first row, rows <= 16, position of the first
    const float* dist_a;      // [H] or null
    const float* dist_b;
    int q_stride, out_stride, bt_stride, H, Hkv;
    float scale;
    int sink;                 // 1: one more term without a value in the softmax's denominator, exp(sink_values[head])
    const float* sink_values; // [H] float32, or null: the term's score is 0
    int window;               // 0: every earlier key; else the last `window` positions, the query's own included
};

__device__ __forceinline__ bf16x8 ag_ld16(const bf16* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

template <int DC, int DT>     // hs = 32 DC, vd = 16 DT
__global__ __launch_bounds__(AG_WAVES * BN_WAVE) void attn_general_prompt_kernel(GenArgs a) {
    constexpr int HS = 32 * DC, VD = 16 * DT;
    const int* tl = a.tiles + 4 * blockIdx.x;
    const int seq = tl[0], row0 = tl[1], n = min(tl[2], 16), pos0 = tl[3];
    const int head = blockIdx.y * AG_WAVES + (threadIdx.x >> 6);
    if (n <= 0 || pos0 < 0 || head >= a.H) return;
    const int lane = threadIdx.x & 63, i = lane & 15, g = lane >> 4;
    const int kvh = head / (a.H / a.Hkv);
    const bool col_ok = i < n;                           // this lane's query column exists
    const int qpos = pos0 + i;
    const int k_hi = pos0 + n;                           // keys of this tile: positions below this

    // Q^T: column i, dimensions 32 c + 8 g .. + 7 (a row that does not exist reads the tile's last one and is never stored)
    bf16x8 qf[DC];
    {
        const bf16* qp = a.q + (size_t)(row0 + min(i, n - 1)) * a.q_stride + (size_t)head * HS + 8 * g;
#pragma unroll
        for (int c = 0; c < DC; ++c) qf[c] = ag_ld16(qp + 32 * c);
    }
    const float scale2 = a.scale * AG_LOG2E;
    const float ba = a.dist_a ? a.dist_a[head] : 0.f, bb = a.dist_a ? a.dist_b[head] : 0.f;
    f32x4 acc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const bf16x8 ones = __builtin_bit_cast(bf16x8, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));
    const int krow = 8 * (i >> 2) + (i & 3);             // this lane's key row of tile 0 inside a block; tile 1: 4 further

    // The keys of a block are asked for one block ahead (the last block asks for itself once more: a load without a
    // branch around it), so that the first product finds its operand there; the values are asked for when the block
    // begins and are used behind the weights.
    bf16x8 kn0[DC], kn1[DC];
    auto ask_keys = [&](int kb) {
        const int page = a.block_table[(size_t)seq * a.bt_stride + kb / BN_PAGE];
        const bf16* kbase = a.k_pages + (((size_t)page * a.Hkv + kvh) * BN_PAGE + kb % BN_PAGE + krow) * HS + 8 * g;
#pragma unroll
        for (int c = 0; c < DC; ++c) { kn0[c] = ag_ld16(kbase + 32 * c); kn1[c] = ag_ld16(kbase + 4 * HS + 32 * c); }
    };
    const int k_lo = a.window > 0 ? max(0, pos0 - a.window + 1) & ~31 : 0;      // the block of the first key any row sees
    const int q_lo = a.window > 0 ? qpos - a.window : -1;                        // keys at or below this are out of sight
    ask_keys(k_lo);
    const int last_block = ((k_hi - 1) / 32) * 32;
    for (int kb = k_lo; kb < k_hi; kb += 32) {
        const int page = a.block_table[(size_t)seq * a.bt_stride + kb / BN_PAGE];
        const int off = kb % BN_PAGE;
        const bf16* vbase = a.v_pages + (((size_t)page * a.Hkv + kvh) * VD + i) * BN_PAGE + off + 8 * g;
        bf16x8 k0[DC], k1[DC];
#pragma unroll
        for (int c = 0; c < DC; ++c) { k0[c] = kn0[c]; k1[c] = kn1[c]; }
        ask_keys(min(kb + 32, last_block));
        f32x4 st0 = (f32x4){0.f, 0.f, 0.f, 0.f}, st1 = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            st0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0[c], qf[c], st0, 0, 0, 0);
            st1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1[c], qf[c], st1, 0, 0, 0);
        }
        // the values' tiles are asked for now and used behind the weights
        bf16x8 va[DT];
#pragma unroll
        for (int t = 0; t < DT; ++t) va[t] = ag_ld16(vbase + (size_t)t * 16 * BN_PAGE);
        // this lane's eight scores: keys kb + 8 g + e, e = 4 h + r
        float s[8];
        float mx = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int key = kb + 8 * g + e;
            float v = (e < 4 ? st0[e & 3] : st1[e & 3]) * scale2;
            if (a.dist_a) v -= ba * __log2f(1.0f + bb * (float)(qpos - key));     // a ln(x) log2(e) = a log2(x)
            if (!col_ok || key > qpos || key >= k_hi || key <= q_lo) v = -INFINITY;
            s[e] = v;
            mx = fmaxf(mx, v);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, BN_WAVE));     // the four lane groups of a column
        mx = fmaxf(mx, __shfl_xor(mx, 32, BN_WAVE));
        const float m_new = fmaxf(m, mx);
        float alpha = 1.f;
        if (m_new == -INFINITY) {
#pragma unroll
            for (int e = 0; e < 8; ++e) s[e] = 0.f;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) s[e] = __builtin_amdgcn_exp2f(s[e] - m_new);
            alpha = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
        }
        m = m_new;
        const f32x8 pv = {s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7]};
        const bf16x8 pb = __builtin_convertvector(pv, bf16x8);
        const f32x4 lsum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb, (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
        l = fmaf(l, alpha, lsum[0]);
        // keys past the tile's last position may hold anything in V^T (0 * NaN is NaN): cleared
        if (kb + 32 > k_hi) {
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                uint4 w = __builtin_bit_cast(uint4, va[t]);
                const int first = kb + 8 * g;
                if (first + 0 >= k_hi) w.x &= 0xffff0000u;
                if (first + 1 >= k_hi) w.x &= 0x0000ffffu;
                if (first + 2 >= k_hi) w.y &= 0xffff0000u;
                if (first + 3 >= k_hi) w.y &= 0x0000ffffu;
                if (first + 4 >= k_hi) w.z &= 0xffff0000u;
                if (first + 5 >= k_hi) w.z &= 0x0000ffffu;
                if (first + 6 >= k_hi) w.w &= 0xffff0000u;
                if (first + 7 >= k_hi) w.w &= 0x0000ffffu;
                va[t] = __builtin_bit_cast(bf16x8, w);
            }
        }
#pragma unroll
        for (int t = 0; t < DT; ++t) {
            acc[t] *= alpha;
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[t], pb, acc[t], 0, 0, 0);
        }
    }
    // the sink: a term 2^(sv - m') with no value, m' = max(m, sv)
    float fa = 1.f;
    if (a.sink) {
        const float sv = a.sink_values ? a.sink_values[head] * AG_LOG2E : 0.f;       // the sink's score in the exponent's base 2
        const float m2 = fmaxf(m, sv);
        fa = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - m2);
        l = fmaf(l, fa, __builtin_amdgcn_exp2f(sv - m2));
    }
    const float inv = l > 0.f ? fa / l : 0.f;
    if (!col_ok) return;
    // acc[t][r] = O^T[value column 16 t + 4 g + r][query i]: four consecutive columns, one 8-byte store
    bf16* op = a.out + (size_t)(row0 + i) * a.out_stride + (size_t)head * VD + 4 * g;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        const bf16 o0 = __float2bfloat16(acc[t][0] * inv), o1 = __float2bfloat16(acc[t][1] * inv);
        const bf16 o2 = __float2bfloat16(acc[t][2] * inv), o3 = __float2bfloat16(acc[t][3] * inv);
        uint2 w;
        w.x = (uint32_t)__builtin_bit_cast(unsigned short, o0) | ((uint32_t)__builtin_bit_cast(unsigned short, o1) << 16);
        w.y = (uint32_t)__builtin_bit_cast(unsigned short, o2) | ((uint32_t)__builtin_bit_cast(unsigned short, o3) << 16);
        *reinterpret_cast<uint2*>(op + 16 * t) = w;
    }
}

struct GenDecodeArgs {
    const bf16* q;            // [n_seqs, q_stride]: head h at h * hs, row b is sequence b's new token
    bf16* out;                // [n_seqs, out_stride]
    const bf16* k_pages;
    const bf16* v_pages;
    const int* block_table;   // [n_seqs, bt_stride]
    const int* seq_lens;      // [n_seqs] keys in the cache, the new one included; 0: a padding row
    const float* dist_a;
    const float* dist_b;
    float* part_o;            // [n_seqs H, n_splits, vd]   (n_splits > 1)
    float* part_ml;           // [n_seqs H, n_splits, 2]: maximum (natural exponent) and sum of the weights
    const int* max_len;       // != null: the longest sequence's key count; the keys per split follow from it
    int q_stride, out_stride, bt_stride, H, Hkv, n_splits, chunk, window, sink;
    const float* sink_values; // [H] float32, or null (score 0)
    float scale;
};

template <int DC, int DT>     // hs = 32 DC, vd = 16 DT
__global__ __launch_bounds__(BN_WAVE) void attn_general_decode_kernel(GenDecodeArgs a) {
    constexpr int HS = 32 * DC, VD = 16 * DT;
    const int seq = blockIdx.x, split = blockIdx.z;
    const int G = a.H / a.Hkv, head_tiles = (G + 15) / 16;
    const int kvh = blockIdx.y / head_tiles, ht = blockIdx.y - kvh * head_tiles;
    const int lane = threadIdx.x, i = lane & 15, g = lane >> 4;
    const bool col_ok = 16 * ht + i < G;                 // this lane's column is a head that exists
    const int head = kvh * G + min(16 * ht + i, G - 1);
    const int len = a.seq_lens[seq], qpos = len - 1;
    int k_lo = 0, k_hi = 0;
    if (len > 0) {
        const int lo = a.window > 0 ? max(0, len - a.window) : 0;
        if (a.n_splits > 1) {
            const int chunk = a.max_len ? bn_split_chunk(*a.max_len, a.n_splits) : a.chunk;
            const int base = a.window > 0 ? (lo / BN_PAGE) * BN_PAGE : 0;
            k_lo = max(lo, base + split * chunk);
            k_hi = min(len, base + (split + 1) * chunk);
        } else {
            k_lo = lo; k_hi = len;
        }
    }
    const size_t prow = ((size_t)seq * a.H + head) * a.n_splits + split;
    if (k_lo >= k_hi) {                                  // no key for this split (or a padding row): zeros and no weight
        if (!col_ok) return;
        if (a.n_splits > 1) {
#pragma unroll
            for (int t = 0; t < DT; ++t)
                *reinterpret_cast<float4*>(a.part_o + prow * VD + 16 * t + 4 * g) = make_float4(0.f, 0.f, 0.f, 0.f);
            if (g == 0) { a.part_ml[2 * prow] = -INFINITY; a.part_ml[2 * prow + 1] = 0.f; }
        } else {
            bf16* op = a.out + (size_t)seq * a.out_stride + (size_t)head * VD + 4 * g;
#pragma unroll
            for (int t = 0; t < DT; ++t) *reinterpret_cast<uint2*>(op + 16 * t) = make_uint2(0u, 0u);
        }
        return;
    }
    bf16x8 qf[DC];
    {
        const bf16* qp = a.q + (size_t)seq * a.q_stride + (size_t)head * HS + 8 * g;
#pragma unroll
        for (int c = 0; c < DC; ++c) qf[c] = ag_ld16(qp + 32 * c);
    }
    const float scale2 = a.scale * AG_LOG2E;
    const float ba = a.dist_a ? a.dist_a[head] : 0.f, bb = a.dist_a ? a.dist_b[head] : 0.f;
    f32x4 acc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const bf16x8 ones = __builtin_bit_cast(bf16x8, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));
    const int krow = 8 * (i >> 2) + (i & 3);
    bf16x8 kn0[DC], kn1[DC];
    auto ask_keys = [&](int kb) {
        const int page = a.block_table[(size_t)seq * a.bt_stride + kb / BN_PAGE];
        const bf16* kbase = a.k_pages + (((size_t)page * a.Hkv + kvh) * BN_PAGE + kb % BN_PAGE + krow) * HS + 8 * g;
#pragma unroll
        for (int c = 0; c < DC; ++c) { kn0[c] = ag_ld16(kbase + 32 * c); kn1[c] = ag_ld16(kbase + 4 * HS + 32 * c); }
    };
    const int first_block = k_lo & ~31, last_block = ((k_hi - 1) / 32) * 32;
    ask_keys(first_block);
    for (int kb = first_block; kb < k_hi; kb += 32) {
        const int page = a.block_table[(size_t)seq * a.bt_stride + kb / BN_PAGE];
        const bf16* vbase = a.v_pages + (((size_t)page * a.Hkv + kvh) * VD + i) * BN_PAGE + kb % BN_PAGE + 8 * g;
        bf16x8 k0[DC], k1[DC];
#pragma unroll
        for (int c = 0; c < DC; ++c) { k0[c] = kn0[c]; k1[c] = kn1[c]; }
        ask_keys(min(kb + 32, last_block));
        f32x4 st0 = (f32x4){0.f, 0.f, 0.f, 0.f}, st1 = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            st0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0[c], qf[c], st0, 0, 0, 0);
            st1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1[c], qf[c], st1, 0, 0, 0);
        }
        bf16x8 va[DT];
#pragma unroll
        for (int t = 0; t < DT; ++t) va[t] = ag_ld16(vbase + (size_t)t * 16 * BN_PAGE);
        float s[8];
        float mx = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int key = kb + 8 * g + e;
            float v = (e < 4 ? st0[e & 3] : st1[e & 3]) * scale2;
            if (a.dist_a) v -= ba * __log2f(1.0f + bb * (float)(qpos - key));
            if (!col_ok || key < k_lo || key >= k_hi) v = -INFINITY;
            s[e] = v;
            mx = fmaxf(mx, v);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, BN_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, BN_WAVE));
        const float m_new = fmaxf(m, mx);
        float alpha = 1.f;
        if (m_new == -INFINITY) {
#pragma unroll
            for (int e = 0; e < 8; ++e) s[e] = 0.f;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) s[e] = __builtin_amdgcn_exp2f(s[e] - m_new);
            alpha = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
        }
        m = m_new;
        const f32x8 pv = {s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7]};
        const bf16x8 pb = __builtin_convertvector(pv, bf16x8);
        const f32x4 lsum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb, (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
        l = fmaf(l, alpha, lsum[0]);
        // positions past the sequence's end may hold anything in V^T (0 * NaN is NaN): cleared
        if (kb + 32 > k_hi) {
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                uint4 w = __builtin_bit_cast(uint4, va[t]);
                const int first = kb + 8 * g;
                if (first + 0 >= k_hi) w.x &= 0xffff0000u;
                if (first + 1 >= k_hi) w.x &= 0x0000ffffu;
                if (first + 2 >= k_hi) w.y &= 0xffff0000u;
                if (first + 3 >= k_hi) w.y &= 0x0000ffffu;
                if (first + 4 >= k_hi) w.z &= 0xffff0000u;
                if (first + 5 >= k_hi) w.z &= 0x0000ffffu;
                if (first + 6 >= k_hi) w.w &= 0xffff0000u;
                if (first + 7 >= k_hi) w.w &= 0x0000ffffu;
                va[t] = __builtin_bit_cast(bf16x8, w);
            }
        }
#pragma unroll
        for (int t = 0; t < DT; ++t) {
            acc[t] *= alpha;
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[t], pb, acc[t], 0, 0, 0);
        }
    }
    if (!col_ok) return;
    if (a.n_splits > 1) {                                // sums relative to the maximum m (base 2), for the merge
#pragma unroll
        for (int t = 0; t < DT; ++t)
            *reinterpret_cast<float4*>(a.part_o + prow * VD + 16 * t + 4 * g) = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
        if (g == 0) { a.part_ml[2 * prow] = m * 0.6931471805599453f; a.part_ml[2 * prow + 1] = l; }
        return;
    }
    float fa = 1.f;
    if (a.sink) {
        const float sv = a.sink_values ? a.sink_values[head] * AG_LOG2E : 0.f;       // the sink's score in the exponent's base 2
        const float m2 = fmaxf(m, sv);
        fa = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - m2);
        l = fmaf(l, fa, __builtin_amdgcn_exp2f(sv - m2));
    }
    const float inv = l > 0.f ? fa / l : 0.f;
    bf16* op = a.out + (size_t)seq * a.out_stride + (size_t)head * VD + 4 * g;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        const bf16 o0 = __float2bfloat16(acc[t][0] * inv), o1 = __float2bfloat16(acc[t][1] * inv);
        const bf16 o2 = __float2bfloat16(acc[t][2] * inv), o3 = __float2bfloat16(acc[t][3] * inv);
        uint2 w;
        w.x = (uint32_t)__builtin_bit_cast(unsigned short, o0) | ((uint32_t)__builtin_bit_cast(unsigned short, o1) << 16);
        w.y = (uint32_t)__builtin_bit_cast(unsigned short, o2) | ((uint32_t)__builtin_bit_cast(unsigned short, o3) << 16);
        *reinterpret_cast<uint2*>(op + 16 * t) = w;
    }
}

// out[row, d] = sum_s e^(m_s - m) o_s[d] / (sum_s e^(m_s - m) l_s [+ e^(-m) for the sink]), the splits in index order;
// one wave a (token, head) row, a lane four value columns at a time
__global__ __launch_bounds__(BN_WAVE) void attn_general_combine_kernel(bf16* __restrict__ out, int out_stride,
                                                                       const float* __restrict__ part_o,
                                                                       const float* __restrict__ part_ml, int H, int vd,
                                                                       int n_splits, int sink,
                                                                       const float* __restrict__ sink_values) {
    const int row = blockIdx.x, tok = row / H, head = row - tok * H;
    const float* ml = part_ml + (size_t)row * n_splits * 2;
    const float sv = sink && sink_values ? sink_values[head] : 0.f;
    float m = sink ? sv : -INFINITY;
    for (int s = 0; s < n_splits; ++s) m = fmaxf(m, ml[2 * s]);
    float den = sink ? expf(sv - m) : 0.f;
    if (m != -INFINITY)
        for (int s = 0; s < n_splits; ++s) den = fmaf(expf(ml[2 * s] - m), ml[2 * s + 1], den);
    const float inv = den > 0.f ? 1.0f / den : 0.f;
    for (int d = 4 * threadIdx.x; d < vd; d += 4 * BN_WAVE) {
        float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
        if (m != -INFINITY) {
            for (int s = 0; s < n_splits; ++s) {
                const float w = expf(ml[2 * s] - m);      // 0 for a split without keys
                if (w == 0.f) continue;
                const float4 o = *reinterpret_cast<const float4*>(part_o + ((size_t)row * n_splits + s) * vd + d);
                num.x = fmaf(w, o.x, num.x); num.y = fmaf(w, o.y, num.y); num.z = fmaf(w, o.z, num.z); num.w = fmaf(w, o.w, num.w);
            }
        }
        bf16* op = out + (size_t)tok * out_stride + (size_t)head * vd + d;
        op[0] = __float2bfloat16(num.x * inv); op[1] = __float2bfloat16(num.y * inv);
        op[2] = __float2bfloat16(num.z * inv); op[3] = __float2bfloat16(num.w * inv);
    }
}

static bool ag_size(int x, int unit) { return x == unit || x == 2 * unit || x == 3 * unit || x == 4 * unit || x == 8 * unit; }

// 1 if the kernels take these head sizes (keys 32, 64, 96, 128 or 256 wide, values 32, 64, 96, 128, 192 or 256)
extern "C" int bn_attn_general_supports(int hs, int vd) { return (ag_size(hs, 32) && (ag_size(vd, 32) || vd == 192)) ? 1 : 0; }

template <int DC>
static int ag_launch_dt(const GenArgs& a, int vd, dim3 grid, hipStream_t s) {
#define AG_CASE(DT) hipLaunchKernelGGL((attn_general_prompt_kernel<DC, DT>), grid, dim3(AG_WAVES * BN_WAVE), 0, s, a); return bn_launch_status()
    switch (vd / 16) {
        case 2: AG_CASE(2);
        case 4: AG_CASE(4);
        case 6: AG_CASE(6);
        case 8: AG_CASE(8);
        case 12: AG_CASE(12);
        case 16: AG_CASE(16);
    }
#undef AG_CASE
    return BN_ERR_ARG;
}

extern "C" int bn_attn_general_prompt(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                                      const void* v_pages, const int* block_table, int bt_stride, const int* tiles, int n_tiles,
                                      int H, int Hkv, int hs, int vd, float scale, const float* dist_a, const float* dist_b,
                                      int sink, const float* sink_values, int window, hipStream_t s) {
    if (n_tiles <= 0 || H <= 0 || Hkv <= 0 || H % Hkv || window < 0 || !bn_attn_general_supports(hs, vd)) return BN_ERR_ARG;
    if (!q || !out || !k_pages || !v_pages || !block_table || !tiles || (dist_a == nullptr) != (dist_b == nullptr)) return BN_ERR_ARG;
    if (q_stride % 8 || out_stride % 4 || (((uintptr_t)q | (uintptr_t)k_pages | (uintptr_t)v_pages) & 15) || ((uintptr_t)out & 7))
        return BN_ERR_ARG;
    GenArgs a;
    a.q = (const bf16*)q; a.out = (bf16*)out; a.k_pages = (const bf16*)k_pages; a.v_pages = (const bf16*)v_pages;
    a.block_table = block_table; a.tiles = tiles; a.dist_a = dist_a; a.dist_b = dist_b;
    a.q_stride = q_stride; a.out_stride = out_stride; a.bt_stride = bt_stride; a.H = H; a.Hkv = Hkv;
    a.scale = scale; a.sink = sink ? 1 : 0; a.sink_values = sink ? sink_values : nullptr; a.window = window;
    const dim3 grid(n_tiles, (H + AG_WAVES - 1) / AG_WAVES);
    switch (hs / 32) {
        case 1: return ag_launch_dt<1>(a, vd, grid, s);
        case 2: return ag_launch_dt<2>(a, vd, grid, s);
        case 3: return ag_launch_dt<3>(a, vd, grid, s);
        case 4: return ag_launch_dt<4>(a, vd, grid, s);
        case 8: return ag_launch_dt<8>(a, vd, grid, s);
    }
    return BN_ERR_ARG;
}

template <int DC>
static int ag_launch_decode_dt(const GenDecodeArgs& a, int vd, dim3 grid, hipStream_t s) {
#define AG_CASE(DT) hipLaunchKernelGGL((attn_general_decode_kernel<DC, DT>), grid, dim3(BN_WAVE), 0, s, a); return bn_launch_status()
    switch (vd / 16) {
        case 2: AG_CASE(2);
        case 4: AG_CASE(4);
        case 6: AG_CASE(6);
        case 8: AG_CASE(8);
        case 12: AG_CASE(12);
        case 16: AG_CASE(16);
    }
#undef AG_CASE
    return BN_ERR_ARG;
}

// Decode form: row b of q is sequence b's new token (seq_lens[b] keys in the cache, 0 for a padding row, whose output is
// zeros).  n_splits > 1: part_o [n_seqs H n_splits, vd] and part_ml [n_seqs H n_splits, 2] float32 work space; the keys per
// split are `chunk` (a multiple of BN_PAGE), or follow the longest sequence's key count in *max_len.
extern "C" int bn_attn_general_decode(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                                      const void* v_pages, const int* block_table, int bt_stride, const int* seq_lens, int n_seqs,
                                      int H, int Hkv, int hs, int vd, float scale, const float* dist_a, const float* dist_b,
                                      int sink, const float* sink_values, int window, int n_splits, int chunk, float* part_o, float* part_ml,
                                      const int* max_len, hipStream_t s) {
    if (n_seqs <= 0 || H <= 0 || Hkv <= 0 || H % Hkv || window < 0 || n_splits < 1 || !bn_attn_general_supports(hs, vd)) return BN_ERR_ARG;
    if (!q || !out || !k_pages || !v_pages || !block_table || !seq_lens || (dist_a == nullptr) != (dist_b == nullptr)) return BN_ERR_ARG;
    if (q_stride % 8 || out_stride % 4 || (((uintptr_t)q | (uintptr_t)k_pages | (uintptr_t)v_pages) & 15) || ((uintptr_t)out & 7))
        return BN_ERR_ARG;
    if (n_splits > 1 && (!part_o || !part_ml || ((uintptr_t)part_o & 15) || (!max_len && (chunk <= 0 || chunk % BN_PAGE)))) return BN_ERR_ARG;
    const int head_tiles = (H / Hkv + 15) / 16;
    if ((long long)Hkv * head_tiles > 65535 || n_splits > 65535) return BN_ERR_ARG;
    GenDecodeArgs a;
    a.q = (const bf16*)q; a.out = (bf16*)out; a.k_pages = (const bf16*)k_pages; a.v_pages = (const bf16*)v_pages;
    a.block_table = block_table; a.seq_lens = seq_lens; a.dist_a = dist_a; a.dist_b = dist_b; a.part_o = part_o; a.part_ml = part_ml;
    a.max_len = n_splits > 1 ? max_len : nullptr;
    a.q_stride = q_stride; a.out_stride = out_stride; a.bt_stride = bt_stride; a.H = H; a.Hkv = Hkv; a.n_splits = n_splits;
    a.chunk = chunk; a.window = window; a.sink = sink ? 1 : 0; a.sink_values = sink ? sink_values : nullptr; a.scale = scale;
    const dim3 grid(n_seqs, Hkv * head_tiles, n_splits);
    int rc = BN_ERR_ARG;
    switch (hs / 32) {
        case 1: rc = ag_launch_decode_dt<1>(a, vd, grid, s); break;
        case 2: rc = ag_launch_decode_dt<2>(a, vd, grid, s); break;
        case 3: rc = ag_launch_decode_dt<3>(a, vd, grid, s); break;
        case 4: rc = ag_launch_decode_dt<4>(a, vd, grid, s); break;
        case 8: rc = ag_launch_decode_dt<8>(a, vd, grid, s); break;
    }
    if (rc != 0 || n_splits == 1) return rc;
    hipLaunchKernelGGL(attn_general_combine_kernel, dim3(n_seqs * H), dim3(BN_WAVE), 0, s, (bf16*)out, out_stride, part_o, part_ml,
                       H, vd, n_splits, sink ? 1 : 0, sink ? sink_values : nullptr);
    return bn_launch_status();
}
