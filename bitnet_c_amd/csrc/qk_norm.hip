// What an attention mixer of the general form does to its projected heads before they meet: an RMSNorm over each query
// and key head (one weight vector of the head size, shared by the heads) or over the whole query projection and the whole
// key projection (weights as wide as the projection); eps inside the root; then a rotation of the first rope_dims
// dimensions of every query and key head by the position, in neighbouring pairs (2i, 2i + 1) or in split-half pairs
// (i, i + rope_dims / 2): (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * inv_freq[i]; then a query
// temperature that grows with the position; and the write of the new keys and values into the pages.  One kernel for
// prompt and decode steps; all arithmetic in float32, the results stored once in the activations' type.
//
//   q_h <- rot_p(q_h / rms * wq) * (1 + coef * ln(floor((p + 1) / every) + 1))
//   k_g <- rot_p(k_g / rms * wk)                       -> page of position p
//   v_g                                                 -> page of position p
//
// v_from_k: the values are the key projections themselves, as projected (before the key's norm and rotation): qkv then
// holds no value heads, and kv head g's value is read from its key's columns, which this kernel leaves as they arrived.
//
// Pages hold a row per position for the keys, [page, kv head, BN_PAGE, hs]; the values lie the same way ("rows" layout,
// [page, kv head, BN_PAGE, vd]) or transposed ([page, kv head, vd, BN_PAGE]), as the caller says.
#include "common.h"
#include <math.h>

#define QKN_WAVES 4
#define QKN_MAX_WAVES 16         // waves of the one workgroup that takes a whole row (norms over the whole projections)
#define QKN_PER_LANE (BN_MAX_HEAD_DIM / BN_WAVE)

struct QkNormArgs {
    void* qkv;                // [T, ld]: q heads (H x hs), k heads (Hkv x hs), v heads (Hkv x vd)
    const int* positions;     // [T]; < 0: a padding row, nothing is written
    const int* seq_index;     // [T] row of the block table
    const int* block_table;   // [n_seqs, bt_stride]
    void* k_pages;
    void* v_pages;            // both null: nothing is stored (the entry reads another entry's cache)
    const float* wq;          // [hs], or [H hs] when norm_all; null: no norm
    const float* wk;          // [hs], or [Hkv hs]
    const float* inv_freq;    // [rope_dims / 2]; null: no rotation
    int ld, bt_stride, H, Hkv, hs, vd;
    int v_transposed;         // the values' pages are [page, kv head, vd, BN_PAGE]
    int norm_all;             // the norms run over the whole projection instead of over each head
    int rope_dims, rope_interleaved;
    float eps, temp_coef;
    int temp_every;           // <= 0: no temperature
    int v_from_k;             // the values are the keys as projected (vd == hs; qkv has no value columns)
};

// sine and cosine of an angle of any size: the angle less the nearest multiple of 2 pi (2 pi as the sum of two floats, the
// products exact inside the fused operations), then the hardware's functions on what is left, which lies in [-pi, pi]
__device__ __forceinline__ void qkn_sincos(float a, float* sn, float* cs) {
    const float k = rintf(a * 0.15915494309189535f);
    float r = fmaf(-k, 6.2831854820251465f, a);
    r = fmaf(-k, -1.7484555e-7f, r);
    *sn = __sinf(r);
    *cs = __cosf(r);
}

// a workgroup takes QKN_WAVES heads of one row, a wave each; heads 0 .. H-1 are queries, then Hkv keys, then Hkv values.
// With norms over the whole projections one workgroup (of up to QKN_MAX_WAVES waves) takes all heads of a row, its waves in turn: the query heads are
// rewritten in place, so the sums of squares over the whole projections must have been formed (by all threads, in front
// of a barrier) before any of them is, and no other workgroup may read the row meanwhile.
template <typename T>
__global__ __launch_bounds__(QKN_MAX_WAVES * BN_WAVE) void qk_norm_store_kernel(QkNormArgs a) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, lane = threadIdx.x & (BN_WAVE - 1), wave = threadIdx.x / BN_WAVE;
    const int pos = a.positions[t];
    if (pos < 0) return;
    T* row = reinterpret_cast<T*>(a.qkv) + (size_t)t * a.ld;
    float fq = 1.0f, fk = 1.0f;
    if (a.norm_all && a.wq) {
        const int nq = a.H * a.hs, nk = a.Hkv * a.hs;
        float sq = 0.f, sk = 0.f;
        for (int d = threadIdx.x; d < nq; d += blockDim.x) { const float x = to_f32(row[d]); sq = fmaf(x, x, sq); }
        for (int d = threadIdx.x; d < nk; d += blockDim.x) { const float x = to_f32(row[nq + d]); sk = fmaf(x, x, sk); }
        sq = block_sum(sq, scratch);
        sk = block_sum(sk, scratch);
        fq = 1.0f / sqrtf(sq / (float)nq + a.eps);
        fk = 1.0f / sqrtf(sk / (float)nk + a.eps);
    }
    const int rd = a.inv_freq ? a.rope_dims : 0, half = rd / 2;
    const int n_heads = a.H + 2 * a.Hkv;
    const int head0 = a.norm_all ? 0 : blockIdx.y * QKN_WAVES, head1 = a.norm_all ? n_heads : min(n_heads, head0 + QKN_WAVES);
    const int n_waves = blockDim.x / BN_WAVE;
    for (int head = head0 + wave; head < head1; head += n_waves) {
        const bool is_q = head < a.H, is_k = !is_q && head < a.H + a.Hkv;
        if (is_q || is_k) {
            if (is_k && !a.k_pages) continue;
            T* v = row + (size_t)head * a.hs;
            const float* w = is_q ? a.wq : a.wk;
            if (w && a.norm_all) w += (size_t)(is_q ? head : head - a.H) * a.hs;
            float f = is_q ? fq : fk;
            if (w && !a.norm_all) {
                float ss = 0.f;
                for (int d = lane; d < a.hs; d += BN_WAVE) { const float x = to_f32(v[d]); ss = fmaf(x, x, ss); }
                ss = wave_sum(ss);
                f = 1.0f / sqrtf(ss / (float)a.hs + a.eps);
            }
            float temp = 1.0f;
            if (is_q && a.temp_every > 0) temp = 1.0f + a.temp_coef * logf((float)((pos + 1) / a.temp_every) + 1.0f);
            // the whole head first (a rotation reads its partner, which another lane or a later turn overwrites)
            float xs[QKN_PER_LANE], ps[QKN_PER_LANE];
#pragma unroll
            for (int j = 0; j < QKN_PER_LANE; ++j) {
                const int d = lane + BN_WAVE * j;
                xs[j] = ps[j] = 0.f;
                if (d < a.hs) {
                    xs[j] = to_f32(v[d]);
                    if (w) xs[j] = xs[j] * f * w[d];
                    if (d < rd) {
                        const int pd = a.rope_interleaved ? (d ^ 1) : (d < half ? d + half : d - half);
                        ps[j] = to_f32(v[pd]);
                        if (w) ps[j] = ps[j] * f * w[pd];
                    }
                }
            }
            T* dst = v;
            if (is_k) {
                const int kvh = head - a.H;
                const int page = a.block_table[(size_t)a.seq_index[t] * a.bt_stride + pos / BN_PAGE];
                dst = reinterpret_cast<T*>(a.k_pages) + (((size_t)page * a.Hkv + kvh) * BN_PAGE + pos % BN_PAGE) * a.hs;
            }
#pragma unroll
            for (int j = 0; j < QKN_PER_LANE; ++j) {
                const int d = lane + BN_WAVE * j;
                if (d >= a.hs) continue;
                float x = xs[j];
                if (d < rd) {
                    const int i = a.rope_interleaved ? (d >> 1) : (d < half ? d : d - half);
                    const bool first = a.rope_interleaved ? !(d & 1) : d < half;
                    float sn, cs;
                    qkn_sincos((float)pos * a.inv_freq[i], &sn, &cs);
                    x = first ? x * cs - ps[j] * sn : x * cs + ps[j] * sn;
                }
                dst[d] = from_f32<T>(x * temp);
            }
        } else {
            if (!a.v_pages) continue;
            const int kvh = head - a.H - a.Hkv;
            const T* v = a.v_from_k ? row + (size_t)(a.H + kvh) * a.hs : row + (size_t)(a.H + a.Hkv) * a.hs + (size_t)kvh * a.vd;
            const int page = a.block_table[(size_t)a.seq_index[t] * a.bt_stride + pos / BN_PAGE];
            if (a.v_transposed) {
                T* dst = reinterpret_cast<T*>(a.v_pages) + ((size_t)page * a.Hkv + kvh) * a.vd * BN_PAGE + pos % BN_PAGE;
                for (int d = lane; d < a.vd; d += BN_WAVE) dst[(size_t)d * BN_PAGE] = v[d];
            } else {
                T* dst = reinterpret_cast<T*>(a.v_pages) + (((size_t)page * a.Hkv + kvh) * BN_PAGE + pos % BN_PAGE) * a.vd;
                for (int d = lane; d < a.vd; d += BN_WAVE) dst[d] = v[d];
            }
        }
    }
}

extern "C" int bn_qk_norm_store(int dtype, void* qkv, int ld, const int* positions, const int* seq_index,
                                const int* block_table, int bt_stride, void* k_pages, void* v_pages, const float* wq,
                                const float* wk, int n_tokens, int H, int Hkv, int hs, int vd, float eps, float temp_coef,
                                int temp_every, int v_transposed, int norm_all, const float* inv_freq, int rope_dims,
                                int rope_interleaved, int v_from_k, hipStream_t s) {
    if (n_tokens <= 0 || H <= 0 || Hkv <= 0 || hs <= 0 || hs > BN_MAX_HEAD_DIM || vd <= 0 || !qkv || !positions) return BN_ERR_ARG;
    if ((k_pages == nullptr) != (v_pages == nullptr) || (k_pages && (!seq_index || !block_table))) return BN_ERR_ARG;
    if ((wq == nullptr) != (wk == nullptr) || ld < H * hs + Hkv * (v_from_k ? hs : hs + vd) || (v_from_k && vd != hs)) return BN_ERR_ARG;
    if (inv_freq && (rope_dims <= 0 || rope_dims % 2 || rope_dims > hs)) return BN_ERR_ARG;
    QkNormArgs a;
    a.qkv = qkv; a.positions = positions; a.seq_index = seq_index; a.block_table = block_table;
    a.k_pages = k_pages; a.v_pages = v_pages; a.wq = wq; a.wk = wk; a.inv_freq = inv_freq;
    a.ld = ld; a.bt_stride = bt_stride; a.H = H; a.Hkv = Hkv; a.hs = hs; a.vd = vd;
    a.eps = eps; a.temp_coef = temp_coef; a.temp_every = temp_every; a.v_transposed = v_transposed ? 1 : 0;
    a.norm_all = norm_all ? 1 : 0; a.rope_dims = inv_freq ? rope_dims : 0; a.rope_interleaved = rope_interleaved ? 1 : 0;
    a.v_from_k = v_from_k ? 1 : 0;
    const int n_heads = H + 2 * Hkv;
    const int waves = norm_all ? (n_heads < QKN_MAX_WAVES ? (n_heads < QKN_WAVES ? QKN_WAVES : n_heads) : QKN_MAX_WAVES) : QKN_WAVES;
    const dim3 grid(n_tokens, norm_all ? 1 : (n_heads + QKN_WAVES - 1) / QKN_WAVES), block(waves * BN_WAVE);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(qk_norm_store_kernel<float>, grid, block, 0, s, a);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(qk_norm_store_kernel<bf16>, grid, block, 0, s, a);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}
