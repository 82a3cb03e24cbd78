// Linear attention with a fixed decay per head ("lightning" attention): per head a matrix state S [dk, dv] in float32,
//
//     S_t = decay S_(t-1) + k_t v_t^T,      o_t = S_t^T q_t,      q, k, v = silu of their projections
//
// for prompt and decode steps alike.  The state lives in the cache's state area, [slot][head][dk][dv] float32; a kernel
// finds a sequence's row through the step's device-side slot ids and its tokens either through a list of tiles (one tile
// a sequence: sequence, first row, rows, position of the first; a tile of no rows is skipped) or, tiles == null, as row
// b = the one new token of sequence b (seq_lens[b] == 0: a padding row, nothing is touched).  A sequence whose first
// position is 0 starts from zeros whatever its state row holds.  Everything that enters the recurrence is float32; the
// projections arrive in the activations' type and pass their silu in float32.
//
//   bn_lightning_scan    the recurrence: a workgroup owns (sequence, head, 64 value columns); a column's rows are spread
//                        over the workgroup's four waves, each thread keeping its rows of S in registers; tokens come in
//                        chunks that all threads stage (silu applied) in shared memory, the waves walk a chunk token by
//                        token and leave their partial sums, which are added in wave order.  The order of every sum is
//                        a function of the sizes alone, so a token's output does not depend on how the step was cut.
//                        This "chain" form serves decode steps, key widths above LC_MAX_DIM and prompt steps of so
//                        many sequences that it fills the chip (bn_lightning_prefers_chunks).
//   the chunked form     other prompt steps: a workgroup owns (sequence, head, 16 value columns) and takes the tokens in
//                        chunks of 64, from a float32 copy of silu(q), silu(k), silu(v) that a kernel in front makes.  With d the decay, S the state before the chunk, n its tokens:
//                            A_ij = (q_i . k_j) d^(i-j) for j <= i,    o_i = sum_j A_ij v_j + d^(i+1) S^T q_i,
//                            S   <- d^n S + sum_j d^(n-1-j) k_j v_j^T
//                        which is the chain's sum in another order.  All four products run on the matrix cores in float32
//                        (v_mfma_f32_16x16x4_f32) from operands staged in shared memory; the powers of d come from a table
//                        made in double precision, so no power is a product of rounded powers.  The state's tiles stay in
//                        the accumulators of the waves that own them, with a copy in shared memory for the other waves.
//   bn_row_norm_gate     y = o / sqrt(mean_row(o^2) + eps) * weight * act(gate): the heads' outputs normed together
#include "common.h"
#include <math.h>

#define LA_THREADS 256
#define LA_CB 64              // value columns of a workgroup: a wave's lanes
#define LA_RG 4               // groups of rows: the workgroup's waves
#define LA_TC 16              // tokens of a staged chunk
#define LA_MAX_DIM 256        // largest key width (value widths are cut into column blocks and have no bound)

struct LaRange { int seq, row0, n, pos0; };

__device__ __forceinline__ LaRange la_range(const int* tiles, const int* seq_lens, int idx) {
    LaRange r;
    if (tiles) {
        const int* t = tiles + 4 * idx;
        r.seq = t[0]; r.row0 = t[1]; r.n = t[2]; r.pos0 = t[3];
    } else {
        r.seq = idx; r.row0 = idx; r.pos0 = seq_lens[idx] - 1; r.n = r.pos0 >= 0 ? 1 : 0;
    }
    return r;
}

__device__ __forceinline__ float la_silu(float z) { return z / (1.0f + expf(-z)); }

struct LaArgs {
    const void* x;            // [T, ld]: the projections side by side
    float* o;                 // [T, H dv] float32
    const float* decay;       // [H]
    float* state;             // [slots, state_stride]: [H][dk][dv]
    size_t state_stride;
    const int* tiles;         // [n, 4] or null
    const int* seq_lens;      // [B] when tiles is null
    const int* slot_ids;      // [sequences of the step]
    int ld, q_col, k_col, v_col, H, dk, dv;
    const float* pq;          // the chunked form's copy of q, k and v (see lightning_prepare_kernel) and its sizes
    const float* pk;
    const float* pv;
    int T, dks, dvs;
};

template <typename T, int RPT>
__global__ __launch_bounds__(LA_THREADS) void lightning_scan_kernel(LaArgs a) {
    constexpr int DKP = RPT * LA_RG;                     // the key rows, rounded up; rows from dk on stay zero
    extern __shared__ __align__(16) float la_smem[];
    float* q_s = la_smem;                                // [LA_TC][DKP]
    float* k_s = q_s + LA_TC * DKP;                      // [LA_TC][DKP]
    float* v_s = k_s + LA_TC * DKP;                      // [LA_TC][LA_CB]
    float* p_s = v_s + LA_TC * LA_CB;                    // [LA_TC][LA_RG][LA_CB]
    const LaRange sr = la_range(a.tiles, a.seq_lens, blockIdx.x);
    if (sr.n <= 0 || sr.pos0 < 0) return;
    const int tid = threadIdx.x, col = tid % LA_CB, rg = tid / LA_CB;
    const int head = blockIdx.y, c0 = blockIdx.z * LA_CB, c = c0 + col, r0 = rg * RPT;
    const bool has = c < a.dv;
    float* sp = a.state + (size_t)a.slot_ids[sr.seq] * a.state_stride + (size_t)head * a.dk * a.dv + c;
    float S[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) S[i] = (has && r0 + i < a.dk && sr.pos0 > 0) ? sp[(size_t)(r0 + i) * a.dv] : 0.f;
    const float decay = a.decay[head];
    const T* x = reinterpret_cast<const T*>(a.x) + (size_t)sr.row0 * a.ld;
    float* o = a.o + (size_t)sr.row0 * a.H * a.dv + (size_t)head * a.dv + c0;
    for (int t0 = 0; t0 < sr.n; t0 += LA_TC) {
        const int nt = min(LA_TC, sr.n - t0);
        for (int idx = tid; idx < LA_TC * DKP; idx += LA_THREADS) {
            const int tt = idx / DKP, r = idx - tt * DKP;
            float qv = 0.f, kv = 0.f;
            if (tt < nt && r < a.dk) {
                const T* row = x + (size_t)(t0 + tt) * a.ld + (size_t)head * a.dk + r;
                qv = la_silu(to_f32(row[a.q_col]));
                kv = la_silu(to_f32(row[a.k_col]));
            }
            q_s[idx] = qv;
            k_s[idx] = kv;
        }
        for (int idx = tid; idx < LA_TC * LA_CB; idx += LA_THREADS) {
            const int tt = idx / LA_CB, cc = idx - tt * LA_CB;
            v_s[idx] = (tt < nt && c0 + cc < a.dv)
                           ? la_silu(to_f32(x[(size_t)(t0 + tt) * a.ld + a.v_col + (size_t)head * a.dv + c0 + cc])) : 0.f;
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float vt = v_s[tt * LA_CB + col];
            const float4* k4 = reinterpret_cast<const float4*>(k_s + tt * DKP + r0);
            const float4* q4 = reinterpret_cast<const float4*>(q_s + tt * DKP + r0);
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < RPT / 4; ++i) {
                const float4 kk = k4[i], qq = q4[i];
                const float kv[4] = {kk.x, kk.y, kk.z, kk.w}, qv[4] = {qq.x, qq.y, qq.z, qq.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    S[4 * i + e] = fmaf(decay, S[4 * i + e], kv[e] * vt);
                    acc[e] = fmaf(S[4 * i + e], qv[e], acc[e]);
                }
            }
            p_s[(tt * LA_RG + rg) * LA_CB + col] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
        }
        __syncthreads();
        for (int idx = tid; idx < nt * LA_CB; idx += LA_THREADS) {
            const int tt = idx / LA_CB, cc = idx - tt * LA_CB;
            if (c0 + cc < a.dv) {
                const float* p = p_s + tt * LA_RG * LA_CB + cc;
                o[(size_t)(t0 + tt) * a.H * a.dv + cc] = (p[0] + p[LA_CB]) + (p[2 * LA_CB] + p[3 * LA_CB]);
            }
        }
        // the next chunk's staging writes q_s, k_s and v_s only, and its barrier stands before the next write of p_s
    }
    if (has) {
#pragma unroll
        for (int i = 0; i < RPT; ++i)
            if (r0 + i < a.dk) sp[(size_t)(r0 + i) * a.dv] = S[i];
    }
}

// ---- the chunked form -------------------------------------------------------------------------------------------------
#define LC_C 64               // tokens of a chunk
#define LC_MAX_DIM 128        // largest key width of the chunked form
#define LC_POW 80             // floats kept for the table of powers (LC_C + 1 used)

typedef float f32x4 __attribute__((ext_vector_type(4)));

// The chunked form reads a copy of the step's q, k and v that one kernel makes first: silu applied, float32, head by
// head ([H][T][dks] for q and for k, then [H][T][dvs] for v; dks and dvs the widths rounded up to a multiple of 4, the
// elements behind a width zero).  A chunk of one head is then one run of consecutive bytes instead of 64 short pieces a
// whole row of projections apart, every load is 16 bytes, and silu is taken once and not by every workgroup that shares
// a head's q and k.
struct LcPrepArgs {
    const void* x;            // [T, ld]
    float* q;                 // [H][T][dks]
    float* k;                 // [H][T][dks]
    float* v;                 // [H][T][dvs]
    int T, ld, q_col, k_col, v_col, H, dk, dv, dks, dvs;
};

template <typename T>
__global__ __launch_bounds__(256) void lightning_prepare_kernel(LcPrepArgs a) {
    const int t = blockIdx.x;
    const T* row = reinterpret_cast<const T*>(a.x) + (size_t)t * a.ld;
    const int nq = a.H * (a.dks / 4), nv = a.H * (a.dvs / 4);
    for (int idx = threadIdx.x; idx < 2 * nq + nv; idx += blockDim.x) {
        const int which = idx < nq ? 0 : idx < 2 * nq ? 1 : 2;
        const int rel = idx - which * nq, per = which == 2 ? a.dvs / 4 : a.dks / 4;
        const int h = rel / per, r = (rel - h * per) * 4, width = which == 2 ? a.dv : a.dk, ws = which == 2 ? a.dvs : a.dks;
        const T* src = row + (which == 0 ? a.q_col : which == 1 ? a.k_col : a.v_col) + (size_t)h * width + r;
        float e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) e[i] = r + i < width ? la_silu(to_f32(src[i])) : 0.f;
        float* dst = (which == 0 ? a.q : which == 1 ? a.k : a.v) + ((size_t)h * a.T + t) * ws + r;
        *reinterpret_cast<float4*>(dst) = make_float4(e[0], e[1], e[2], e[3]);
    }
}

// A barrier of the workgroup that orders its shared memory only: loads and stores of global memory stay in flight.
__device__ __forceinline__ void lc_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// A product D[16 x 16] += A[16 x K] B[K x 16] is walked in blocks of 16 along K; inside a block lane m + 16 g supplies
// the four indices 4 g .. 4 g + 3 in turn (A[m][.] and B[.][m]), so an operand that is contiguous along K is one 16-byte
// read of shared memory per block.  D's element r of lane m + 16 g is row 4 g + r, column m.
#define LC_MFMA(a_, b_, c_) __builtin_amdgcn_mfma_f32_16x16x4f32((a_), (b_), (c_), 0, 0, 0)

// RT: row tiles (of 16 key rows) of the state that a wave owns, the key width rounded up to 64 RT; NCT: column tiles of 16
template <int RT, int NCT>
__global__ __launch_bounds__(LA_THREADS) void lightning_chunk_kernel(LaArgs a) {
    constexpr int DKP = 64 * RT, CB = 16 * NCT;
    constexpr int LDQ = DKP + 4, LDV = CB + 4, LDA = LC_C + 4;     // rows 16 bytes apart from a multiple of 128: few bank conflicts
    extern __shared__ __align__(16) float la_smem[];
    float* Q_s = la_smem;                                 // [LC_C][LDQ]   silu(q), rows from the chunk's tokens on zero
    float* K_s = Q_s + LC_C * LDQ;                        // [LC_C][LDQ]
    float* V_s = K_s + LC_C * LDQ;                        // [LC_C][LDV]
    float* A_s = V_s + LC_C * LDV;                        // [LC_C][LDA]   decayed scores, the causal half
    float* S_s = A_s + LC_C * LDA;                        // [DKP][LDV]    the state before the chunk
    float* P_s = S_s + DKP * LDV;                         // [LC_POW]      decay^0 .. decay^LC_C
    const LaRange sr = la_range(a.tiles, a.seq_lens, blockIdx.x);
    if (sr.n <= 0 || sr.pos0 < 0) return;
    const int tid = threadIdx.x, wave = tid / BN_WAVE, lane = tid % BN_WAVE, m = lane % 16, g = lane / 16;
    const int head = blockIdx.y, c0 = blockIdx.z * CB;
    float* sp = a.state + (size_t)a.slot_ids[sr.seq] * a.state_stride + (size_t)head * a.dk * a.dv;
    if (tid <= LC_C) P_s[tid] = (float)pow((double)a.decay[head], (double)tid);
    f32x4 S[RT][NCT];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = 16 * (wave + 4 * i) + 4 * g + r, c = c0 + 16 * ct + m;
                const float v = (sr.pos0 > 0 && row < a.dk && c < a.dv) ? sp[(size_t)row * a.dv + c] : 0.f;
                S[i][ct][r] = v;
                S_s[row * LDV + 16 * ct + m] = v;
            }
    const float* pq = a.pq + ((size_t)head * a.T + sr.row0) * a.dks;
    const float* pk = a.pk + ((size_t)head * a.T + sr.row0) * a.dks;
    const float* pv = a.pv + ((size_t)head * a.T + sr.row0) * a.dvs;
    float* o = a.o + (size_t)sr.row0 * a.H * a.dv + (size_t)head * a.dv + c0;
    // what a thread stages of a chunk: NQ runs of four elements of q and of k, NV of v, asked for a chunk ahead; a run
    // past the chunk's tokens or the head's width is loaded from a place that exists and dropped when it is stored
    constexpr int NQ = LC_C * (DKP / 4) / LA_THREADS, NV = LC_C * (CB / 4) / LA_THREADS;
    f32x4 qraw[NQ], kraw[NQ], vraw[NV];
    auto fetch = [&](int t0) {
        const int nt = min(LC_C, sr.n - t0);
#pragma unroll
        for (int it = 0; it < NQ; ++it) {
            const int idx = tid + it * LA_THREADS, tt = idx / (DKP / 4), r = (idx - tt * (DKP / 4)) * 4;
            const bool live = tt < nt && r < a.dks;
            const size_t at = (size_t)(t0 + (live ? tt : 0)) * a.dks + (live ? r : 0);
            qraw[it] = *reinterpret_cast<const f32x4*>(pq + at);
            kraw[it] = *reinterpret_cast<const f32x4*>(pk + at);
        }
#pragma unroll
        for (int it = 0; it < NV; ++it) {
            const int idx = tid + it * LA_THREADS, tt = idx / (CB / 4), cc = (idx - tt * (CB / 4)) * 4;
            const bool live = tt < nt && c0 + cc < a.dvs;
            vraw[it] = *reinterpret_cast<const f32x4*>(pv + (size_t)(t0 + (live ? tt : 0)) * a.dvs + (live ? c0 + cc : 0));
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < sr.n; t0 += LC_C) {
        const int nt = min(LC_C, sr.n - t0);
        const int nb = (nt + 15) / 16;                    // blocks of 16 tokens that hold any
        // ---- the chunk's q, k and v go to shared memory; the next chunk's are asked for ----
        const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int it = 0; it < NQ; ++it) {
            const int idx = tid + it * LA_THREADS, tt = idx / (DKP / 4), r = (idx - tt * (DKP / 4)) * 4;
            const bool live = tt < nt && r < a.dks;
            *reinterpret_cast<f32x4*>(Q_s + tt * LDQ + r) = live ? qraw[it] : zero4;
            *reinterpret_cast<f32x4*>(K_s + tt * LDQ + r) = live ? kraw[it] : zero4;
        }
#pragma unroll
        for (int it = 0; it < NV; ++it) {
            const int idx = tid + it * LA_THREADS, tt = idx / (CB / 4), cc = (idx - tt * (CB / 4)) * 4;
            *reinterpret_cast<f32x4*>(V_s + tt * LDV + cc) = (tt < nt && c0 + cc < a.dvs) ? vraw[it] : zero4;
        }
        if (t0 + LC_C < sr.n) fetch(t0 + LC_C);
        lc_barrier();
        // ---- A = (Q K^T) with the decay, the ten tiles on and under the diagonal dealt to the waves ----
        for (int ti = wave; ti < 10; ti += 4) {
            const int ib = ti < 4 ? 3 : ti < 7 ? 2 : ti < 9 ? 1 : 0;
            const int jb = ti - (ti < 4 ? 0 : ti < 7 ? 4 : ti < 9 ? 7 : 9);
            if (ib >= nb) continue;                        // no token in these rows (the same for the whole wave)
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            const float* qp = Q_s + (16 * ib + m) * LDQ + 4 * g;
            const float* kp = K_s + (16 * jb + m) * LDQ + 4 * g;
#pragma unroll 4
            for (int u = 0; u < DKP / 16; ++u) {
                const float4 qa = *reinterpret_cast<const float4*>(qp + 16 * u);
                const float4 kb = *reinterpret_cast<const float4*>(kp + 16 * u);
                acc = LC_MFMA(qa.x, kb.x, acc);
                acc = LC_MFMA(qa.y, kb.y, acc);
                acc = LC_MFMA(qa.z, kb.z, acc);
                acc = LC_MFMA(qa.w, kb.w, acc);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 16 * ib + 4 * g + r, j = 16 * jb + m;
                A_s[i * LDA + j] = i >= j ? acc[r] * P_s[max(i - j, 0)] : 0.f;
            }
        }
        lc_barrier();
        // ---- o = A V + d^(i+1) Q S: a wave takes 16 tokens ----
        if (wave < nb) {
            f32x4 av[NCT], qs[NCT];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) { av[ct] = (f32x4){0.f, 0.f, 0.f, 0.f}; qs[ct] = (f32x4){0.f, 0.f, 0.f, 0.f}; }
            const float* ap = A_s + (16 * wave + m) * LDA + 4 * g;
            for (int u = 0; u <= wave; ++u) {
                const float4 a4 = *reinterpret_cast<const float4*>(ap + 16 * u);
                const float* vp = V_s + (16 * u + 4 * g) * LDV + m;
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) {
                    av[ct] = LC_MFMA(a4.x, vp[16 * ct], av[ct]);
                    av[ct] = LC_MFMA(a4.y, vp[LDV + 16 * ct], av[ct]);
                    av[ct] = LC_MFMA(a4.z, vp[2 * LDV + 16 * ct], av[ct]);
                    av[ct] = LC_MFMA(a4.w, vp[3 * LDV + 16 * ct], av[ct]);
                }
            }
            const float* qp = Q_s + (16 * wave + m) * LDQ + 4 * g;
#pragma unroll 2
            for (int u = 0; u < DKP / 16; ++u) {
                const float4 a4 = *reinterpret_cast<const float4*>(qp + 16 * u);
                const float* vp = S_s + (16 * u + 4 * g) * LDV + m;
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) {
                    qs[ct] = LC_MFMA(a4.x, vp[16 * ct], qs[ct]);
                    qs[ct] = LC_MFMA(a4.y, vp[LDV + 16 * ct], qs[ct]);
                    qs[ct] = LC_MFMA(a4.z, vp[2 * LDV + 16 * ct], qs[ct]);
                    qs[ct] = LC_MFMA(a4.w, vp[3 * LDV + 16 * ct], qs[ct]);
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 16 * wave + 4 * g + r;
                const float carry = P_s[min(i + 1, LC_C)];
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct)
                    if (i < nt && c0 + 16 * ct + m < a.dv)
                        o[(size_t)(t0 + i) * a.H * a.dv + 16 * ct + m] = av[ct][r] + carry * qs[ct][r];
            }
        }
        // ---- S <- d^n S + K^T (d^(n-1-j) V): a wave's own tiles, in its accumulators ----
        {
            const float whole = P_s[nt];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) {
                float b[4][4];
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int j = 16 * u + 4 * g + e;
                        b[u][e] = j < nt ? V_s[j * LDV + 16 * ct + m] * P_s[max(nt - 1 - j, 0)] : 0.f;
                    }
#pragma unroll
                for (int i = 0; i < RT; ++i) {
                    f32x4 acc = S[i][ct] * whole;
                    const float* kp = K_s + (4 * g) * LDQ + 16 * (wave + 4 * i) + m;
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        if (u < nb) {                      // blocks of 16 tokens that hold any
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc = LC_MFMA(kp[(16 * u + e) * LDQ], b[u][e], acc);
                        }
                    S[i][ct] = acc;
                }
            }
        }
        lc_barrier();                                      // every wave has read the old state and this chunk's q, k, v
#pragma unroll
        for (int i = 0; i < RT; ++i)
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int r = 0; r < 4; ++r) S_s[(16 * (wave + 4 * i) + 4 * g + r) * LDV + 16 * ct + m] = S[i][ct][r];
        // the next chunk's barrier behind its staging stands before any read of S_s
    }
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = 16 * (wave + 4 * i) + 4 * g + r, c = c0 + 16 * ct + m;
                if (row < a.dk && c < a.dv) sp[(size_t)row * a.dv + c] = S[i][ct][r];
            }
}

static int la_compute_units() {
    static int n[64] = {0};                 // per device
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (n[dev] == 0) {
        int v = 0;
        n[dev] = (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) ? v : 256;
    }
    return n[dev];
}

template <int RT, int NCT>
static int lc_launch(const LaArgs& a, int n_seqs, hipStream_t s) {
    constexpr int DKP = 64 * RT, CB = 16 * NCT;
    constexpr size_t smem = sizeof(float) * (2 * LC_C * (DKP + 4) + LC_C * (CB + 4) + LC_C * (LC_C + 4) + DKP * (CB + 4) + LC_POW);
    static_assert(smem <= 160 * 1024, "the chunked form's shared memory");
    static bool raised = false;              // beyond the default limit of dynamic shared memory
    if (smem > 64 * 1024 && !raised) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(lightning_chunk_kernel<RT, NCT>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return (int)e;
        raised = true;
    }
    const dim3 grid(n_seqs, a.H, (a.dv + CB - 1) / CB), block(LA_THREADS);
    hipLaunchKernelGGL((lightning_chunk_kernel<RT, NCT>), grid, block, smem, s, a);
    return bn_launch_status();
}

static int lc_dispatch(int dtype, LaArgs& a, int n_seqs, int n_rows, float* prepared, hipStream_t s) {
    LcPrepArgs p;
    p.x = a.x; p.T = n_rows; p.ld = a.ld; p.q_col = a.q_col; p.k_col = a.k_col; p.v_col = a.v_col; p.H = a.H; p.dk = a.dk; p.dv = a.dv;
    p.dks = (a.dk + 3) / 4 * 4; p.dvs = (a.dv + 3) / 4 * 4;
    p.q = prepared; p.k = p.q + (size_t)a.H * n_rows * p.dks; p.v = p.k + (size_t)a.H * n_rows * p.dks;
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(lightning_prepare_kernel<float>, dim3(n_rows), dim3(256), 0, s, p);
    else hipLaunchKernelGGL(lightning_prepare_kernel<bf16>, dim3(n_rows), dim3(256), 0, s, p);
    const int rc = bn_launch_status();
    if (rc != 0) return rc;
    a.pq = p.q; a.pk = p.k; a.pv = p.v; a.T = n_rows; a.dks = p.dks; a.dvs = p.dvs;
    // a workgroup takes 16 value columns: blocks of 32 and 64 columns (which share one Q K^T among more columns) took as
    // long per column when they were measured, with a fourth of the workgroups
    return a.dk <= 64 ? lc_launch<1, 1>(a, n_seqs, s) : lc_launch<2, 1>(a, n_seqs, s);
}

extern "C" int bn_lightning_supports(int dk, int dv) { return (dk >= 1 && dk <= LA_MAX_DIM && dv >= 1) ? 1 : 0; }

// 1 when prompt steps of these sizes can take the chunked form
extern "C" int bn_lightning_chunked(int dk, int dv) { return (dk >= 1 && dk <= LC_MAX_DIM && dv >= 1) ? 1 : 0; }
// 1 when a prompt step of n_seqs sequences should: the chain form walks a sequence token by token and has a workgroup per
// (sequence, head, 64 columns); from two workgroups a CU on it fills the chip and is the faster one (32 prompts of 256
// tokens, 16 heads of 128 x 128: 0.31 ms against 0.44), below that the chunks are (one prompt of 2,048: 0.26 ms against 1.58)
extern "C" int bn_lightning_prefers_chunks(int n_seqs, int H, int dk, int dv) {
    if (!bn_lightning_chunked(dk, dv) || n_seqs <= 0 || H <= 0) return 0;
    return (long long)n_seqs * H * ((dv + LA_CB - 1) / LA_CB) < 2LL * la_compute_units() ? 1 : 0;
}

// x [T, ld] holds q at q_col, k at k_col (H dk wide each) and v at v_col (H dv wide); n_seqs: tiles, or rows of a decode step;
// prepared: room for the chunked form's copy of q, k and v, n_rows H (2 dks + dvs) floats with n_rows the rows of x and dks,
// dvs the widths rounded up to a multiple of 4; null: the chain form also where the chunked form would run
extern "C" int bn_lightning_scan(int dtype, const void* x, int ld, int q_col, int k_col, int v_col, const float* decay, float* o,
                                 float* state, long long state_stride, const int* tiles, int n_seqs, const int* seq_lens,
                                 const int* slot_ids, int H, int dk, int dv, int n_rows, float* prepared, hipStream_t s) {
    if (n_seqs <= 0 || H <= 0 || !bn_lightning_supports(dk, dv) || !x || !decay || !o || !state || !slot_ids) return BN_ERR_ARG;
    if ((!tiles && !seq_lens) || state_stride < (long long)H * dk * dv || q_col < 0 || k_col < 0 || v_col < 0) return BN_ERR_ARG;
    if (ld < q_col + H * dk || ld < k_col + H * dk || ld < v_col + H * dv) return BN_ERR_ARG;
    LaArgs a;
    a.x = x; a.o = o; a.decay = decay; a.state = state; a.state_stride = (size_t)state_stride; a.tiles = tiles;
    a.seq_lens = seq_lens; a.slot_ids = slot_ids; a.ld = ld; a.q_col = q_col; a.k_col = k_col; a.v_col = v_col;
    a.H = H; a.dk = dk; a.dv = dv;
    if (dtype != BN_DT_F32 && dtype != BN_DT_BF16) return BN_ERR_DTYPE;
    if (tiles && prepared && bn_lightning_chunked(dk, dv)) {
        if (n_rows <= 0 || (uintptr_t)prepared % 16 != 0) return BN_ERR_ARG;
        return lc_dispatch(dtype, a, n_seqs, n_rows, prepared, s);
    }
    const int rpt = dk <= 32 ? 8 : dk <= 64 ? 16 : dk <= 128 ? 32 : 64;
    const size_t smem = (size_t)LA_TC * (2 * rpt * LA_RG + LA_CB + LA_RG * LA_CB) * sizeof(float);
    const dim3 grid(n_seqs, H, (dv + LA_CB - 1) / LA_CB), block(LA_THREADS);
#define LA_GO(RPT_)                                                                                         \
    if (dtype == BN_DT_F32) hipLaunchKernelGGL((lightning_scan_kernel<float, RPT_>), grid, block, smem, s, a); \
    else hipLaunchKernelGGL((lightning_scan_kernel<bf16, RPT_>), grid, block, smem, s, a)
    if (rpt == 8) { LA_GO(8); }
    else if (rpt == 16) { LA_GO(16); }
    else if (rpt == 32) { LA_GO(32); }
    else { LA_GO(64); }
#undef LA_GO
    return bn_launch_status();
}

// ---- the heads' outputs normed together, the weight and the gate -------------------------------------------------------
// one workgroup a row: y = o / sqrt(mean(o^2) + eps) * weight * act(gate), act one of bn_unary_act's kinds
template <typename T>
__global__ __launch_bounds__(256) void row_norm_gate_kernel(T* __restrict__ y, const float* __restrict__ o, const T* __restrict__ gate,
                                                            int ldg, const float* __restrict__ weight, int W, float eps, int act) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const float* ov = o + (size_t)t * W;
    float ss = 0.f;
    for (int e = threadIdx.x; e < W; e += blockDim.x) ss = fmaf(ov[e], ov[e], ss);
    ss = block_sum(ss, scratch);
    const float f = 1.0f / sqrtf(ss / (float)W + eps);
    for (int e = threadIdx.x; e < W; e += blockDim.x)
        y[(size_t)t * W + e] = from_f32<T>(ov[e] * f * weight[e] * bn_unary_act(to_f32(gate[(size_t)t * ldg + e]), act));
}

extern "C" int bn_row_norm_gate(int dtype, void* y, const float* o, const void* gate, int ldg, const float* weight, int n_rows,
                                int W, float eps, int act, hipStream_t s) {
    if (n_rows <= 0 || W <= 0 || !y || !o || !gate || !weight || ldg < W || act < 0 || act >= BN_UNARY_KINDS) return BN_ERR_ARG;
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(row_norm_gate_kernel<float>, dim3(n_rows), dim3(256), 0, s, (float*)y, o, (const float*)gate, ldg, weight,
                           W, eps, act);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(row_norm_gate_kernel<bf16>, dim3(n_rows), dim3(256), 0, s, (bf16*)y, o, (const bf16*)gate, ldg, weight,
                           W, eps, act);
    else
        return BN_ERR_DTYPE;
    return bn_launch_status();
}
