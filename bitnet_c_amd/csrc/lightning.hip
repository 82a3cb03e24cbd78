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

extern "C" int bn_lightning_supports(int dk, int dv) { return (dk >= 1 && dk <= LA_MAX_DIM && dv >= 1) ? 1 : 0; }

// x [T, ld] holds q at q_col, k at k_col (H dk wide each) and v at v_col (H dv wide); n_seqs: tiles, or rows of a decode step
extern "C" int bn_lightning_scan(int dtype, const void* x, int ld, int q_col, int k_col, int v_col, const float* decay, float* o,
                                 float* state, long long state_stride, const int* tiles, int n_seqs, const int* seq_lens,
                                 const int* slot_ids, int H, int dk, int dv, hipStream_t s) {
    if (n_seqs <= 0 || H <= 0 || !bn_lightning_supports(dk, dv) || !x || !decay || !o || !state || !slot_ids) return BN_ERR_ARG;
    if ((!tiles && !seq_lens) || state_stride < (long long)H * dk * dv || q_col < 0 || k_col < 0 || v_col < 0) return BN_ERR_ARG;
    if (ld < q_col + H * dk || ld < k_col + H * dk || ld < v_col + H * dv) return BN_ERR_ARG;
    LaArgs a;
    a.x = x; a.o = o; a.decay = decay; a.state = state; a.state_stride = (size_t)state_stride; a.tiles = tiles;
    a.seq_lens = seq_lens; a.slot_ids = slot_ids; a.ld = ld; a.q_col = q_col; a.k_col = k_col; a.v_col = v_col;
    a.H = H; a.dk = dk; a.dv = dv;
    const int rpt = dk <= 32 ? 8 : dk <= 64 ? 16 : dk <= 128 ? 32 : 64;
    const size_t smem = (size_t)LA_TC * (2 * rpt * LA_RG + LA_CB + LA_RG * LA_CB) * sizeof(float);
    const dim3 grid(n_seqs, H, (dv + LA_CB - 1) / LA_CB), block(LA_THREADS);
    if (dtype != BN_DT_F32 && dtype != BN_DT_BF16) return BN_ERR_DTYPE;
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
