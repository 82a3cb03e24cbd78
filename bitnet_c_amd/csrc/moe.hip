// A mixture-of-experts feed-forward.  Expert e is  W_down[e] act(W_up[e] x)  (no gate), or, in the gated form,
// W_down[e] glu(W_gate[e] x, W_up[e] x)  with the clamped unit  glu(g, u) = g' sigmoid(slope g') (u' + shift),
// g' = min(g, limit), u' = clamp(u, -limit, limit)  (gate and up rows stacked, [E, 2 F, D]).
//
//   bn_moe_route     router logits z = W_r h (+ a bias per expert) in float32 (one workgroup a token), scores sigmoid(z) or softmax(z), the top_k
//                    largest (ties: the lower index; with a choice bias the largest score + bias, the weights staying the
//                    plain scores), optionally divided by their sum (+ floor), times a constant -> expert ids and weights
//                    [T, top_k]; optionally also sigmoid(w_g . h) per token, the gate of a shared expert
//   bn_gated_unit    rows of stacked (gate | up) products -> the clamped unit, optionally times a factor per row
//   bn_moe_experts   for every (token, choice) pair: y = W_down[e] act(W_up[e] (w h)) when the weight multiplies the
//                    expert's input, w * W_down[e] act(W_up[e] h) when it multiplies the output; a pair reads its expert's
//                    two matrices once, their rows spread over workgroups.  The products accumulate in float32; the scaled
//                    input and the hidden vector are rounded to the activations' type as a product of that type would
//                    see them.
//   bn_moe_group     (bf16, steps of many rows) pairs ordered by expert, tiles of rows of one expert each, and the inputs
//                    gathered in that order, for the grouped matrix products of gemm_mfma.hip
// The outputs of a token's choices land in slab j of y [top_k, T, D] (float32) and are added by whoever consumes y.
#include "common.h"
#include <math.h>

#define MOE_MAX_EXPERTS 1024
#define MOE_PER_LANE (MOE_MAX_EXPERTS / BN_WAVE)
#define MOE_SCORE_SIGMOID 0
#define MOE_SCORE_SOFTMAX 1

struct RouteArgs {
    const void* h;            // [T, ld]
    const float* wr;          // [E, D] float32
    int* ids;                 // [T, K]
    float* wts;               // [T, K]
    int ld, D, E, K, scoring, renorm;
    const float* bias;        // [E] added to the scores for the choice alone; null: the choice goes by the scores
    const float* zbias;       // [E] added to the logits themselves (a router with a bias); null: none
    const float* gate_w;      // [D]: gate_out[t] = sigmoid(gate_w . h); null: none
    float* gate_out;          // [T]
    float floor, scale;       // weights = score / (sum of the chosen + floor) (when renorm) * scale
};

#define MOE_ROUTE_THREADS 256

// One workgroup a token: its waves take the experts in turn (a row of the router as 16-byte loads across the lanes, several
// in flight), the first wave then chooses.
template <typename T>
__global__ __launch_bounds__(MOE_ROUTE_THREADS) void moe_route_kernel(RouteArgs a) {
    extern __shared__ __align__(16) float hs[];          // the token's row as float32, then the experts' logits
    float* zs = hs + ((a.D + 3) & ~3);
    const int t = blockIdx.x, lane = threadIdx.x & (BN_WAVE - 1), wave = threadIdx.x / BN_WAVE;
    const T* h = reinterpret_cast<const T*>(a.h) + (size_t)t * a.ld;
    for (int d = threadIdx.x; d < a.D; d += MOE_ROUTE_THREADS) hs[d] = to_f32(h[d]);
    __syncthreads();
    // the shared expert's gate is one more row: it takes its turn among the waves after the experts
    for (int e = wave; e < a.E + (a.gate_w ? 1 : 0); e += MOE_ROUTE_THREADS / BN_WAVE) {
        const float* w = e < a.E ? a.wr + (size_t)e * a.D : a.gate_w;
        float s = 0.f;
        if (a.D % 4 == 0) {
#pragma unroll 4
            for (int d = 4 * lane; d < a.D; d += 4 * BN_WAVE) {
                const float4 wv = *reinterpret_cast<const float4*>(w + d), xv = *reinterpret_cast<const float4*>(hs + d);
                s = fmaf(xv.x, wv.x, s); s = fmaf(xv.y, wv.y, s); s = fmaf(xv.z, wv.z, s); s = fmaf(xv.w, wv.w, s);
            }
        } else {
            for (int d = lane; d < a.D; d += BN_WAVE) s = fmaf(hs[d], w[d], s);
        }
        s = wave_sum(s);
        if (lane == 0) {
            if (e < a.E) zs[e] = a.zbias ? s + a.zbias[e] : s;
            else a.gate_out[t] = 1.0f / (1.0f + expf(-s));
        }
    }
    __syncthreads();
    if (wave != 0) return;
    float z[MOE_PER_LANE];                               // expert lane + 64 j
#pragma unroll
    for (int j = 0; j < MOE_PER_LANE; ++j) z[j] = lane + BN_WAVE * j < a.E ? zs[lane + BN_WAVE * j] : -INFINITY;
    float zmax = -INFINITY, denom = 1.f;
    if (a.scoring == MOE_SCORE_SOFTMAX) {
#pragma unroll
        for (int j = 0; j < MOE_PER_LANE; ++j) zmax = fmaxf(zmax, z[j]);
        zmax = wave_max(zmax);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < MOE_PER_LANE; ++j) sum += z[j] == -INFINITY ? 0.f : expf(z[j] - zmax);
        denom = wave_sum(sum);
    }
    // with a choice bias the experts are ranked by score + bias: the scores of all experts are formed first and z holds
    // the ranking value from here on
    float sc[MOE_PER_LANE];
    if (a.bias) {
#pragma unroll
        for (int j = 0; j < MOE_PER_LANE; ++j) {
            const int e = lane + BN_WAVE * j;
            sc[j] = 0.f;
            if (e < a.E) {
                sc[j] = a.scoring == MOE_SCORE_SOFTMAX ? expf(z[j] - zmax) / denom : 1.0f / (1.0f + expf(-z[j]));
                z[j] = sc[j] + a.bias[e];
            }
        }
    }
    float total = 0.f, mine_w = 0.f;
    int mine_id = 0;
    for (int k = 0; k < a.K; ++k) {
        float best = -INFINITY;
        int at = MOE_MAX_EXPERTS;
#pragma unroll
        for (int j = 0; j < MOE_PER_LANE; ++j)
            if (z[j] > best) { best = z[j]; at = lane + BN_WAVE * j; }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, BN_WAVE);
            const int oa = __shfl_xor(at, o, BN_WAVE);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
        if (at >= a.E) at = k;                           // a row of NaNs (a padding row's garbage): still an expert that exists
        float own = 0.f;                                 // the chosen expert's plain score, held by the lane that owns it
#pragma unroll
        for (int j = 0; j < MOE_PER_LANE; ++j)
            if (at == lane + BN_WAVE * j) { z[j] = -INFINITY; if (a.bias) own = sc[j]; }
        const float score = a.bias ? wave_sum(own)
                          : a.scoring == MOE_SCORE_SOFTMAX ? expf(best - zmax) / denom : 1.0f / (1.0f + expf(-best));
        total += score;
        if (lane == k % BN_WAVE && k < BN_WAVE) { mine_w = score; mine_id = at; }
        if (k >= BN_WAVE && lane == 0) {                  // more choices than lanes: stored as they come
            a.ids[(size_t)t * a.K + k] = at;
            a.wts[(size_t)t * a.K + k] = score;
        }
    }
    const float norm = (a.renorm ? 1.0f / (total + a.floor) : 1.0f) * a.scale;
    if (lane < a.K) {
        a.ids[(size_t)t * a.K + lane] = mine_id;
        a.wts[(size_t)t * a.K + lane] = mine_w * norm;
    }
    if ((a.renorm || a.scale != 1.0f) && a.K > BN_WAVE && lane == 0)
        for (int k = BN_WAVE; k < a.K; ++k) a.wts[(size_t)t * a.K + k] *= norm;
}

extern "C" int bn_moe_route(int dtype, const void* h, int ld, const float* wr, int* ids, float* wts, int n_tokens, int D, int E,
                            int K, int scoring, int renorm, const float* bias, float floor, float scale, const float* gate_w,
                            float* gate_out, const float* zbias, hipStream_t s) {
    if ((gate_w == nullptr) != (gate_out == nullptr) || ((uintptr_t)gate_w & 15) || !(floor >= 0.f)) return BN_ERR_ARG;
    if (n_tokens <= 0 || D <= 0 || E <= 0 || E > MOE_MAX_EXPERTS || K <= 0 || K > E || ld < D || !h || !wr || !ids || !wts)
        return BN_ERR_ARG;
    if (scoring != MOE_SCORE_SIGMOID && scoring != MOE_SCORE_SOFTMAX) return BN_ERR_ARG;
    if ((size_t)(D + 4 + E) * sizeof(float) > 64 * 1024 || ((uintptr_t)wr & 15)) return BN_ERR_ARG;
    RouteArgs a;
    a.h = h; a.wr = wr; a.ids = ids; a.wts = wts; a.ld = ld; a.D = D; a.E = E; a.K = K; a.scoring = scoring; a.renorm = renorm ? 1 : 0;
    a.bias = bias; a.zbias = zbias; a.gate_w = gate_w; a.gate_out = gate_out; a.floor = floor; a.scale = scale;
    const size_t shm = (size_t)(((D + 3) & ~3) + E) * sizeof(float);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(moe_route_kernel<float>, dim3(n_tokens), dim3(MOE_ROUTE_THREADS), shm, s, a);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(moe_route_kernel<bf16>, dim3(n_tokens), dim3(MOE_ROUTE_THREADS), shm, s, a);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- a (token, choice) pair at a time ----------------------------------------------------------------------------------
// Steps of few rows: every pair reads its expert's two matrices once, and the rows of a matrix are spread over many
// workgroups so that one pair alone fills the chip (two launches: the hidden vector, then the output).  A workgroup stages
// the pair's input vector in shared memory as float32, each of its waves takes MOE_PAIR_ROWS / 4 rows of the matrix, a row
// as 16-byte loads across the lanes (bf16 rows of whole 8-element groups) or element by element, and sums in float32.
#define MOE_PAIR_THREADS 256
#define MOE_PAIR_ROWS 8

struct PairArgs {
    const void* h;            // [T, ld]
    const void* w_up;         // [E, F, D]
    const void* w_down;       // [E, D, F]
    const int* ids;           // [T, K]
    const float* wts;         // [T, K]
    float* hidden;            // [T K, F] float32 holding values of the activations' type
    float* y;                 // [K, T, D]
    int ld, T, D, F, K, act, weight_on_input;      // T: the rows of a slab of y
    int gated;                // w_up is [E, 2 F, D]: F gate rows, then F up rows; hidden = the clamped unit of the two
    float limit, slope, shift;
};

// the clamped gated unit: g' sigmoid(slope g') (u' + shift), g' = min(g, limit), u' = clamp(u, -limit, limit)
__device__ __forceinline__ float moe_clamped_unit(float g, float u, float limit, float slope, float shift) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.0f + expf(-slope * g)) * (u + shift);
}

// sum over n of x[i] w[i]: x in shared memory, w a row in global memory; every lane gets the sum
template <typename T>
__device__ __forceinline__ float moe_row_dot(const T* __restrict__ w, const float* __restrict__ x, int n, int lane) {
    float s = 0.f;
    for (int i = lane; i < n; i += BN_WAVE) s = fmaf(x[i], to_f32(w[i]), s);
    return wave_sum(s);
}
template <>
__device__ __forceinline__ float moe_row_dot<bf16>(const bf16* __restrict__ w, const float* __restrict__ x, int n, int lane) {
    float s = 0.f;
    if (n % 8 == 0 && ((uintptr_t)w & 15) == 0) {
#pragma unroll 4
        for (int i = 8 * lane; i < n; i += 8 * BN_WAVE) {
            const uint4 p = *reinterpret_cast<const uint4*>(w + i);
            const float4 a = *reinterpret_cast<const float4*>(x + i), b = *reinterpret_cast<const float4*>(x + i + 4);
            s = fmaf(a.x, bf16lo_to_f32(p.x), s); s = fmaf(a.y, bf16hi_to_f32(p.x), s);
            s = fmaf(a.z, bf16lo_to_f32(p.y), s); s = fmaf(a.w, bf16hi_to_f32(p.y), s);
            s = fmaf(b.x, bf16lo_to_f32(p.z), s); s = fmaf(b.y, bf16hi_to_f32(p.z), s);
            s = fmaf(b.z, bf16lo_to_f32(p.w), s); s = fmaf(b.w, bf16hi_to_f32(p.w), s);
        }
    } else {
        for (int i = lane; i < n; i += BN_WAVE) s = fmaf(x[i], to_f32(w[i]), s);
    }
    return wave_sum(s);
}

// hidden[pair][f] = act(W_up[e][f] . (w h[t])) for the workgroup's rows f
template <typename T>
__global__ __launch_bounds__(MOE_PAIR_THREADS) void moe_pair_up_kernel(PairArgs a) {
    extern __shared__ __align__(16) float xs[];          // [D]
    const int pair = blockIdx.y, t = pair / a.K;
    const int lane = threadIdx.x & (BN_WAVE - 1), wave = threadIdx.x / BN_WAVE;
    const int e = a.ids[pair];
    const float in_scale = a.weight_on_input ? a.wts[pair] : 1.0f;
    const T* h = reinterpret_cast<const T*>(a.h) + (size_t)t * a.ld;
    for (int d = threadIdx.x; d < a.D; d += MOE_PAIR_THREADS) xs[d] = to_f32(from_f32<T>(to_f32(h[d]) * in_scale));
    __syncthreads();
    const T* wu = reinterpret_cast<const T*>(a.w_up) + (size_t)e * (a.gated ? 2 : 1) * a.F * a.D;
    const int f0 = blockIdx.x * MOE_PAIR_ROWS;
    if (a.gated) {
        // a gate row and its up row one after the other, both rows' loads in flight; the products are rounded to the
        // activations' type, as the rows of a stacked product of that type are, before they meet in the unit
        float g[MOE_PAIR_ROWS / (MOE_PAIR_THREADS / BN_WAVE)], u[MOE_PAIR_ROWS / (MOE_PAIR_THREADS / BN_WAVE)];
#pragma unroll
        for (int k = 0; k < MOE_PAIR_ROWS / (MOE_PAIR_THREADS / BN_WAVE); ++k) {
            const int f = f0 + wave + k * (MOE_PAIR_THREADS / BN_WAVE);
            g[k] = f < a.F ? moe_row_dot<T>(wu + (size_t)f * a.D, xs, a.D, lane) : 0.f;
            u[k] = f < a.F ? moe_row_dot<T>(wu + (size_t)(a.F + f) * a.D, xs, a.D, lane) : 0.f;
        }
#pragma unroll
        for (int k = 0; k < MOE_PAIR_ROWS / (MOE_PAIR_THREADS / BN_WAVE); ++k) {
            const int f = f0 + wave + k * (MOE_PAIR_THREADS / BN_WAVE);
            if (f < a.F && lane == 0)
                a.hidden[(size_t)pair * a.F + f] = to_f32(from_f32<T>(moe_clamped_unit(
                    to_f32(from_f32<T>(g[k])), to_f32(from_f32<T>(u[k])), a.limit, a.slope, a.shift)));
        }
        return;
    }
    // a wave's two rows (MOE_PAIR_ROWS / 4) one after the other without a dependence between them: both rows' loads are
    // in flight before the first sum is needed
    float sums[MOE_PAIR_ROWS / (MOE_PAIR_THREADS / BN_WAVE)];
#pragma unroll
    for (int k = 0; k < MOE_PAIR_ROWS / (MOE_PAIR_THREADS / BN_WAVE); ++k) {
        const int f = f0 + wave + k * (MOE_PAIR_THREADS / BN_WAVE);
        sums[k] = f < a.F ? moe_row_dot<T>(wu + (size_t)f * a.D, xs, a.D, lane) : 0.f;
    }
#pragma unroll
    for (int k = 0; k < MOE_PAIR_ROWS / (MOE_PAIR_THREADS / BN_WAVE); ++k) {
        const int f = f0 + wave + k * (MOE_PAIR_THREADS / BN_WAVE);
        if (f < a.F && lane == 0) a.hidden[(size_t)pair * a.F + f] = to_f32(from_f32<T>(bn_unary_act(sums[k], a.act)));
    }
}

// y[j][t][d] = W_down[e][d] . hidden[pair] (times w when the weight multiplies the output) for the workgroup's rows d
template <typename T>
__global__ __launch_bounds__(MOE_PAIR_THREADS) void moe_pair_down_kernel(PairArgs a) {
    extern __shared__ __align__(16) float hid[];         // [F]
    const int pair = blockIdx.y, t = pair / a.K, j = pair - t * a.K;
    const int lane = threadIdx.x & (BN_WAVE - 1), wave = threadIdx.x / BN_WAVE;
    const int e = a.ids[pair];
    const float out_scale = a.weight_on_input ? 1.0f : a.wts[pair];
    for (int f = threadIdx.x; f < a.F; f += MOE_PAIR_THREADS) hid[f] = a.hidden[(size_t)pair * a.F + f];
    __syncthreads();
    const T* wd = reinterpret_cast<const T*>(a.w_down) + (size_t)e * a.D * a.F;
    float* y = a.y + ((size_t)j * a.T + t) * a.D;
    const int d0 = blockIdx.x * MOE_PAIR_ROWS;
    float sums[MOE_PAIR_ROWS / (MOE_PAIR_THREADS / BN_WAVE)];
#pragma unroll
    for (int k = 0; k < MOE_PAIR_ROWS / (MOE_PAIR_THREADS / BN_WAVE); ++k) {
        const int d = d0 + wave + k * (MOE_PAIR_THREADS / BN_WAVE);
        sums[k] = d < a.D ? moe_row_dot<T>(wd + (size_t)d * a.F, hid, a.F, lane) : 0.f;
    }
#pragma unroll
    for (int k = 0; k < MOE_PAIR_ROWS / (MOE_PAIR_THREADS / BN_WAVE); ++k) {
        const int d = d0 + wave + k * (MOE_PAIR_THREADS / BN_WAVE);
        if (d < a.D && lane == 0) y[d] = sums[k] * out_scale;
    }
}

// hidden: float32 work space [n_tokens K, F]; y_rows: the rows of a slab of y (>= n_tokens: the call may take a run of a
// step's tokens, y then points at the run's first row of slab 0)
extern "C" int bn_moe_experts(int dtype, const void* h, int ld, const void* w_up, const void* w_down, const int* ids,
                              const float* wts, float* y, float* hidden, int n_tokens, int y_rows, int D, int F, int K, int act,
                              int weight_on_input, int gated, float limit, float slope, float shift, hipStream_t s) {
    if (n_tokens <= 0 || y_rows < n_tokens || D <= 0 || F <= 0 || K <= 0 || ld < D) return BN_ERR_ARG;
    if (gated ? !(limit > 0.f) : (act < 0 || act >= BN_UNARY_KINDS)) return BN_ERR_ARG;
    if (!h || !w_up || !w_down || !ids || !wts || !y || !hidden) return BN_ERR_ARG;
    if ((size_t)D * sizeof(float) > 64 * 1024 || (size_t)F * sizeof(float) > 64 * 1024 || (size_t)n_tokens * K > 65535) return BN_ERR_ARG;
    PairArgs a;
    a.h = h; a.w_up = w_up; a.w_down = w_down; a.ids = ids; a.wts = wts; a.y = y; a.hidden = hidden;
    a.ld = ld; a.T = y_rows; a.D = D; a.F = F; a.K = K; a.act = act; a.weight_on_input = weight_on_input ? 1 : 0;
    a.gated = gated ? 1 : 0; a.limit = limit; a.slope = slope; a.shift = shift;
    const dim3 block(MOE_PAIR_THREADS);
    const dim3 up((F + MOE_PAIR_ROWS - 1) / MOE_PAIR_ROWS, n_tokens * K), down((D + MOE_PAIR_ROWS - 1) / MOE_PAIR_ROWS, n_tokens * K);
    if (dtype == BN_DT_F32) {
        hipLaunchKernelGGL(moe_pair_up_kernel<float>, up, block, (size_t)D * sizeof(float), s, a);
        hipLaunchKernelGGL(moe_pair_down_kernel<float>, down, block, (size_t)F * sizeof(float), s, a);
    } else if (dtype == BN_DT_BF16) {
        hipLaunchKernelGGL(moe_pair_up_kernel<bf16>, up, block, (size_t)D * sizeof(float), s, a);
        hipLaunchKernelGGL(moe_pair_down_kernel<bf16>, down, block, (size_t)F * sizeof(float), s, a);
    } else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- steps of many rows: pairs ordered by expert (bf16) ---------------------------------------------------------------
// The pairs of a step are ordered by expert and cut into tiles of up to tile_rows rows of one expert; the inputs are
// gathered in that order (scaled by the pair's weight and rounded, when the weight multiplies the input), and the two
// products run as grouped matrix products over the tiles (gemm_mfma.hip).  Everything a tile needs to know lies in device
// memory, so the launches do not depend on the routing.
#define MOE_PLAN_THREADS 1024

// order [T K]: the pairs (t K + j) by expert; tiles [max_tiles][3] = expert, first place in `order`, rows; n_tiles [1]
__global__ __launch_bounds__(MOE_PLAN_THREADS) void moe_plan_kernel(const int* __restrict__ ids, int n_pairs, int E, int tile_rows,
                                                                    int* __restrict__ order, int* __restrict__ tiles,
                                                                    int* __restrict__ n_tiles) {
    __shared__ int count[MOE_MAX_EXPERTS], first[MOE_MAX_EXPERTS + 1], tile0[MOE_MAX_EXPERTS + 1];
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) atomicAdd(&count[ids[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, tl = 0;
        for (int e = 0; e < E; ++e) {
            first[e] = at; tile0[e] = tl;
            at += count[e];
            tl += (count[e] + tile_rows - 1) / tile_rows;
        }
        first[E] = at; tile0[E] = tl;
        n_tiles[0] = tl;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        const int n = count[e];
        for (int r = 0, k = tile0[e]; r < n; r += tile_rows, ++k) {
            tiles[3 * k] = e; tiles[3 * k + 1] = first[e] + r; tiles[3 * k + 2] = min(tile_rows, n - r);
        }
        count[e] = 0;                                    // now the cursor of the scatter
    }
    __syncthreads();
    // the places inside an expert's run are handed out in whatever order the lanes arrive: a row's result does not depend
    // on its place
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int e = ids[p];
        order[first[e] + atomicAdd(&count[e], 1)] = p;
    }
}

// xg[place] = h[token of the pair at that place] (times the pair's weight, rounded to bf16, when scale_input); row_map[place]
// = the pair's row of y seen as [K T, D]; row_scale[place] = the pair's weight.  One workgroup a place, 16 bytes a thread.
__global__ __launch_bounds__(256) void moe_gather_kernel(const bf16* __restrict__ h, int ld, const int* __restrict__ order,
                                                         const float* __restrict__ wts, bf16* __restrict__ xg,
                                                         int* __restrict__ row_map, float* __restrict__ row_scale, int T, int D,
                                                         int K, int scale_input) {
    const int place = blockIdx.x, pair = order[place], t = pair / K, j = pair - t * K;
    const float w = wts[pair];
    if (threadIdx.x == 0) { row_map[place] = j * T + t; row_scale[place] = w; }
    const bf16* src = h + (size_t)t * ld;
    bf16* dst = xg + (size_t)place * D;
    for (int d = 8 * threadIdx.x; d < D; d += 8 * 256) {
        uint4 p = *reinterpret_cast<const uint4*>(src + d);
        if (scale_input) {
            uint32_t* q = reinterpret_cast<uint32_t*>(&p);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const bf16 lo = __float2bfloat16(bf16lo_to_f32(q[k]) * w), hi = __float2bfloat16(bf16hi_to_f32(q[k]) * w);
                q[k] = (uint32_t)__builtin_bit_cast(unsigned short, lo) | ((uint32_t)__builtin_bit_cast(unsigned short, hi) << 16);
            }
        }
        *reinterpret_cast<uint4*>(dst + d) = p;
    }
}

extern "C" int bn_moe_grouped_tiles(int n_pairs, int E, int tile_rows) {
    return tile_rows > 0 ? (n_pairs + tile_rows - 1) / tile_rows + E : 0;
}

// work: int32 [2 n_pairs + 3 max_tiles + 1] = order, row_map, tiles, n_tiles; row_scale: float32 [n_pairs]; xg: bf16 [n_pairs, D]
extern "C" int bn_moe_group(const void* h, int ld, const int* ids, const float* wts, int* work, float* row_scale, void* xg,
                            int n_tokens, int D, int E, int K, int tile_rows, int scale_input, hipStream_t s) {
    if (n_tokens <= 0 || K <= 0 || E <= 0 || E > MOE_MAX_EXPERTS || D <= 0 || D % 8 || ld < D || ld % 8 || tile_rows <= 0) return BN_ERR_ARG;
    if (!h || !ids || !wts || !work || !row_scale || !xg || (((uintptr_t)h | (uintptr_t)xg) & 15)) return BN_ERR_ARG;
    const int n_pairs = n_tokens * K, max_tiles = bn_moe_grouped_tiles(n_pairs, E, tile_rows);
    int* order = work;
    int* row_map = work + n_pairs;
    int* tiles = row_map + n_pairs;
    int* n_tiles = tiles + 3 * max_tiles;
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(MOE_PLAN_THREADS), 0, s, ids, n_pairs, E, tile_rows, order, tiles, n_tiles);
    hipLaunchKernelGGL(moe_gather_kernel, dim3(n_pairs), dim3(256), 0, s, (const bf16*)h, ld, order, wts, (bf16*)xg, row_map,
                       row_scale, n_tokens, D, K, scale_input ? 1 : 0);
    return bn_launch_status();
}

// ---- the clamped gated unit over rows of stacked products ------------------------------------------------------------
// out[r, f] = unit(gu[r, f], gu[r, F + f]) (times row_scale[r]), rounded once to the activations' type: what follows a
// product with stacked gate and up rows, for the grouped experts and for a shared expert (whose factor is its gate)
template <typename T>
__global__ void gated_unit_kernel(T* __restrict__ out, const T* __restrict__ gu, int ld, const float* __restrict__ row_scale,
                                  int n_rows, int F, float limit, float slope, float shift) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)n_rows * F) return;
    const int r = (int)(i / F), f = (int)(i - (size_t)r * F);
    const T* row = gu + (size_t)r * ld;
    float v = moe_clamped_unit(to_f32(row[f]), to_f32(row[F + f]), limit, slope, shift);
    if (row_scale) v *= row_scale[r];
    out[i] = from_f32<T>(v);
}

extern "C" int bn_gated_unit(int dtype, void* out, const void* gu, int ld, const float* row_scale, int n_rows, int F, float limit,
                             float slope, float shift, hipStream_t s) {
    if (n_rows <= 0 || F <= 0 || ld < 2 * F || !out || !gu || !(limit > 0.f)) return BN_ERR_ARG;
    const size_t n = (size_t)n_rows * F;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(gated_unit_kernel<float>, grid, block, 0, s, (float*)out, (const float*)gu, ld, row_scale, n_rows, F, limit, slope, shift);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(gated_unit_kernel<bf16>, grid, block, 0, s, (bf16*)out, (const bf16*)gu, ld, row_scale, n_rows, F, limit, slope, shift);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}
