// Kernels of the latent attention mixer: keys and values are both projections of one normed vector c per token (the
// latent), which is all that the cache keeps.  Because k_h = U_h c and v_h = V_h c are linear in c, the mixer attends in
// the latent's space: the query of head h becomes q'_h = U_h^T q_h, all heads share the one cached vector as key and as
// value (score = q'_h . c, o'_h = sum_j p_j c_j), and the value projection runs once on the result, o_h = V_h o'_h.
//
//   bn_latent_store   c = x / sqrt(mean(x^2) + eps) * w over the latent's columns of a projected row -> the page of the
//                     row's position, once as a key row and once into the transposed value page
//   bn_head_linear    y[t, h, :] = x[t, h, :] . M_h for every head (M_h [in, out]), optionally times sigmoid(gate[t, h, :])
//   bn_sigmoid_gate   y *= sigmoid(gate), element by element
// All arithmetic in float32; results are stored once in the activations' type.
#include "common.h"
#include <math.h>

struct LatentStoreArgs {
    const void* x;            // [T, ld]; the latent's columns start at column `col`, the rotated key part follows them
    const int* positions;     // [T]; < 0: a padding row, nothing is written
    const int* seq_index;     // [T] row of the block table
    const int* block_table;   // [n_seqs, bt_stride]
    void* k_pages;            // [pages, 1, BN_PAGE, rank + rot]: the latent, then the rotated part
    void* v_pages;            // [pages, 1, rank, BN_PAGE]
    const float* w;           // [rank]
    const float* inv_freq;    // [rot / 2] or null (rot 0)
    int ld, col, rank, bt_stride, rot;
    float eps, rot_mult;      // rot_mult multiplies every cosine and sine
};

template <typename T>
__global__ __launch_bounds__(256) void latent_store_kernel(LatentStoreArgs a) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const int pos = a.positions[t];
    if (pos < 0) return;
    const T* x = reinterpret_cast<const T*>(a.x) + (size_t)t * a.ld + a.col;
    float ss = 0.f;
    for (int d = threadIdx.x; d < a.rank; d += blockDim.x) { const float v = to_f32(x[d]); ss = fmaf(v, v, ss); }
    ss = block_sum(ss, scratch);
    const float f = 1.0f / sqrtf(ss / (float)a.rank + a.eps);
    const int page = a.block_table[(size_t)a.seq_index[t] * a.bt_stride + pos / BN_PAGE], slot = pos % BN_PAGE;
    T* kd = reinterpret_cast<T*>(a.k_pages) + ((size_t)page * BN_PAGE + slot) * (a.rank + a.rot);
    T* vd = reinterpret_cast<T*>(a.v_pages) + (size_t)page * a.rank * BN_PAGE + slot;
    for (int d = threadIdx.x; d < a.rank; d += blockDim.x) {
        const T c = from_f32<T>(to_f32(x[d]) * f * a.w[d]);
        kd[d] = c;
        vd[(size_t)d * BN_PAGE] = c;
    }
    // the key part that all heads share: not normed, dimension i turned with dimension i + rot / 2 by pos * f_i
    const int half = a.rot / 2;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float sn, cs;
        sincosf((float)pos * a.inv_freq[i], &sn, &cs);
        sn *= a.rot_mult; cs *= a.rot_mult;
        const float u = to_f32(x[a.rank + i]), v = to_f32(x[a.rank + half + i]);
        kd[a.rank + i] = from_f32<T>(u * cs - v * sn);
        kd[a.rank + half + i] = from_f32<T>(v * cs + u * sn);
    }
}

extern "C" int bn_latent_store(int dtype, const void* x, int ld, int col, const int* positions, const int* seq_index,
                               const int* block_table, int bt_stride, void* k_pages, void* v_pages, const float* w, int n_tokens,
                               int rank, float eps, int rot, const float* inv_freq, float rot_mult, hipStream_t s) {
    if (n_tokens <= 0 || rank <= 0 || col < 0 || rot < 0 || rot % 2 || ld < col + rank + rot || (rot > 0 && !inv_freq)) return BN_ERR_ARG;
    if (!x || !positions || !seq_index || !block_table || !k_pages || !v_pages || !w) return BN_ERR_ARG;
    LatentStoreArgs a;
    a.x = x; a.positions = positions; a.seq_index = seq_index; a.block_table = block_table; a.k_pages = k_pages;
    a.v_pages = v_pages; a.w = w; a.ld = ld; a.col = col; a.rank = rank; a.bt_stride = bt_stride; a.eps = eps;
    a.rot = rot; a.inv_freq = inv_freq; a.rot_mult = rot_mult;
    const dim3 grid(n_tokens), block(rank > 128 ? 256 : 64);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(latent_store_kernel<float>, grid, block, 0, s, a);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(latent_store_kernel<bf16>, grid, block, 0, s, a);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- a product per head ---------------------------------------------------------------------------------------------
#define HL_ROWS 8             // rows of x that a workgroup takes
#define HL_COLS 64            // output columns of a workgroup
#define HL_SLICES 4           // parts of the input dimension, a wave each; their sums meet in shared memory

struct HeadLinearArgs {
    const void* x;            // [T, ldx]: head h at h * I
    const void* w;            // [H, I, O]
    void* y;                  // [T, ldy]: head h at h * O
    const void* gate;         // [T, ldg]: the gate of output column n is entry n / gate_group (1: one a column; O: one a head); null: none
    int ldx, ldy, ldg, T, H, I, O, gate_group;
};

// The rows of x are staged in shared memory as float32 and read by every lane of a wave at the same address; a lane owns
// an output column and walks its wave's part of the input dimension with one coalesced load of the weights a step, eight
// steps' loads in flight.
template <typename T>
__global__ __launch_bounds__(HL_COLS * HL_SLICES) void head_linear_kernel(HeadLinearArgs a) {
    extern __shared__ float xs[];                        // [HL_ROWS][I], then the slices' sums [HL_SLICES][HL_ROWS][HL_COLS]
    float* red = xs + HL_ROWS * a.I;
    const int h = blockIdx.y, t0 = blockIdx.z * HL_ROWS, c = threadIdx.x & (HL_COLS - 1), slice = threadIdx.x / HL_COLS;
    const int o = blockIdx.x * HL_COLS + c;
    const int rows = min(HL_ROWS, a.T - t0);
    const T* x = reinterpret_cast<const T*>(a.x);
    for (int idx = threadIdx.x; idx < HL_ROWS * a.I; idx += HL_COLS * HL_SLICES) {
        const int r = idx / a.I, i = idx - r * a.I;
        xs[idx] = r < rows ? to_f32(x[(size_t)(t0 + r) * a.ldx + (size_t)h * a.I + i]) : 0.f;
    }
    __syncthreads();
    float acc[HL_ROWS];
#pragma unroll
    for (int r = 0; r < HL_ROWS; ++r) acc[r] = 0.f;
    const int per = (a.I + HL_SLICES - 1) / HL_SLICES, i0 = slice * per, i1 = min(a.I, i0 + per);
    if (o < a.O) {
        const T* w = reinterpret_cast<const T*>(a.w) + (size_t)h * a.I * a.O + o;
#pragma unroll 8
        for (int i = i0; i < i1; ++i) {
            const float wv = to_f32(w[(size_t)i * a.O]);
#pragma unroll
            for (int r = 0; r < HL_ROWS; ++r) acc[r] = fmaf(xs[r * a.I + i], wv, acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < HL_ROWS; ++r) red[(slice * HL_ROWS + r) * HL_COLS + c] = acc[r];
    __syncthreads();
    if (slice != 0 || o >= a.O) return;
    T* y = reinterpret_cast<T*>(a.y);
    const T* g = reinterpret_cast<const T*>(a.gate);
#pragma unroll
    for (int r = 0; r < HL_ROWS; ++r) {
        if (r >= rows) break;
        float v = 0.f;
#pragma unroll
        for (int k = 0; k < HL_SLICES; ++k) v += red[(k * HL_ROWS + r) * HL_COLS + c];
        if (g) v *= 1.0f / (1.0f + expf(-to_f32(g[(size_t)(t0 + r) * a.ldg + ((size_t)h * a.O + o) / a.gate_group])));
        y[(size_t)(t0 + r) * a.ldy + (size_t)h * a.O + o] = from_f32<T>(v);
    }
}

// The same product with 16-byte loads of the weights: a lane owns HLW_VEC consecutive output columns (8 bf16 or 4 float32),
// O / HLW_VEC lanes cover a row of the head's matrix, and the 256 / (O / HLW_VEC) groups of lanes take the input dimension
// in turn; their sums meet in shared memory.  One workgroup a (head, four rows of x): at one row a head's matrix is read
// with sixteen loads a lane instead of one load an input row.
#define HLW_ROWS 4
#define HLW_THREADS 256

template <typename T> struct HlwVec;
template <> struct HlwVec<bf16> {
    static constexpr int N = 8;
    static __device__ __forceinline__ void load(const bf16* p, float (&v)[8]) {
        const uint4 w = *reinterpret_cast<const uint4*>(p);
        v[0] = bf16lo_to_f32(w.x); v[1] = bf16hi_to_f32(w.x); v[2] = bf16lo_to_f32(w.y); v[3] = bf16hi_to_f32(w.y);
        v[4] = bf16lo_to_f32(w.z); v[5] = bf16hi_to_f32(w.z); v[6] = bf16lo_to_f32(w.w); v[7] = bf16hi_to_f32(w.w);
    }
};
template <> struct HlwVec<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const float4 w = *reinterpret_cast<const float4*>(p);
        v[0] = w.x; v[1] = w.y; v[2] = w.z; v[3] = w.w;
    }
};

template <typename T>
__global__ __launch_bounds__(HLW_THREADS) void head_linear_wide_kernel(HeadLinearArgs a) {
    constexpr int V = HlwVec<T>::N;
    extern __shared__ float xs[];                        // [HLW_ROWS][I], then the groups' sums [groups][HLW_ROWS][O]
    float* red = xs + HLW_ROWS * a.I;
    const int h = blockIdx.x, t0 = blockIdx.y * HLW_ROWS;
    const int lanes = a.O / V, groups = HLW_THREADS / lanes;         // lanes <= 256
    const int grp = threadIdx.x / lanes, cg = threadIdx.x - grp * lanes;
    const int rows = min(HLW_ROWS, a.T - t0);
    const T* x = reinterpret_cast<const T*>(a.x);
    for (int idx = threadIdx.x; idx < HLW_ROWS * a.I; idx += HLW_THREADS) {
        const int r = idx / a.I, i = idx - r * a.I;
        xs[idx] = r < rows ? to_f32(x[(size_t)(t0 + r) * a.ldx + (size_t)h * a.I + i]) : 0.f;
    }
    __syncthreads();
    float acc[HLW_ROWS][V];
#pragma unroll
    for (int r = 0; r < HLW_ROWS; ++r)
#pragma unroll
        for (int k = 0; k < V; ++k) acc[r][k] = 0.f;
    if (grp < groups) {
        const T* w = reinterpret_cast<const T*>(a.w) + (size_t)h * a.I * a.O + (size_t)cg * V;
#pragma unroll 4
        for (int i = grp; i < a.I; i += groups) {
            float wv[V];
            HlwVec<T>::load(w + (size_t)i * a.O, wv);
#pragma unroll
            for (int r = 0; r < HLW_ROWS; ++r) {
                const float xv = xs[r * a.I + i];
#pragma unroll
                for (int k = 0; k < V; ++k) acc[r][k] = fmaf(xv, wv[k], acc[r][k]);
            }
        }
#pragma unroll
        for (int r = 0; r < HLW_ROWS; ++r)
#pragma unroll
            for (int k = 0; k < V; ++k) red[((size_t)grp * HLW_ROWS + r) * a.O + cg * V + k] = acc[r][k];
    }
    __syncthreads();
    T* y = reinterpret_cast<T*>(a.y);
    const T* g = reinterpret_cast<const T*>(a.gate);
    for (int idx = threadIdx.x; idx < rows * a.O; idx += HLW_THREADS) {
        const int r = idx / a.O, o = idx - r * a.O;
        float v = 0.f;
        for (int k = 0; k < groups; ++k) v += red[((size_t)k * HLW_ROWS + r) * a.O + o];
        if (g) v *= 1.0f / (1.0f + expf(-to_f32(g[(size_t)(t0 + r) * a.ldg + ((size_t)h * a.O + o) / a.gate_group])));
        y[(size_t)(t0 + r) * a.ldy + (size_t)h * a.O + o] = from_f32<T>(v);
    }
}

template <typename T>
static bool hlw_takes(const void* w, int I, int O) {
    constexpr int V = HlwVec<T>::N;
    if (O % V || O / V > HLW_THREADS || ((uintptr_t)w & 15)) return false;
    const int groups = HLW_THREADS / (O / V);
    return (size_t)HLW_ROWS * ((size_t)I + (size_t)groups * O) * sizeof(float) <= 64 * 1024;
}

extern "C" int bn_head_linear(int dtype, const void* x, int ldx, const void* w, void* y, int ldy, const void* gate, int ldg,
                              int gate_group, int n_rows, int H, int I, int O, hipStream_t s) {
    if (n_rows <= 0 || H <= 0 || I <= 0 || O <= 0 || !x || !w || !y) return BN_ERR_ARG;
    if (gate && (gate_group < 1 || (H * O) % gate_group)) return BN_ERR_ARG;
    if (ldx < H * I || ldy < H * O || (gate && ldg < H * O / gate_group) || (size_t)HL_ROWS * (I + HL_SLICES * HL_COLS) * sizeof(float) > 64 * 1024 || H > 65535) return BN_ERR_ARG;
    const int row_tiles = (n_rows + HL_ROWS - 1) / HL_ROWS;
    if (row_tiles > 65535) return BN_ERR_ARG;
    HeadLinearArgs a;
    a.x = x; a.w = w; a.y = y; a.gate = gate; a.ldx = ldx; a.ldy = ldy; a.ldg = ldg; a.T = n_rows; a.H = H; a.I = I; a.O = O; a.gate_group = gate ? gate_group : 1;
    if (dtype != BN_DT_F32 && dtype != BN_DT_BF16) return BN_ERR_DTYPE;
    const bool wide = dtype == BN_DT_F32 ? hlw_takes<float>(w, I, O) : hlw_takes<bf16>(w, I, O);
    if (wide && (n_rows + HLW_ROWS - 1) / HLW_ROWS <= 65535) {
        const int vec = dtype == BN_DT_F32 ? 4 : 8, groups = HLW_THREADS / (O / vec);
        const dim3 wgrid(H, (n_rows + HLW_ROWS - 1) / HLW_ROWS);
        const size_t wshm = (size_t)HLW_ROWS * ((size_t)I + (size_t)groups * O) * sizeof(float);
        if (dtype == BN_DT_F32) hipLaunchKernelGGL(head_linear_wide_kernel<float>, wgrid, dim3(HLW_THREADS), wshm, s, a);
        else hipLaunchKernelGGL(head_linear_wide_kernel<bf16>, wgrid, dim3(HLW_THREADS), wshm, s, a);
        return bn_launch_status();
    }
    const dim3 grid((O + HL_COLS - 1) / HL_COLS, H, row_tiles), block(HL_COLS * HL_SLICES);
    const size_t shm = (size_t)HL_ROWS * (I + HL_SLICES * HL_COLS) * sizeof(float);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(head_linear_kernel<float>, grid, block, shm, s, a);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(head_linear_kernel<bf16>, grid, block, shm, s, a);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- y *= sigmoid(gate) ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ y, int ldy, const T* __restrict__ g, int ldg, int n_rows, int n_cols, int group) {
    const size_t n = (size_t)n_rows * n_cols;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) {
        const size_t r = idx / n_cols, c = idx - r * n_cols;
        const float v = to_f32(y[r * ldy + c]) / (1.0f + expf(-to_f32(g[r * ldg + c / group])));
        y[r * ldy + c] = from_f32<T>(v);
    }
}

extern "C" int bn_sigmoid_gate(int dtype, void* y, int ldy, const void* gate, int ldg, int group, int n_rows, int n_cols, hipStream_t s) {
    if (n_rows <= 0 || n_cols <= 0 || group < 1 || n_cols % group || ldy < n_cols || ldg < n_cols / group || !y || !gate) return BN_ERR_ARG;
    const size_t n = (size_t)n_rows * n_cols;
    const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(sigmoid_gate_kernel<float>, dim3(blocks), dim3(256), 0, s, (float*)y, ldy, (const float*)gate, ldg, n_rows, n_cols, group);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(sigmoid_gate_kernel<bf16>, dim3(blocks), dim3(256), 0, s, (bf16*)y, ldy, (const bf16*)gate, ldg, n_rows, n_cols, group);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- a rotation of part of every head, in place ------------------------------------------------------------------------
// x[t, h * head_stride + off + i] is turned with x[t, h * head_stride + off + i + rot / 2] by the angle pos_t * f_i; both
// cosine and sine times `mult`.  Rows with position < 0 are left alone.  Angles, cosines and sines in float32.
template <typename T>
__global__ void rope_heads_kernel(T* __restrict__ x, int ld, const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                  int n_rows, int H, int head_stride, int off, int rot, float mult) {
    const int half = rot / 2;
    const size_t n = (size_t)n_rows * H * half;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) {
        const int i = (int)(idx % half);
        const size_t th = idx / half;
        const int h = (int)(th % H);
        const size_t t = th / H;
        const int pos = positions[t];
        if (pos < 0) continue;
        float sn, cs;
        sincosf((float)pos * inv_freq[i], &sn, &cs);
        sn *= mult; cs *= mult;
        T* p = x + t * ld + (size_t)h * head_stride + off;
        const float u = to_f32(p[i]), v = to_f32(p[half + i]);
        p[i] = from_f32<T>(u * cs - v * sn);
        p[half + i] = from_f32<T>(v * cs + u * sn);
    }
}

extern "C" int bn_rope_heads(int dtype, void* x, int ld, const int* positions, const float* inv_freq, int n_rows, int H,
                             int head_stride, int off, int rot, float mult, hipStream_t s) {
    if (n_rows <= 0 || H <= 0 || rot <= 0 || rot % 2 || off < 0 || head_stride < off + rot || ld < (H - 1) * head_stride + off + rot
        || !x || !positions || !inv_freq) return BN_ERR_ARG;
    const size_t n = (size_t)n_rows * H * (rot / 2);
    const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(rope_heads_kernel<float>, dim3(blocks), dim3(256), 0, s, (float*)x, ld, positions, inv_freq, n_rows, H, head_stride, off, rot, mult);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(rope_heads_kernel<bf16>, dim3(blocks), dim3(256), 0, s, (bf16*)x, ld, positions, inv_freq, n_rows, H, head_stride, off, rot, mult);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}
