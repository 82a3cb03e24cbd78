// A residual that is several streams (hyper-connections), and the norm without statistics that reads it.
//
// The residual of a model with n streams is x_1 .. x_n, each [T, D] float32.  A sublayer reads u = sum_s in[s] x_s and
// its output y rebuilds all streams at once from the old ones: x_t <- sum_s mix[s, t] x_s + mult * out[t] * y.  Both are
// sums over s at one (token, column), so one kernel does the held-back write of the sublayer before, the read for the
// sublayer after and its norm in one pass over the streams:
//
//   bn_hc_step   x' = mix^T x + mult out y   (skipped when there is no y; stored unless only a choice of rows is wanted)
//                u  = sum_s in[s] x'_s       (in null: the plain sum, which is the model's residual at its end)
//                h  = tanh(alpha u) * w + b  (w null: u itself), stored in the activations' type or float32
//
// The streams may be read with a stride of 0: a model's first sublayer reads the embedding's rows as every stream.
// y is one tensor in the activations' type or float32, or several float32 slabs that are added in slab order.
// n = 1 with in = out = mix = 1 is the plain residual x <- x + mult y.
//
//   bn_dyt_norm  x += delta (optional), h = tanh(alpha x) * w + b for all rows or a choice of rows: the norm alone, for
//                a residual of one stream that is held by other code.
// All arithmetic in float32.
#include "common.h"
#include <math.h>

#define BN_HC_MAX_STREAMS 8       // the Python side reads this line

struct HcArgs {
    const float* lanes_in;        // stream s at s * in_stride (0: all streams are the same rows)
    float* lanes_out;             // stream s at s * out_stride; null: the new streams are not stored
    const void* delta;            // y: [T, D] (or n_slabs float32 slabs slab_stride apart); null: no write is held back
    const float* mix;             // [n, n] from, to
    const float* outc;            // [n]
    const float* inc;             // [n]; null: ones
    const float* w;               // [D]; null: no norm
    const float* b;               // [D]
    const float* alpha;           // one number in device memory
    void* h;                      // [rows, D]; null: nothing is read out
    const int* rows;              // a choice of rows; null: all
    long long in_stride, out_stride, slab_stride;
    int n_rows, T, D, n, n_slabs;
    float mult;
};

// One thread a (row, column); the coefficients wait in shared memory.
template <typename TD, typename TH>
__global__ __launch_bounds__(256) void hc_step_kernel(HcArgs a) {
    __shared__ float cm[BN_HC_MAX_STREAMS * BN_HC_MAX_STREAMS], co[BN_HC_MAX_STREAMS], ci[BN_HC_MAX_STREAMS];
    const int n = a.n;
    if (threadIdx.x < n * n) cm[threadIdx.x] = a.delta ? a.mix[threadIdx.x] : 0.f;
    if (threadIdx.x < n) {
        co[threadIdx.x] = a.delta ? a.outc[threadIdx.x] : 0.f;
        ci[threadIdx.x] = a.inc ? a.inc[threadIdx.x] : 1.0f;
    }
    __syncthreads();
    const int r = blockIdx.x, d = blockIdx.y * blockDim.x + threadIdx.x;
    const int t = a.rows ? a.rows[r] : r;
    if (t < 0 || t >= a.T || d >= a.D) return;
    const TD* delta = reinterpret_cast<const TD*>(a.delta);
    TH* h = reinterpret_cast<TH*>(a.h);
    const size_t at = (size_t)t * a.D + d;
    float x[BN_HC_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < BN_HC_MAX_STREAMS; ++s) x[s] = s < n ? a.lanes_in[(size_t)s * a.in_stride + at] : 0.f;
    if (delta) {
        float y = 0.f;
        for (int p = 0; p < a.n_slabs; ++p) y += to_f32(delta[(size_t)p * a.slab_stride + at]);
        y *= a.mult;
        float nx[BN_HC_MAX_STREAMS];
#pragma unroll
        for (int to = 0; to < BN_HC_MAX_STREAMS; ++to) {
            float v = 0.f;
#pragma unroll
            for (int s = 0; s < BN_HC_MAX_STREAMS; ++s)
                if (s < n && to < n) v = fmaf(cm[s * n + to], x[s], v);
            nx[to] = to < n ? fmaf(co[to], y, v) : 0.f;
        }
#pragma unroll
        for (int s = 0; s < BN_HC_MAX_STREAMS; ++s) x[s] = nx[s];
        if (a.lanes_out) {
#pragma unroll
            for (int s = 0; s < BN_HC_MAX_STREAMS; ++s)
                if (s < n) a.lanes_out[(size_t)s * a.out_stride + at] = x[s];
        }
    } else if (a.lanes_out && a.lanes_out != a.lanes_in) {
#pragma unroll
        for (int s = 0; s < BN_HC_MAX_STREAMS; ++s)
            if (s < n) a.lanes_out[(size_t)s * a.out_stride + at] = x[s];
    }
    if (!h) return;
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < BN_HC_MAX_STREAMS; ++s)
        if (s < n) u = a.inc ? fmaf(ci[s], x[s], u) : u + x[s];
    const float v = a.w ? fmaf(tanhf(a.alpha[0] * u), a.w[d], a.b[d]) : u;
    h[(size_t)r * a.D + d] = from_f32<TH>(v);
}

// delta_dtype / h_dtype: BN_DT_F32 or BN_DT_BF16.
extern "C" int bn_hc_step(int delta_dtype, int h_dtype, const float* lanes_in, long long in_stride, float* lanes_out,
                          long long out_stride, const void* delta, int n_slabs, long long slab_stride, const float* mix,
                          const float* outc, float mult, const float* inc, const float* w, const float* b, const float* alpha,
                          void* h, const int* rows, int n_rows, int T, int D, int n, hipStream_t s) {
    if (n_rows <= 0 || T <= 0 || D <= 0 || n < 1 || n > BN_HC_MAX_STREAMS || !lanes_in) return BN_ERR_ARG;
    if (delta && (!mix || !outc || n_slabs < 1 || (delta_dtype == BN_DT_BF16 && n_slabs != 1))) return BN_ERR_ARG;
    if (w && (!b || !alpha)) return BN_ERR_ARG;
    if (!rows && n_rows != T) return BN_ERR_ARG;
    if (rows && lanes_out) return BN_ERR_ARG;              // a choice of rows stores no streams
    HcArgs a;
    a.lanes_in = lanes_in; a.lanes_out = lanes_out; a.delta = delta; a.mix = mix; a.outc = outc; a.inc = inc; a.w = w; a.b = b;
    a.alpha = alpha; a.h = h; a.rows = rows; a.in_stride = in_stride; a.out_stride = out_stride; a.slab_stride = slab_stride;
    a.n_rows = n_rows; a.T = T; a.D = D; a.n = n; a.n_slabs = delta ? n_slabs : 0; a.mult = mult;
    const int threads = D >= 256 ? 256 : 64;
    if ((D + threads - 1) / threads > 65535) return BN_ERR_ARG;
    const dim3 grid(n_rows, (D + threads - 1) / threads), block(threads);
    const bool df = delta_dtype == BN_DT_F32, hf = h_dtype == BN_DT_F32;
    if ((delta_dtype != BN_DT_F32 && delta_dtype != BN_DT_BF16) || (h_dtype != BN_DT_F32 && h_dtype != BN_DT_BF16)) return BN_ERR_DTYPE;
    if (df && hf) hipLaunchKernelGGL((hc_step_kernel<float, float>), grid, block, 0, s, a);
    else if (df) hipLaunchKernelGGL((hc_step_kernel<float, bf16>), grid, block, 0, s, a);
    else if (hf) hipLaunchKernelGGL((hc_step_kernel<bf16, float>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((hc_step_kernel<bf16, bf16>), grid, block, 0, s, a);
    return bn_launch_status();
}

// ---- the norm alone -------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void dyt_norm_kernel(float* __restrict__ x, const T* __restrict__ delta, const float* __restrict__ w,
                                                       const float* __restrict__ b, const float* __restrict__ alpha,
                                                       T* __restrict__ out, const int* __restrict__ rows, int D) {
    const int r = blockIdx.x, t = rows ? rows[r] : r;
    const float al = alpha[0];
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float v = x[(size_t)t * D + d];
        if (delta) {
            v += to_f32(delta[(size_t)t * D + d]);
            x[(size_t)t * D + d] = v;
        }
        out[(size_t)r * D + d] = from_f32<T>(fmaf(tanhf(al * v), w[d], b[d]));
    }
}

extern "C" int bn_dyt_norm(int dtype, float* x, const void* delta, const float* w, const float* b, const float* alpha, void* out,
                           const int* rows, int n_rows, int D, hipStream_t s) {
    if (n_rows <= 0 || D <= 0 || !x || !w || !b || !alpha || !out || (rows && delta)) return BN_ERR_ARG;
    const dim3 grid(n_rows), block(D >= 1024 ? 256 : 128);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(dyt_norm_kernel<float>, grid, block, 0, s, x, (const float*)delta, w, b, alpha, (float*)out, rows, D);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(dyt_norm_kernel<bf16>, grid, block, 0, s, x, (const bf16*)delta, w, b, alpha, (bf16*)out, rows, D);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}
