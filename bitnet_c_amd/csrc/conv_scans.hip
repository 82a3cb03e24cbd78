// Short causal convolutions over time and two recurrences with a float32 state per sequence.
//
//   bn_short_conv   y_t = sum_j w[:, j] u_(t - taps + 1 + j) (+ bias) on every channel of a projection, zeros before a
//                   sequence's first token.  The last taps - 1 inputs of a sequence are part of its state: a step's
//                   first tokens read them from there, and the step leaves its own last inputs behind.
//   bn_lru_gates    the gates of a real-gated linear recurrent unit: the input in `blocks` equal parts, in part b
//                   r = sigmoid(Wa[b] u_b + ba), i = sigmoid(Wi[b] u_b + bi); a = exp(c r) with c = -8 softplus(lam) per
//                   channel; the unit's two operands a and sqrt(1 - a^2) i u leave as float32 rows
//   bn_lru_scan     S <- a S + b per channel, the result times gelu_tanh of the other branch
//   bn_gla_scan     gated linear attention: per head S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t with a decay per key
//                   channel and token, alpha = sigmoid(z)^(1 / tau); token by token, the tokens staged two runs deep
//
// Everything that enters a recurrence is float32: gates, decays and their logarithms, exponentials, the state.  Every
// chain is the same operations in the same order whatever else a step holds, so a sequence's values do not depend on
// how its tokens were cut into steps or on the batch.
#include "common.h"
#include <math.h>

#define BN_CONV_MAX_TAPS 16       // the Python side reads this line
#define GLA_MAX_DIM 256           // key channels of a head (the Python side reads this line)
#define GLA_COLS 16               // value columns of a wave
#define GLA_SLICES 4              // parts of the key channels, 16 lanes each

struct SeqRange { int seq, row0, n, pos0; };

__device__ __forceinline__ SeqRange seq_range(const int* tiles, const int* seq_lens, int idx) {
    SeqRange r;
    if (tiles) {
        const int* t = tiles + 4 * idx;
        r.seq = t[0]; r.row0 = t[1]; r.n = t[2]; r.pos0 = t[3];
    } else {
        r.seq = idx; r.row0 = idx; r.pos0 = seq_lens[idx] - 1; r.n = r.pos0 >= 0 ? 1 : 0;
    }
    return r;
}

// ---- short convolution ----------------------------------------------------------------------------------------------
struct ConvArgs {
    const void* x;            // [T, ldx]; the channels start at column col
    void* y;                  // [T, ldy]: the channels from column 0
    const float* w;           // [C, taps]; the last column meets the current token
    const float* bias;        // [C] or null
    float* state;             // row of a slot: [taps - 1][C], the inputs before the step's first token, oldest first
    const int* positions;     // [T]; < 0: a padding row
    const int* seq_index;     // [T]
    const int* slot_ids;      // [sequences]
    const int* tiles;         // [n, 4] one tile a sequence (prompt form) or null
    const int* seq_lens;      // decode form: row b is sequence b's one token
    long long state_stride;
    int ldx, ldy, col, T, C, taps;
};

// One thread a (row, channel).  The token j places back is the row j places up when that row is the same sequence's
// token at that position; from the first j0 for which it is not, the state holds it: position pos0 - 1 - (j - j0) is
// state entry taps - 2 - (j - j0).  Reads the state only.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void short_conv_rows_kernel(ConvArgs a) {
    const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= a.C) return;
    TO* y = reinterpret_cast<TO*>(a.y) + (size_t)t * a.ldy + c;
    const int pos = a.positions[t];
    if (pos < 0) { *y = from_f32<TO>(0.f); return; }
    const int seq = a.seq_index[t];
    const TI* x = reinterpret_cast<const TI*>(a.x) + a.col + c;
    const float* w = a.w + (size_t)c * a.taps;
    const float* st = a.state + (size_t)a.slot_ids[seq] * a.state_stride + c;
    float acc = a.bias ? a.bias[c] : 0.f;
    int j0 = -1;
    for (int j = 0; j < a.taps && j <= pos; ++j) {
        if (j0 < 0 && !(t - j >= 0 && a.seq_index[t - j] == seq && a.positions[t - j] == pos - j)) j0 = j;
        const float u = j0 < 0 ? to_f32(x[(size_t)(t - j) * a.ldx]) : st[(size_t)(a.taps - 2 - (j - j0)) * a.C];
        acc = fmaf(w[a.taps - 1 - j], u, acc);
    }
    *y = from_f32<TO>(acc);
}

// One thread a (sequence, channel): the state after the step holds the inputs at the last taps - 1 positions, which are
// rows of the step or, for a step shorter than that, entries of the old state further up (read before they are written).
template <typename TI>
__global__ __launch_bounds__(256) void short_conv_state_kernel(ConvArgs a) {
    const SeqRange sr = seq_range(a.tiles, a.seq_lens, blockIdx.x);
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (sr.n <= 0 || sr.pos0 < 0 || c >= a.C) return;
    const TI* x = reinterpret_cast<const TI*>(a.x) + a.col + c;
    float* st = a.state + (size_t)a.slot_ids[sr.seq] * a.state_stride + c;
    const int keep = a.taps - 1;
    for (int i = 0; i < keep; ++i) {
        const int p = sr.pos0 + sr.n - keep + i;             // the position that entry i will hold
        float v = 0.f;
        if (p >= sr.pos0) v = to_f32(x[(size_t)(sr.row0 + (p - sr.pos0)) * a.ldx]);
        else if (p >= 0) v = st[(size_t)(keep + (p - sr.pos0)) * a.C];
        st[(size_t)i * a.C] = v;
    }
}

// Decode form, both in one: one thread a (sequence, channel) reads the state and the new input, leaves the output and
// the state moved on by one.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void short_conv_decode_kernel(ConvArgs a) {
    const int b = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= a.C) return;
    TO* y = reinterpret_cast<TO*>(a.y) + (size_t)b * a.ldy + c;
    const int pos = a.seq_lens[b] - 1;
    if (pos < 0) { *y = from_f32<TO>(0.f); return; }
    const float u0 = to_f32(reinterpret_cast<const TI*>(a.x)[(size_t)b * a.ldx + a.col + c]);
    const float* w = a.w + (size_t)c * a.taps;
    float* st = a.state + (size_t)a.slot_ids[b] * a.state_stride + c;
    const int keep = a.taps - 1;
    float acc = fmaf(w[keep], u0, a.bias ? a.bias[c] : 0.f);
    for (int j = 1; j <= keep; ++j) {                       // the token j places back is state entry keep - j
        const float u = j <= pos ? st[(size_t)(keep - j) * a.C] : 0.f;
        acc = fmaf(w[keep - j], u, acc);
    }
    for (int i = 0; i + 1 < keep; ++i) st[(size_t)i * a.C] = (keep - 1 - i) <= pos ? st[(size_t)(i + 1) * a.C] : 0.f;
    if (keep > 0) st[(size_t)(keep - 1) * a.C] = u0;
    *y = from_f32<TO>(acc);
}

// in_dtype: x's type; out_dtype: y's.  n_seqs: tiles (prompt form) or sequences (decode form: tiles null, seq_lens given).
extern "C" int bn_short_conv(int in_dtype, int out_dtype, const void* x, int ldx, int col, void* y, int ldy, const float* w,
                             const float* bias, float* state, long long state_stride, const int* positions,
                             const int* seq_index, const int* slot_ids, const int* tiles, const int* seq_lens, int n_seqs,
                             int T, int C, int taps, hipStream_t s) {
    if (T <= 0 || C <= 0 || taps < 1 || taps > BN_CONV_MAX_TAPS || n_seqs <= 0) return BN_ERR_ARG;
    if (!x || !y || !w || !state || !positions || !seq_index || !slot_ids || (!tiles && !seq_lens)) return BN_ERR_ARG;
    if (ldx < col + C || ldy < C || state_stride < (long long)(taps - 1) * C) return BN_ERR_ARG;
    if (!tiles && n_seqs != T) return BN_ERR_ARG;
    ConvArgs a;
    a.x = x; a.y = y; a.w = w; a.bias = bias; a.state = state; a.positions = positions; a.seq_index = seq_index;
    a.slot_ids = slot_ids; a.tiles = tiles; a.seq_lens = seq_lens; a.state_stride = state_stride; a.ldx = ldx; a.ldy = ldy;
    a.col = col; a.T = T; a.C = C; a.taps = taps;
    const int threads = C >= 256 ? 256 : 64;
    const int cb = (C + threads - 1) / threads;
    const bool fi = in_dtype == BN_DT_F32, fo = out_dtype == BN_DT_F32;
    if ((!fi && in_dtype != BN_DT_BF16) || (!fo && out_dtype != BN_DT_BF16)) return BN_ERR_DTYPE;
    if (!tiles) {
        const dim3 grid(T, cb);
        if (fi && fo) hipLaunchKernelGGL((short_conv_decode_kernel<float, float>), grid, dim3(threads), 0, s, a);
        else if (fi) hipLaunchKernelGGL((short_conv_decode_kernel<float, bf16>), grid, dim3(threads), 0, s, a);
        else if (fo) hipLaunchKernelGGL((short_conv_decode_kernel<bf16, float>), grid, dim3(threads), 0, s, a);
        else hipLaunchKernelGGL((short_conv_decode_kernel<bf16, bf16>), grid, dim3(threads), 0, s, a);
        return bn_launch_status();
    }
    const dim3 grid(T, cb);
    if (fi && fo) hipLaunchKernelGGL((short_conv_rows_kernel<float, float>), grid, dim3(threads), 0, s, a);
    else if (fi) hipLaunchKernelGGL((short_conv_rows_kernel<float, bf16>), grid, dim3(threads), 0, s, a);
    else if (fo) hipLaunchKernelGGL((short_conv_rows_kernel<bf16, float>), grid, dim3(threads), 0, s, a);
    else hipLaunchKernelGGL((short_conv_rows_kernel<bf16, bf16>), grid, dim3(threads), 0, s, a);
    if (taps > 1) {
        const dim3 sgrid(n_seqs, cb);
        if (fi) hipLaunchKernelGGL(short_conv_state_kernel<float>, sgrid, dim3(threads), 0, s, a);
        else hipLaunchKernelGGL(short_conv_state_kernel<bf16>, sgrid, dim3(threads), 0, s, a);
    }
    return bn_launch_status();
}

// ---- gates of the real-gated linear recurrent unit ----------------------------------------------------------------
#define LRU_ROWS 8
#define LRU_COLS 64
#define LRU_SLICES 8

// One workgroup a (eight rows, block of the input, 64 output channels of the block).  The rows' part of u is staged in
// shared memory; a thread owns an output channel and one of eight runs of the part's inputs, which it walks in order with
// both matrices (they lie [block][in][out], so the threads of a wave read neighbouring words); the runs' sums meet in
// shared memory and are added in run order.  The sums of a row are the same operations whatever the step holds.
__global__ __launch_bounds__(LRU_COLS * LRU_SLICES) void lru_gates_kernel(const float* __restrict__ u, const float* __restrict__ wa,
                                                                          const float* __restrict__ ba, const float* __restrict__ wi,
                                                                          const float* __restrict__ bi, const float* __restrict__ c_neg,
                                                                          float* __restrict__ a_out, float* __restrict__ b_out, int T,
                                                                          int W, int bw) {
    extern __shared__ float us[];                        // [LRU_ROWS][bw], then the runs' sums [LRU_SLICES][LRU_ROWS][2][LRU_COLS]
    float* red = us + LRU_ROWS * bw;
    const int t0 = blockIdx.x * LRU_ROWS, blk = blockIdx.y, c = threadIdx.x & (LRU_COLS - 1), slice = threadIdx.x / LRU_COLS;
    const int o = blockIdx.z * LRU_COLS + c;
    const int rows = min(LRU_ROWS, T - t0);
    for (int idx = threadIdx.x; idx < LRU_ROWS * bw; idx += LRU_COLS * LRU_SLICES) {
        const int r = idx / bw, i = idx - r * bw;
        us[idx] = r < rows ? u[(size_t)(t0 + r) * W + (size_t)blk * bw + i] : 0.f;
    }
    __syncthreads();
    float acc_a[LRU_ROWS], acc_i[LRU_ROWS];
#pragma unroll
    for (int r = 0; r < LRU_ROWS; ++r) { acc_a[r] = 0.f; acc_i[r] = 0.f; }
    const int per = (bw + LRU_SLICES - 1) / LRU_SLICES, i0 = slice * per, i1 = min(bw, i0 + per);
    if (o < bw) {
        const float* pa = wa + (size_t)blk * bw * bw + o;
        const float* pi = wi + (size_t)blk * bw * bw + o;
#pragma unroll 8
        for (int i = i0; i < i1; ++i) {
            const float va = pa[(size_t)i * bw], vi = pi[(size_t)i * bw];
#pragma unroll
            for (int r = 0; r < LRU_ROWS; ++r) {
                const float x = us[r * bw + i];
                acc_a[r] = fmaf(va, x, acc_a[r]);
                acc_i[r] = fmaf(vi, x, acc_i[r]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < LRU_ROWS; ++r) {
        red[((slice * LRU_ROWS + r) * 2 + 0) * LRU_COLS + c] = acc_a[r];
        red[((slice * LRU_ROWS + r) * 2 + 1) * LRU_COLS + c] = acc_i[r];
    }
    __syncthreads();
    if (slice != 0 || o >= bw) return;
    const int ch = blk * bw + o;
    const float biasa = ba[ch], biasi = bi[ch], cn = c_neg[ch];
#pragma unroll
    for (int r = 0; r < LRU_ROWS; ++r) {
        if (r >= rows) break;
        float sa = 0.f, si = 0.f;
#pragma unroll
        for (int k = 0; k < LRU_SLICES; ++k) {
            sa += red[((k * LRU_ROWS + r) * 2 + 0) * LRU_COLS + c];
            si += red[((k * LRU_ROWS + r) * 2 + 1) * LRU_COLS + c];
        }
        const float rg = 1.0f / (1.0f + expf(-(sa + biasa)));
        const float ig = 1.0f / (1.0f + expf(-(si + biasi)));
        const float la = cn * rg;                                  // log a <= 0
        const float m = sqrtf(fmaxf(-expm1f(2.0f * la), 0.f));      // sqrt(1 - a^2) without the cancellation near a = 1
        a_out[(size_t)(t0 + r) * W + ch] = expf(la);
        b_out[(size_t)(t0 + r) * W + ch] = m * ig * us[r * bw + o];
    }
}

extern "C" int bn_lru_gates(const float* u, const float* wa, const float* ba, const float* wi, const float* bi,
                            const float* c_neg, float* a_out, float* b_out, int T, int W, int blocks, hipStream_t s) {
    if (T <= 0 || W <= 0 || blocks <= 0 || W % blocks || !u || !wa || !ba || !wi || !bi || !c_neg || !a_out || !b_out) return BN_ERR_ARG;
    const int bw = W / blocks;
    const size_t shm = ((size_t)LRU_ROWS * bw + (size_t)LRU_SLICES * LRU_ROWS * 2 * LRU_COLS) * sizeof(float);
    const int row_tiles = (T + LRU_ROWS - 1) / LRU_ROWS;
    if (shm > 64 * 1024 || blocks > 65535 || (bw + LRU_COLS - 1) / LRU_COLS > 65535) return BN_ERR_ARG;
    const dim3 grid(row_tiles, blocks, (bw + LRU_COLS - 1) / LRU_COLS);
    hipLaunchKernelGGL(lru_gates_kernel, grid, dim3(LRU_COLS * LRU_SLICES), shm, s, u, wa, ba, wi, bi, c_neg, a_out, b_out, T, W, bw);
    return bn_launch_status();
}

// ---- S <- a S + b, times the other branch ---------------------------------------------------------------------------
#define LRU_AHEAD 8

// One thread a (sequence, channel) walks the sequence's tokens; the loads of the next LRU_AHEAD tokens are in flight
// while the chain advances.
template <typename T>
__global__ __launch_bounds__(64) void lru_scan_kernel(const float* __restrict__ av, const float* __restrict__ bv,
                                                      const T* __restrict__ ypre, int ldy, T* __restrict__ out,
                                                      float* __restrict__ state, long long state_stride,
                                                      const int* __restrict__ tiles, const int* __restrict__ seq_lens,
                                                      const int* __restrict__ slot_ids, int W) {
    const SeqRange sr = seq_range(tiles, seq_lens, blockIdx.x);
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (sr.n <= 0 || sr.pos0 < 0 || c >= W) return;
    float* sp = state + (size_t)slot_ids[sr.seq] * state_stride + c;
    float S = sr.pos0 > 0 ? *sp : 0.f;
    const float* ap = av + (size_t)sr.row0 * W + c;
    const float* bp = bv + (size_t)sr.row0 * W + c;
    const T* yp = ypre + (size_t)sr.row0 * ldy + c;
    T* op = out + (size_t)sr.row0 * W + c;
    for (int t0 = 0; t0 < sr.n; t0 += LRU_AHEAD) {
        float a[LRU_AHEAD], b[LRU_AHEAD], y[LRU_AHEAD];
#pragma unroll
        for (int i = 0; i < LRU_AHEAD; ++i) {
            const int t = min(t0 + i, sr.n - 1);
            a[i] = ap[(size_t)t * W]; b[i] = bp[(size_t)t * W]; y[i] = to_f32(yp[(size_t)t * ldy]);
        }
#pragma unroll
        for (int i = 0; i < LRU_AHEAD; ++i) {
            if (t0 + i >= sr.n) break;
            S = fmaf(a[i], S, b[i]);
            op[(size_t)(t0 + i) * W] = from_f32<T>(S * bn_gate_act(y[i], BN_ACT_GELU_TANH));
        }
    }
    *sp = S;
}

// Long prompts in pieces side by side, as the gated linear attention's: a thread owns (sequence, piece, channel).
//   phase 1  the piece's own chain from nothing and the product of its decays -> carry[.][0 / 1][channel]
//   carry    the sequence's S through the pieces in order; carry[.][0] then holds what a piece starts from
//   phase 2  the piece's chain from there, the outputs
template <typename T>
__global__ __launch_bounds__(64) void lru_scan_pieces_kernel(const float* __restrict__ av, const float* __restrict__ bv,
                                                             const T* __restrict__ ypre, int ldy, T* __restrict__ out,
                                                             float* __restrict__ carry, const int* __restrict__ tiles, int W,
                                                             int piece, int max_pieces, int phase) {
    SeqRange sr = seq_range(tiles, nullptr, blockIdx.x / max_pieces);
    const int c = blockIdx.y * blockDim.x + threadIdx.x, first = (blockIdx.x % max_pieces) * piece;
    if (sr.n <= 0 || sr.pos0 < 0 || first >= sr.n || c >= W) return;
    const int n = min(piece, sr.n - first), row0 = sr.row0 + first;
    float* cp = carry + (size_t)blockIdx.x * 2 * W + c;
    float S = phase == 2 ? cp[0] : 0.f, P = 1.0f;
    const float* ap = av + (size_t)row0 * W + c;
    const float* bp = bv + (size_t)row0 * W + c;
    const T* yp = ypre + (size_t)row0 * ldy + c;
    T* op = out + (size_t)row0 * W + c;
    for (int t0 = 0; t0 < n; t0 += LRU_AHEAD) {
        float a[LRU_AHEAD], b[LRU_AHEAD], y[LRU_AHEAD];
#pragma unroll
        for (int i = 0; i < LRU_AHEAD; ++i) {
            const int t = min(t0 + i, n - 1);
            a[i] = ap[(size_t)t * W]; b[i] = bp[(size_t)t * W]; y[i] = phase == 2 ? to_f32(yp[(size_t)t * ldy]) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < LRU_AHEAD; ++i) {
            if (t0 + i >= n) break;
            S = fmaf(a[i], S, b[i]);
            if (phase == 2) op[(size_t)(t0 + i) * W] = from_f32<T>(S * bn_gate_act(y[i], BN_ACT_GELU_TANH));
            else P *= a[i];
        }
    }
    if (phase == 1) { cp[0] = S; cp[W] = P; }
}

__global__ __launch_bounds__(64) void lru_carry_kernel(float* __restrict__ carry, float* __restrict__ state, long long state_stride,
                                                       const int* __restrict__ tiles, const int* __restrict__ slot_ids, int W,
                                                       int piece, int max_pieces) {
    const SeqRange sr = seq_range(tiles, nullptr, blockIdx.x);
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (sr.n <= 0 || sr.pos0 < 0 || c >= W) return;
    float* sp = state + (size_t)slot_ids[sr.seq] * state_stride + c;
    float S = sr.pos0 > 0 ? *sp : 0.f;
    const int pieces = (sr.n + piece - 1) / piece;
    for (int p = 0; p < pieces; ++p) {
        float* cp = carry + ((size_t)blockIdx.x * max_pieces + p) * 2 * W + c;
        const float own = cp[0], f = cp[W];
        cp[0] = S;
        S = fmaf(f, S, own);
    }
    *sp = S;
}

// carry: [n_tiles max_pieces, 2, W] float32 work space.  Results differ from bn_lru_scan's by rounding alone.
extern "C" int bn_lru_scan_pieces(int dtype, const float* av, const float* bv, const void* ypre, int ldy, void* out, float* state,
                                  long long state_stride, const int* tiles, int n_tiles, const int* slot_ids, int W, int piece,
                                  int max_pieces, float* carry, hipStream_t s) {
    if (n_tiles <= 0 || W <= 0 || !av || !bv || !ypre || !out || !state || !slot_ids || !tiles || !carry || ldy < W) return BN_ERR_ARG;
    if (state_stride < W || piece < 1 || max_pieces < 1 || (long long)n_tiles * max_pieces > 0x7fffffffLL) return BN_ERR_ARG;
    if (dtype != BN_DT_F32 && dtype != BN_DT_BF16) return BN_ERR_DTYPE;
    const dim3 grid(n_tiles * max_pieces, (W + 63) / 64), cgrid(n_tiles, (W + 63) / 64);
    for (int phase = 1; phase <= 2; ++phase) {
        if (dtype == BN_DT_F32)
            hipLaunchKernelGGL(lru_scan_pieces_kernel<float>, grid, dim3(64), 0, s, av, bv, (const float*)ypre, ldy, (float*)out, carry,
                               tiles, W, piece, max_pieces, phase);
        else
            hipLaunchKernelGGL(lru_scan_pieces_kernel<bf16>, grid, dim3(64), 0, s, av, bv, (const bf16*)ypre, ldy, (bf16*)out, carry,
                               tiles, W, piece, max_pieces, phase);
        if (phase == 1)
            hipLaunchKernelGGL(lru_carry_kernel, cgrid, dim3(64), 0, s, carry, state, state_stride, tiles, slot_ids, W, piece, max_pieces);
    }
    return bn_launch_status();
}

extern "C" int bn_lru_scan(int dtype, const float* av, const float* bv, const void* ypre, int ldy, void* out, float* state,
                           long long state_stride, const int* tiles, int n_seqs, const int* seq_lens, const int* slot_ids,
                           int W, hipStream_t s) {
    if (n_seqs <= 0 || W <= 0 || !av || !bv || !ypre || !out || !state || !slot_ids || (!tiles && !seq_lens) || ldy < W) return BN_ERR_ARG;
    if (state_stride < W) return BN_ERR_ARG;
    const dim3 grid(n_seqs, (W + 63) / 64);
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(lru_scan_kernel<float>, grid, dim3(64), 0, s, av, bv, (const float*)ypre, ldy, (float*)out, state,
                           state_stride, tiles, seq_lens, slot_ids, W);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(lru_scan_kernel<bf16>, grid, dim3(64), 0, s, av, bv, (const bf16*)ypre, ldy, (bf16*)out, state,
                           state_stride, tiles, seq_lens, slot_ids, W);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- gated linear attention -----------------------------------------------------------------------------------------
struct GlaArgs {
    const void* x;            // [T, ld]: q at q_col, k at k_col (head h at h * dk), v at v_col (head h at h * dv)
    const float* z;           // [T, H dk]: the decay's logits, bias included
    float* o;                 // [T, H dv] float32
    float* state;             // row of a slot: [H][dk][dv]
    const int* tiles;
    const int* seq_lens;
    const int* slot_ids;
    long long state_stride;
    int ld, q_col, k_col, v_col, H, dk, dv;
    float q_scale, inv_tau;
    // Long prompts in pieces that run side by side (phase > 0): a sequence's tokens are cut into pieces of `piece`; every
    // (sequence, piece) has a [H][dk][dv] matrix in `carry` and a [H][dk] row in `fade`.
    //   phase 1  every piece from nothing: its own sum of decayed k v^T into carry (no outputs)
    //   (bn_gla_fade: the product of a piece's decays per key channel; bn_gla_carry: S_in of every piece from the
    //    sequence's state, the pieces' sums and fades in order, left in carry; the sequence's state after its last piece)
    //   phase 2  every piece from its S_in: the outputs
    int phase, piece, max_pieces;
    float* carry;
    float* fade;
};

// A wave owns (sequence, head, 16 value columns); a workgroup is NW such waves over neighbouring columns of one head, so
// that q, k and the decays of a token are staged once for 16 NW columns.  Lane = (slice s of the key channels, column c):
// it keeps rows s RPL .. s RPL + RPL - 1 of its column of S in registers and reads their q, k and decays from shared memory
// four at a time (a slice's run of a staged row is padded so that the four slices' reads fall into different banks).
// Tokens come in runs: all threads turn a
// run into q (scaled), k, alpha = exp(logsigmoid(z) / tau) and v as float32 in shared memory, in two buffers: the next
// run's loads are asked for before the current run is walked and parked behind it, so the chain waits for no memory.
// The four slices' parts of o meet through two lane exchanges in a fixed order; the chain of a column is the same
// operations in the same order whatever the step holds and however many waves share the workgroup.
template <typename T, int RPL, int NW>
__global__ __launch_bounds__(BN_WAVE * NW) void gla_scan_kernel(GlaArgs a) {
    constexpr int DKP = GLA_SLICES * RPL;                 // staged key channels (those past dk are zeros)
    constexpr int SLP = RPL + 4, DKL = GLA_SLICES * SLP;  // a slice's channels and four floats of padding; a staged row
    constexpr int RUN = 4;                                // tokens of a run
    constexpr int NT = BN_WAVE * NW, VC = GLA_COLS * NW;
    constexpr int PF = (RUN * DKP + NT - 1) / NT, PV = (RUN * VC + NT - 1) / NT;
    __shared__ __align__(16) float q_s[2][RUN][DKL], k_s[2][RUN][DKL], a_s[2][RUN][DKL];
    __shared__ float v_s[2][RUN][VC];
    SeqRange sr = seq_range(a.tiles, a.seq_lens, a.phase ? blockIdx.x / a.max_pieces : blockIdx.x);
    if (sr.n <= 0 || sr.pos0 < 0) return;
    const int head = blockIdx.y, colb = blockIdx.z * VC;
    float* carry = nullptr;
    if (a.phase) {                                        // this workgroup's piece of the sequence
        const int first = (blockIdx.x % a.max_pieces) * a.piece;
        if (first >= sr.n) return;
        carry = a.carry + ((size_t)blockIdx.x * a.H + head) * a.dk * a.dv;
        sr.row0 += first;
        sr.n = min(a.piece, sr.n - first);
    }
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, sl = lane >> 4, c = lane & 15;
    const int col = colb + wave * GLA_COLS + c;
    const bool has = col < a.dv;
    const T* x = reinterpret_cast<const T*>(a.x);
    float* sp = a.phase ? carry + (has ? col : 0)
                        : a.state + (size_t)a.slot_ids[sr.seq] * a.state_stride + (size_t)head * a.dk * a.dv + (has ? col : 0);
    float S[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
        const int i = sl * RPL + r;
        const bool from_memory = a.phase == 2 || (a.phase == 0 && sr.pos0 > 0);
        S[r] = (from_memory && has && i < a.dk) ? sp[(size_t)i * a.dv] : 0.f;
    }
    float rq[PF], rk[PF], rz[PF], rv[PV];
    // loads from clamped places, unconditional: what lies outside the run or the head is never parked
    auto fetch = [&](int t0) {
        const int run = min(RUN, sr.n - t0);
#pragma unroll
        for (int k = 0; k < PF; ++k) {
            const int e = tid + k * NT, tt = min(e / DKP, run - 1), i = min(e % DKP, a.dk - 1);
            const size_t row = (size_t)(sr.row0 + t0 + tt);
            rq[k] = to_f32(x[row * a.ld + a.q_col + head * a.dk + i]);
            rk[k] = to_f32(x[row * a.ld + a.k_col + head * a.dk + i]);
            rz[k] = a.z[row * (size_t)(a.H * a.dk) + (size_t)head * a.dk + i];
        }
#pragma unroll
        for (int k = 0; k < PV; ++k) {
            const int e = tid + k * NT, tt = min(e / VC, run - 1), cc = min(colb + e % VC, a.dv - 1);
            rv[k] = to_f32(x[(size_t)(sr.row0 + t0 + tt) * a.ld + a.v_col + head * a.dv + cc]);
        }
    };
    auto park = [&](int buf, int t0) {
        const int run = min(RUN, sr.n - t0);
#pragma unroll
        for (int k = 0; k < PF; ++k) {
            const int e = tid + k * NT, tt = e / DKP, i = e % DKP;
            if (e >= RUN * DKP) break;
            const bool ok = tt < run && i < a.dk;
            const int at = (i / RPL) * SLP + i % RPL;
            q_s[buf][tt][at] = ok ? rq[k] * a.q_scale : 0.f;
            k_s[buf][tt][at] = ok ? rk[k] : 0.f;
            a_s[buf][tt][at] = ok ? expf((fminf(rz[k], 0.f) - log1pf(expf(-fabsf(rz[k])))) * a.inv_tau) : 1.0f;
        }
#pragma unroll
        for (int k = 0; k < PV; ++k) {
            const int e = tid + k * NT, tt = e / VC, cc = e % VC;
            if (e >= RUN * VC) break;
            v_s[buf][tt][cc] = (tt < run && colb + cc < a.dv) ? rv[k] : 0.f;
        }
    };
    fetch(0);
    park(0, 0);
    __syncthreads();
    int buf = 0;
    for (int t0 = 0; t0 < sr.n; t0 += RUN, buf ^= 1) {
        const int run = min(RUN, sr.n - t0);
        const bool more = t0 + RUN < sr.n;
        if (more) fetch(t0 + RUN);
        // Rows outside, tokens inside: four rows of S walk the run's tokens while the next four rows' q, k and decays are
        // on their way from shared memory, and the slices' parts of the run's outputs meet once, behind the run.  A place
        // of the run without a token is staged as the identity (decay 1, k = q = v = 0): S passes it unchanged.
        float vj[RUN], o[RUN];
#pragma unroll
        for (int tt = 0; tt < RUN; ++tt) { vj[tt] = v_s[buf][tt][wave * GLA_COLS + c]; o[tt] = 0.f; }
        float4 av[2][RUN], kv[2][RUN], qv[2][RUN];
        auto rows4 = [&](int set, int r) {
#pragma unroll
            for (int tt = 0; tt < RUN; ++tt) {
                av[set][tt] = *reinterpret_cast<const float4*>(&a_s[buf][tt][sl * SLP + r]);
                kv[set][tt] = *reinterpret_cast<const float4*>(&k_s[buf][tt][sl * SLP + r]);
                qv[set][tt] = *reinterpret_cast<const float4*>(&q_s[buf][tt][sl * SLP + r]);
            }
        };
        rows4(0, 0);
#pragma unroll
        for (int r = 0; r < RPL; r += 4) {
            const int set = (r / 4) & 1;
            if (r + 4 < RPL) rows4(set ^ 1, r + 4);             // asked for before this group's rows are walked
#pragma unroll
            for (int tt = 0; tt < RUN; ++tt) {
                S[r] = fmaf(av[set][tt].x, S[r], kv[set][tt].x * vj[tt]);         o[tt] = fmaf(S[r], qv[set][tt].x, o[tt]);
                S[r + 1] = fmaf(av[set][tt].y, S[r + 1], kv[set][tt].y * vj[tt]); o[tt] = fmaf(S[r + 1], qv[set][tt].y, o[tt]);
                S[r + 2] = fmaf(av[set][tt].z, S[r + 2], kv[set][tt].z * vj[tt]); o[tt] = fmaf(S[r + 2], qv[set][tt].z, o[tt]);
                S[r + 3] = fmaf(av[set][tt].w, S[r + 3], kv[set][tt].w * vj[tt]); o[tt] = fmaf(S[r + 3], qv[set][tt].w, o[tt]);
            }
            __builtin_amdgcn_sched_barrier(0);                   // the compiler keeps to one group ahead (registers)
        }
#pragma unroll
        for (int tt = 0; tt < RUN; ++tt) {
            float v = o[tt];
            v += __shfl_xor(v, 16, BN_WAVE);
            v += __shfl_xor(v, 32, BN_WAVE);
            if (tt < run && sl == 0 && has && a.phase != 1) a.o[(size_t)(sr.row0 + t0 + tt) * (a.H * a.dv) + (size_t)head * a.dv + col] = v;
        }
        if (more) park(buf ^ 1, t0 + RUN);
        __syncthreads();
    }
    if (has && a.phase != 2) {
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
            const int i = sl * RPL + r;
            if (i < a.dk) sp[(size_t)i * a.dv] = S[r];
        }
    }
}

// The product of a piece's decays per key channel, as the exponential of the sum of their logarithms.
__global__ __launch_bounds__(256) void gla_fade_kernel(GlaArgs a) {
    const SeqRange sr = seq_range(a.tiles, a.seq_lens, blockIdx.x / a.max_pieces);
    const int first = (blockIdx.x % a.max_pieces) * a.piece, ch = blockIdx.y * blockDim.x + threadIdx.x;
    if (sr.n <= 0 || sr.pos0 < 0 || first >= sr.n || ch >= a.H * a.dk) return;
    const int n = min(a.piece, sr.n - first);
    const float* z = a.z + (size_t)(sr.row0 + first) * (a.H * a.dk) + ch;
    float sum = 0.f;
    for (int t = 0; t < n; ++t) {
        const float zz = z[(size_t)t * (a.H * a.dk)];
        sum += (fminf(zz, 0.f) - log1pf(expf(-fabsf(zz)))) * a.inv_tau;
    }
    a.fade[(size_t)blockIdx.x * (a.H * a.dk) + ch] = expf(sum);
}

// One thread an element of a head's matrix: it walks the sequence's pieces in order, leaves in carry what every piece
// starts from, and in the state what the sequence ends with.
__global__ __launch_bounds__(256) void gla_carry_kernel(GlaArgs a) {
    const int tile = blockIdx.x, head = blockIdx.y, e = blockIdx.z * blockDim.x + threadIdx.x;
    const SeqRange sr = seq_range(a.tiles, a.seq_lens, tile);
    if (sr.n <= 0 || sr.pos0 < 0 || e >= a.dk * a.dv) return;
    const int i = e / a.dv;
    float* sp = a.state + (size_t)a.slot_ids[sr.seq] * a.state_stride + (size_t)head * a.dk * a.dv + e;
    float S = sr.pos0 > 0 ? *sp : 0.f;
    const int pieces = (sr.n + a.piece - 1) / a.piece;
    for (int p = 0; p < pieces; ++p) {
        const size_t at = (size_t)tile * a.max_pieces + p;
        float* c = a.carry + (at * a.H + head) * a.dk * a.dv + e;
        const float own = *c, f = a.fade[(at * a.H + head) * a.dk + i];
        *c = S;
        S = fmaf(f, S, own);
    }
    *sp = S;
}

extern "C" int bn_gla_supports(int dk, int dv) { return (dk >= 1 && dk <= GLA_MAX_DIM && dv >= 1) ? 1 : 0; }

// waves of a workgroup: four (64 value columns share a staged run) unless a head has no more than one wave's columns;
// more waves a workgroup would share the staging further but put several chains on one SIMD
static int gla_waves(int dv) { return dv <= GLA_COLS ? 1 : 4; }

template <typename T, int NW>
static int gla_launch_nw(const GlaArgs& a, int n_seqs, hipStream_t s) {
    const dim3 grid(a.phase ? n_seqs * a.max_pieces : n_seqs, a.H, (a.dv + GLA_COLS * NW - 1) / (GLA_COLS * NW)), block(BN_WAVE * NW);
    const int rpl = (a.dk + GLA_SLICES - 1) / GLA_SLICES;
    if (rpl <= 8) hipLaunchKernelGGL((gla_scan_kernel<T, 8, NW>), grid, block, 0, s, a);
    else if (rpl <= 16) hipLaunchKernelGGL((gla_scan_kernel<T, 16, NW>), grid, block, 0, s, a);
    else if (rpl <= 32) hipLaunchKernelGGL((gla_scan_kernel<T, 32, NW>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((gla_scan_kernel<T, 64, NW>), grid, block, 0, s, a);
    return bn_launch_status();
}

template <typename T>
static int gla_launch(const GlaArgs& a, int n_seqs, hipStream_t s) {
    switch (gla_waves(a.dv)) {
        case 1: return gla_launch_nw<T, 1>(a, n_seqs, s);
        default: return gla_launch_nw<T, 4>(a, n_seqs, s);
    }
}

extern "C" int bn_gla_scan(int dtype, const void* x, int ld, int q_col, int k_col, int v_col, const float* z, float* o,
                           float* state, long long state_stride, const int* tiles, int n_seqs, const int* seq_lens,
                           const int* slot_ids, int H, int dk, int dv, float q_scale, float inv_tau, hipStream_t s) {
    if (n_seqs <= 0 || H <= 0 || !bn_gla_supports(dk, dv) || !x || !z || !o || !state || !slot_ids || (!tiles && !seq_lens)) return BN_ERR_ARG;
    if (ld < q_col + H * dk || ld < k_col + H * dk || ld < v_col + H * dv || state_stride < (long long)H * dk * dv) return BN_ERR_ARG;
    if (H > 65535 || (dv + GLA_COLS - 1) / GLA_COLS > 65535) return BN_ERR_ARG;
    GlaArgs a;
    a.x = x; a.z = z; a.o = o; a.state = state; a.tiles = tiles; a.seq_lens = seq_lens; a.slot_ids = slot_ids;
    a.state_stride = state_stride; a.ld = ld; a.q_col = q_col; a.k_col = k_col; a.v_col = v_col; a.H = H; a.dk = dk; a.dv = dv;
    a.q_scale = q_scale; a.inv_tau = inv_tau;
    a.phase = 0; a.piece = 0; a.max_pieces = 1; a.carry = nullptr; a.fade = nullptr;
    if (dtype == BN_DT_F32) return gla_launch<float>(a, n_seqs, s);
    if (dtype == BN_DT_BF16) return gla_launch<bf16>(a, n_seqs, s);
    return BN_ERR_DTYPE;
}

// The same over long prompts, their pieces side by side (prompt form only).  carry: [n_tiles max_pieces, H dk dv] and
// fade: [n_tiles max_pieces, H dk] float32 work space; max_pieces covers the longest sequence's pieces.  A sequence's
// outputs and state differ from the plain walk's by rounding alone (a piece's own sum is formed from nothing and joined
// to what came before it by one multiplication and addition).
extern "C" int bn_gla_scan_pieces(int dtype, const void* x, int ld, int q_col, int k_col, int v_col, const float* z, float* o,
                                  float* state, long long state_stride, const int* tiles, int n_tiles, const int* slot_ids, int H,
                                  int dk, int dv, float q_scale, float inv_tau, int piece, int max_pieces, float* carry,
                                  float* fade, hipStream_t s) {
    if (n_tiles <= 0 || H <= 0 || !bn_gla_supports(dk, dv) || !x || !z || !o || !state || !slot_ids || !tiles || !carry || !fade) return BN_ERR_ARG;
    if (ld < q_col + H * dk || ld < k_col + H * dk || ld < v_col + H * dv || state_stride < (long long)H * dk * dv) return BN_ERR_ARG;
    if (piece < 1 || max_pieces < 1 || H > 65535 || (long long)n_tiles * max_pieces > 0x7fffffffLL) return BN_ERR_ARG;
    if (dtype != BN_DT_F32 && dtype != BN_DT_BF16) return BN_ERR_DTYPE;
    GlaArgs a;
    a.x = x; a.z = z; a.o = o; a.state = state; a.tiles = tiles; a.seq_lens = nullptr; a.slot_ids = slot_ids;
    a.state_stride = state_stride; a.ld = ld; a.q_col = q_col; a.k_col = k_col; a.v_col = v_col; a.H = H; a.dk = dk; a.dv = dv;
    a.q_scale = q_scale; a.inv_tau = inv_tau; a.piece = piece; a.max_pieces = max_pieces; a.carry = carry; a.fade = fade;
    a.phase = 1;
    int rc = dtype == BN_DT_F32 ? gla_launch<float>(a, n_tiles, s) : gla_launch<bf16>(a, n_tiles, s);
    if (rc != 0) return rc;
    hipLaunchKernelGGL(gla_fade_kernel, dim3(n_tiles * max_pieces, (H * dk + 255) / 256), dim3(256), 0, s, a);
    hipLaunchKernelGGL(gla_carry_kernel, dim3(n_tiles, H, (dk * dv + 255) / 256), dim3(256), 0, s, a);
    if ((rc = bn_launch_status()) != 0) return rc;
    a.phase = 2;
    return dtype == BN_DT_F32 ? gla_launch<float>(a, n_tiles, s) : gla_launch<bf16>(a, n_tiles, s);
}
