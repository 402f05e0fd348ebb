// The residual stream's general norm step, for layers that put a norm behind a sublayer as well as
// before it:   x += norm_d(delta);   out = norm_o(x).
//
// x float32 [n, H] is the stream.  delta, what a sublayer left (a tensor of the activation type or a
// float32 stack of partial sums added in stack order), is normalised by a norm of its own before it is
// added: none, RMS (d / sqrt(mean(d^2) + eps) * (offset + w)) or layer norm without a bias
// ((d - mean) / sqrt(mean((d - mean)^2) + eps) * (offset + w)).  The sum is written back to x unless
// the rows are gathered (`rows`: logits of a few places; x is then left alone).  `out`, if asked
// for, is the new x under the second norm (the same three kinds; "none" is a cast), in the
// activation type.  Everything is float32: means, variances as means of squared deviations (two
// passes over a row held in shared memory), the sum.  One workgroup a row.
//
// `conv` (a step in which every row is its request's one new token): out is not a norm of the new x but the new x
// through a short convolution over time, out[c] = x[c] + sum_k w[k, c] * (the request's k-th carried row, the last tap
// x itself), and the carried rows (float32 [taps - 1, H] from `carried_offset` of row state_slots[row] of `state`)
// move up by one and take x: what `stream_conv` does for single tokens, in the launch that settles the stream.
#include "common.h"

struct NormConv {
    const float* weight;       // [taps, H], a row a tap; null: no convolution
    float* state;
    long long state_stride;
    long long carried_offset;
    const int* state_slots;
    int taps;
};

constexpr int kNormNone = 0, kNormRms = 1, kNormLayer = 2;

// v (a thread's elements of the row, in shared memory `row`) under a norm; returns through `row`.
// Every thread of the workgroup calls it.
__device__ __forceinline__ void row_stats(const float* row, int hidden, int kind, float eps, float* scratch, float& mean,
                                          float& inv) {
    mean = 0.f;
    inv = 1.f;
    if (kind == kNormNone) return;
    const float count = static_cast<float>(hidden);
    if (kind == kNormLayer) {
        float s = 0.f;
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) s += row[i];
        mean = block_sum(s, scratch) / count;
    }
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float d = row[i] - mean;
        ss += d * d;
    }
    inv = 1.f / sqrtf(block_sum(ss, scratch) / count + eps);
}

template <typename TD, typename TO>
__global__ void __launch_bounds__(1024)
norm_add_kernel(float* __restrict__ x, const TD* __restrict__ delta, int splits, size_t split_stride, int d_kind,
                const float* __restrict__ d_weight, float d_eps, float d_offset, const int* __restrict__ rows,
                TO* __restrict__ out, int o_kind, const float* __restrict__ o_weight, float o_eps, float o_offset,
                int hidden, NormConv conv) {
    extern __shared__ float row[];
    __shared__ float scratch[16];
    const int orow = blockIdx.x;
    const int irow = rows ? rows[orow] : orow;
    float* xr = x + static_cast<size_t>(irow) * hidden;
    // The convolution's taps and the carried rows of this thread's (at most two) elements are asked for before anything
    // else, so that they arrive while the sublayer's product is normalised: a row's time is its chain of trips to memory.
    constexpr int kHeldTaps = 8;
    float held_w[2][kHeldTaps], held_c[2][kHeldTaps];
    const bool held = conv.weight && conv.taps <= kHeldTaps && hidden <= 2 * static_cast<int>(blockDim.x);
    if (held) {
        const float* carried = conv.state + static_cast<size_t>(conv.state_slots[orow]) * conv.state_stride + conv.carried_offset;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int i = threadIdx.x + e * blockDim.x;
#pragma unroll
            for (int k = 0; k < kHeldTaps; ++k) {
                held_w[e][k] = (i < hidden && k < conv.taps) ? conv.weight[static_cast<size_t>(k) * hidden + i] : 0.f;
                held_c[e][k] = (i < hidden && k + 1 < conv.taps) ? carried[static_cast<size_t>(k) * hidden + i] : 0.f;
            }
        }
    }
    if (delta) {
        const TD* dr = delta + static_cast<size_t>(irow) * hidden;
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
            float d;
            if (sizeof(TD) == sizeof(float) && splits > 1) d = stack_sum(reinterpret_cast<const float*>(dr) + i, splits, split_stride);
            else d = to_float(dr[i]);
            row[i] = d;
        }
        __syncthreads();
        float mean, inv;
        row_stats(row, hidden, d_kind, d_eps, scratch, mean, inv);
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
            float d = row[i];                       // this thread's own elements: no other thread writes them
            if (d_kind != kNormNone) d = (d - mean) * inv * (d_offset + d_weight[i]);
            const float v = xr[i] + d;
            if (!rows) xr[i] = v;
            row[i] = v;
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) row[i] = xr[i];
    }
    if (!out) return;
    TO* o = out + static_cast<size_t>(orow) * hidden;
    if (conv.weight) {
        // (a thread's own elements of the row, and its own columns of the carried rows)
        float* carried = conv.state + static_cast<size_t>(conv.state_slots[orow]) * conv.state_stride + conv.carried_offset;
        const int taps = conv.taps;
        if (held) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int i = threadIdx.x + e * blockDim.x;
                if (i >= hidden) break;
                const float now = row[i];
                float acc = now;
#pragma unroll
                for (int k = 0; k < kHeldTaps; ++k) {
                    if (k + 1 < taps) {
                        acc = fmaf(held_w[e][k], held_c[e][k], acc);
                        if (k > 0) carried[static_cast<size_t>(k - 1) * hidden + i] = held_c[e][k];
                    } else if (k + 1 == taps) {
                        acc = fmaf(held_w[e][k], now, acc);
                    }
                }
                if (taps > 1) carried[static_cast<size_t>(taps - 2) * hidden + i] = now;
                o[i] = from_float<TO>(acc);
            }
            return;
        }
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
            const float now = row[i];
            float acc = now;
            for (int k = 0; k + 1 < taps; ++k) {
                const float v = carried[static_cast<size_t>(k) * hidden + i];
                acc = fmaf(conv.weight[static_cast<size_t>(k) * hidden + i], v, acc);
                if (k > 0) carried[static_cast<size_t>(k - 1) * hidden + i] = v;
            }
            acc = fmaf(conv.weight[static_cast<size_t>(taps - 1) * hidden + i], now, acc);
            if (taps > 1) carried[static_cast<size_t>(taps - 2) * hidden + i] = now;
            o[i] = from_float<TO>(acc);
        }
        return;
    }
    __syncthreads();
    float mean, inv;
    row_stats(row, hidden, o_kind, o_eps, scratch, mean, inv);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v = row[i];
        if (o_kind != kNormNone) v = (v - mean) * inv * (o_offset + o_weight[i]);
        o[i] = from_float<TO>(v);
    }
}

// delta_type / out_type: 0 float32, 1 bfloat16.  Returns 0, a HIP error code, or -1 for sizes it does not take.
WLLM_API int wllm_norm_add(float* x, const void* delta, int delta_type, int splits, long long split_stride, int d_kind,
                           const float* d_weight, float d_eps, float d_offset, const int* rows, void* out, int out_type,
                           int o_kind, const float* o_weight, float o_eps, float o_offset, int num_rows, int hidden,
                           const float* conv_weight, int conv_taps, float* conv_state, long long conv_state_stride,
                           long long conv_carried_offset, const int* conv_state_slots, hipStream_t stream) {
    if (num_rows <= 0) return 0;
    if (conv_weight && (!out || rows || o_kind != kNormNone || conv_taps < 1 || conv_taps > 64 || !conv_state || !conv_state_slots))
        return -1;
    const NormConv conv{conv_weight, conv_state, conv_state_stride, conv_carried_offset, conv_state_slots, conv_taps};
    if (hidden <= 0 || hidden > 16384 || !x) return -1;
    if (d_kind < 0 || d_kind > 2 || o_kind < 0 || o_kind > 2) return -1;
    if (delta && d_kind != kNormNone && !d_weight) return -1;
    if (out && o_kind != kNormNone && !o_weight) return -1;
    if (!delta && !out) return 0;
    const size_t smem = sizeof(float) * static_cast<size_t>(hidden);
    // The few rows of a decode step: a row's time is that of its chain of trips to memory (a stack of partial
    // sums to add, the stream, the weights), so as many threads as give each two elements; many rows: 256.
    int threads = 256;
    if (num_rows <= 256) {
        threads = (hidden / 2 + 63) / 64 * 64;
        threads = threads < 64 ? 64 : (threads > 1024 ? 1024 : threads);
    }
#define LAUNCH(TD, TO)                                                                                               \
    norm_add_kernel<TD, TO><<<num_rows, threads, smem, stream>>>(x, static_cast<const TD*>(delta), splits,            \
                                                              static_cast<size_t>(split_stride), d_kind, d_weight,   \
                                                              d_eps, d_offset, rows, static_cast<TO*>(out), o_kind,   \
                                                              o_weight, o_eps, o_offset, hidden, conv)
    if (delta_type && out_type) LAUNCH(bf16, bf16);
    else if (delta_type) LAUNCH(bf16, float);
    else if (out_type) LAUNCH(float, bf16);
    else LAUNCH(float, float);
#undef LAUNCH
    return launch_status();
}

// ---- RMS norm of a band of columns of every row, with a weight: out = v / sqrt(sum(v^2) / count + eps) * w,
// where v is the band, plus a bias (float32, one a column) if the band has one: a projection's bias that
// belongs in front of its norm.  The band [rows, cols] lies in a wider tensor (row stride); `count` is the number of elements the
// mean is taken over (less than cols where a band carries padding that is always zero); out may be
// the band itself or another band, and where it is wider than cols the further columns become zero.
// Up to two bands a launch (blockIdx.y), each with its own operands. ----
struct NormBand {
    const void* src;
    long long src_stride;
    int cols;
    const float* weight;
    float count;
    void* out;
    long long out_stride;
    int out_cols;
    const float* bias;
};

template <typename T>
__global__ void __launch_bounds__(256) band_norm_kernel(NormBand b0, NormBand b1, float eps) {
    __shared__ float scratch[16];
    const NormBand b = blockIdx.y == 0 ? b0 : b1;
    const T* s = static_cast<const T*>(b.src) + static_cast<size_t>(blockIdx.x) * b.src_stride;
    T* o = static_cast<T*>(b.out) + static_cast<size_t>(blockIdx.x) * b.out_stride;
    float ss = 0.f;
    for (int i = threadIdx.x; i < b.cols; i += blockDim.x) {
        const float v = to_float(s[i]) + (b.bias ? b.bias[i] : 0.f);
        ss += v * v;
    }
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / b.count + eps);
    for (int i = threadIdx.x; i < b.out_cols; i += blockDim.x)
        o[i] = from_float<T>(i < b.cols ? (to_float(s[i]) + (b.bias ? b.bias[i] : 0.f)) * inv * b.weight[i] : 0.f);
}

WLLM_API int wllm_band_norm(const void* src0, long long src_stride0, int cols0, const float* weight0, float count0,
                            void* out0, long long out_stride0, int out_cols0, const float* bias0, const void* src1,
                            long long src_stride1, int cols1, const float* weight1, float count1, void* out1,
                            long long out_stride1, int out_cols1, const float* bias1, float eps, int is_bf16, int rows,
                            hipStream_t stream) {
    if (rows <= 0) return 0;
    if (!src0 || !out0 || !weight0 || cols0 <= 0 || out_cols0 < cols0 || !(count0 > 0.f)) return -1;
    if (src1 && (!out1 || !weight1 || cols1 <= 0 || out_cols1 < cols1 || !(count1 > 0.f))) return -1;
    const NormBand b0{src0, src_stride0, cols0, weight0, count0, out0, out_stride0, out_cols0, bias0};
    const NormBand b1{src1, src_stride1, cols1, weight1, count1, out1, out_stride1, out_cols1, bias1};
    const dim3 grid(rows, src1 ? 2 : 1);
    if (is_bf16) band_norm_kernel<bf16><<<grid, 256, 0, stream>>>(b0, b1, eps);
    else band_norm_kernel<float><<<grid, 256, 0, stream>>>(b0, b1, eps);
    return launch_status();
}

// ---- out[r, c] = act(gate[r, c]) * table[ids[r], col0 + c]: a small projection of the stream,
// bent and multiplied by the token's own entry of a table (a band of `cols` columns of its row) ----
template <typename T, int ACT>
__global__ void gated_lookup_kernel(const T* __restrict__ gate, const int* __restrict__ ids, const T* __restrict__ table,
                                    long long table_stride, int col0, T* __restrict__ out, int rows, int cols) {
    const long long total = static_cast<long long>(rows) * cols;
    for (long long e = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; e < total;
         e += static_cast<long long>(gridDim.x) * blockDim.x) {
        const int r = static_cast<int>(e / cols), c = static_cast<int>(e - static_cast<long long>(r) * cols);
        const float entry = to_float(table[static_cast<size_t>(ids[r]) * table_stride + col0 + c]);
        out[e] = from_float<T>(activate<ACT>(to_float(gate[e])) * entry);
    }
}

WLLM_API int wllm_gated_lookup(const void* gate, const int* ids, const void* table, long long table_stride, int col0,
                               void* out, int is_bf16, int activation, int rows, int cols, hipStream_t stream) {
    if (rows <= 0 || cols <= 0) return 0;
    if (activation < 0 || activation >= kActivations || col0 < 0 || col0 + cols > table_stride) return -1;
    const long long total = static_cast<long long>(rows) * cols;
    const int blocks = static_cast<int>(total / 256 + 1 < 4096 ? total / 256 + 1 : 4096);
#define LAUNCH(T)                                                                                                     \
    WLLM_BY_ACTIVATION(activation, (gated_lookup_kernel<T, ACT><<<blocks, 256, 0, stream>>>(                           \
                                       static_cast<const T*>(gate), ids, static_cast<const T*>(table), table_stride,  \
                                       col0, static_cast<T*>(out), rows, cols)))
    if (is_bf16) { LAUNCH(bf16); } else { LAUNCH(float); }
#undef LAUNCH
    return launch_status();
}

// ---- a product head by head: y[r, h * O + o] = sum_k x[r, h * K + k] * w[h, o, k].  x and y are
// bands of wider tensors (row strides); w is [heads, O, K].  float32 sums in ascending order of k,
// so a row's result does not depend on the rows beside it.  A workgroup makes 32 rows by 64 outputs
// of one head, a thread 2 by 4 of them, from chunks of 32 keys staged in shared memory. ----
constexpr int kHlRows = 32, kHlOuts = 64, kHlKeys = 32;

template <typename T>
__global__ void __launch_bounds__(256)
head_linear_kernel(const T* __restrict__ x, long long x_stride, const T* __restrict__ w, T* __restrict__ y,
                   long long y_stride, int rows, int heads, int outs, int keys) {
    __shared__ float xs[kHlRows][kHlKeys + 1];
    __shared__ float ws[kHlOuts][kHlKeys + 1];
    const int h = blockIdx.y;
    const int r0 = blockIdx.x * kHlRows, o0 = blockIdx.z * kHlOuts;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;       // outputs 4 tx .. +4, rows 2 ty .. +2
    const T* wh = w + static_cast<size_t>(h) * outs * keys;
    float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int k0 = 0; k0 < keys; k0 += kHlKeys) {
        for (int e = threadIdx.x; e < kHlRows * kHlKeys; e += blockDim.x) {
            const int r = e / kHlKeys, k = e % kHlKeys;
            xs[r][k] = (r0 + r < rows && k0 + k < keys)
                           ? to_float(x[static_cast<size_t>(r0 + r) * x_stride + static_cast<size_t>(h) * keys + k0 + k]) : 0.f;
        }
        for (int e = threadIdx.x; e < kHlOuts * kHlKeys; e += blockDim.x) {
            const int o = e / kHlKeys, k = e % kHlKeys;
            ws[o][k] = (o0 + o < outs && k0 + k < keys) ? to_float(wh[static_cast<size_t>(o0 + o) * keys + k0 + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int k = 0; k < kHlKeys; ++k) {
            const float a0 = xs[2 * ty][k], a1 = xs[2 * ty + 1][k];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float b = ws[4 * tx + j][k];
                acc[0][j] = fmaf(a0, b, acc[0][j]);
                acc[1][j] = fmaf(a1, b, acc[1][j]);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = r0 + 2 * ty + i;
        if (r >= rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int o = o0 + 4 * tx + j;
            if (o < outs) y[static_cast<size_t>(r) * y_stride + static_cast<size_t>(h) * outs + o] = from_float<T>(acc[i][j]);
        }
    }
}

// The few rows of a decode step: a workgroup takes one head and 64 outputs, all rows (at most 16).  Thread
// (o, q) multiplies the q-th quarter of output o's row of w (read once, in runs of consecutive elements) with
// every row of x, which lies in shared memory; the quarters are added in ascending order, so the sum's order
// is k ascending within a quarter and quarter by quarter.
constexpr int kHlFewRows = 16;

template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
head_linear_few_kernel(const T* __restrict__ x, long long x_stride, const T* __restrict__ w, T* __restrict__ y,
                       long long y_stride, int rows, int heads, int outs, int keys) {
    extern __shared__ float hl_smem[];
    float* xs = hl_smem;                                  // [rows][keys]
    float* part = hl_smem + rows * keys;                  // [4][rows][64]
    const int h = blockIdx.x, o0 = blockIdx.y * kHlOuts;
    for (int e = threadIdx.x; e < rows * keys; e += blockDim.x) {
        const int r = e / keys, k = e - r * keys;
        xs[e] = to_float(x[static_cast<size_t>(r) * x_stride + static_cast<size_t>(h) * keys + k]);
    }
    __syncthreads();
    const int o = threadIdx.x % kHlOuts, q = threadIdx.x / kHlOuts;
    const int per = (keys + 3) / 4, k_begin = q * per, k_end = min(keys, k_begin + per);
    float acc[kHlFewRows];
#pragma unroll
    for (int r = 0; r < kHlFewRows; ++r) acc[r] = 0.f;
    if (o0 + o < outs) {
        const T* wr = w + (static_cast<size_t>(h) * outs + o0 + o) * keys;
        if (VEC) {
            // the quarter is a whole number of 16-byte pieces that begin at multiples of 16 bytes: the row of w
            // streams in as such pieces, several asked for before the first is multiplied
            constexpr int kPiece = 16 / sizeof(T);
#pragma unroll 4
            for (int k = k_begin; k < k_end; k += kPiece) {
                const uint4 piece = load_streamed(wr + k);
                float wv[kPiece];
                if (sizeof(T) == 2) {
                    const uint32_t words[4] = {piece.x, piece.y, piece.z, piece.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        wv[2 * j] = __uint_as_float(words[j] << 16);
                        wv[2 * j + 1] = __uint_as_float(words[j] & 0xffff0000u);
                    }
                } else {
                    wv[0] = __uint_as_float(piece.x);
                    wv[1] = __uint_as_float(piece.y);
                    wv[2] = __uint_as_float(piece.z);
                    wv[3] = __uint_as_float(piece.w);
                }
#pragma unroll
                for (int j = 0; j < kPiece; ++j)
#pragma unroll
                    for (int r = 0; r < kHlFewRows; ++r)
                        if (r < rows) acc[r] = fmaf(xs[r * keys + k + j], wv[j], acc[r]);
            }
        } else {
            for (int k = k_begin; k < k_end; ++k) {
                const float wv = to_float(wr[k]);
#pragma unroll
                for (int r = 0; r < kHlFewRows; ++r)
                    if (r < rows) acc[r] = fmaf(xs[r * keys + k], wv, acc[r]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < kHlFewRows; ++r)
        if (r < rows) part[(q * rows + r) * kHlOuts + o] = acc[r];
    __syncthreads();
    for (int e = threadIdx.x; e < rows * kHlOuts; e += blockDim.x) {
        const int r = e / kHlOuts, oo = e % kHlOuts;
        if (o0 + oo >= outs) continue;
        float total = part[r * kHlOuts + oo];
#pragma unroll
        for (int qq = 1; qq < 4; ++qq) total += part[(qq * rows + r) * kHlOuts + oo];
        y[static_cast<size_t>(r) * y_stride + static_cast<size_t>(h) * outs + o0 + oo] = from_float<T>(total);
    }
}

WLLM_API int wllm_head_linear(const void* x, long long x_stride, const void* w, void* y, long long y_stride, int is_bf16,
                              int rows, int heads, int outs, int keys, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (heads <= 0 || outs <= 0 || keys <= 0 || heads > 65535) return -1;
    const dim3 grid((rows + kHlRows - 1) / kHlRows, heads, (outs + kHlOuts - 1) / kHlOuts);
    if (grid.z > 65535) return -1;
    const size_t smem = sizeof(float) * (static_cast<size_t>(rows) * keys + 4 * static_cast<size_t>(rows) * kHlOuts);
    if (rows <= kHlFewRows && smem <= 48 * 1024) {
        const dim3 few(heads, (outs + kHlOuts - 1) / kHlOuts);
        // whole 16-byte pieces a quarter of a row of w, each at a multiple of 16 bytes
        const int piece = is_bf16 ? 8 : 4;
        const bool vec = keys % (4 * piece) == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
#define LAUNCH_FEW(T, V)                                                                                               \
    head_linear_few_kernel<T, V><<<few, 256, smem, stream>>>(static_cast<const T*>(x), x_stride, static_cast<const T*>(w), \
                                                             static_cast<T*>(y), y_stride, rows, heads, outs, keys)
        if (is_bf16) { if (vec) LAUNCH_FEW(bf16, true); else LAUNCH_FEW(bf16, false); }
        else { if (vec) LAUNCH_FEW(float, true); else LAUNCH_FEW(float, false); }
#undef LAUNCH_FEW
        return launch_status();
    }
    if (is_bf16)
        head_linear_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(x), x_stride, static_cast<const bf16*>(w),
                                                           static_cast<bf16*>(y), y_stride, rows, heads, outs, keys);
    else
        head_linear_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(x), x_stride,
                                                            static_cast<const float*>(w), static_cast<float*>(y), y_stride,
                                                            rows, heads, outs, keys);
    return launch_status();
}
