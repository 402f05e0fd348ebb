// A selective state-space mixer (the recurrence of Mamba-2) on a flat batch of segments: the short
// causal convolution with its carried inputs, the recurrence with its carried state, and the gated
// norm in groups behind it.  A segment is the next tokens of one request; what a request carries from
// step to step lies in one float32 row of `state` per request (row state_slots[segment]):
//   [heads, N, P] the recurrence's state S, then [taps - 1, channels] the convolution's last inputs
//   (the oldest first).
// A fresh request's row is all zeros, which is both "S starts at zero" and "zeros before the start".
// Everything that enters the recurrence is float32: step sizes, decays, the state, the sums.
#include "common.h"

// ---- convolution: out[t, c] = silu(bias[c] + sum_k w[c, k] * in[t - (taps - 1) + k, c]), the inputs
// before the segment's first token taken from the carried rows.  in is a band of a wider row. ----
template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ in, long long in_stride, const float* __restrict__ weight,
                   const float* __restrict__ bias, const float* __restrict__ state, long long state_stride,
                   long long carried_offset, const int* __restrict__ token_segment, const int* __restrict__ seg_q_start,
                   const int* __restrict__ state_slots, T* __restrict__ out, int channels, int taps) {
    const int token = blockIdx.x;
    const int seg = token_segment[token];
    const int local = token - seg_q_start[seg];
    const float* carried = state + static_cast<size_t>(state_slots[seg]) * state_stride + carried_offset;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
        float acc = bias[c];
        for (int k = 0; k < taps; ++k) {
            const int src = local - (taps - 1) + k;          // place in the segment; negative: a carried input
            const float v = src >= 0 ? to_float(in[static_cast<size_t>(token - local + src) * in_stride + c])
                                     : carried[static_cast<size_t>(taps - 1 + src) * channels + c];
            acc = fmaf(weight[static_cast<size_t>(c) * taps + k], v, acc);
        }
        out[static_cast<size_t>(token) * channels + c] = from_float<T>(acc / (1.f + expf(-acc)));
    }
}

// ---- after the convolution of a step: the carried rows take the segment's last taps - 1 inputs (of
// a segment shorter than that, the carried rows move up).  Row j's new value comes from a row above
// it or from the step's inputs, so a thread that walks j upwards never reads what it wrote. ----
template <typename T>
__global__ void __launch_bounds__(256)
conv_carry_kernel(const T* __restrict__ in, long long in_stride, float* __restrict__ state, long long state_stride,
                  long long carried_offset, const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                  const int* __restrict__ state_slots, int channels, int taps) {
    const int seg = blockIdx.x;
    const int q_len = seg_q_len[seg], q_start = seg_q_start[seg];
    if (q_len <= 0) return;
    float* carried = state + static_cast<size_t>(state_slots[seg]) * state_stride + carried_offset;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
        for (int j = 0; j < taps - 1; ++j) {
            const int src = q_len - (taps - 1) + j;
            carried[static_cast<size_t>(j) * channels + c] =
                src >= 0 ? to_float(in[static_cast<size_t>(q_start + src) * in_stride + c])
                         : carried[static_cast<size_t>(j + q_len) * channels + c];
        }
    }
}

WLLM_API int wllm_causal_conv(const void* in, long long in_stride, const float* weight, const float* bias, float* state,
                              long long state_stride, long long carried_offset, const int* token_segment,
                              const int* seg_q_start, const int* seg_q_len, const int* state_slots, void* out,
                              int is_bf16, int tokens, int segments, int channels, int taps, hipStream_t stream) {
    if (tokens <= 0 || segments <= 0) return 0;
    if (channels <= 0 || taps < 1 || taps > 64) return -1;
    const int tiles = (channels + 255) / 256 < 64 ? (channels + 255) / 256 : 64;
    const dim3 grid(tokens, tiles), carry_grid(segments, tiles);
    if (is_bf16)
        causal_conv_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(in), in_stride, weight, bias, state,
                                                           state_stride, carried_offset, token_segment, seg_q_start,
                                                           state_slots, static_cast<bf16*>(out), channels, taps);
    else
        causal_conv_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(in), in_stride, weight, bias, state,
                                                            state_stride, carried_offset, token_segment, seg_q_start,
                                                            state_slots, static_cast<float*>(out), channels, taps);
    if (const int err = launch_status()) return err;
    if (taps == 1) return 0;
    if (is_bf16)
        conv_carry_kernel<bf16><<<carry_grid, 256, 0, stream>>>(static_cast<const bf16*>(in), in_stride, state, state_stride,
                                                                carried_offset, seg_q_start, seg_q_len, state_slots, channels,
                                                                taps);
    else
        conv_carry_kernel<float><<<carry_grid, 256, 0, stream>>>(static_cast<const float*>(in), in_stride, state,
                                                                 state_stride, carried_offset, seg_q_start, seg_q_len,
                                                                 state_slots, channels, taps);
    return launch_status();
}

// ---- the same convolution on the residual stream itself, in front of a sublayer that reads the stream:
// out[t, c] = x[t, c] + sum_k w[k, c] * x[t - (taps - 1) + k, c] (w a row a tap, [taps, channels]), float32 sums in this order, no bias and no
// activation; x float32 [tokens, channels], out the activation type.  The carried rows (the request's last
// taps - 1 rows of x, the oldest first) are kept by `conv_carry_kernel`, as above; or, CARRY (a step of single
// tokens, where no other token of the launch reads a request's carried rows), by the token's own threads, each
// moving its channel's rows up by one as it reads them: one launch instead of two, the same sums. ----
template <typename T, bool CARRY>
__global__ void __launch_bounds__(256)
stream_conv_kernel(const float* __restrict__ x, const float* __restrict__ weight, float* __restrict__ state,
                   long long state_stride, long long carried_offset, const int* __restrict__ token_segment,
                   const int* __restrict__ seg_q_start, const int* __restrict__ state_slots, T* __restrict__ out,
                   int channels, int taps) {
    const int token = blockIdx.x;
    const int seg = token_segment[token];
    const int local = token - seg_q_start[seg];
    float* carried = state + static_cast<size_t>(state_slots[seg]) * state_stride + carried_offset;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
        float acc = x[static_cast<size_t>(token) * channels + c];
        if (CARRY) {
            // the segment is this one token: every earlier input is a carried row
            const float now = acc;
            for (int k = 0; k + 1 < taps; ++k) {
                const float v = carried[static_cast<size_t>(k) * channels + c];
                acc = fmaf(weight[static_cast<size_t>(k) * channels + c], v, acc);
                if (k > 0) carried[static_cast<size_t>(k - 1) * channels + c] = v;
            }
            acc = fmaf(weight[static_cast<size_t>(taps - 1) * channels + c], now, acc);
            if (taps > 1) carried[static_cast<size_t>(taps - 2) * channels + c] = now;
            out[static_cast<size_t>(token) * channels + c] = from_float<T>(acc);
            continue;
        }
        for (int k = 0; k < taps; ++k) {
            const int src = local - (taps - 1) + k;
            const float v = src >= 0 ? x[static_cast<size_t>(token - local + src) * channels + c]
                                     : carried[static_cast<size_t>(taps - 1 + src) * channels + c];
            acc = fmaf(weight[static_cast<size_t>(k) * channels + c], v, acc);
        }
        out[static_cast<size_t>(token) * channels + c] = from_float<T>(acc);
    }
}

// The same sums, four consecutive channels a thread with 16-byte loads of x and of the carried rows (a prompt's
// portion: the kernel is bound by what it moves).  Channels, the carried rows' offset and the state's row are
// multiples of four floats.
template <typename T> struct alignas(4 * sizeof(T)) ConvFour { T v[4]; };

template <typename T>
__global__ void __launch_bounds__(256)
stream_conv_four_kernel(const float* __restrict__ x, const float* __restrict__ weight, const float* __restrict__ state,
                        long long state_stride, long long carried_offset, const int* __restrict__ token_segment,
                        const int* __restrict__ seg_q_start, const int* __restrict__ state_slots, T* __restrict__ out,
                        int channels, int taps) {
    const int token = blockIdx.x;
    const int seg = token_segment[token];
    const int local = token - seg_q_start[seg];
    const float* carried = state + static_cast<size_t>(state_slots[seg]) * state_stride + carried_offset;
    for (int c = (blockIdx.y * blockDim.x + threadIdx.x) * 4; c < channels; c += gridDim.y * blockDim.x * 4) {
        const float4 now = *reinterpret_cast<const float4*>(x + static_cast<size_t>(token) * channels + c);
        float acc[4] = {now.x, now.y, now.z, now.w};
        for (int k = 0; k < taps; ++k) {
            const int src = local - (taps - 1) + k;
            const float4 v = *reinterpret_cast<const float4*>(
                src >= 0 ? x + static_cast<size_t>(token - local + src) * channels + c
                         : carried + static_cast<size_t>(taps - 1 + src) * channels + c);
            const float4 w = *reinterpret_cast<const float4*>(weight + static_cast<size_t>(k) * channels + c);
            acc[0] = fmaf(w.x, v.x, acc[0]);
            acc[1] = fmaf(w.y, v.y, acc[1]);
            acc[2] = fmaf(w.z, v.z, acc[2]);
            acc[3] = fmaf(w.w, v.w, acc[3]);
        }
        ConvFour<T> r;
#pragma unroll
        for (int u = 0; u < 4; ++u) r.v[u] = from_float<T>(acc[u]);
        *reinterpret_cast<ConvFour<T>*>(out + static_cast<size_t>(token) * channels + c) = r;
    }
}

WLLM_API int wllm_stream_conv(const float* x, const float* weight, float* state, long long state_stride,
                              long long carried_offset, const int* token_segment, const int* seg_q_start,
                              const int* seg_q_len, const int* state_slots, void* out, int out_bf16, int tokens,
                              int segments, int channels, int taps, int single_tokens, hipStream_t stream) {
    if (tokens <= 0 || segments <= 0) return 0;
    if (channels <= 0 || taps < 1 || taps > 64) return -1;
    if (single_tokens && tokens != segments) return -1;      // `single_tokens`: every segment is one token
    const int tiles = (channels + 255) / 256 < 64 ? (channels + 255) / 256 : 64;
    const dim3 grid(tokens, tiles), carry_grid(segments, tiles);
    const bool four = !single_tokens && channels % 4 == 0 && state_stride % 4 == 0 && carried_offset % 4 == 0 &&
                      reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(state) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(weight) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(out) % 16 == 0;
    if (four) {
        const dim3 grid4(tokens, (channels / 4 + 255) / 256);
        if (out_bf16)
            stream_conv_four_kernel<bf16><<<grid4, 256, 0, stream>>>(x, weight, state, state_stride, carried_offset,
                                                                     token_segment, seg_q_start, state_slots,
                                                                     static_cast<bf16*>(out), channels, taps);
        else
            stream_conv_four_kernel<float><<<grid4, 256, 0, stream>>>(x, weight, state, state_stride, carried_offset,
                                                                      token_segment, seg_q_start, state_slots,
                                                                      static_cast<float*>(out), channels, taps);
        if (const int err = launch_status()) return err;
        if (taps == 1) return 0;
        conv_carry_kernel<float><<<carry_grid, 256, 0, stream>>>(x, channels, state, state_stride, carried_offset, seg_q_start,
                                                                 seg_q_len, state_slots, channels, taps);
        return launch_status();
    }
#define LAUNCH(T, CARRY)                                                                                              \
    stream_conv_kernel<T, CARRY><<<grid, 256, 0, stream>>>(x, weight, state, state_stride, carried_offset, token_segment, \
                                                           seg_q_start, state_slots, static_cast<T*>(out), channels, taps)
    if (out_bf16) { if (single_tokens) LAUNCH(bf16, true); else LAUNCH(bf16, false); }
    else { if (single_tokens) LAUNCH(float, true); else LAUNCH(float, false); }
#undef LAUNCH
    if (const int err = launch_status()) return err;
    if (taps == 1 || single_tokens) return 0;
    conv_carry_kernel<float><<<carry_grid, 256, 0, stream>>>(x, channels, state, state_stride, carried_offset, seg_q_start,
                                                             seg_q_len, state_slots, channels, taps);
    return launch_status();
}

// ---- the recurrence.  Per head h (group g = h / (heads / groups)), token by token:
//   dt = softplus(dt_in + dt_bias[h]);  S = exp(-exp(A_log[h]) * dt) * S + dt * B_t x_t^T;  y_t = S^T C_t + D[h] x_t
// with S [N, P], B_t and C_t [N] of the group, x_t [P] of the head.  xbc [tokens, heads*P + 2*groups*N]
// holds x, then B, then C.  The step sizes and decays of all tokens and heads are made first, by a
// kernel of their own (`ssm_steps_kernel`: softplus and two exponentials a value, out of the token
// loop).  Then a workgroup owns (head, segment, 16 columns of P) and walks the segment's tokens in
// order.  N is cut into 32 slices: a lane is (column, one of four slices), a wavefront four slices,
// the workgroup's eight wavefronts all of them; a lane keeps its R rows of its column of S in
// registers.  So a head of 64 columns is four workgroups, a prompt's 64 heads fill 256 compute units
// with two wavefronts a SIMD (one multiplies while the other waits for shared memory), and a lane's
// chain of dependent multiply-adds a token is R long (4 at N = 128).  Measured at 64 heads of 64 with
// 128 rows of state, a prompt of 2,048 tokens / 64 decoded tokens / 8 portions of 256: four wavefronts
// a workgroup 787 / 83 / 290 us, eight 572 / 88 / 291, sixteen 682 / 113 / 466; eight with 32 tokens a
// chunk 564 / 105 / 335; 8 columns a workgroup (a lane's 32 bytes of a row of S are half a memory
// transaction) 654 / 134 / 409.  Tokens are staged 16 at a time through shared memory
// (B, C, x, step, decay), the next 16 fetched into registers meanwhile; a token's y is the slices'
// partial sums added in a fixed order (within the wavefront, then wavefront by wavefront), so it has
// the same bits whether the token came alone or inside a prompt. ----
constexpr int kScanTokens = 16;
constexpr int kScanWaves = 8;
constexpr int kScanCols = 16;                       // columns of P a workgroup owns
constexpr int kScanLaneSlices = kWave / kScanCols;  // slices of N side by side in a wavefront
constexpr int kScanSlices = kScanWaves * kScanLaneSlices;
constexpr int kScanFetchers = kWave * kScanWaves / kScanTokens;    // threads that fetch one token's B, C and x of a chunk
static_assert(kScanFetchers >= kScanCols && (kScanLaneSlices == 4 || kScanLaneSlices == 8),
              "a token's fetchers cover its columns of x; the lane sums below are for 4 or 8 slices");

__device__ __forceinline__ float softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// steps[0][t][h] = softplus(dt_in[t][h] + dt_bias[h]); steps[1][t][h] = exp(-exp(a_log[h]) * steps[0][t][h])
template <typename T>
__global__ void ssm_steps_kernel(const T* __restrict__ dt_in, long long dt_stride, const float* __restrict__ dt_bias,
                                 const float* __restrict__ a_log, float* __restrict__ steps, int tokens, int heads) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= tokens * heads) return;
    const int t = e / heads, h = e - t * heads;
    const float dt = softplus(to_float(dt_in[static_cast<size_t>(t) * dt_stride + h]) + dt_bias[h]);
    steps[e] = dt;
    steps[static_cast<size_t>(tokens) * heads + e] = expf(-expf(a_log[h]) * dt);
}

// VEC: N is a multiple of 4 and so is R, so a lane's rows of B and C are runs of float4 in shared memory.
// F: elements of B (of C) one of a token's 16 fetchers brings.
template <typename T, int R, int F, bool VEC>
__global__ void __launch_bounds__(kWave * kScanWaves)
ssm_scan_kernel(const T* __restrict__ xbc, const float* __restrict__ steps, int tokens,
                const float* __restrict__ d_skip, float* __restrict__ state, long long state_stride, const int* __restrict__ seg_q_start,
                const int* __restrict__ seg_q_len, const int* __restrict__ state_slots, float* __restrict__ y, int heads,
                int groups, int n_state, int p_dim) {
    extern __shared__ __align__(16) float smem[];
    const int h = blockIdx.x, seg = blockIdx.y, p0 = blockIdx.z * kScanCols;
    const int q_len = seg_q_len[seg], q_start = seg_q_start[seg];
    if (q_len <= 0) return;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int col = lane % kScanCols, slice = wave * kScanLaneSlices + lane / kScanCols;
    const int p = p0 + col;
    const bool live = p < p_dim;
    const int g = h / (heads / groups);
    const int inner = heads * p_dim, channels = inner + 2 * groups * n_state;
    const int b_col = inner + g * n_state, c_col = inner + groups * n_state + g * n_state;
    const int n_pad = (n_state + 3) / 4 * 4;             // a token's row of B (of C) in shared memory
    float* b_s = smem;                                   // [kScanTokens][n_pad]
    float* c_s = b_s + kScanTokens * n_pad;              // [kScanTokens][n_pad]
    float* x_s = c_s + kScanTokens * n_pad;              // [kScanTokens][kScanCols]
    float* dt_s = x_s + kScanTokens * kScanCols;         // [kScanTokens]
    float* decay_s = dt_s + kScanTokens;                 // [kScanTokens]
    float* part_s = decay_s + kScanTokens;               // [kScanTokens][kScanWaves][kScanCols]
    float* s_rows = state + static_cast<size_t>(state_slots[seg]) * state_stride + static_cast<size_t>(h) * n_state * p_dim;
    const int n0 = slice * R;
    float s[R];
#pragma unroll
    for (int i = 0; i < R; ++i) s[i] = (live && n0 + i < n_state) ? s_rows[static_cast<size_t>(n0 + i) * p_dim + p] : 0.f;
    const float skip = d_skip[h];
    // What a thread fetches of a chunk of 16 tokens, into registers while the chunk before is worked on:
    // of token `ft` of the chunk, F elements of B and of C (thread = 16 ft + fq takes the fq-th run), one
    // element of x, and (the first 16 threads) a token's step size and decay.
    const int ft = threadIdx.x / kScanFetchers, fq = threadIdx.x % kScanFetchers;
    float pb[F], pc[F], px = 0.f, pdt = 0.f, pdecay = 0.f;
    auto fetch = [&](int t0) {
        const int count = min(kScanTokens, q_len - t0);
        if (ft < count) {
            const T* row = xbc + static_cast<size_t>(q_start + t0 + ft) * channels;
#pragma unroll
            for (int i = 0; i < F; ++i) {
                const int n = fq * F + i;
                pb[i] = n < n_state ? to_float(row[b_col + n]) : 0.f;
                pc[i] = n < n_state ? to_float(row[c_col + n]) : 0.f;
            }
            px = (fq < kScanCols && p0 + fq < p_dim) ? to_float(row[h * p_dim + p0 + fq]) : 0.f;
        }
        if (threadIdx.x < count) {
            const size_t at = static_cast<size_t>(q_start + t0 + threadIdx.x) * heads + h;
            pdt = steps[at];
            pdecay = steps[static_cast<size_t>(tokens) * heads + at];
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < q_len; t0 += kScanTokens) {
        const int count = min(kScanTokens, q_len - t0);
        __syncthreads();                                 // the chunk before is read out
        if (ft < count) {
#pragma unroll
            for (int i = 0; i < F; ++i) {
                const int n = fq * F + i;
                if (n < n_pad) {
                    b_s[ft * n_pad + n] = pb[i];
                    c_s[ft * n_pad + n] = pc[i];
                }
            }
            if (fq < kScanCols) x_s[ft * kScanCols + fq] = px;
        }
        if (threadIdx.x < count) {
            dt_s[threadIdx.x] = pdt;
            decay_s[threadIdx.x] = pdecay;
        }
        __syncthreads();
        if (t0 + kScanTokens < q_len) fetch(t0 + kScanTokens);      // in flight while this chunk is worked on
        // (unrolled: a token's reads of shared memory are asked for while the token before it is multiplied)
#pragma unroll 4
        for (int t = 0; t < count; ++t) {
            const float decay = decay_s[t], dx = dt_s[t] * x_s[t * kScanCols + col];
            const float* bt = b_s + t * n_pad + n0;
            const float* ct = c_s + t * n_pad + n0;
            float part = 0.f;
            if (VEC) {
#pragma unroll
                for (int i = 0; i < R; i += 4) {
                    if (n0 + i < n_state) {              // whole groups of four: N and R are multiples of 4
                        const float4 bv = *reinterpret_cast<const float4*>(bt + i), cv = *reinterpret_cast<const float4*>(ct + i);
                        s[i] = fmaf(decay, s[i], dx * bv.x);
                        s[i + 1] = fmaf(decay, s[i + 1], dx * bv.y);
                        s[i + 2] = fmaf(decay, s[i + 2], dx * bv.z);
                        s[i + 3] = fmaf(decay, s[i + 3], dx * bv.w);
                        part = fmaf(s[i], cv.x, part);
                        part = fmaf(s[i + 1], cv.y, part);
                        part = fmaf(s[i + 2], cv.z, part);
                        part = fmaf(s[i + 3], cv.w, part);
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    if (n0 + i < n_state) {
                        s[i] = fmaf(decay, s[i], dx * bt[i]);
                        part = fmaf(s[i], ct[i], part);
                    }
                }
            }
            // the wavefront's slices of this column, in a fixed order
            part = sum_across(sum_across(part, 32), 16);
            if (kScanLaneSlices == 8) part += row_permuted<0x128>(part);
            if (lane < kScanCols) part_s[(t * kScanWaves + wave) * kScanCols + col] = part;
        }
        __syncthreads();
        for (int e = threadIdx.x; e < count * kScanCols; e += blockDim.x) {
            const int t = e / kScanCols, l = e % kScanCols;
            if (p0 + l >= p_dim) continue;
            float total = part_s[(t * kScanWaves) * kScanCols + l];
#pragma unroll
            for (int w = 1; w < kScanWaves; ++w) total += part_s[(t * kScanWaves + w) * kScanCols + l];
            total = fmaf(skip, x_s[e], total);
            y[static_cast<size_t>(q_start + t0 + t) * inner + h * p_dim + p0 + l] = total;
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < R; ++i)
            if (n0 + i < n_state) s_rows[static_cast<size_t>(n0 + i) * p_dim + p] = s[i];
    }
}

// `steps`: scratch of 2 * tokens * heads floats (the step sizes, then the decays).
WLLM_API int wllm_ssm_scan(const void* xbc, const void* dt_in, long long dt_stride, const float* dt_bias, const float* a_log,
                           const float* d_skip, float* state, long long state_stride, const int* seg_q_start,
                           const int* seg_q_len, const int* state_slots, float* y, float* steps, int is_bf16, int tokens,
                           int segments, int heads, int groups, int n_state, int p_dim, hipStream_t stream) {
    if (segments <= 0 || tokens <= 0) return 0;
    if (!steps) return -1;
    if (heads <= 0 || groups <= 0 || heads % groups != 0 || n_state <= 0 || n_state > 16 * kScanSlices || p_dim <= 0) return -1;
    if (segments > 65535 || (p_dim + kScanCols - 1) / kScanCols > 65535) return -1;
    const int r = (n_state + kScanSlices - 1) / kScanSlices;
    {
        const int total = tokens * heads, blocks = (total + 255) / 256;
        if (is_bf16)
            ssm_steps_kernel<bf16><<<blocks, 256, 0, stream>>>(static_cast<const bf16*>(dt_in), dt_stride, dt_bias, a_log, steps,
                                                               tokens, heads);
        else
            ssm_steps_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<const float*>(dt_in), dt_stride, dt_bias, a_log,
                                                                steps, tokens, heads);
        if (const int err = launch_status()) return err;
    }
    const int n_pad = (n_state + 3) / 4 * 4;
    const dim3 grid(heads, segments, (p_dim + kScanCols - 1) / kScanCols);
    const size_t smem = sizeof(float) * (2 * kScanTokens * n_pad + kScanTokens * kScanCols + 2 * kScanTokens +
                                         kScanTokens * kScanWaves * kScanCols);
#define LAUNCH(T, R, V)                                                                                             \
    ssm_scan_kernel<T, R, (R * kScanSlices + kScanFetchers - 1) / kScanFetchers, V><<<grid, kWave * kScanWaves, smem, stream>>>( \
        static_cast<const T*>(xbc), steps, tokens, d_skip, state, state_stride, seg_q_start, seg_q_len, state_slots, y, \
        heads, groups, n_state, p_dim)
#define LAUNCH_R(T)                                                                          \
    if (r <= 1) LAUNCH(T, 1, false);                                                         \
    else if (r <= 2) LAUNCH(T, 2, false);                                                    \
    else if (r <= 4) { if (n_state % 4 == 0) LAUNCH(T, 4, true); else LAUNCH(T, 4, false); }   \
    else if (r <= 8) { if (n_state % 4 == 0) LAUNCH(T, 8, true); else LAUNCH(T, 8, false); }   \
    else { if (n_state % 4 == 0) LAUNCH(T, 16, true); else LAUNCH(T, 16, false); }
    if (is_bf16) { LAUNCH_R(bf16) } else { LAUNCH_R(float) }
#undef LAUNCH_R
#undef LAUNCH
    return launch_status();
}

// ---- out = rms_norm_in_groups(y * silu(z)) * weight: the recurrence's result (float32) gated by
// z (a band of a wider row, the activation type), then every one of `groups` equal parts of the row
// divided by its own root mean square, times the weight; out in the activation type.  One workgroup
// a (token, part). ----
template <typename T>
__global__ void __launch_bounds__(256)
gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ z, long long z_stride,
                        const float* __restrict__ weight, T* __restrict__ out, int width, int groups, float eps) {
    __shared__ float scratch[16];
    const int token = blockIdx.x, part = blockIdx.y;
    const int size = width / groups, c0 = part * size;
    const float* yr = y + static_cast<size_t>(token) * width + c0;
    const T* zr = z + static_cast<size_t>(token) * z_stride + c0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < size; i += blockDim.x) {
        const float zv = to_float(zr[i]);
        const float v = yr[i] * (zv / (1.f + expf(-zv)));
        ss += v * v;
    }
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(size) + eps);
    T* o = out + static_cast<size_t>(token) * width + c0;
    for (int i = threadIdx.x; i < size; i += blockDim.x) {
        const float zv = to_float(zr[i]);
        const float v = yr[i] * (zv / (1.f + expf(-zv)));
        o[i] = from_float<T>(v * inv * weight[c0 + i]);
    }
}

WLLM_API int wllm_gated_group_norm(const float* y, const void* z, long long z_stride, const float* weight, void* out,
                                   int is_bf16, int tokens, int width, int groups, float eps, hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (width <= 0 || groups <= 0 || width % groups != 0 || groups > 65535) return -1;
    const dim3 grid(tokens, groups);
    if (is_bf16)
        gated_group_norm_kernel<bf16><<<grid, 256, 0, stream>>>(y, static_cast<const bf16*>(z), z_stride, weight,
                                                                static_cast<bf16*>(out), width, groups, eps);
    else
        gated_group_norm_kernel<float><<<grid, 256, 0, stream>>>(y, static_cast<const float*>(z), z_stride, weight,
                                                                 static_cast<float*>(out), width, groups, eps);
    return launch_status();
}
