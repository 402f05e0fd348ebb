// A recurrent mixer whose state is a matrix a head (linear attention in its recurrent form) on a flat
// batch of segments.  A segment is the next tokens of one request; what a request carries from step to
// step lies in one float32 row of `state` per request (row state_slots[segment]):
//   [heads, D, P] the memory S, then (exponential gating only) [heads, D] the normaliser n and [heads] the
//   running maximum m.
// A fresh request's row is all zeros: S, n and m all start at zero.  Per head and token
//   S_t = a_t S_(t-1) + b_t k_t v_t^T,    o_t = S_t^T q_t / den_t
// with (a, b) either (the head's fixed decay, 1) and den = 1, or made from the two gates by `memory_gates`; then
// the normaliser n_t = a_t n_(t-1) + b_t k_t is one more column of the memory (a value that is always 1), the
// recurrence leaves n_t . q_t beside the columns' sums, and den_t = max(|n_t . q_t|, exp(-m_t)) + eps divides them
// where the heads are normed (`head_norm_gate`).
// Everything that enters the recurrence is float32: the rotated queries and keys, the gates, their
// exponentials, the maximum, the normaliser, the state and every sum.
#include "common.h"

// ---- queries and keys as the recurrence takes them: qk[0] = q_scale * rot(q), qk[1] = k_scale * rot(k), float32.
// row [n, >= 2 * heads * D] begins with the query heads, then the key heads.  The first rot_dims elements
// of a head turn by position * inv_freq[j], element j paired with j + rot_dims / 2. ----
template <typename T>
__global__ void __launch_bounds__(256)
memory_inputs_kernel(const T* __restrict__ row, long long row_stride, const int* __restrict__ positions,
                     const float* __restrict__ inv_freq, float* __restrict__ qk, int tokens, int heads, int d, int rot_dims,
                     float q_scale, float k_scale) {
    const int token = blockIdx.x;
    const int width = heads * d, half = rot_dims / 2;
    const float pos = static_cast<float>(positions[token]);
    const T* r = row + static_cast<size_t>(token) * row_stride;
    for (int e = blockIdx.y * blockDim.x + threadIdx.x; e < 2 * width; e += gridDim.y * blockDim.x) {
        const int which = e / width, j = e % d;
        float v = to_float(r[e]);
        if (j < rot_dims) {
            const int f = j < half ? j : j - half;
            float sn, cs, ra, rb;
            sincosf(pos * inv_freq[f], &sn, &cs);
            if (j < half) {
                rotate_pair(v, to_float(r[e + half]), sn, cs, ra, rb);
                v = ra;
            } else {
                rotate_pair(to_float(r[e - half]), v, sn, cs, ra, rb);
                v = rb;
            }
        }
        qk[static_cast<size_t>(which) * tokens * width + static_cast<size_t>(token) * width + (e - which * width)] =
            v * (which ? k_scale : q_scale);
    }
}

WLLM_API int wllm_memory_inputs(const void* row, long long row_stride, const int* positions, const float* inv_freq,
                                float* qk, int is_bf16, int tokens, int heads, int d, int rot_dims, float q_scale,
                                float k_scale, hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (heads <= 0 || d <= 0 || rot_dims < 0 || rot_dims > d || rot_dims % 2 || (rot_dims && !inv_freq)) return -1;
    const int tiles = (2 * heads * d + 255) / 256 < 64 ? (2 * heads * d + 255) / 256 : 64;
    const dim3 grid(tokens, tiles);
    if (is_bf16)
        memory_inputs_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(row), row_stride, positions, inv_freq,
                                                             qk, tokens, heads, d, rot_dims, q_scale, k_scale);
    else
        memory_inputs_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(row), row_stride, positions,
                                                              inv_freq, qk, tokens, heads, d, rot_dims, q_scale, k_scale);
    return launch_status();
}

// ---- a forget gate a channel that also decides what is written (the gating of HGRN2): from a row that begins
// with the query heads and then the forget gate's projection z (heads * D columns each),
//   f = lower + (1 - lower) * sigmoid(z + bias),   qkf[0] = act(q) (0: as it is, 1: silu),   qkf[1] = 1 - f,   qkf[2] = f
// all float32: the recurrence S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T then is `memory_scan` with 1 - f in the
// keys' place and f as a decay a row. ----
template <typename T>
__global__ void __launch_bounds__(256)
memory_forget_inputs_kernel(const T* __restrict__ row, long long row_stride, const float* __restrict__ bias,
                            const float* __restrict__ lower, float* __restrict__ qkf, int tokens, int width, int q_act) {
    const int token = blockIdx.x;
    const T* r = row + static_cast<size_t>(token) * row_stride;
    const size_t plane = static_cast<size_t>(tokens) * width;
    for (int e = blockIdx.y * blockDim.x + threadIdx.x; e < width; e += gridDim.y * blockDim.x) {
        const float q = to_float(r[e]);
        const float z = to_float(r[width + e]) + (bias ? bias[e] : 0.f);
        const float l = lower ? lower[e] : 0.f;
        const float f = l + (1.f - l) * (1.f / (1.f + expf(-z)));
        const size_t at = static_cast<size_t>(token) * width + e;
        qkf[at] = q_act == 1 ? q / (1.f + expf(-q)) : q;
        qkf[plane + at] = 1.f - f;
        qkf[2 * plane + at] = f;
    }
}

WLLM_API int wllm_memory_forget_inputs(const void* row, long long row_stride, const float* bias, const float* lower,
                                       float* qkf, int is_bf16, int tokens, int width, int q_act, hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (width <= 0 || q_act < 0 || q_act > 1) return -1;
    const int tiles = (width + 255) / 256 < 64 ? (width + 255) / 256 : 64;
    const dim3 grid(tokens, tiles);
    if (is_bf16)
        memory_forget_inputs_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(row), row_stride, bias, lower,
                                                                    qkf, tokens, width, q_act);
    else
        memory_forget_inputs_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(row), row_stride, bias, lower,
                                                                     qkf, tokens, width, q_act);
    return launch_status();
}

// ---- exponential gates held in range by a running maximum.  Per head and token, with the gate
// projections z_i, z_f (a band [n, 2 * heads] of a wider row: the input gates, then the forget gates):
//   i = cap * tanh((z_i + bias_i) / cap)                 (cap <= 0: no cap)
//   f = logsigmoid(cap * tanh((z_f + bias_f) / cap))
//   m_t = max(f + m_(t-1), i);  a = exp(f + m_(t-1) - m_t);  b = exp(i - m_t);  floor = exp(-m_t)
// steps[0], [1], [2] [n, heads] take a, b and floor; m is read from and left in the request's row (one float a
// head from `m_offset`).  One wavefront a (head, segment), 64 tokens at a time: a lane bends its token's gates,
// the chain of maxima (an addition and a maximum a token, the same operations in the same order however the
// tokens are cut into steps) runs over the 64 in turn with every lane following it, and a lane takes the
// exponentials of its own token. ----
__device__ __forceinline__ float from_lane(float v, int lane) {      // `lane` is the same in every lane
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), lane));
}
__device__ __forceinline__ float bent(float z, float cap) { return cap > 0.f ? cap * tanhf(z / cap) : z; }
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename T>
__global__ void __launch_bounds__(kWave)
memory_gates_kernel(const T* __restrict__ gates, long long gates_stride, const float* __restrict__ i_bias,
                    const float* __restrict__ f_bias, float cap, float* __restrict__ state, long long state_stride,
                    long long m_offset, const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                    const int* __restrict__ state_slots, float* __restrict__ steps, int tokens, int heads) {
    const int h = blockIdx.x, seg = blockIdx.y, lane = threadIdx.x;
    const int q_len = seg_q_len[seg], q_start = seg_q_start[seg];
    if (q_len <= 0) return;
    const size_t all = static_cast<size_t>(tokens) * heads;
    float* m_at = state + static_cast<size_t>(state_slots[seg]) * state_stride + m_offset + h;
    float m = *m_at;
    const float bi = i_bias ? i_bias[h] : 0.f, bf = f_bias ? f_bias[h] : 0.f;
    for (int t0 = 0; t0 < q_len; t0 += kWave) {
        const int count = min(kWave, q_len - t0);
        float li = 0.f, lf = 0.f;
        if (lane < count) {
            const T* g = gates + static_cast<size_t>(q_start + t0 + lane) * gates_stride;
            li = bent(to_float(g[h]) + bi, cap);
            lf = log_sigmoid(bent(to_float(g[heads + h]) + bf, cap));
        }
        float m_before = 0.f, m_mine = 0.f;
        auto follow = [&](int t) {
            const float m_new = fmaxf(from_lane(lf, t) + m, from_lane(li, t));
            if (lane == t) {
                m_before = m;
                m_mine = m_new;
            }
            m = m_new;
        };
        if (count == kWave) {
#pragma unroll
            for (int t = 0; t < kWave; ++t) follow(t);
        } else {
            for (int t = 0; t < count; ++t) follow(t);
        }
        if (lane < count) {
            const size_t at = static_cast<size_t>(q_start + t0 + lane) * heads + h;
            steps[at] = expf(lf + m_before - m_mine);
            steps[all + at] = expf(li - m_mine);
            steps[2 * all + at] = expf(-m_mine);
        }
    }
    if (lane == 0) *m_at = m;
}

WLLM_API int wllm_memory_gates(const void* gates, long long gates_stride, const float* i_bias, const float* f_bias, float cap,
                               float* state, long long state_stride, long long m_offset, const int* seg_q_start,
                               const int* seg_q_len, const int* state_slots, float* steps, int is_bf16, int tokens,
                               int segments, int heads, hipStream_t stream) {
    if (tokens <= 0 || segments <= 0) return 0;
    if (heads <= 0 || segments > 65535) return -1;
    const dim3 grid(heads, segments);
    if (is_bf16)
        memory_gates_kernel<bf16><<<grid, kWave, 0, stream>>>(static_cast<const bf16*>(gates), gates_stride, i_bias, f_bias, cap,
                                                              state, state_stride, m_offset, seg_q_start, seg_q_len,
                                                              state_slots, steps, tokens, heads);
    else
        memory_gates_kernel<float><<<grid, kWave, 0, stream>>>(static_cast<const float*>(gates), gates_stride, i_bias, f_bias,
                                                               cap, state, state_stride, m_offset, seg_q_start, seg_q_len,
                                                               state_slots, steps, tokens, heads);
    return launch_status();
}

// ---- the recurrence itself.  A workgroup owns (head, segment, 16 columns of P) and walks the segment's
// tokens in order.  D is cut into 32 slices: a lane is (column, one of four slices), a wavefront four
// slices, the workgroup's eight wavefronts all of them; a lane keeps its R rows of its column of S in
// registers.  Tokens go 16 at a time through shared memory (q, k, v, a, b), the next 16 fetched into registers
// while these are walked; a token's sum is the slices' partial sums added in a fixed order (within the
// wavefront, then wavefront by wavefront), so it has the same bits whether the token came alone or inside a
// prompt.  With `steps` the column behind the last (p = P) is the normaliser: its value is 1 for every token,
// its rows lie at `n_offset` of the request's row, and its sums go to `nq` [tokens, heads]. ----
constexpr int kMemTokens = 16;
constexpr int kMemWaves = 8;
constexpr int kMemCols = 16;
constexpr int kMemSlices = kMemWaves * (kWave / kMemCols);
constexpr int kMemThreads = kWave * kMemWaves;

template <typename T, int R, bool ROWS>
__global__ void __launch_bounds__(kMemThreads)
memory_scan_kernel(const float* __restrict__ qk, const T* __restrict__ v, long long v_stride, const float* __restrict__ steps,
                   const float* __restrict__ decays, float* __restrict__ state, long long state_stride, long long n_offset,
                   const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len, const int* __restrict__ state_slots,
                   float* __restrict__ y, float* __restrict__ nq, int tokens, int heads, int d, int p_dim) {
    constexpr int kRow = kMemSlices * R;                   // a token's row of q (and of k) in shared memory: d and zeros
    constexpr int kPasses = kMemTokens * kRow / kMemThreads;      // elements of q (and of k) a thread stages: R
    constexpr int kRowsPass = kMemThreads / kRow;          // tokens a pass covers
    __shared__ __align__(16) float q_s[kMemTokens * kRow];
    __shared__ __align__(16) float k_s[kMemTokens * kRow];
    __shared__ __align__(16) float f_s[ROWS ? kMemTokens * kRow : 1];      // ROWS: a decay a row of S and token
    __shared__ float v_s[kMemTokens * kMemCols];
    __shared__ float a_s[kMemTokens], b_s[kMemTokens];
    __shared__ float part_s[kMemTokens * kMemWaves * kMemCols];
    const int h = blockIdx.x, seg = blockIdx.y, p0 = blockIdx.z * kMemCols;
    const int q_len = seg_q_len[seg], q_start = seg_q_start[seg];
    if (q_len <= 0) return;
    const int tid = threadIdx.x;
    const int lane = tid % kWave, wave = tid / kWave;
    const int col = lane % kMemCols, slice = wave * (kWave / kMemCols) + lane / kMemCols;
    const int p = p0 + col;
    const bool norm_col = steps != nullptr && p == p_dim;
    const bool live = p < p_dim || norm_col;
    const size_t width = static_cast<size_t>(heads) * d, all = static_cast<size_t>(tokens) * heads;
    float* request = state + static_cast<size_t>(state_slots[seg]) * state_stride;
    // this lane's column of the state: rows p_dim apart in S, or the normaliser's rows one after the other
    float* s_rows = norm_col ? request + n_offset + static_cast<size_t>(h) * d : request + static_cast<size_t>(h) * d * p_dim + p;
    const size_t s_step = norm_col ? 1 : p_dim;
    const int n0 = slice * R;
    float s[R];
#pragma unroll
    for (int i = 0; i < R; ++i) s[i] = (live && n0 + i < d) ? s_rows[static_cast<size_t>(n0 + i) * s_step] : 0.f;
    const float fixed = decays ? decays[h] : 1.f;

    // what this thread stages of every 16 tokens: element `sj` of the rows of tokens st, st + kRowsPass, ... of q and of
    // k (zeros beyond d: a row of S that is not there stays zero and adds nothing), one value of v, one token's a and b
    const int sj = tid % kRow, st = tid / kRow;
    const int vt = tid / kMemCols, vc = tid % kMemCols;
    float q_r[kPasses], k_r[kPasses], f_r[ROWS ? kPasses : 1], v_r = 0.f, a_r = 1.f, b_r = 1.f;
    auto fetch = [&](int t0) {
        const int count = min(kMemTokens, q_len - t0);
#pragma unroll
        for (int u = 0; u < kPasses; ++u) {
            const int t = st + u * kRowsPass;
            q_r[u] = k_r[u] = 0.f;
            if (ROWS) f_r[u] = 0.f;
            if (sj < d && t < count) {
                const size_t at = static_cast<size_t>(q_start + t0 + t) * width + static_cast<size_t>(h) * d + sj;
                q_r[u] = qk[at];
                k_r[u] = qk[static_cast<size_t>(tokens) * width + at];
                if (ROWS) f_r[u] = qk[2 * static_cast<size_t>(tokens) * width + at];
            }
        }
        if (tid < kMemTokens * kMemCols) {
            v_r = 0.f;
            if (vt < count) {
                if (p0 + vc < p_dim)
                    v_r = to_float(v[static_cast<size_t>(q_start + t0 + vt) * v_stride + static_cast<size_t>(h) * p_dim + p0 + vc]);
                else if (steps != nullptr && p0 + vc == p_dim)
                    v_r = 1.f;
            }
        }
        if (tid < count) {
            const size_t at = static_cast<size_t>(q_start + t0 + tid) * heads + h;
            a_r = steps ? steps[at] : fixed;
            b_r = steps ? steps[all + at] : 1.f;
        }
    };
    auto place = [&]() {
#pragma unroll
        for (int u = 0; u < kPasses; ++u) {
            q_s[(st + u * kRowsPass) * kRow + sj] = q_r[u];
            k_s[(st + u * kRowsPass) * kRow + sj] = k_r[u];
            if (ROWS) f_s[(st + u * kRowsPass) * kRow + sj] = f_r[u];
        }
        if (tid < kMemTokens * kMemCols) v_s[tid] = v_r;
        if (tid < kMemTokens) {
            a_s[tid] = a_r;
            b_s[tid] = b_r;
        }
    };
    auto token = [&](int t) {
        const float a = a_s[t], bv = b_s[t] * v_s[t * kMemCols + col];
        const float* kt = k_s + t * kRow + n0;
        const float* qt = q_s + t * kRow + n0;
        const float* ft = f_s + (ROWS ? t * kRow + n0 : 0);
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            s[i] = fmaf(ROWS ? ft[i] : a, s[i], bv * kt[i]);
            part = fmaf(s[i], qt[i], part);
        }
        part = sum_across(sum_across(part, 32), 16);      // the wavefront's four slices of this column
        if (lane < kMemCols) part_s[(t * kMemWaves + wave) * kMemCols + col] = part;
    };

    fetch(0);
    for (int t0 = 0; t0 < q_len; t0 += kMemTokens) {
        const int count = min(kMemTokens, q_len - t0);
        place();
        __syncthreads();
        if (t0 + kMemTokens < q_len) fetch(t0 + kMemTokens);     // on their way while these 16 are walked
        if (count == kMemTokens) {
#pragma unroll
            for (int t = 0; t < kMemTokens; ++t) token(t);
        } else {
            for (int t = 0; t < count; ++t) token(t);
        }
        __syncthreads();
        for (int e = tid; e < count * kMemCols; e += kMemThreads) {
            const int t = e / kMemCols, l = e % kMemCols;
            if (p0 + l > p_dim || (p0 + l == p_dim && steps == nullptr)) continue;
            float total = part_s[(t * kMemWaves) * kMemCols + l];
#pragma unroll
            for (int w = 1; w < kMemWaves; ++w) total += part_s[(t * kMemWaves + w) * kMemCols + l];
            if (p0 + l == p_dim) nq[static_cast<size_t>(q_start + t0 + t) * heads + h] = total;
            else y[static_cast<size_t>(q_start + t0 + t) * heads * p_dim + static_cast<size_t>(h) * p_dim + p0 + l] = total;
        }
        // (the next round's `place` writes q, k, v, a, b, which nobody reads any more; its barrier stands between
        // these reads of the partial sums and the next writes to them)
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < R; ++i)
            if (n0 + i < d) s_rows[static_cast<size_t>(n0 + i) * s_step] = s[i];
    }
}

// `steps` (float32 [3, tokens, heads], of which a and b are read; then `nq` float32 [tokens, heads] takes the
// normaliser's sums and the normaliser lies at `n_offset` of a request's row) or, if null, `decays` (float32 [heads]; b = 1),
// or, with `row_decays`, neither: then qk has a third plane [tokens, heads * d] of decays a row and token (b = 1).
WLLM_API int wllm_memory_scan(const float* qk, const void* v, long long v_stride, const float* steps, const float* decays,
                              float* state, long long state_stride, long long n_offset, const int* seg_q_start,
                              const int* seg_q_len, const int* state_slots, float* y, float* nq, int is_bf16, int tokens,
                              int segments, int heads, int d, int p_dim, int row_decays, hipStream_t stream) {
    if (segments <= 0 || tokens <= 0) return 0;
    if (row_decays ? (steps || decays) : ((!steps) == (!decays) || (steps && !nq))) return -1;
    if (heads <= 0 || d <= 0 || d > 8 * kMemSlices || p_dim <= 0) return -1;
    if (segments > 65535 || (p_dim + kMemCols) / kMemCols > 65535) return -1;
    const int r = (d + kMemSlices - 1) / kMemSlices;
    const int columns = p_dim + (steps ? 1 : 0);
    const dim3 grid(heads, segments, (columns + kMemCols - 1) / kMemCols);
#define LAUNCH(T, R, ROWS)                                                                                          \
    memory_scan_kernel<T, R, ROWS><<<grid, kMemThreads, 0, stream>>>(qk, static_cast<const T*>(v), v_stride, steps, decays, \
                                                                     state, state_stride, n_offset, seg_q_start, seg_q_len, \
                                                                     state_slots, y, nq, tokens, heads, d, p_dim)
#define LAUNCH_R(T, ROWS)                  \
    if (r <= 1) LAUNCH(T, 1, ROWS);        \
    else if (r <= 2) LAUNCH(T, 2, ROWS);   \
    else if (r <= 4) LAUNCH(T, 4, ROWS);   \
    else LAUNCH(T, 8, ROWS);
    if (row_decays) {
        if (is_bf16) { LAUNCH_R(bf16, true) } else { LAUNCH_R(float, true) }
    } else {
        if (is_bf16) { LAUNCH_R(bf16, false) } else { LAUNCH_R(float, false) }
    }
#undef LAUNCH_R
#undef LAUNCH
    return launch_status();
}

// ---- out = o / rms_of_the_head(o) * weight * act(gate) * scale with o = y / den: the recurrence's sums (float32),
// divided by the head's denominator den = max(|nq|, floor) + den_eps if there is one (nq, floor float32 [tokens, heads]),
// every head divided by its own root mean square (eps inside the root), times a weight over the whole row (if
// any), times the gate's activation (0: sigmoid, 1: silu; 2: there is no gate) of a band of a wider row; out (the activation
// type) may be a band too.  One wavefront a (token, head). ----
template <typename T, int GATE>
__global__ void __launch_bounds__(kWave)
head_norm_gate_kernel(const float* __restrict__ y, const T* __restrict__ gate, long long gate_stride,
                      const float* __restrict__ weight, T* __restrict__ out, long long out_stride,
                      const float* __restrict__ nq, const float* __restrict__ floor, float den_eps, int heads, int p_dim,
                      float eps, float scale) {
    const int token = blockIdx.x, h = blockIdx.y;
    const float* yr = y + (static_cast<size_t>(token) * heads + h) * p_dim;
    const size_t th = static_cast<size_t>(token) * heads + h;
    const float den = nq ? fmaxf(fabsf(nq[th]), floor[th]) + den_eps : 1.f;
    float ss = 0.f;
    for (int i = threadIdx.x; i < p_dim; i += kWave) {
        const float o = yr[i] / den;
        ss = fmaf(o, o, ss);
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) / static_cast<float>(p_dim) + eps);
    const T* g = GATE == 2 ? nullptr : gate + static_cast<size_t>(token) * gate_stride + static_cast<size_t>(h) * p_dim;
    T* o = out + static_cast<size_t>(token) * out_stride + static_cast<size_t>(h) * p_dim;
    for (int i = threadIdx.x; i < p_dim; i += kWave) {
        float val = yr[i] / den * inv;
        if (weight) val *= weight[h * p_dim + i];
        if (GATE != 2) {
            const float z = to_float(g[i]);
            const float sg = 1.f / (1.f + expf(-z));
            val *= GATE == 0 ? sg : z * sg;
        }
        o[i] = from_float<T>(val * scale);
    }
}

WLLM_API int wllm_head_norm_gate(const float* y, const void* gate, long long gate_stride, const float* weight, void* out,
                                 long long out_stride, const float* nq, const float* floor, float den_eps, int is_bf16,
                                 int gate_kind, int tokens, int heads, int p_dim, float eps, float scale, hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (heads <= 0 || heads > 65535 || p_dim <= 0 || gate_kind < 0 || gate_kind > 2 || (!nq) != (!floor)) return -1;
    if (gate_kind != 2 && !gate) return -1;
    const dim3 grid(tokens, heads);
#define LAUNCH(T, G)                                                                                                   \
    head_norm_gate_kernel<T, G><<<grid, kWave, 0, stream>>>(y, static_cast<const T*>(gate), gate_stride, weight,       \
                                                            static_cast<T*>(out), out_stride, nq, floor, den_eps, heads, \
                                                            p_dim, eps, scale)
    if (is_bf16) { if (gate_kind == 0) LAUNCH(bf16, 0); else if (gate_kind == 1) LAUNCH(bf16, 1); else LAUNCH(bf16, 2); }
    else { if (gate_kind == 0) LAUNCH(float, 0); else if (gate_kind == 1) LAUNCH(float, 1); else LAUNCH(float, 2); }
#undef LAUNCH
    return launch_status();
}
