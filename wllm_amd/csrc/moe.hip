// A mixture of gated feed-forward experts on a flat batch of tokens: the router, the plan that sorts a
// step's (token, chosen expert) pairs by expert, and the two grouped products on the matrix cores.
//
//   router   z = W_r x (float32), s = softmax(z) over all experts; only experts of the `keep` best of
//            `groups` equal groups of neighbours (a group's score: its largest s) may be chosen; the `top`
//            allowed experts with the largest s are chosen, weights s / (sum of the chosen + eps)
//   plan     an assignment is a = token * top + slot.  The assignments of one expert lie together, in
//            tiles of 16 rows (the last tile of an expert padded with -1):
//            plan[0] = tiles in use; plan[1 + t] = expert of tile t; plan[1 + max_tiles + 16 t + r] = a or -1
//   up       act[a] = activation(x[token] Wg_e^T) * (x[token] Wu_e^T)
//   down     out[slot][token] = weight[a] * (act[a] Wd_e^T), float32: a stack of `top` partial sums that
//            whoever adds the feed-forward to the stream adds in order
// A row's sums run over k in ascending chunks whatever tile the row lies in, so a token's result does
// not depend on what else the batch holds.  Nothing is read on the host: the grid has room for the most
// tiles a step of its size can need and a workgroup beyond plan[0] leaves at once.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kMoeTile = 16;            // rows of a tile
constexpr int kMoeMaxExperts = 256;

// ---- the router: one wavefront a token ----
template <typename T>
__global__ void __launch_bounds__(256)
moe_route_kernel(const T* __restrict__ x, const float* __restrict__ router, int* __restrict__ ids, float* __restrict__ weights,
                 int tokens, int width, int experts, int top, int groups, int keep, float eps) {
    __shared__ float score_s[4][kMoeMaxExperts];
    __shared__ unsigned char open_s[4][kMoeMaxExperts];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int token = blockIdx.x * 4 + wave;
    if (token >= tokens) return;
    const T* xr = x + static_cast<size_t>(token) * width;
    float* sc = score_s[wave];
    unsigned char* open = open_s[wave];
    for (int e = 0; e < experts; ++e) {
        const float* w = router + static_cast<size_t>(e) * width;
        float dot = 0.f;
        for (int c = lane; c < width; c += kWave) dot = fmaf(to_float(xr[c]), w[c], dot);
        dot = wave_sum(dot);
        if (lane == 0) sc[e] = dot;
    }
    asm volatile("" ::: "memory");
    if (lane != 0) return;
    float mx = sc[0];
    for (int e = 1; e < experts; ++e) mx = fmaxf(mx, sc[e]);
    float sum = 0.f;
    for (int e = 0; e < experts; ++e) {
        sc[e] = expf(sc[e] - mx);
        sum += sc[e];
    }
    for (int e = 0; e < experts; ++e) {
        sc[e] /= sum;
        open[e] = 1;
    }
    if (keep < groups) {
        // a group is closed unless it is among the `keep` best: take the best open-able group `keep` times
        const int per = experts / groups;
        for (int e = 0; e < experts; ++e) open[e] = 0;
        for (int pick = 0; pick < keep; ++pick) {
            int best = -1;
            float best_score = -1.f;
            for (int g = 0; g < groups; ++g) {
                if (open[g * per]) continue;
                float top_of = sc[g * per];
                for (int j = 1; j < per; ++j) top_of = fmaxf(top_of, sc[g * per + j]);
                if (top_of > best_score) {
                    best_score = top_of;
                    best = g;
                }
            }
            for (int j = 0; j < per; ++j) open[best * per + j] = 1;
        }
    }
    float chosen_sum = 0.f;
    int* id = ids + static_cast<size_t>(token) * top;
    float* wt = weights + static_cast<size_t>(token) * top;
    for (int slot = 0; slot < top; ++slot) {
        int best = -1;
        float best_score = -1.f;
        for (int e = 0; e < experts; ++e) {
            if (open[e] == 1 && sc[e] > best_score) {
                best_score = sc[e];
                best = e;
            }
        }
        open[best] = 2;
        id[slot] = best;
        wt[slot] = best_score;
        chosen_sum += best_score;
    }
    const float denom = chosen_sum + eps;
    for (int slot = 0; slot < top; ++slot) wt[slot] /= denom;
}

WLLM_API int wllm_moe_route(const void* x, const float* router, int* ids, float* weights, int is_bf16, int tokens, int width,
                            int experts, int top, int groups, int keep, float eps, hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (experts <= 0 || experts > kMoeMaxExperts || groups <= 0 || experts % groups || keep <= 0 || keep > groups || top <= 0 ||
        top > keep * (experts / groups) || width <= 0)
        return -1;
    const int blocks = (tokens + 3) / 4;
    if (is_bf16)
        moe_route_kernel<bf16><<<blocks, 256, 0, stream>>>(static_cast<const bf16*>(x), router, ids, weights, tokens, width,
                                                           experts, top, groups, keep, eps);
    else
        moe_route_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<const float*>(x), router, ids, weights, tokens, width,
                                                            experts, top, groups, keep, eps);
    return launch_status();
}

// ---- the plan: one workgroup counts the assignments of every expert, gives each expert its tiles and
// every assignment a row.  Which row of its expert's tiles an assignment gets depends on the order in
// which threads arrive; a row's result does not depend on its place. ----
__global__ void __launch_bounds__(1024)
moe_plan_kernel(const int* __restrict__ ids, int* __restrict__ plan, int assignments, int experts, int max_tiles) {
    __shared__ int count_s[kMoeMaxExperts];
    __shared__ int first_s[kMoeMaxExperts + 1];      // first tile of every expert; [experts]: tiles in use
    int* tile_expert = plan + 1;
    int* rows = plan + 1 + max_tiles;
    for (int e = threadIdx.x; e < experts; e += blockDim.x) count_s[e] = 0;
    __syncthreads();
    for (int a = threadIdx.x; a < assignments; a += blockDim.x) atomicAdd(&count_s[ids[a]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int tiles = 0;
        for (int e = 0; e < experts; ++e) {
            first_s[e] = tiles;
            tiles += (count_s[e] + kMoeTile - 1) / kMoeTile;
        }
        first_s[experts] = tiles;
        plan[0] = tiles;
    }
    __syncthreads();
    const int tiles = first_s[experts];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) {
        for (int t = first_s[e]; t < first_s[e + 1]; ++t) tile_expert[t] = e;
        count_s[e] = 0;                              // from here on: rows of the expert already given out
    }
    for (int i = threadIdx.x; i < tiles * kMoeTile; i += blockDim.x) rows[i] = -1;
    __syncthreads();
    for (int a = threadIdx.x; a < assignments; a += blockDim.x) {
        const int e = ids[a];
        rows[first_s[e] * kMoeTile + atomicAdd(&count_s[e], 1)] = a;
    }
}

WLLM_API int wllm_moe_plan(const int* ids, int* plan, int assignments, int experts, int max_tiles, hipStream_t stream) {
    if (assignments <= 0) return 0;
    if (experts <= 0 || experts > kMoeMaxExperts || max_tiles < assignments / kMoeTile + experts) return -1;
    moe_plan_kernel<<<1, 1024, 0, stream>>>(ids, plan, assignments, experts, max_tiles);
    return launch_status();
}

// ---- fragments of the two products.  The weights are the A operand (a wavefront owns 16 output columns:
// lane (i, g) holds w[c0 + i][k + 8g .. +8]), a tile's rows the B operand (lane (i, g) holds row i's
// x[k + 8g .. +8]); the result lands as C[column 4g + v][row i].  bfloat16: v_mfma_f32_16x16x32_bf16, 32 keys
// an instruction.  float32: v_mfma_f32_16x16x4_f32 (IEEE float32 in and out), a lane holding 4 keys of a
// chunk of 16 and the t-th of four instructions taking keys 4g + t. ----
template <typename T> struct MoeFrag;
template <> struct MoeFrag<bf16> {
    static constexpr int kChunk = 32, kPer = 8;
    bf16x8_t v;
    __device__ __forceinline__ void load(const bf16* p, int k, int K, bool live) {
        union { uint4 u; bf16x8_t v; uint16_t s[8]; } t;
        t.u = make_uint4(0, 0, 0, 0);
        if (live) {
            if (K % 8 == 0) {
                if (k < K) t.u = *reinterpret_cast<const uint4*>(p + k);
            } else {
                for (int j = 0; j < 8; ++j) t.s[j] = k + j < K ? p[k + j].bits : 0;
            }
        }
        v = t.v;
    }
    static __device__ __forceinline__ float4_t mma(const MoeFrag& a, const MoeFrag& b, float4_t acc) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc, 0, 0, 0);
    }
};
template <> struct MoeFrag<float> {
    static constexpr int kChunk = 16, kPer = 4;
    float v[4];
    __device__ __forceinline__ void load(const float* p, int k, int K, bool live) {
        for (int j = 0; j < 4; ++j) v[j] = 0.f;
        if (live) {
            if (K % 4 == 0) {
                if (k < K) {
                    const float4 t = *reinterpret_cast<const float4*>(p + k);
                    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
                }
            } else {
                for (int j = 0; j < 4; ++j) v[j] = k + j < K ? p[k + j] : 0.f;
            }
        }
    }
    static __device__ __forceinline__ float4_t mma(const MoeFrag& a, const MoeFrag& b, float4_t acc) {
#pragma unroll
        for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[t], b.v[t], acc, 0, 0, 0);
        return acc;
    }
};

// act[a, c] = activation(x[token(a)] . Wg[e][c]) * (x[token(a)] . Wu[e][c]); w [experts, 2 * ff, K]: an
// expert's gate rows, then its up rows.  Grid (tiles, bands of 64 columns); a wavefront 16 columns.
template <typename T, int ACT>
__global__ void __launch_bounds__(256)
moe_up_kernel(const T* __restrict__ x, const T* __restrict__ w, const int* __restrict__ plan, int max_tiles,
              T* __restrict__ act, int K, int ff, int top) {
    const int tile = blockIdx.x;
    if (tile >= plan[0]) return;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int i = lane % 16, g = lane / 16;
    const int c0 = (blockIdx.y * 4 + wave) * 16;
    if (c0 >= ff) return;
    const int e = plan[1 + tile];
    const int* rows = plan + 1 + max_tiles + tile * kMoeTile;
    const int a_i = rows[i];
    const T* xr = x + static_cast<size_t>(a_i >= 0 ? a_i / top : 0) * K;
    const bool w_live = c0 + i < ff;
    const T* wg = w + (static_cast<size_t>(e) * 2 * ff + (w_live ? c0 + i : 0)) * K;
    const T* wu = wg + static_cast<size_t>(ff) * K;
    float4_t acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
    constexpr int kChunk = MoeFrag<T>::kChunk, kPer = MoeFrag<T>::kPer;
    for (int k0 = 0; k0 < K; k0 += kChunk) {
        MoeFrag<T> fx, fg, fu;
        const int k = k0 + g * kPer;
        fx.load(xr, k, K, a_i >= 0);
        fg.load(wg, k, K, w_live);
        fu.load(wu, k, K, w_live);
        acc_g = MoeFrag<T>::mma(fg, fx, acc_g);
        acc_u = MoeFrag<T>::mma(fu, fx, acc_u);
    }
    if (a_i < 0) return;
    T* out = act + static_cast<size_t>(a_i) * ff;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int c = c0 + 4 * g + v;
        if (c < ff) out[c] = from_float<T>(activate<ACT>(acc_g[v]) * acc_u[v]);
    }
}

WLLM_API int wllm_moe_up(const void* x, const void* w, const int* plan, int max_tiles, void* act, int is_bf16, int activation,
                         int K, int ff, int top, hipStream_t stream) {
    if (max_tiles <= 0) return 0;
    if (K <= 0 || ff <= 0 || top <= 0 || activation < 0 || activation >= kActivations || (ff + 63) / 64 > 65535) return -1;
    const dim3 grid(max_tiles, (ff + 63) / 64);
#define LAUNCH(T)                                                                                                     \
    WLLM_BY_ACTIVATION(activation, (moe_up_kernel<T, ACT><<<grid, 256, 0, stream>>>(                                  \
                                       static_cast<const T*>(x), static_cast<const T*>(w), plan, max_tiles,           \
                                       static_cast<T*>(act), K, ff, top)))
    if (is_bf16) { LAUNCH(bf16); } else { LAUNCH(float); }
#undef LAUNCH
    return launch_status();
}

// out[a % top][a / top][c] = weight[a] * (act[a] . Wd[e][c]); w [experts, width, ff]; out float32 [top, tokens, width].
template <typename T>
__global__ void __launch_bounds__(256)
moe_down_kernel(const T* __restrict__ act, const T* __restrict__ w, const int* __restrict__ plan, int max_tiles,
                const float* __restrict__ weights, float* __restrict__ out, int tokens, int ff, int width, int top) {
    const int tile = blockIdx.x;
    if (tile >= plan[0]) return;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int i = lane % 16, g = lane / 16;
    const int c0 = (blockIdx.y * 4 + wave) * 16;
    if (c0 >= width) return;
    const int e = plan[1 + tile];
    const int* rows = plan + 1 + max_tiles + tile * kMoeTile;
    const int a_i = rows[i];
    const T* xr = act + static_cast<size_t>(a_i >= 0 ? a_i : 0) * ff;
    const bool w_live = c0 + i < width;
    const T* wd = w + (static_cast<size_t>(e) * width + (w_live ? c0 + i : 0)) * ff;
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    constexpr int kChunk = MoeFrag<T>::kChunk, kPer = MoeFrag<T>::kPer;
    for (int k0 = 0; k0 < ff; k0 += kChunk) {
        MoeFrag<T> fx, fw;
        const int k = k0 + g * kPer;
        fx.load(xr, k, ff, a_i >= 0);
        fw.load(wd, k, ff, w_live);
        acc = MoeFrag<T>::mma(fw, fx, acc);
    }
    if (a_i < 0) return;
    const float weight = weights[a_i];
    float* o = out + (static_cast<size_t>(a_i % top) * tokens + a_i / top) * width;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int c = c0 + 4 * g + v;
        if (c < width) o[c] = weight * acc[v];
    }
}

WLLM_API int wllm_moe_down(const void* act, const void* w, const int* plan, int max_tiles, const float* weights, float* out,
                           int is_bf16, int tokens, int ff, int width, int top, hipStream_t stream) {
    if (max_tiles <= 0 || tokens <= 0) return 0;
    if (ff <= 0 || width <= 0 || top <= 0 || (width + 63) / 64 > 65535) return -1;
    const dim3 grid(max_tiles, (width + 63) / 64);
    if (is_bf16)
        moe_down_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(act), static_cast<const bf16*>(w), plan,
                                                        max_tiles, weights, out, tokens, ff, width, top);
    else
        moe_down_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(act), static_cast<const float*>(w), plan,
                                                         max_tiles, weights, out, tokens, ff, width, top);
    return launch_status();
}
