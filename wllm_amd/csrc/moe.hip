// A mixture of gated feed-forward experts on a flat batch of tokens: the router, the plan that sorts a
// step's (token, chosen expert) pairs by expert, and the two grouped products on the matrix cores.
//
//   router   z = W_r x (float32), s = softmax(z) over all experts (or, `scoring` 1, s = sigmoid(z) of each); only experts of the `keep` best of
//            `groups` equal groups of neighbours (a group's score: its largest s) may be chosen; the `top`
//            allowed experts with the largest s are chosen, weights s / (sum of the chosen + eps) (or, `normalize` 0, s itself)
//   plan     an assignment is a = token * top + slot.  The assignments of one expert lie together, in
//            tiles of R rows (16, 32, 64 or 128; the last tile of an expert padded with -1):
//            plan[0] = tiles in use; plan[1 + t] = expert of tile t; plan[1 + max_tiles + R t + r] = a or -1
//   up       act[a] = activation(x[token] Wg_e^T) * (x[token] Wu_e^T); with `in_weights` both products are multiplied by
//            in_weights[a] first: the expert's input is in_weights[a] * x[token] (the factor taken out of the sums)
//   down     out[slot][token] = weight[a] * (act[a] Wd_e^T) (weight 1 without `weights`), float32: a stack of `top` partial sums that
//            whoever adds the feed-forward to the stream adds in order
// A row's sums run over k in ascending chunks whatever tile the row lies in, so a token's result does
// not depend on what else the batch holds.  Nothing is read on the host: the grid has room for the most
// tiles a step of its size can need and a workgroup beyond plan[0] leaves at once.
#include "common.h"

#include <type_traits>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kMoeTile = 16;            // rows of a tile
constexpr int kMoeMaxExperts = 256;

// ---- the router: one workgroup a token.  The four wavefronts share the experts' dot products (a lane sums its
// columns in ascending order, the lanes are added in the butterfly's order: the same bits whatever the batch);
// then the first wavefront, a lane holding the experts lane, lane + 64, ..., takes the softmax, shuts the groups
// out and picks the top, every choice a maximum over the wavefront and, among equals, the lowest index. ----
constexpr int kRoutePer = kMoeMaxExperts / kWave;        // experts a lane holds

__device__ __forceinline__ int wave_lowest(int v) { return -static_cast<int>(wave_max(-static_cast<float>(v))); }

template <typename T>
__global__ void __launch_bounds__(256)
moe_route_kernel(const T* __restrict__ x, const float* __restrict__ router, int* __restrict__ ids, float* __restrict__ weights,
                 int tokens, int width, int experts, int top, int groups, int keep, float eps, int scoring, int normalize) {
    __shared__ float z_s[kMoeMaxExperts];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int token = blockIdx.x;
    const T* xr = x + static_cast<size_t>(token) * width;
    for (int e = wave; e < experts; e += 4) {
        const float* w = router + static_cast<size_t>(e) * width;
        float dot = 0.f;
        if (width % 4 == 0) {
#pragma unroll 4
            for (int c = lane * 4; c < width; c += kWave * 4) {
                const float4 wv = *reinterpret_cast<const float4*>(w + c);
                dot = fmaf(to_float(xr[c]), wv.x, dot);
                dot = fmaf(to_float(xr[c + 1]), wv.y, dot);
                dot = fmaf(to_float(xr[c + 2]), wv.z, dot);
                dot = fmaf(to_float(xr[c + 3]), wv.w, dot);
            }
        } else {
            for (int c = lane; c < width; c += kWave) dot = fmaf(to_float(xr[c]), w[c], dot);
        }
        dot = wave_sum(dot);
        if (lane == 0) z_s[e] = dot;
    }
    __syncthreads();
    if (wave != 0) return;
    // softmax over all experts
    float sc[kRoutePer];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < kRoutePer; ++j) {
        const int e = lane + kWave * j;
        sc[j] = e < experts ? z_s[e] : -INFINITY;
        mx = fmaxf(mx, sc[j]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    if (scoring == 1) {
        // a score of each expert by itself: in the terms of the softmax's code below, exp(z - mx) / sum with mx = 0
        // and sum = 1 would not do (it overflows), so the sigmoid is written into sc and z_s as it is
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < kRoutePer; ++j) {
            const int e = lane + kWave * j;
            sc[j] = e < experts ? 1.f / (1.f + expf(-sc[j])) : 0.f;
            if (e < experts) z_s[e] = sc[j];
        }
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        sum = 1.f;
    } else {
#pragma unroll
        for (int j = 0; j < kRoutePer; ++j) {
            sc[j] = lane + kWave * j < experts ? expf(sc[j] - mx) : 0.f;
            sum += sc[j];
        }
        sum = wave_sum(sum);
    }
    // a score that may still be chosen is >= 0; one that may not is -1
#pragma unroll
    for (int j = 0; j < kRoutePer; ++j) sc[j] = lane + kWave * j < experts ? sc[j] / sum : -1.f;
    if (keep < groups) {
        const int per = experts / groups;
        float gs[kRoutePer];                     // the scores of the groups lane, lane + 64, ...: their largest member's
        bool allowed[kRoutePer];
#pragma unroll
        for (int j = 0; j < kRoutePer; ++j) {
            const int g = lane + kWave * j;
            gs[j] = -1.f;
            allowed[j] = false;
            if (g < groups)
                for (int m = 0; m < per; ++m)
                    gs[j] = fmaxf(gs[j], scoring == 1 ? z_s[g * per + m] : expf(z_s[g * per + m] - mx) / sum);
        }
        for (int pick = 0; pick < keep; ++pick) {
            float best = -1.f;
#pragma unroll
            for (int j = 0; j < kRoutePer; ++j) best = fmaxf(best, gs[j]);
            best = wave_max(best);
            int which = kMoeMaxExperts;
#pragma unroll
            for (int j = kRoutePer - 1; j >= 0; --j)
                if (gs[j] == best) which = lane + kWave * j;
            which = wave_lowest(which);
#pragma unroll
            for (int j = 0; j < kRoutePer; ++j) {
                if (lane + kWave * j == which) gs[j] = -1.f;
                if ((lane + kWave * j) / per == which) allowed[j] = true;
            }
        }
#pragma unroll
        for (int j = 0; j < kRoutePer; ++j)
            if (!allowed[j]) sc[j] = -1.f;
    }
    float chosen_sum = 0.f;
    int* id = ids + static_cast<size_t>(token) * top;
    float* wt = weights + static_cast<size_t>(token) * top;
    for (int slot = 0; slot < top; ++slot) {
        float best = -1.f;
#pragma unroll
        for (int j = 0; j < kRoutePer; ++j) best = fmaxf(best, sc[j]);
        best = wave_max(best);
        int which = kMoeMaxExperts;
#pragma unroll
        for (int j = kRoutePer - 1; j >= 0; --j)
            if (sc[j] == best) which = lane + kWave * j;
        which = wave_lowest(which);
#pragma unroll
        for (int j = 0; j < kRoutePer; ++j)
            if (lane + kWave * j == which) sc[j] = -1.f;
        chosen_sum += best;
        if (lane == 0) {
            id[slot] = which;
            wt[slot] = best;
        }
    }
    if (lane == 0 && normalize) {
        const float denom = chosen_sum + eps;
        for (int slot = 0; slot < top; ++slot) wt[slot] /= denom;
    }
}

WLLM_API int wllm_moe_route(const void* x, const float* router, int* ids, float* weights, int is_bf16, int tokens, int width,
                            int experts, int top, int groups, int keep, float eps, int scoring, int normalize,
                            hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (scoring < 0 || scoring > 1) return -1;
    if (experts <= 0 || experts > kMoeMaxExperts || groups <= 0 || experts % groups || keep <= 0 || keep > groups || top <= 0 ||
        top > keep * (experts / groups) || width <= 0)
        return -1;
    if (is_bf16)
        moe_route_kernel<bf16><<<tokens, 256, 0, stream>>>(static_cast<const bf16*>(x), router, ids, weights, tokens, width,
                                                           experts, top, groups, keep, eps, scoring, normalize);
    else
        moe_route_kernel<float><<<tokens, 256, 0, stream>>>(static_cast<const float*>(x), router, ids, weights, tokens, width,
                                                            experts, top, groups, keep, eps, scoring, normalize);
    return launch_status();
}

// ---- the plan: one workgroup counts the assignments of every expert, gives each expert its tiles (of
// `tile_rows` rows: 16 for the kernels that stream an expert's weights past a few rows, 128 for the kernel that
// tiles many rows through shared memory) and every assignment a row.  Which row of its expert's tiles an
// assignment gets depends on the order in which threads arrive; a row's result does not depend on its place. ----
__global__ void __launch_bounds__(1024)
moe_plan_kernel(const int* __restrict__ ids, int* __restrict__ plan, int assignments, int experts, int max_tiles, int tile_rows) {
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
            tiles += (count_s[e] + tile_rows - 1) / tile_rows;
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
    for (int i = threadIdx.x; i < tiles * tile_rows; i += blockDim.x) rows[i] = -1;
    __syncthreads();
    for (int a = threadIdx.x; a < assignments; a += blockDim.x) {
        const int e = ids[a];
        rows[first_s[e] * tile_rows + atomicAdd(&count_s[e], 1)] = a;
    }
}

WLLM_API int wllm_moe_plan(const int* ids, int* plan, int assignments, int experts, int max_tiles, int tile_rows,
                           hipStream_t stream) {
    if (assignments <= 0) return 0;
    if (experts <= 0 || experts > kMoeMaxExperts || tile_rows <= 0 || max_tiles < assignments / tile_rows + experts) return -1;
    moe_plan_kernel<<<1, 1024, 0, stream>>>(ids, plan, assignments, experts, max_tiles, tile_rows);
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
    template <bool STREAM = false>
    __device__ __forceinline__ void whole(const bf16* p) {           // 8 keys that are all there, 16-byte aligned
        union { uint4 u; bf16x8_t v; } t;
        t.u = STREAM ? load_streamed(p) : *reinterpret_cast<const uint4*>(p);
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
    template <bool STREAM = false>
    __device__ __forceinline__ void whole(const float* p) {
        const float4 t = *reinterpret_cast<const float4*>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
    static __device__ __forceinline__ float4_t mma(const MoeFrag& a, const MoeFrag& b, float4_t acc) {
#pragma unroll
        for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[t], b.v[t], acc, 0, 0, 0);
        return acc;
    }
};

// act[a, c] = activation(x[token(a)] . Wg[e][c]) * (x[token(a)] . Wu[e][c]); w [experts, 2 * ff, K]: an
// expert's gate rows, then its up rows.  Grid (tiles, bands of 64 columns); a wavefront 16 columns.  A tile is MT
// sub-tiles of 16 rows (the plan's tiles have 16 MT rows): a fragment of the weights feeds MT products, so an expert
// with up to 16 MT rows reads its weights once.
// `tiles`: the weights' tile-major copy (bfloat16: per band of 16 rows of the stacked [experts * 2 * ff, K] matrix and
// step of 32 keys one KiB in lane order, as `wllm_tile_weight` writes it; ff a multiple of 16), or null: then a
// wavefront's load of a fragment is one contiguous KiB instead of 16 pieces a row apart.
template <typename T, int ACT, int MT>
__global__ void __launch_bounds__(256)
moe_up_kernel(const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ tiles, const int* __restrict__ plan,
              int max_tiles, T* __restrict__ act, int K, int ff, int top, const float* __restrict__ in_weights) {
    constexpr int U = MT == 4 ? 2 : 4;          // chunks whose loads are asked for before the first product
    const int tile = blockIdx.x;
    if (tile >= plan[0]) return;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int i = lane % 16, g = lane / 16;
    const int c0 = (blockIdx.y * 4 + wave) * 16;
    if (c0 >= ff) return;
    const int e = plan[1 + tile];
    const int* rows = plan + 1 + max_tiles + tile * (kMoeTile * MT);
    int a_i[MT];
    const T* xr[MT];
    float4_t acc_g[MT], acc_u[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        a_i[m] = rows[16 * m + i];
        xr[m] = x + static_cast<size_t>(a_i[m] >= 0 ? a_i[m] / top : 0) * K;
        acc_g[m] = acc_u[m] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    const bool w_live = c0 + i < ff;
    const T* wg = w + (static_cast<size_t>(e) * 2 * ff + (w_live ? c0 + i : 0)) * K;
    const T* wu = wg + static_cast<size_t>(ff) * K;
    constexpr int kChunk = MoeFrag<T>::kChunk, kPer = MoeFrag<T>::kPer;
    if (K % (4 * kChunk) == 0) {
        // every fragment is whole (rows that stand for nothing read row 0, and their sums are dropped)
        const bool tiled = tiles != nullptr;
        const size_t per_band = static_cast<size_t>(K / kChunk) * kWave * kPer;        // elements of a band's tiles
        const T* tg = tiled ? tiles + (static_cast<size_t>(e) * 2 * ff + c0) / 16 * per_band + lane * kPer : wg + g * kPer;
        const T* tu = tiled ? tiles + (static_cast<size_t>(e) * 2 * ff + ff + c0) / 16 * per_band + lane * kPer : wu + g * kPer;
        // (the step from a chunk's fragment to the next chunk's is a constant either way, so that the loads of a
        // round differ by immediate offsets)
        auto walk = [&](auto step) {
            constexpr int kStep = decltype(step)::value;
            for (int k0 = 0; k0 < K; k0 += U * kChunk) {
                MoeFrag<T> fx[U][MT], fg[U], fu[U];
                const T* pg = tg + static_cast<size_t>(k0 / kChunk) * kStep;
                const T* pu = tu + static_cast<size_t>(k0 / kChunk) * kStep;
#pragma unroll
                for (int u = 0; u < U; ++u) {
#pragma unroll
                    for (int m = 0; m < MT; ++m) fx[u][m].whole(xr[m] + k0 + u * kChunk + g * kPer);
                    fg[u].template whole<true>(pg + u * kStep);
                    fu[u].template whole<true>(pu + u * kStep);
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        acc_g[m] = MoeFrag<T>::mma(fg[u], fx[u][m], acc_g[m]);
                        acc_u[m] = MoeFrag<T>::mma(fu[u], fx[u][m], acc_u[m]);
                    }
            }
        };
        if (tiled) walk(std::integral_constant<int, kWave * kPer>{});
        else walk(std::integral_constant<int, kChunk>{});
    } else {
        for (int k0 = 0; k0 < K; k0 += kChunk) {
            MoeFrag<T> fg, fu;
            const int k = k0 + g * kPer;
            fg.load(wg, k, K, w_live);
            fu.load(wu, k, K, w_live);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                MoeFrag<T> fx;
                fx.load(xr[m], k, K, a_i[m] >= 0);
                acc_g[m] = MoeFrag<T>::mma(fg, fx, acc_g[m]);
                acc_u[m] = MoeFrag<T>::mma(fu, fx, acc_u[m]);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if (a_i[m] < 0) continue;
        T* out = act + static_cast<size_t>(a_i[m]) * ff;
        const float scale = in_weights ? in_weights[a_i[m]] : 1.f;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int c = c0 + 4 * g + v;
            if (c < ff) out[c] = from_float<T>(activate<ACT>(acc_g[m][v] * scale) * (acc_u[m][v] * scale));
        }
    }
}

// `tile_rows`: the rows of the plan's tiles, 16, 32 or 64.
WLLM_API int wllm_moe_up(const void* x, const void* w, const void* tiles, const int* plan, int max_tiles, int tile_rows,
                         void* act, int is_bf16, int activation, int K, int ff, int top, const float* in_weights,
                         hipStream_t stream) {
    if (max_tiles <= 0) return 0;
    if (K <= 0 || ff <= 0 || top <= 0 || activation < 0 || activation >= kActivations || (ff + 63) / 64 > 65535) return -1;
    if (tile_rows != 16 && tile_rows != 32 && tile_rows != 64) return -1;
    if (tiles && (!is_bf16 || ff % 16 || K % 32)) return -1;
    const dim3 grid(max_tiles, (ff + 63) / 64);
#define LAUNCH_MT(T, MT)                                                                                              \
    WLLM_BY_ACTIVATION(activation, (moe_up_kernel<T, ACT, MT><<<grid, 256, 0, stream>>>(                              \
                                       static_cast<const T*>(x), static_cast<const T*>(w), static_cast<const T*>(tiles), \
                                       plan, max_tiles, static_cast<T*>(act), K, ff, top, in_weights)))
#define LAUNCH(T)                                    \
    if (tile_rows == 16) { LAUNCH_MT(T, 1); }        \
    else if (tile_rows == 32) { LAUNCH_MT(T, 2); }   \
    else { LAUNCH_MT(T, 4); }
    if (is_bf16) { LAUNCH(bf16) } else { LAUNCH(float) }
#undef LAUNCH
#undef LAUNCH_MT
    return launch_status();
}

// out[a % top][a / top][c] = weight[a] * (act[a] . Wd[e][c]); w [experts, width, ff]; out float32 [top, tokens, width].
template <typename T, int MT>
__global__ void __launch_bounds__(256)
moe_down_kernel(const T* __restrict__ act, const T* __restrict__ w, const T* __restrict__ tiles, const int* __restrict__ plan,
                int max_tiles, const float* __restrict__ weights, float* __restrict__ out, int tokens, int ff, int width,
                int top) {
    constexpr int U = 4;
    const int tile = blockIdx.x;
    if (tile >= plan[0]) return;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int i = lane % 16, g = lane / 16;
    const int c0 = (blockIdx.y * 4 + wave) * 16;
    if (c0 >= width) return;
    const int e = plan[1 + tile];
    const int* rows = plan + 1 + max_tiles + tile * (kMoeTile * MT);
    int a_i[MT];
    const T* xr[MT];
    float4_t acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        a_i[m] = rows[16 * m + i];
        xr[m] = act + static_cast<size_t>(a_i[m] >= 0 ? a_i[m] : 0) * ff;
        acc[m] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    const bool w_live = c0 + i < width;
    const T* wd = w + (static_cast<size_t>(e) * width + (w_live ? c0 + i : 0)) * ff;
    constexpr int kChunk = MoeFrag<T>::kChunk, kPer = MoeFrag<T>::kPer;
    if (ff % (4 * kChunk) == 0) {
        const bool tiled = tiles != nullptr;
        const size_t per_band = static_cast<size_t>(ff / kChunk) * kWave * kPer;
        const T* td = tiled ? tiles + (static_cast<size_t>(e) * width + c0) / 16 * per_band + lane * kPer : wd + g * kPer;
        auto walk = [&](auto step) {
            constexpr int kStep = decltype(step)::value;
            for (int k0 = 0; k0 < ff; k0 += U * kChunk) {
                MoeFrag<T> fx[U][MT], fw[U];
                const T* pd = td + static_cast<size_t>(k0 / kChunk) * kStep;
#pragma unroll
                for (int u = 0; u < U; ++u) {
#pragma unroll
                    for (int m = 0; m < MT; ++m) fx[u][m].whole(xr[m] + k0 + u * kChunk + g * kPer);
                    fw[u].template whole<true>(pd + u * kStep);
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int m = 0; m < MT; ++m) acc[m] = MoeFrag<T>::mma(fw[u], fx[u][m], acc[m]);
            }
        };
        if (tiled) walk(std::integral_constant<int, kWave * kPer>{});
        else walk(std::integral_constant<int, kChunk>{});
    } else {
        for (int k0 = 0; k0 < ff; k0 += kChunk) {
            MoeFrag<T> fw;
            const int k = k0 + g * kPer;
            fw.load(wd, k, ff, w_live);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                MoeFrag<T> fx;
                fx.load(xr[m], k, ff, a_i[m] >= 0);
                acc[m] = MoeFrag<T>::mma(fw, fx, acc[m]);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if (a_i[m] < 0) continue;
        const float weight = weights ? weights[a_i[m]] : 1.f;
        float* o = out + (static_cast<size_t>(a_i[m] % top) * tokens + a_i[m] / top) * width;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int c = c0 + 4 * g + v;
            if (c < width) o[c] = weight * acc[m][v];
        }
    }
}

WLLM_API int wllm_moe_down(const void* act, const void* w, const void* tiles, const int* plan, int max_tiles, int tile_rows,
                           const float* weights, float* out, int is_bf16, int tokens, int ff, int width, int top,
                           hipStream_t stream) {
    if (max_tiles <= 0 || tokens <= 0) return 0;
    if (ff <= 0 || width <= 0 || top <= 0 || (width + 63) / 64 > 65535) return -1;
    if (tile_rows != 16 && tile_rows != 32 && tile_rows != 64) return -1;
    if (tiles && (!is_bf16 || width % 16 || ff % 32)) return -1;
    const dim3 grid(max_tiles, (width + 63) / 64);
#define LAUNCH_MT(T, MT)                                                                                              \
    moe_down_kernel<T, MT><<<grid, 256, 0, stream>>>(static_cast<const T*>(act), static_cast<const T*>(w),             \
                                                     static_cast<const T*>(tiles), plan, max_tiles, weights, out, tokens, \
                                                     ff, width, top)
#define LAUNCH(T)                                    \
    if (tile_rows == 16) LAUNCH_MT(T, 1);            \
    else if (tile_rows == 32) LAUNCH_MT(T, 2);       \
    else LAUNCH_MT(T, 4);
    if (is_bf16) { LAUNCH(bf16) } else { LAUNCH(float) }
#undef LAUNCH
#undef LAUNCH_MT
    return launch_status();
}

// ---- many rows an expert: the two products in tiles of 128 rows of one expert by 128 rows of its weights,
// through shared memory, as the framework's tiled product does it (four wavefronts of 64 x 64, stages of 64 keys
// that go from memory straight into shared memory in an XOR-swizzled order, two stages in turn, two workgroups a
// compute unit).  What differs: a tile's rows of x are gathered (row r of tile t is the assignment the plan names:
// the token's row of x for the first product, the assignment's row of act for the second), the weights are the
// tile's expert's, and a row's result goes where its assignment belongs.  A row's sums run over k in ascending
// stages whatever tile it lies in.  Workgroups that share an expert's rows of w lie 8 indices apart, on one XCD.
// bfloat16; K a multiple of 64. ----
constexpr int kBigRows = 128;
constexpr int kBigKeys = 64;
constexpr int kBigRowBytes = kBigKeys * 2;
constexpr int kBigStageBytes = 2 * kBigRows * kBigRowBytes;

union MoeTFrag {
    uint4 u;
    bf16x8_t v;
};

// 16 bytes a lane from base + offset into shared memory at dst + 16 * lane (M0 is put back as it was).
static __device__ __forceinline__ void moe_load_to_shared(const void* base, uint32_t offset, void* dst) {
    const uint32_t lds_address = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)dst)));
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0) : "v"(offset), "s"(base), "s"(lds_address) : "memory");
}

// GATED: 0 the second product (out32[a % top][a / top][n] = weight[a] * sum), 1 + the activation's number the
// first (act[a][n] = activation(gate) * up; w holds an expert's N gate rows, then its N up rows).
template <int GATED>
__global__ void __launch_bounds__(256, 2)
moe_tile_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, const int* __restrict__ plan, int max_tiles,
                bf16* __restrict__ act, float* __restrict__ out32, const float* __restrict__ weights, int N, int K, int top,
                int tokens) {
    // (`weights`: of the second product the factor of a row's result, 1 if null; of the first the factor of a row's
    // input, taken out of both sums, none if null)
    constexpr int kWaves = 4, kStages = 2;
    constexpr int kWBytes = kBigRows * kBigRowBytes;
    constexpr int kLoads = 2 * kBigRows / 8 / kWaves;
    extern __shared__ __align__(16) unsigned char tiles_s[];
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int i = lane % 16, g = lane / 16;
    const int wm = wave / 2, wn = wave % 2;
    const int xcd = blockIdx.x % 8, j = blockIdx.x / 8;
    const int m_tile = j % max_tiles;
    const int n_tile = (j / max_tiles) * 8 + xcd;
    constexpr int kColumns = GATED ? kBigRows / 2 : kBigRows;
    const int n_base = n_tile * kColumns;
    if (m_tile >= plan[0] || n_base >= N) return;
    const int e = plan[1 + m_tile];
    const int* rows = plan + 1 + max_tiles + m_tile * kBigRows;
    const int stages = K / kBigKeys;
    const bf16* we = w + static_cast<size_t>(e) * (GATED ? 2 : 1) * N * K;

    const int chunk = (lane % 8) ^ (lane / 8);
    uint32_t offset[kLoads];
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int r = 8 * (wave + kWaves * u) + lane / 8;
        size_t row;
        if (r < kBigRows) {
            if (GATED) row = r < 64 ? min(n_base + r, N - 1) : N + min(n_base + r - 64, N - 1);
            else row = min(n_base + r, N - 1);
        } else {
            const int a = rows[r - kBigRows];
            row = a < 0 ? 0 : (GATED ? a / top : a);
        }
        offset[u] = static_cast<uint32_t>((row * K + chunk * 8) * 2);
    }
    const unsigned char* w_bytes = reinterpret_cast<const unsigned char*>(we);
    const unsigned char* x_bytes = reinterpret_cast<const unsigned char*>(x);
    auto issue = [&](int stage, int s) {
        const unsigned char* wb = w_bytes + static_cast<size_t>(s) * kBigRowBytes;
        const unsigned char* xb = x_bytes + static_cast<size_t>(s) * kBigRowBytes;
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int q = wave + kWaves * u;
            moe_load_to_shared(q < kBigRows / 8 ? wb : xb, offset[u], tiles_s + stage * kBigStageBytes + q * 1024);
        }
    };

    float4_t acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};
    int w_row_s[4], x_row_s[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        w_row_s[a] = GATED ? (a < 2 ? wn * 32 + 16 * a + i : 64 + wn * 32 + 16 * (a - 2) + i) : wn * 64 + 16 * a + i;
        x_row_s[a] = wm * 64 + 16 * a + i;
    }
    issue(0, 0);
    for (int s = 0; s < stages; ++s) {
        const int stage = s % kStages;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (s + 1 < stages) issue((s + 1) % kStages, s + 1);
        const unsigned char* ws = tiles_s + stage * kBigStageBytes;
        const unsigned char* xs = ws + kWBytes;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int place = ((ks * 4 + g) ^ (i % 8)) * 16;
            MoeTFrag fw[4], fx[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                fw[a].u = *reinterpret_cast<const uint4*>(ws + w_row_s[a] * 128 + place);
                fx[a].u = *reinterpret_cast<const uint4*>(xs + x_row_s[a] * 128 + place);
            }
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[a].v, fx[b].v, acc[a][b], 0, 0, 0);
        }
    }

    // lane (i, g) holds, of tile (a, b), the tile's row 16 b + i and columns 4g .. 4g + 3 of the tile's 16
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const int asg = rows[wm * 64 + 16 * b + i];
        if (asg < 0) continue;
        if (GATED) {
            bf16* o_row = act + static_cast<size_t>(asg) * N;
            const float scale = weights ? weights[asg] : 1.f;
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const int n = n_base + wn * 32 + 16 * a + 4 * g;
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < N)
                        o_row[n + v] = from_float<bf16>(activate<(GATED > 0 ? GATED - 1 : 0)>(acc[a][b][v] * scale) *
                                                        (acc[a + 2][b][v] * scale));
            }
        } else {
            const float weight = weights ? weights[asg] : 1.f;
            float* o_row = out32 + (static_cast<size_t>(asg % top) * tokens + asg / top) * N;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const int n = n_base + wn * 64 + 16 * a + 4 * g;
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < N) o_row[n + v] = weight * acc[a][b][v];
            }
        }
    }
}

// The first product (activation >= 0: `act` [assignments, N] from x [tokens, K] and w [experts, 2N, K]) or the second
// (activation < 0: out32 [top, tokens, N] from x = act [assignments, K] and w [experts, N, K]) over a plan of tiles of
// 128 rows.  Returns -1 for sizes it does not take (K no multiple of 64, operands of 4 GiB).
WLLM_API int wllm_moe_tiles(const void* x, const void* w, const int* plan, int max_tiles, void* act, float* out32,
                            const float* weights, int activation, int x_rows, int N, int K, int top, int tokens,
                            hipStream_t stream) {
    if (max_tiles <= 0 || x_rows <= 0) return 0;
    if (N <= 0 || K < kBigKeys || K % kBigKeys || top <= 0 || tokens <= 0 || activation >= kActivations) return -1;
    const bool gated = activation >= 0;
    if ((gated && !act) || (!gated && !out32)) return -1;
    if (static_cast<size_t>(gated ? 2 : 1) * N * K * 2 >= (size_t(1) << 32) || static_cast<size_t>(x_rows) * K * 2 >= (size_t(1) << 32))
        return -1;
    const int columns = gated ? kBigRows / 2 : kBigRows;
    const int n_tiles = (N + columns - 1) / columns;
    const long long blocks = static_cast<long long>((n_tiles + 7) / 8 * 8) * max_tiles;
    if (blocks > 0x7fffffffLL) return -1;
    const dim3 grid(static_cast<unsigned>(blocks));
    const bf16* xp = static_cast<const bf16*>(x);
    const bf16* wp = static_cast<const bf16*>(w);
#define LAUNCH(GATED)                                                                                                 \
    moe_tile_kernel<GATED><<<grid, 256, 2 * kBigStageBytes, stream>>>(xp, wp, plan, max_tiles, static_cast<bf16*>(act), \
                                                                      out32, weights, N, K, top, tokens)
    if (!gated) { LAUNCH(0); }
    else { WLLM_BY_ACTIVATION(activation, LAUNCH(ACT + 1)) }
#undef LAUNCH
    return launch_status();
}
