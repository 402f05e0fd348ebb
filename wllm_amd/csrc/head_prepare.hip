// What lies between the projection of an attention block and its attention, for blocks that do
// more there than rotate: per head a rotation (either pairing, the whole head or its first
// elements), a unit norm of queries and keys, values that are the keys as projected, and columns
// beyond the heads that only take their bias and the sum of their partial sums.  And three small
// steps of the residual stream and of a block's output: a gate on the attention's result, a copy
// into a band of columns, and a sum into the stream.  Everything here computes in float32.
#include "common.h"

constexpr int kPrepareWaves = 4;
constexpr int kPrepareMaxHead = 256;
constexpr int kPerLane = kPrepareMaxHead / kWave;
constexpr int kRestColumns = kWave * kPrepareWaves * 4;      // columns beyond the heads that one workgroup takes

template <typename T> struct alignas(4 * sizeof(T)) Four { T v[4]; };

// A row is
//   [num_heads query heads | num_kv_heads key heads | num_kv_heads value heads, unless the values are the keys | the rest]
// of head_dim elements a head.  In the order of the steps, for every query and key head:
//   1. the element is the row's (or the sum of the stack of partial sums `parts`), plus its bias
//      (the bias covers the row's first bias_width columns);
//   2. where the values are the keys, the key head as it is now goes to the cache's values;
//   2b. with pre_eps >= 0 the head is divided by sqrt(sum of its squares / norm_dim + pre_eps) and multiplied
//      element by element by a weight of head_dim numbers (pre_q for query heads, pre_k for key heads): an RMS
//      norm with a weight over each head, in front of the rotation;
//   3. the first rotary_dim elements turn by position * inv_freq[j]: pair j is (2j, 2j + 1)
//      (interleaved) or (j, j + rotary_dim / 2); sine and cosine are multiplied by rot_scale;
//   4. with norm_eps >= 0 the head is divided by sqrt(sum of its squares / norm_dim + norm_eps) (norm_dim is
//      head_dim, or less where the last elements of a head are padding that is always zero);
//   5. it is written back to the row, and a key head to the cache's keys.
// Value heads of their own and the rest of the row take step 1 only.  Keys lie in the cache as
// [page_size, head_dim], values transposed as [head_dim, page_size].
//
// The grid is (token, piece): the first pieces are groups of four heads, a wavefront a head; the others
// take kRestColumns columns each of what lies behind the query and key heads.  A decode step's few
// tokens so fill some tens of workgroups instead of one a token, whose wavefronts would walk the heads
// and the stack of partial sums one after the other.  FOUR: head_dim and the row's width are multiples
// of four and the pairs are neighbours (or nothing turns), so a lane owns four consecutive elements with
// both partners of its pairs and moves 8 or 16 bytes at a time; else a lane owns elements 64 apart and
// finds a partner in shared memory.
template <typename T, bool FOUR>
__global__ void __launch_bounds__(kWave * kPrepareWaves)
head_prepare_kernel(T* __restrict__ rows, int row_width, const float* __restrict__ parts, int splits, size_t split_stride,
                    const float* __restrict__ bias, int bias_width, const int* __restrict__ positions,
                    const float* __restrict__ inv_freq, const int* __restrict__ slots, T* __restrict__ cache,
                    long long num_pages, int num_heads, int num_kv_heads, int head_dim, int rotary_dim,
                    int interleaved, float norm_eps, int norm_dim, int values_are_keys, int page_size, int head_pieces,
                    const float* __restrict__ pre_q, const float* __restrict__ pre_k, float pre_eps, float rot_scale) {
    __shared__ float staged[kPrepareWaves][FOUR ? 1 : kPrepareMaxHead];
    const int token = blockIdx.x;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    T* row = rows + static_cast<size_t>(token) * row_width;
    const float* prow = parts ? parts + static_cast<size_t>(token) * row_width : nullptr;
    auto value = [&](int idx) -> float {
        const float v = prow ? stack_sum(prow + idx, splits, split_stride) : to_float(row[idx]);
        return idx < bias_width ? v + bias[idx] : v;
    };
    const size_t page_elems = static_cast<size_t>(2) * num_kv_heads * page_size * head_dim;
    T* kpage = nullptr;
    T* vpage = nullptr;
    int off = 0;
    if (cache) {
        const int slot = slots[token];
        const long long page = slot / page_size;
        off = slot % page_size;
        if (slot >= 0 && page < num_pages) {
            kpage = cache + page * page_elems;
            vpage = kpage + static_cast<size_t>(num_kv_heads) * page_size * head_dim;
        }
    }
    const int turned_heads = num_heads + num_kv_heads;
    if (static_cast<int>(blockIdx.y) >= head_pieces) {
        // ---- behind the query and key heads: value heads of their own, then the rest of the row ----
        const int begin = turned_heads * head_dim;
        const int values_end = values_are_keys ? begin : begin + num_kv_heads * head_dim;
        const int idx0 = begin + (static_cast<int>(blockIdx.y) - head_pieces) * kRestColumns + threadIdx.x * 4;
        for (int u = 0; u < 4; ++u) {
            const int idx = idx0 + u;
            if (idx >= row_width) break;
            const bool rewrite = prow || idx < bias_width;
            if (!rewrite && !(idx < values_end && vpage)) continue;
            T v = row[idx];
            if (rewrite) {
                v = from_float<T>(value(idx));
                row[idx] = v;
            }
            if (idx < values_end && vpage) {
                const int head = (idx - begin) / head_dim, j = (idx - begin) % head_dim;
                vpage[(static_cast<size_t>(head) * head_dim + j) * page_size + off] = v;
            }
        }
        return;
    }
    const int head = static_cast<int>(blockIdx.y) * kPrepareWaves + wave;
    if (head >= turned_heads) return;
    const float pos = static_cast<float>(positions[token]);
    const int base = head * head_dim;
    const int kvh = head - num_heads;                 // >= 0: a key head
    const int half = rotary_dim / 2;
    if (FOUR) {
        const int e = 4 * lane;
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        const bool live = e < head_dim;
        if (live) {
            if (prow) {
                // the partial sums are added in stack order, eight slices asked for at a time
                const float* p = prow + base + e;
                Four<float> t = *reinterpret_cast<const Four<float>*>(p);
#pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = t.v[u];
                for (int s0 = 1; s0 < splits; s0 += 8) {
                    Four<float> q[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        q[j] = *reinterpret_cast<const Four<float>*>(p + static_cast<size_t>(min(s0 + j, splits - 1)) * split_stride);
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        if (s0 + j >= splits) break;
#pragma unroll
                        for (int u = 0; u < 4; ++u) v[u] += q[j].v[u];
                    }
                }
            } else {
                const Four<T> t = *reinterpret_cast<const Four<T>*>(row + base + e);
#pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = to_float(t.v[u]);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (base + e + u < bias_width) v[u] += bias[base + e + u];
            if (values_are_keys && kvh >= 0 && vpage) {
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    vpage[(static_cast<size_t>(kvh) * head_dim + e + u) * page_size + off] = from_float<T>(v[u]);
            }
        }
        if (pre_eps >= 0.f) {
            // (every lane of the wavefront takes part in the sum; lanes beyond the head hold zeros)
            const float ss = wave_sum(v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3]);
            const float pre = rsqrtf(ss / static_cast<float>(norm_dim) + pre_eps);
            if (live) {
                const float* pw = (kvh >= 0 ? pre_k : pre_q) + e;
#pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = v[u] * pre * pw[u];
            }
        }
        if (live) {
            if (inv_freq) {
#pragma unroll
                for (int u = 0; u < 4; u += 2) {
                    if (e + u < rotary_dim) {
                        float sn, cs, ra, rb;
                        sincosf(pos * inv_freq[(e + u) >> 1], &sn, &cs);
                        rotate_pair(v[u], v[u + 1], sn * rot_scale, cs * rot_scale, ra, rb);
                        v[u] = ra;
                        v[u + 1] = rb;
                    }
                }
            }
        }
        float inv = 1.f;
        if (norm_eps >= 0.f) {
            const float ss = wave_sum(v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3]);
            inv = rsqrtf(ss / static_cast<float>(norm_dim) + norm_eps);
        }
        if (live) {
            Four<T> r;
#pragma unroll
            for (int u = 0; u < 4; ++u) r.v[u] = from_float<T>(v[u] * inv);
            *reinterpret_cast<Four<T>*>(row + base + e) = r;
            if (kvh >= 0 && kpage)
                *reinterpret_cast<Four<T>*>(kpage + (static_cast<size_t>(kvh) * page_size + off) * head_dim + e) = r;
        }
        return;
    }
    // ---- any sizes, either pairing: the lane's elements are lane, lane + 64, ... ----
    float* mine = staged[wave];
    float v[kPerLane];
#pragma unroll
    for (int k = 0; k < kPerLane; ++k) {
        const int e = lane + k * kWave;
        v[k] = e < head_dim ? value(base + e) : 0.f;
        if (values_are_keys && kvh >= 0 && vpage && e < head_dim)
            vpage[(static_cast<size_t>(kvh) * head_dim + e) * page_size + off] = from_float<T>(v[k]);
    }
    if (pre_eps >= 0.f) {
        float pss = 0.f;
#pragma unroll
        for (int k = 0; k < kPerLane; ++k) pss += v[k] * v[k];
        const float pre = rsqrtf(wave_sum(pss) / static_cast<float>(norm_dim) + pre_eps);
        const float* pw = kvh >= 0 ? pre_k : pre_q;
#pragma unroll
        for (int k = 0; k < kPerLane; ++k) {
            const int e = lane + k * kWave;
            if (e < head_dim) v[k] = v[k] * pre * pw[e];
        }
    }
#pragma unroll
    for (int k = 0; k < kPerLane; ++k) {
        const int e = lane + k * kWave;
        if (e < head_dim) mine[e] = v[k];
    }
    // lanes read below what other lanes of the wavefront wrote above
    __builtin_amdgcn_wave_barrier();
    asm volatile("" ::: "memory");
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < kPerLane; ++k) {
        const int e = lane + k * kWave;
        if (inv_freq && e < rotary_dim) {
            const bool first = interleaved ? (e & 1) == 0 : e < half;
            const int partner = interleaved ? (e ^ 1) : (first ? e + half : e - half);
            const int j = interleaved ? e >> 1 : (first ? e : e - half);
            const float other = mine[partner];
            float sn, cs, ra, rb;
            sincosf(pos * inv_freq[j], &sn, &cs);
            rotate_pair(first ? v[k] : other, first ? other : v[k], sn * rot_scale, cs * rot_scale, ra, rb);
            v[k] = first ? ra : rb;
        }
        ss += v[k] * v[k];
    }
    float inv = 1.f;
    if (norm_eps >= 0.f) inv = rsqrtf(wave_sum(ss) / static_cast<float>(norm_dim) + norm_eps);
#pragma unroll
    for (int k = 0; k < kPerLane; ++k) {
        const int e = lane + k * kWave;
        if (e < head_dim) {
            const T r = from_float<T>(v[k] * inv);
            row[base + e] = r;
            if (kvh >= 0 && kpage) kpage[(static_cast<size_t>(kvh) * page_size + off) * head_dim + e] = r;
        }
    }
}

// Returns 0, a HIP error code, or -1 for sizes the kernel does not take.  `bias` covers the first
// `bias_width` columns of a row (0: no bias).
WLLM_API int wllm_head_prepare(void* rows, int is_bf16, int row_width, const float* parts, int splits,
                               long long split_stride, const float* bias, int bias_width, const int* positions,
                               const float* inv_freq, const int* slots, void* cache, long long num_pages, int n,
                               int num_heads, int num_kv_heads, int head_dim, int rotary_dim, int interleaved,
                               float norm_eps, int norm_dim, int values_are_keys, int page_size, const float* pre_q,
                               const float* pre_k, float pre_eps, float rot_scale, hipStream_t stream) {
    if (pre_eps >= 0.f && (pre_q == nullptr || (pre_k == nullptr && num_kv_heads > 0))) return -1;
    const int heads = num_heads + (values_are_keys ? 1 : 2) * num_kv_heads;
    if (head_dim <= 0 || head_dim > kPrepareMaxHead || rotary_dim < 0 || rotary_dim > head_dim || rotary_dim % 2 != 0 ||
        row_width < heads * head_dim || num_heads < 0 || num_kv_heads < 0 || page_size <= 0 || bias_width < 0 ||
        bias_width > row_width || (bias == nullptr && bias_width != 0) || norm_dim <= 0 || norm_dim > head_dim)
        return -1;
    if (inv_freq == nullptr && rotary_dim != 0) return -1;
    if (n <= 0) return 0;
    const int turned = (num_heads + num_kv_heads) * head_dim;
    const int head_pieces = (num_heads + num_kv_heads + kPrepareWaves - 1) / kPrepareWaves;
    // what lies behind the query and key heads needs a workgroup only if something is to be done there
    const bool rest = row_width > turned && (parts != nullptr || bias_width > turned || (!values_are_keys && cache != nullptr));
    const int rest_pieces = rest ? (row_width - turned + kRestColumns - 1) / kRestColumns : 0;
    if (head_pieces + rest_pieces > 65535) return -1;
    const dim3 grid(n, head_pieces + rest_pieces);
    const bool four = head_dim % 4 == 0 && row_width % 4 == 0 && (interleaved || rotary_dim == 0) &&
                      (parts == nullptr || split_stride % 4 == 0) &&
                      reinterpret_cast<uintptr_t>(rows) % 16 == 0 && reinterpret_cast<uintptr_t>(parts) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(cache) % 16 == 0;
#define LAUNCH(T, FOUR)                                                                                             \
    head_prepare_kernel<T, FOUR><<<grid, kWave * kPrepareWaves, 0, stream>>>(                                       \
        static_cast<T*>(rows), row_width, parts, splits, static_cast<size_t>(split_stride), bias, bias_width, positions, \
        inv_freq, slots, static_cast<T*>(cache), num_pages, num_heads, num_kv_heads, head_dim, rotary_dim, interleaved, \
        norm_eps, norm_dim, values_are_keys, page_size, head_pieces, pre_q, pre_k, pre_eps, rot_scale)
    if (is_bf16) {
        if (four) LAUNCH(bf16, true); else LAUNCH(bf16, false);
    } else {
        if (four) LAUNCH(float, true); else LAUNCH(float, false);
    }
#undef LAUNCH
    return launch_status();
}

// ---- out[r, c] = a[r, c] * sigmoid(gate[r, c]); every operand has a row stride of its own, so the
// gate may be a band of a wider row and the result a band of a wider buffer ----------------------
// FOUR: every row begins at a multiple of four elements and has a multiple of four: 8 or 16 bytes a lane.
template <typename T, bool FOUR>
__global__ void sigmoid_gate_kernel(const T* __restrict__ a, long long a_stride, const T* __restrict__ gate,
                                    long long gate_stride, T* __restrict__ out, long long out_stride, int rows,
                                    int cols, int per) {
    constexpr int W = FOUR ? 4 : 1;
    for (int r = blockIdx.y; r < rows; r += gridDim.y) {
        const T* ar = a + r * a_stride;
        const T* gr = gate + r * gate_stride;
        T* o = out + r * out_stride;
        for (int c = (blockIdx.x * blockDim.x + threadIdx.x) * W; c < cols; c += gridDim.x * blockDim.x * W) {
            if (FOUR) {
                const Four<T> av = *reinterpret_cast<const Four<T>*>(ar + c);
                Four<T> gv, ov;
                // `per` > 1: one gate for every `per` consecutive columns (a number a head)
                if (per > 1) {
#pragma unroll
                    for (int u = 0; u < 4; ++u) gv.v[u] = gr[(c + u) / per];
                } else {
                    gv = *reinterpret_cast<const Four<T>*>(gr + c);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) ov.v[u] = from_float<T>(to_float(av.v[u]) / (1.f + expf(-to_float(gv.v[u]))));
                *reinterpret_cast<Four<T>*>(o + c) = ov;
            } else {
                o[c] = from_float<T>(to_float(ar[c]) / (1.f + expf(-to_float(gr[c / per]))));
            }
        }
    }
}

WLLM_API int wllm_sigmoid_gate(const void* a, long long a_stride, const void* gate, long long gate_stride, void* out,
                               long long out_stride, int is_bf16, int rows, int cols, int per, hipStream_t stream) {
    if (rows <= 0 || cols <= 0) return 0;
    if (per < 1) return -1;
    const size_t four_bytes = 4 * (is_bf16 ? 2 : 4);
    const bool gate_four = per > 1 || (gate_stride % 4 == 0 && reinterpret_cast<uintptr_t>(gate) % four_bytes == 0);
    const bool four = cols % 4 == 0 && a_stride % 4 == 0 && gate_four && out_stride % 4 == 0 &&
                      reinterpret_cast<uintptr_t>(a) % four_bytes == 0 &&
                      reinterpret_cast<uintptr_t>(out) % four_bytes == 0;
    const int per_row = four ? cols / 4 : cols;
    const dim3 grid(per_row < 4096 ? (per_row + 255) / 256 : 16, rows < 16384 ? rows : 16384);
#define LAUNCH(T, FOUR)                                                                                              \
    sigmoid_gate_kernel<T, FOUR><<<grid, 256, 0, stream>>>(static_cast<const T*>(a), a_stride, static_cast<const T*>(gate), \
                                                           gate_stride, static_cast<T*>(out), out_stride, rows, cols, per)
    if (is_bf16) {
        if (four) LAUNCH(bf16, true); else LAUNCH(bf16, false);
    } else {
        if (four) LAUNCH(float, true); else LAUNCH(float, false);
    }
#undef LAUNCH
    return launch_status();
}

// ---- out[r, c] = src[r, c] * scale with row strides: a tensor into a band of columns of a wider one
// (scale 1: the same bits) ------
template <typename T>
__global__ void copy_columns_kernel(const T* __restrict__ src, long long src_stride, T* __restrict__ out,
                                    long long out_stride, int rows, int cols, float scale) {
    for (int r = blockIdx.y; r < rows; r += gridDim.y) {
        const T* s = src + r * src_stride;
        T* o = out + r * out_stride;
        if (scale == 1.f) {
            for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < cols; c += gridDim.x * blockDim.x) o[c] = s[c];
        } else {
            for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < cols; c += gridDim.x * blockDim.x)
                o[c] = from_float<T>(to_float(s[c]) * scale);
        }
    }
}

WLLM_API int wllm_copy_columns(const void* src, long long src_stride, void* out, long long out_stride, int is_bf16,
                               int rows, int cols, float scale, hipStream_t stream) {
    if (rows <= 0 || cols <= 0) return 0;
    const dim3 grid(cols < 4096 ? (cols + 255) / 256 : 16, rows < 16384 ? rows : 16384);
    if (is_bf16)
        copy_columns_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(src), src_stride, static_cast<bf16*>(out),
                                                            out_stride, rows, cols, scale);
    else
        copy_columns_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(src), src_stride,
                                                             static_cast<float*>(out), out_stride, rows, cols, scale);
    return launch_status();
}

// ---- the residual stream takes what is pending and one more addend, in float32:
// x = ((x + delta) + bias) + addend, with delta a tensor of the activation type or a stack of float32
// partial sums added in stack order, bias a row, addend a tensor of x's shape; each may be absent ----
template <typename TD>
__global__ void stream_add_kernel(float* __restrict__ x, const TD* __restrict__ delta, int splits, size_t split_stride,
                                  const float* __restrict__ bias, const float* __restrict__ addend, long long total,
                                  int hidden) {
    const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
    for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
        float v = x[i];
        if (delta) {
            if (sizeof(TD) == sizeof(float) && splits > 1)
                v += stack_sum(reinterpret_cast<const float*>(delta) + i, splits, split_stride);
            else
                v += to_float(delta[i]);
        }
        if (bias) v += bias[i % hidden];
        if (addend) v += addend[i];
        x[i] = v;
    }
}

WLLM_API int wllm_stream_add(float* x, const void* delta, int delta_bf16, int splits, long long split_stride,
                             const float* bias, const float* addend, int rows, int hidden, hipStream_t stream) {
    const long long total = static_cast<long long>(rows) * hidden;
    if (total <= 0) return 0;
    long long blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (delta_bf16)
        stream_add_kernel<bf16><<<static_cast<int>(blocks), 256, 0, stream>>>(
            x, static_cast<const bf16*>(delta), splits, static_cast<size_t>(split_stride), bias, addend, total, hidden);
    else
        stream_add_kernel<float><<<static_cast<int>(blocks), 256, 0, stream>>>(
            x, static_cast<const float*>(delta), splits, static_cast<size_t>(split_stride), bias, addend, total, hidden);
    return launch_status();
}
