// A mixture of gated experts: float32 router with top-k choice, rows grouped by expert on the device, the experts'
// products as grouped products on the matrix cores, and the weighted sum of a token's choices in a fixed order.
//
//   egpt_moe_route     logits = x R^T + b (float32), the `top` largest, softmax over those; or the softmax over all
//                      experts, the choice by score + a correction per expert, the chosen scores over their sum
//   egpt_moe_up        act = relu(x Wu^T)^2 per grouped row: experts without a gate
//   egpt_moe_group     (token, choice) rows grouped by expert; tiles of rows, each of one expert
//   egpt_moe_gate_up   act = silu(x Wg^T) * (x Wu^T) per grouped row, with that row's expert
//   egpt_moe_down      y = act Wd^T per grouped row (float32)
//   egpt_moe_combine   out[t] = sum_c weight[t][c] * y[place[t][c]]
//
// Nothing is read back by the host: the grid of the grouped products is sized for the most tiles that the rows can
// make (rows / tile + experts), and a workgroup whose tile does not exist leaves at once.  A row's result does not
// depend on the rows around it (a tile's rows share their products' weight operands, not their sums), so a token's
// output is the same in any batch.  Products accumulate in float32: bfloat16 operands on v_mfma_f32_16x16x32_bf16,
// float32 operands on v_mfma_f32_16x16x4_f32.
#include "api.h"
#include "common.h"

namespace egpt {

typedef __attribute__((ext_vector_type(8))) __bf16 m_bf16x8;
typedef __attribute__((ext_vector_type(4))) float m_f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int m_u32x4;

// acc[i][j] += sum_k A[i][k] B[j][k] over the 4 * E values of k that the wavefront holds: lane (j = lane % 16,
// g = lane / 16) brings 16 bytes of row i = lane % 16 of A and of row j of B at k = g * E ..; it gets acc[4 g + v][j].
template <typename T>
__device__ __forceinline__ m_f32x4 mma16(const m_u32x4& a, const m_u32x4& b, m_f32x4 acc) {
    if constexpr (sizeof(T) == 2) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(m_bf16x8, a), __builtin_bit_cast(m_bf16x8, b), acc, 0, 0, 0);
    } else {
        const m_f32x4 av = __builtin_bit_cast(m_f32x4, a), bv = __builtin_bit_cast(m_f32x4, b);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], bv[i], acc, 0, 0, 0);
        return acc;
    }
}

// 16 bytes of a row at element k (E elements); zeros beyond the row's end `n`.  Rows whose length is no multiple of E
// are not 16-byte aligned and are read element by element.
template <typename T>
__device__ __forceinline__ m_u32x4 row_piece(const T* row, int k, int n, bool aligned) {
    constexpr int E = 16 / sizeof(T);
    m_u32x4 out = m_u32x4{0u, 0u, 0u, 0u};
    if (row == nullptr || k >= n) return out;
    if (aligned && k + E <= n) return *reinterpret_cast<const m_u32x4*>(row + k);
    struct { T v[E]; } tmp;
#pragma unroll
    for (int e = 0; e < E; ++e) tmp.v[e] = k + e < n ? row[k + e] : from_float<T>(0.f);
    return __builtin_bit_cast(m_u32x4, tmp);
}

constexpr int kMaxExperts = 1024;

// One workgroup of four wavefronts per token.  A wavefront takes the experts four at a time (all loads of the four rows
// in flight together, then the four sums), wavefront w the groups w, w + 4, ...; the first wavefront then picks.
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ x, const T* __restrict__ router,
                                                        const T* __restrict__ bias, int32_t* __restrict__ chosen,
                                                        float* __restrict__ weight, int n_tokens, int hidden, int experts,
                                                        int top, int score_all, const float* __restrict__ correction,
                                                        float weight_scale) {
    extern __shared__ float logits_s[];          // [experts]
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int t = blockIdx.x;
    float* z = logits_s;
    const T* xr = x + static_cast<size_t>(t) * hidden;
    for (int e0 = wave * 4; e0 < experts; e0 += 16) {
        float dot[4] = {0.f, 0.f, 0.f, 0.f};
        const T* wr[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) wr[i] = router + static_cast<size_t>(min(e0 + i, experts - 1)) * hidden;
        for (int j = lane; j < hidden; j += kWave) {
            const float xv = to_float(xr[j]);
#pragma unroll
            for (int i = 0; i < 4; ++i) dot[i] = fmaf(xv, to_float(wr[i][j]), dot[i]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float total = wave_sum(dot[i]);
            if (lane == 0 && e0 + i < experts) z[e0 + i] = total + (bias ? to_float(bias[e0 + i]) : 0.f);
        }
    }
    __syncthreads();
    if (wave != 0) return;
    if (score_all) {
        // scores s = softmax(z) over all experts; an expert is chosen by s + correction and weighs s over the sum of
        // the chosen scores.  z[] keeps the choice scores, score_s[] (behind it) the scores themselves.
        float* score_s = logits_s + experts;
        float mx = -INFINITY;
        for (int e = lane; e < experts; e += kWave) mx = fmaxf(mx, z[e]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int e = lane; e < experts; e += kWave) sum += expf(z[e] - mx);
        const float inv_sum = 1.0f / wave_sum(sum);
        for (int e = lane; e < experts; e += kWave) {
            const float sc = expf(z[e] - mx) * inv_sum;
            score_s[e] = sc;
            z[e] = sc + (correction ? correction[e] : 0.f);
        }
        float chosen_sum = 0.f;
        for (int c = 0; c < top; ++c) {
            float best = -INFINITY;
            int best_e = 0x7fffffff;
            for (int e = lane; e < experts; e += kWave) {
                const float v = z[e];
                if (v > best || (v == best && e < best_e)) {
                    best = v;
                    best_e = e;
                }
            }
#pragma unroll
            for (int off = kWave / 2; off > 0; off >>= 1) {
                const float ov = __shfl_xor(best, off, kWave);
                const int oe = __shfl_xor(best_e, off, kWave);
                if (ov > best || (ov == best && oe < best_e)) {
                    best = ov;
                    best_e = oe;
                }
            }
            const float sc = score_s[best_e];
            chosen_sum += sc;
            if (lane == 0) {
                chosen[static_cast<size_t>(t) * top + c] = best_e;
                weight[static_cast<size_t>(t) * top + c] = sc;
            }
            if (lane == best_e % kWave) z[best_e] = -INFINITY;
        }
        if (lane == 0) {
            const float f = weight_scale / (chosen_sum + 1e-20f);
            for (int c = 0; c < top; ++c) weight[static_cast<size_t>(t) * top + c] *= f;
        }
        return;
    }
    // the top choices one after the other: the largest logit not yet taken, the lowest index among equals
    float first = 0.f, total = 0.f;
    for (int c = 0; c < top; ++c) {
        float best = -INFINITY;
        int best_e = 0x7fffffff;
        for (int e = lane; e < experts; e += kWave) {
            const float v = z[e];
            if (v > best || (v == best && e < best_e)) {
                best = v;
                best_e = e;
            }
        }
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            const float ov = __shfl_xor(best, off, kWave);
            const int oe = __shfl_xor(best_e, off, kWave);
            if (ov > best || (ov == best && oe < best_e)) {
                best = ov;
                best_e = oe;
            }
        }
        if (c == 0) first = best;
        const float p = expf(best - first);      // the first choice is the largest
        total += p;
        if (lane == 0) {
            chosen[static_cast<size_t>(t) * top + c] = best_e;
            weight[static_cast<size_t>(t) * top + c] = p;      // divided by the total below
        }
        if (lane == best_e % kWave) z[best_e] = -INFINITY;     // the lane that reads this entry takes it out
    }
    if (lane == 0) {
        const float inv = 1.0f / total;
        for (int c = 0; c < top; ++c) weight[static_cast<size_t>(t) * top + c] *= inv;
    }
}

// One workgroup: counts per expert, their first rows, every (token, choice)'s row, and the table of tiles.
__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t* __restrict__ chosen, int32_t* __restrict__ row_token,
                                                         int32_t* __restrict__ place, int32_t* __restrict__ tiles,
                                                         int32_t* __restrict__ counts, int n_rows, int top, int experts,
                                                         int tile_rows) {
    __shared__ int count_s[kMaxExperts];
    __shared__ int first_s[kMaxExperts + 1];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) count_s[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n_rows; i += blockDim.x) atomicAdd(&count_s[chosen[i]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, n_tiles = 0;
        for (int e = 0; e < experts; ++e) {
            first_s[e] = at;
            const int c = count_s[e];
            for (int r = 0; r < c; r += tile_rows) {
                int32_t* tile = tiles + 1 + 3 * n_tiles++;
                tile[0] = e;
                tile[1] = at + r;
                tile[2] = min(tile_rows, c - r);
            }
            at += c;
        }
        first_s[experts] = at;
        tiles[0] = n_tiles;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += blockDim.x) {
        counts[e] = count_s[e];
        count_s[e] = 0;                          // now the cursor within the expert's rows
    }
    __syncthreads();
    // which row of its expert a (token, choice) gets does not matter to its result, only that it gets one
    for (int i = threadIdx.x; i < n_rows; i += blockDim.x) {
        const int e = chosen[i];
        const int row = first_s[e] + atomicAdd(&count_s[e], 1);
        row_token[row] = i / top;
        place[i] = row;
    }
}

// A workgroup of NW wavefronts takes one tile of rows (RT tiles of 16) and NW * 16 columns; a wavefront 16 columns of the
// gate and the same 16 of the up product.  Operands come straight from memory, 16 bytes a lane: a row of x and a row of
// W are both contiguous along k, which is the order in which the matrix cores take them.
template <typename T, int RT>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                          const int32_t* __restrict__ row_token,
                                                          const int32_t* __restrict__ tiles, T* __restrict__ act, int hidden,
                                                          int ff) {
    constexpr int E = 16 / sizeof(T);
    if (static_cast<int>(blockIdx.x) >= tiles[0]) return;
    const int32_t* tile = tiles + 1 + 3 * blockIdx.x;
    const int expert = tile[0], row0 = tile[1], n_rows = tile[2];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int lj = lane % 16, lg = lane / 16;
    const int n0 = (blockIdx.y * (blockDim.x / kWave) + wave) * 16;
    if (n0 >= ff) return;
    const bool aligned = hidden % E == 0;
    const T* wg = n0 + lj < ff ? w + (static_cast<size_t>(expert) * 2 * ff + n0 + lj) * hidden : nullptr;
    const T* wu = n0 + lj < ff ? w + (static_cast<size_t>(expert) * 2 * ff + ff + n0 + lj) * hidden : nullptr;
    const T* xr[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
        xr[r] = r * 16 + lj < n_rows ? x + static_cast<size_t>(row_token[row0 + r * 16 + lj]) * hidden : nullptr;
    m_f32x4 g[RT], u[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) g[r] = u[r] = m_f32x4{0.f, 0.f, 0.f, 0.f};
    // the loads of U steps of k are issued together, so that a step waits for memory once in U
    constexpr int U = RT >= 4 ? 2 : 4;
    for (int k0 = 0; k0 < hidden; k0 += 4 * E * U) {
        m_u32x4 a[U], b[U], xv[U][RT];
#pragma unroll
        for (int s = 0; s < U; ++s) {
            const int k = k0 + s * 4 * E + lg * E;
            a[s] = row_piece<T>(wg, k, hidden, aligned);
            b[s] = row_piece<T>(wu, k, hidden, aligned);
#pragma unroll
            for (int r = 0; r < RT; ++r) xv[s][r] = row_piece<T>(xr[r], k, hidden, aligned);
        }
#pragma unroll
        for (int s = 0; s < U; ++s)
#pragma unroll
            for (int r = 0; r < RT; ++r) {
                g[r] = mma16<T>(a[s], xv[s][r], g[r]);
                u[r] = mma16<T>(b[s], xv[s][r], u[r]);
            }
    }
    // the lane holds columns n0 + 4 lg + v of row lj of every tile of 16
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        if (r * 16 + lj >= n_rows) continue;
        T* o = act + static_cast<size_t>(row0 + r * 16 + lj) * ff;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int n = n0 + 4 * lg + v;
            const float gate = g[r][v];
            if (n < ff) o[n] = from_float<T>(gate / (1.0f + expf(-gate)) * u[r][v]);
        }
    }
}

// Experts without a gate: act = relu(x Wu^T)^2; w [experts][ff][hidden].  The same tiling with one product a wavefront.
template <typename T, int RT>
__global__ __launch_bounds__(256) void moe_up_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                     const int32_t* __restrict__ row_token, const int32_t* __restrict__ tiles,
                                                     T* __restrict__ act, int hidden, int ff) {
    constexpr int E = 16 / sizeof(T);
    if (static_cast<int>(blockIdx.x) >= tiles[0]) return;
    const int32_t* tile = tiles + 1 + 3 * blockIdx.x;
    const int expert = tile[0], row0 = tile[1], n_rows = tile[2];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int lj = lane % 16, lg = lane / 16;
    const int n0 = (blockIdx.y * (blockDim.x / kWave) + wave) * 16;
    if (n0 >= ff) return;
    const bool aligned = hidden % E == 0;
    const T* wu = n0 + lj < ff ? w + (static_cast<size_t>(expert) * ff + n0 + lj) * hidden : nullptr;
    const T* xr[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
        xr[r] = r * 16 + lj < n_rows ? x + static_cast<size_t>(row_token[row0 + r * 16 + lj]) * hidden : nullptr;
    m_f32x4 u[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) u[r] = m_f32x4{0.f, 0.f, 0.f, 0.f};
    constexpr int U = RT >= 4 ? 2 : 4;
    for (int k0 = 0; k0 < hidden; k0 += 4 * E * U) {
        m_u32x4 b[U], xv[U][RT];
#pragma unroll
        for (int s = 0; s < U; ++s) {
            const int k = k0 + s * 4 * E + lg * E;
            b[s] = row_piece<T>(wu, k, hidden, aligned);
#pragma unroll
            for (int r = 0; r < RT; ++r) xv[s][r] = row_piece<T>(xr[r], k, hidden, aligned);
        }
#pragma unroll
        for (int s = 0; s < U; ++s)
#pragma unroll
            for (int r = 0; r < RT; ++r) u[r] = mma16<T>(b[s], xv[s][r], u[r]);
    }
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        if (r * 16 + lj >= n_rows) continue;
        T* o = act + static_cast<size_t>(row0 + r * 16 + lj) * ff;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int n = n0 + 4 * lg + v;
            const float z = fmaxf(u[r][v], 0.f);
            if (n < ff) o[n] = from_float<T>(z * z);
        }
    }
}

template <typename T, int RT>
__global__ __launch_bounds__(256) void moe_down_kernel(const T* __restrict__ act, const T* __restrict__ w,
                                                       const int32_t* __restrict__ tiles, float* __restrict__ y, int hidden,
                                                       int ff) {
    constexpr int E = 16 / sizeof(T);
    if (static_cast<int>(blockIdx.x) >= tiles[0]) return;
    const int32_t* tile = tiles + 1 + 3 * blockIdx.x;
    const int expert = tile[0], row0 = tile[1], n_rows = tile[2];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int lj = lane % 16, lg = lane / 16;
    const int n0 = (blockIdx.y * (blockDim.x / kWave) + wave) * 16;
    if (n0 >= hidden) return;
    const bool aligned = ff % E == 0;
    const T* wd = n0 + lj < hidden ? w + (static_cast<size_t>(expert) * hidden + n0 + lj) * ff : nullptr;
    const T* ar[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) ar[r] = r * 16 + lj < n_rows ? act + static_cast<size_t>(row0 + r * 16 + lj) * ff : nullptr;
    m_f32x4 acc[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) acc[r] = m_f32x4{0.f, 0.f, 0.f, 0.f};
    constexpr int U = RT >= 4 ? 2 : 4;
    for (int k0 = 0; k0 < ff; k0 += 4 * E * U) {
        m_u32x4 a[U], av[U][RT];
#pragma unroll
        for (int s = 0; s < U; ++s) {
            const int k = k0 + s * 4 * E + lg * E;
            a[s] = row_piece<T>(wd, k, ff, aligned);
#pragma unroll
            for (int r = 0; r < RT; ++r) av[s][r] = row_piece<T>(ar[r], k, ff, aligned);
        }
#pragma unroll
        for (int s = 0; s < U; ++s)
#pragma unroll
            for (int r = 0; r < RT; ++r) acc[r] = mma16<T>(a[s], av[s][r], acc[r]);
    }
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        if (r * 16 + lj >= n_rows) continue;
        float* o = y + static_cast<size_t>(row0 + r * 16 + lj) * hidden;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int n = n0 + 4 * lg + v;
            if (n < hidden) o[n] = acc[r][v];
        }
    }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int32_t* __restrict__ place,
                                                          const float* __restrict__ weight, float* __restrict__ out, int top,
                                                          int hidden) {
    const int t = blockIdx.x;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        float acc = 0.f;
        for (int c = 0; c < top; ++c)
            acc = fmaf(weight[static_cast<size_t>(t) * top + c], y[static_cast<size_t>(place[static_cast<size_t>(t) * top + c]) * hidden + j], acc);
        out[static_cast<size_t>(t) * hidden + j] = acc;
    }
}

}  // namespace egpt

using namespace egpt;

extern "C" int egpt_moe_route(const void* x, const void* router, const void* bias, int32_t* chosen, float* weight, int n_tokens,
                              int hidden, int experts, int top, int score_all, const float* correction, float weight_scale,
                              int dtype, void* stream) {
    if (!x || !router || !chosen || !weight || n_tokens < 0 || hidden <= 0 || experts <= 0 || top <= 0 || top > experts ||
        (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (experts > kMaxExperts) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t lds = 2 * static_cast<size_t>(experts) * sizeof(float);
    const unsigned blocks = n_tokens;
    if (dtype == 0)
        moe_route_kernel<float><<<blocks, 256, lds, s>>>(static_cast<const float*>(x), static_cast<const float*>(router),
                                                         static_cast<const float*>(bias), chosen, weight, n_tokens, hidden,
                                                         experts, top, score_all, correction, weight_scale);
    else
        moe_route_kernel<bf16_t><<<blocks, 256, lds, s>>>(static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(router),
                                                          static_cast<const bf16_t*>(bias), chosen, weight, n_tokens, hidden,
                                                          experts, top, score_all, correction, weight_scale);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_moe_group(const int32_t* chosen, int32_t* row_token, int32_t* place, int32_t* tiles, int32_t* counts,
                              int n_tokens, int top, int experts, int tile_rows, void* stream) {
    if (!chosen || !row_token || !place || !tiles || !counts || n_tokens < 0 || top <= 0 || experts <= 0 ||
        (tile_rows != 16 && tile_rows != 32 && tile_rows != 64))
        return EGPT_BAD_ARGUMENT;
    if (experts > kMaxExperts) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    moe_group_kernel<<<1, 1024, 0, static_cast<hipStream_t>(stream)>>>(chosen, row_token, place, tiles, counts, n_tokens * top, top,
                                                                       experts, tile_rows);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

static inline int moe_waves(int max_tiles, int cols) {
    // few tiles: a wavefront to a workgroup, so that the columns spread over more compute units
    return static_cast<long long>(max_tiles) * ((cols + 63) / 64) < 512 ? 1 : 4;
}

extern "C" int egpt_moe_gate_up(const void* x, const void* w_gate_up, const int32_t* row_token, const int32_t* tiles, void* act,
                                int n_rows, int hidden, int ff, int experts, int tile_rows, int dtype, void* stream) {
    if (!x || !w_gate_up || !row_token || !tiles || !act || n_rows < 0 || hidden <= 0 || ff <= 0 || experts <= 0 ||
        (tile_rows != 16 && tile_rows != 32 && tile_rows != 64) || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (n_rows == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int max_tiles = n_rows / tile_rows + experts + 1;
    const int nw = moe_waves(max_tiles, ff);
    dim3 grid(max_tiles, (ff + nw * 16 - 1) / (nw * 16));
    if (grid.y > 65535) return EGPT_UNSUPPORTED_SIZE;
#define EGPT_MOE_GU(T_, RT_)                                                                                             \
    moe_gate_up_kernel<T_, RT_><<<grid, nw * 64, 0, s>>>(static_cast<const T_*>(x), static_cast<const T_*>(w_gate_up), row_token, \
                                                         tiles, static_cast<T_*>(act), hidden, ff)
    if (dtype == 0) {
        if (tile_rows == 16) EGPT_MOE_GU(float, 1); else if (tile_rows == 32) EGPT_MOE_GU(float, 2); else EGPT_MOE_GU(float, 4);
    } else {
        if (tile_rows == 16) EGPT_MOE_GU(bf16_t, 1); else if (tile_rows == 32) EGPT_MOE_GU(bf16_t, 2); else EGPT_MOE_GU(bf16_t, 4);
    }
#undef EGPT_MOE_GU
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_moe_up(const void* x, const void* w_up, const int32_t* row_token, const int32_t* tiles, void* act, int n_rows,
                           int hidden, int ff, int experts, int tile_rows, int dtype, void* stream) {
    if (!x || !w_up || !row_token || !tiles || !act || n_rows < 0 || hidden <= 0 || ff <= 0 || experts <= 0 ||
        (tile_rows != 16 && tile_rows != 32 && tile_rows != 64) || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (n_rows == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int max_tiles = n_rows / tile_rows + experts + 1;
    const int nw = moe_waves(max_tiles, ff);
    dim3 grid(max_tiles, (ff + nw * 16 - 1) / (nw * 16));
    if (grid.y > 65535) return EGPT_UNSUPPORTED_SIZE;
#define EGPT_MOE_UP(T_, RT_)                                                                                        \
    moe_up_kernel<T_, RT_><<<grid, nw * 64, 0, s>>>(static_cast<const T_*>(x), static_cast<const T_*>(w_up), row_token, \
                                                    tiles, static_cast<T_*>(act), hidden, ff)
    if (dtype == 0) {
        if (tile_rows == 16) EGPT_MOE_UP(float, 1); else if (tile_rows == 32) EGPT_MOE_UP(float, 2); else EGPT_MOE_UP(float, 4);
    } else {
        if (tile_rows == 16) EGPT_MOE_UP(bf16_t, 1); else if (tile_rows == 32) EGPT_MOE_UP(bf16_t, 2); else EGPT_MOE_UP(bf16_t, 4);
    }
#undef EGPT_MOE_UP
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_moe_down(const void* act, const void* w_down, const int32_t* tiles, float* y, int n_rows, int hidden, int ff,
                             int experts, int tile_rows, int dtype, void* stream) {
    if (!act || !w_down || !tiles || !y || n_rows < 0 || hidden <= 0 || ff <= 0 || experts <= 0 ||
        (tile_rows != 16 && tile_rows != 32 && tile_rows != 64) || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (n_rows == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int max_tiles = n_rows / tile_rows + experts + 1;
    const int nw = moe_waves(max_tiles, hidden);
    dim3 grid(max_tiles, (hidden + nw * 16 - 1) / (nw * 16));
    if (grid.y > 65535) return EGPT_UNSUPPORTED_SIZE;
#define EGPT_MOE_DOWN(T_, RT_)                                                                                          \
    moe_down_kernel<T_, RT_><<<grid, nw * 64, 0, s>>>(static_cast<const T_*>(act), static_cast<const T_*>(w_down), tiles, y, \
                                                      hidden, ff)
    if (dtype == 0) {
        if (tile_rows == 16) EGPT_MOE_DOWN(float, 1); else if (tile_rows == 32) EGPT_MOE_DOWN(float, 2); else EGPT_MOE_DOWN(float, 4);
    } else {
        if (tile_rows == 16) EGPT_MOE_DOWN(bf16_t, 1); else if (tile_rows == 32) EGPT_MOE_DOWN(bf16_t, 2); else EGPT_MOE_DOWN(bf16_t, 4);
    }
#undef EGPT_MOE_DOWN
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_moe_combine(const float* y, const int32_t* place, const float* weight, float* out, int n_tokens, int top,
                                int hidden, void* stream) {
    if (!y || !place || !weight || !out || n_tokens < 0 || top <= 0 || hidden <= 0) return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    moe_combine_kernel<<<n_tokens, 256, 0, static_cast<hipStream_t>(stream)>>>(y, place, weight, out, top, hidden);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
