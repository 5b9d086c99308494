// Activations of feed-forward layers that have no gate product: the square of relu, and a polynomial of the inner
// values whose three powers are each divided by their root mean square over the token's inner values.  Optionally the
// whole row is multiplied by the sigmoid of one more column of the same product (a gate of one number per token, whose
// weights ride as one more row of the up matrix).  Statistics and the activation are float32; the result is rounded
// once, when it is written in the activation type for the product that follows.
#include "api.h"
#include "common.h"

#include <type_traits>

namespace egpt {

constexpr int kKeep = 32;      // inner values that a thread keeps in registers between the statistics and the result

// 16 bytes of a row as floats, and back
__device__ __forceinline__ void load_piece(const float* p, float* v) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
__device__ __forceinline__ void load_piece(const bf16_t* p, float* v) {
    const uint4 x = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
__device__ __forceinline__ void store_piece(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
}
__device__ __forceinline__ void store_piece(bf16_t* p, const float* v) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        w[i] = static_cast<uint32_t>(f32_to_bf16_bits(v[2 * i])) | (static_cast<uint32_t>(f32_to_bf16_bits(v[2 * i + 1])) << 16);
    *reinterpret_cast<uint4*>(p) = uint4{w[0], w[1], w[2], w[3]};
}

// E values of a row, from the activation type or from float32
template <int E>
__device__ __forceinline__ void load_values(const float* p, float* v) {
#pragma unroll
    for (int i = 0; i < E; i += 4) load_piece(p + i, v + i);
}
template <int E>
__device__ __forceinline__ void load_values(const bf16_t* p, float* v) {
    static_assert(E == 8, "a piece of bfloat16 is 8 values");
    load_piece(p, v);
}

// MODE 0: the square of relu.  MODE 1: the polynomial of normed powers; a row of up to 256 * kKeep values is read once
// and kept in registers, a longer one is read twice.  S: void, the product as it comes (any number of partial sums,
// any width); else its element type (the activation type of a whole product, float for a product written out in
// float32), read and written in pieces of 16 bytes of the result: rows start on 16 bytes then.
template <typename T, int MODE, typename S>
__global__ __launch_bounds__(256) void ff_activation_kernel(ProductView<T> z, int z_width, int cols, const float* __restrict__ coef,
                                                            float eps, int gate_col, T* __restrict__ out) {
    __shared__ float scratch[16];
    constexpr int E = 16 / sizeof(T);
    constexpr bool PIECES = !std::is_void<S>::value;
    using Src = typename std::conditional<PIECES, S, T>::type;
    const Src* src = nullptr;
    if constexpr (PIECES) {
        if constexpr (std::is_same<S, T>::value) src = z.n_splits == 0 ? z.whole : reinterpret_cast<const Src*>(z.partial);
        else src = reinterpret_cast<const Src*>(z.partial);
    }
    const size_t row = static_cast<size_t>(blockIdx.x) * z_width;
    T* o = out + static_cast<size_t>(blockIdx.x) * cols;
    float gate = 1.0f;
    if (gate_col >= 0) gate = 1.0f / (1.0f + expf(-z.at(row + gate_col)));
    if constexpr (MODE == 0) {
        if constexpr (PIECES) {
            for (int j = threadIdx.x * E; j < cols; j += 256 * E) {
                float v[E];
                load_values<E>(src + row + j, v);
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const float r = fmaxf(v[e], 0.f);
                    v[e] = r * r * gate;
                }
                store_piece(o + j, v);
            }
        } else {
            for (int j = threadIdx.x; j < cols; j += blockDim.x) {
                const float v = fmaxf(z.at(row + j), 0.f);
                o[j] = from_float<T>(v * v * gate);
            }
        }
    } else {
        // mean squares of z, z^2 and z^3 over the row
        const bool kept = cols <= 256 * kKeep;
        float v[kKeep];
        float s1 = 0.f, s2 = 0.f, s3 = 0.f;
        auto take = [&](float x) {
            const float x2 = x * x;
            s1 += x2;
            s2 = fmaf(x2, x2, s2);
            s3 = fmaf(x2 * x, x2 * x, s3);
        };
        if (kept) {
            if constexpr (PIECES) {
#pragma unroll
                for (int i = 0; i < kKeep / E; ++i) {
                    const int j = (threadIdx.x + i * 256) * E;
                    if (j < cols) {
                        load_values<E>(src + row + j, v + i * E);
#pragma unroll
                        for (int e = 0; e < E; ++e) take(v[i * E + e]);
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < kKeep; ++i) {
                    const int j = threadIdx.x + i * 256;
                    v[i] = j < cols ? z.at(row + j) : 0.f;
                    take(v[i]);
                }
            }
        } else {
            for (int j = threadIdx.x; j < cols; j += blockDim.x) take(z.at(row + j));
        }
        const float inv_n = 1.0f / static_cast<float>(cols);
        const float n1 = coef[0] / sqrtf(block_sum(s1, scratch) * inv_n + eps);
        const float n2 = coef[1] / sqrtf(block_sum(s2, scratch) * inv_n + eps);
        const float n3 = coef[2] / sqrtf(block_sum(s3, scratch) * inv_n + eps);
        const float c3 = coef[3];
        auto poly = [&](float x) {
            const float x2 = x * x;
            return (n1 * x + n2 * x2 + n3 * (x2 * x) + c3) * gate;
        };
        if (kept) {
            if constexpr (PIECES) {
#pragma unroll
                for (int i = 0; i < kKeep / E; ++i) {
                    const int j = (threadIdx.x + i * 256) * E;
                    if (j < cols) {
#pragma unroll
                        for (int e = 0; e < E; ++e) v[i * E + e] = poly(v[i * E + e]);
                        store_piece(o + j, v + i * E);
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < kKeep; ++i) {
                    const int j = threadIdx.x + i * 256;
                    if (j < cols) o[j] = from_float<T>(poly(v[i]));
                }
            }
        } else {
            for (int j = threadIdx.x; j < cols; j += blockDim.x) o[j] = from_float<T>(poly(z.at(row + j)));
        }
    }
}

}  // namespace egpt

using namespace egpt;

template <typename T>
static void launch_activation(const void* z, int z_splits, int z_width, int cols, int mode, const float* coef, float eps,
                              int gate_col, void* out, int n_tokens, hipStream_t s) {
    ProductView<T> v;
    v.whole = z_splits == 0 ? static_cast<const T*>(z) : nullptr;
    v.partial = z_splits > 0 ? static_cast<const float*>(z) : nullptr;
    v.n_splits = z_splits;
    v.split_stride = static_cast<size_t>(n_tokens) * z_width;
    // in pieces of 16 bytes where the product is whole or written out in float32 once, and its rows and the result's
    // start on 16 bytes
    constexpr int E = 16 / sizeof(T);
    const bool aligned = z_width % E == 0 && cols % E == 0 && reinterpret_cast<uintptr_t>(z) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(out) % 16 == 0;
    const int src = !aligned || z_splits > 1 ? 0 : (z_splits == 0 ? 1 : 2);      // as it comes; of T; of float
    T* o = static_cast<T*>(out);
#define EGPT_ACTIVATION(MODE, S) ff_activation_kernel<T, MODE, S><<<n_tokens, 256, 0, s>>>(v, z_width, cols, coef, eps, gate_col, o)
    if (mode == 0) {
        if (src == 0) EGPT_ACTIVATION(0, void);
        else if (src == 1) EGPT_ACTIVATION(0, T);
        else EGPT_ACTIVATION(0, float);
    } else {
        if (src == 0) EGPT_ACTIVATION(1, void);
        else if (src == 1) EGPT_ACTIVATION(1, T);
        else EGPT_ACTIVATION(1, float);
    }
#undef EGPT_ACTIVATION
}

extern "C" int egpt_ff_activation(const void* z, int z_splits, int z_width, int cols, int mode, const float* coef, float eps,
                                  int gate_col, void* out, int n_tokens, int dtype, void* stream) {
    if (!z || !out || z_splits < 0 || cols <= 0 || cols > z_width || n_tokens < 0 || (mode != 0 && mode != 1) ||
        (mode == 1 && !coef) || gate_col >= z_width || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == 0)
        launch_activation<float>(z, z_splits, z_width, cols, mode, coef, eps, gate_col, out, n_tokens, s);
    else
        launch_activation<bf16_t>(z, z_splits, z_width, cols, mode, coef, eps, gate_col, out, n_tokens, s);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
