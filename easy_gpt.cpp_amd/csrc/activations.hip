// Activations of feed-forward layers that have no gate product: the square of relu, and a polynomial of the inner
// values whose three powers are each divided by their root mean square over the token's inner values.  Optionally the
// whole row is multiplied by the sigmoid of one more column of the same product (a gate of one number per token, whose
// weights ride as one more row of the up matrix).  Statistics and the activation are float32; the result is rounded
// once, when it is written in the activation type for the product that follows.
#include "api.h"
#include "common.h"

namespace egpt {

template <typename T, int MODE>
__global__ __launch_bounds__(256) void ff_activation_kernel(ProductView<T> z, int z_width, int cols, const float* __restrict__ coef,
                                                            float eps, int gate_col, T* __restrict__ out) {
    __shared__ float scratch[16];
    const size_t row = static_cast<size_t>(blockIdx.x) * z_width;
    T* o = out + static_cast<size_t>(blockIdx.x) * cols;
    float gate = 1.0f;
    if (gate_col >= 0) gate = 1.0f / (1.0f + expf(-z.at(row + gate_col)));
    if constexpr (MODE == 0) {
        for (int j = threadIdx.x; j < cols; j += blockDim.x) {
            const float v = fmaxf(z.at(row + j), 0.f);
            o[j] = from_float<T>(v * v * gate);
        }
    } else {
        // mean squares of z, z^2 and z^3 over the row
        float s1 = 0.f, s2 = 0.f, s3 = 0.f;
        for (int j = threadIdx.x; j < cols; j += blockDim.x) {
            const float v = z.at(row + j);
            const float v2 = v * v;
            s1 += v2;
            s2 = fmaf(v2, v2, s2);
            s3 = fmaf(v2 * v, v2 * v, s3);
        }
        const float inv_n = 1.0f / static_cast<float>(cols);
        const float n1 = coef[0] / sqrtf(block_sum(s1, scratch) * inv_n + eps);
        const float n2 = coef[1] / sqrtf(block_sum(s2, scratch) * inv_n + eps);
        const float n3 = coef[2] / sqrtf(block_sum(s3, scratch) * inv_n + eps);
        const float c3 = coef[3];
        for (int j = threadIdx.x; j < cols; j += blockDim.x) {
            const float v = z.at(row + j);
            const float v2 = v * v;
            o[j] = from_float<T>((n1 * v + n2 * v2 + n3 * (v2 * v) + c3) * gate);
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
    if (mode == 0)
        ff_activation_kernel<T, 0><<<n_tokens, 256, 0, s>>>(v, z_width, cols, coef, eps, gate_col, static_cast<T*>(out));
    else
        ff_activation_kernel<T, 1><<<n_tokens, 256, 0, s>>>(v, z_width, cols, coef, eps, gate_col, static_cast<T*>(out));
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
