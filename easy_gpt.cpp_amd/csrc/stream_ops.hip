// Operations on the residual stream and on logits for designs that do not norm by the root mean square alone:
// an embedding gather with a constant factor, the layer norm with weight and bias fused with the addition into the
// stream, the mean of two RMS-normed branch outputs, and the tanh cap on logits.  Statistics and sums are float32;
// values are rounded once, when they are written in the activation type.
#include "api.h"
#include "common.h"

namespace egpt {

namespace {
template <typename T>
ProductView<T> stream_view(const void* p, int n_splits, size_t stride) {
    ProductView<T> v;
    v.whole = n_splits == 0 ? static_cast<const T*>(p) : nullptr;
    v.partial = n_splits > 0 ? static_cast<const float*>(p) : nullptr;
    v.n_splits = n_splits;
    v.split_stride = stride;
    return v;
}
}  // namespace

// x[t, :] = E[id_t, :] * factor, written as the float32 residual stream.
template <typename T>
__global__ __launch_bounds__(256) void embed_scaled_kernel(const int32_t* __restrict__ ids, const T* __restrict__ table,
                                                           float factor, float* __restrict__ out, int hidden, int vocab) {
    const int t = blockIdx.x;
    int id = ids[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);      // ids are range-checked on the host; never read outside
    const T* row = table + static_cast<size_t>(id) * hidden;
    float* o = out + static_cast<size_t>(t) * hidden;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) o[j] = to_float(row[j]) * factor;
}

// h += delta (float32, written back unless rows are selected), then out = (h - mean) / sqrt(var + eps) * w + b with
// var the mean of the squared deviations.  Two passes over a row that lies in LDS: the mean first, then the
// deviations, so that a row with a large mean loses nothing to cancellation.
template <typename T>
__global__ __launch_bounds__(256) void add_layernorm_kernel(float* __restrict__ h, ProductView<T> delta,
                                                            const int32_t* __restrict__ rows, const T* __restrict__ weight,
                                                            const T* __restrict__ bias, float eps, T* __restrict__ out,
                                                            int hidden) {
    extern __shared__ float row_s[];
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
    float* hrow = h + src * hidden;
    const bool has_delta = delta.present();
    const bool write_back = rows == nullptr && has_delta;
    float sum = 0.f;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        float v = hrow[j];
        if (has_delta) v += delta.at(src * hidden + j);
        if (write_back) hrow[j] = v;
        row_s[j] = v;
        sum += v;
    }
    const float mean = block_sum(sum, scratch) / static_cast<float>(hidden);
    float dev = 0.f;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        const float d = row_s[j] - mean;
        dev = fmaf(d, d, dev);
    }
    const float inv = 1.0f / sqrtf(block_sum(dev, scratch) / static_cast<float>(hidden) + eps);
    T* orow = out + static_cast<size_t>(r) * hidden;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        float y = (row_s[j] - mean) * inv * to_float(weight[j]);
        if (bias) y += to_float(bias[j]);
        orow[j] = from_float<T>(y);
    }
}

// out[t, :] = factor_a * a[t, :] / rms(a[t, :]) * wa + factor_b * b[t, :] / rms(b[t, :]) * wb, float32: what two branches
// that are normed before they are joined leave for the residual stream.  Without weights (wa null) the branches are not
// normed: out = factor_a * a + factor_b * b.
template <typename T>
__global__ __launch_bounds__(256) void normed_pair_mean_kernel(ProductView<T> a, ProductView<T> b, const T* __restrict__ bias_a,
                                                               const T* __restrict__ bias_b, const T* __restrict__ wa,
                                                               const T* __restrict__ wb, float eps, float factor_a, float factor_b,
                                                               float* __restrict__ out, int hidden) {
    extern __shared__ float pair_s[];
    __shared__ float scratch[16];
    float* a_s = pair_s;
    float* b_s = pair_s + hidden;
    const size_t base = static_cast<size_t>(blockIdx.x) * hidden;
    float ssa = 0.f, ssb = 0.f;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        float x = a.at(base + j), y = b.at(base + j);
        if (bias_a) x += to_float(bias_a[j]);
        if (bias_b) y += to_float(bias_b[j]);
        a_s[j] = x;
        b_s[j] = y;
        ssa = fmaf(x, x, ssa);
        ssb = fmaf(y, y, ssb);
    }
    if (wa == nullptr) {
        for (int j = threadIdx.x; j < hidden; j += blockDim.x) out[base + j] = factor_a * a_s[j] + factor_b * b_s[j];
        return;
    }
    const float inv_a = inv_rms(block_sum(ssa, scratch), 1.0f / static_cast<float>(hidden), eps);
    const float inv_b = inv_rms(block_sum(ssb, scratch), 1.0f / static_cast<float>(hidden), eps);
    for (int j = threadIdx.x; j < hidden; j += blockDim.x)
        out[base + j] = factor_a == factor_b ? factor_a * (a_s[j] * inv_a * to_float(wa[j]) + b_s[j] * inv_b * to_float(wb[j]))
                                             : factor_a * (a_s[j] * inv_a * to_float(wa[j])) + factor_b * (b_s[j] * inv_b * to_float(wb[j]));
}

// x[t, :] = E[id_t, :] + P[position_t, :]: a token's vector plus a learned vector of its position, added in float32
// and written as the float32 residual stream.
template <typename T>
__global__ __launch_bounds__(256) void embed_positions_kernel(const int32_t* __restrict__ ids, const int32_t* __restrict__ positions,
                                                              const T* __restrict__ table, const T* __restrict__ pos_table,
                                                              float* __restrict__ out, int hidden, int vocab, int max_pos) {
    const int t = blockIdx.x;
    int id = ids[t], p = positions[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);      // both are range-checked on the host; never read outside
    p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
    const T* row = table + static_cast<size_t>(id) * hidden;
    const T* prow = pos_table + static_cast<size_t>(p) * hidden;
    float* o = out + static_cast<size_t>(t) * hidden;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) o[j] = to_float(row[j]) + to_float(prow[j]);
}

// A branch's output joins the stream behind a norm of its own:  x = h + mult * LN(y) * post_w  (LN without bias, the
// statistics of y's row in two passes over LDS).  With a second product y2 the branch is fy * y + fy2 * y2.  With a history (every earlier result of the depth, float32
// [n_hist + 1][rows][hidden]) x is kept as result n_hist and what goes on is the weighted sum
// v = sum_(j <= n_hist) mix[j] * hist[j]; otherwise v = x.  v is written to h_out (which may be h itself), and with a
// next norm's weight LN(v) * next_w is written to `out` in the activation type.  One workgroup per row.
template <typename T>
__global__ __launch_bounds__(256) void post_norm_add_kernel(const float* h, ProductView<T> y, ProductView<T> y2, float fy, float fy2,
                                                            const T* __restrict__ post_w, float eps, float mult,
                                                            float* hist, int n_hist, size_t hist_stride,
                                                            const float* __restrict__ mix, float* h_out,
                                                            const T* __restrict__ next_w, T* __restrict__ out, int hidden) {
    extern __shared__ float row_s[];
    __shared__ float scratch[16];
    const size_t base = static_cast<size_t>(blockIdx.x) * hidden;
    const float inv_n = 1.0f / static_cast<float>(hidden);
    float sum = 0.f;
    const bool two = y2.present();                       // the branch is fy * y + fy2 * y2: two products not yet added up
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        float v = y.at(base + j);
        if (two) v = fy * v + fy2 * y2.at(base + j);
        row_s[j] = v;
        sum += v;
    }
    float mean = block_sum(sum, scratch) * inv_n;
    float dev = 0.f;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        const float d = row_s[j] - mean;
        dev = fmaf(d, d, dev);
    }
    float inv = 1.0f / sqrtf(block_sum(dev, scratch) * inv_n + eps);
    sum = 0.f;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        float x = h[base + j] + mult * ((row_s[j] - mean) * inv * to_float(post_w[j]));
        if (hist != nullptr) {
            hist[static_cast<size_t>(n_hist) * hist_stride + base + j] = x;
            float v = 0.f;
            for (int i = 0; i < n_hist; ++i) v = fmaf(mix[i], hist[static_cast<size_t>(i) * hist_stride + base + j], v);
            x = fmaf(mix[n_hist], x, v);
        }
        h_out[base + j] = x;
        row_s[j] = x;
        sum += x;
    }
    if (next_w == nullptr) return;
    mean = block_sum(sum, scratch) * inv_n;
    dev = 0.f;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        const float d = row_s[j] - mean;
        dev = fmaf(d, d, dev);
    }
    inv = 1.0f / sqrtf(block_sum(dev, scratch) * inv_n + eps);
    for (int j = threadIdx.x; j < hidden; j += blockDim.x)
        out[base + j] = from_float<T>((row_s[j] - mean) * inv * to_float(next_w[j]));
}

// x <- x * scale, then (cap > 0) x <- cap * tanh(x / cap)
__global__ __launch_bounds__(256) void tanh_cap_kernel(float* __restrict__ x, float scale, float cap, size_t n) {
    const float inv = cap > 0.f ? 1.0f / cap : 0.f;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const float v = x[i] * scale;
        x[i] = cap > 0.f ? cap * tanhf(v * inv) : v;
    }
}

}  // namespace egpt

using namespace egpt;

extern "C" int egpt_embed_scaled(const int32_t* ids, const void* table, float factor, float* out, int n_tokens, int hidden,
                                 int vocab, int dtype, void* stream) {
    if (!ids || !table || !out || n_tokens < 0 || hidden <= 0 || vocab <= 0 || (dtype != 0 && dtype != 1)) return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == 0)
        embed_scaled_kernel<float><<<n_tokens, 256, 0, s>>>(ids, static_cast<const float*>(table), factor, out, hidden, vocab);
    else
        embed_scaled_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(ids, static_cast<const bf16_t*>(table), factor, out, hidden, vocab);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_add_layernorm(float* h, const void* delta, int delta_splits, int delta_rows, const int32_t* rows,
                                  const void* weight, const void* bias, float eps, void* out, int n_rows, int hidden,
                                  int dtype, void* stream) {
    if (!h || !weight || !out || n_rows < 0 || hidden <= 0 || delta_splits < 0 || (dtype != 0 && dtype != 1)) return EGPT_BAD_ARGUMENT;
    if (delta && delta_rows <= 0) return EGPT_BAD_ARGUMENT;
    if (hidden > 16384) return EGPT_UNSUPPORTED_SIZE;          // a row lies in LDS
    if (n_rows == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t stride = static_cast<size_t>(delta_rows) * hidden;
    const size_t lds = static_cast<size_t>(hidden) * sizeof(float);
    if (dtype == 0)
        add_layernorm_kernel<float><<<n_rows, 256, lds, s>>>(h, stream_view<float>(delta, delta_splits, stride), rows,
                                                             static_cast<const float*>(weight), static_cast<const float*>(bias),
                                                             eps, static_cast<float*>(out), hidden);
    else
        add_layernorm_kernel<bf16_t><<<n_rows, 256, lds, s>>>(h, stream_view<bf16_t>(delta, delta_splits, stride), rows,
                                                              static_cast<const bf16_t*>(weight), static_cast<const bf16_t*>(bias),
                                                              eps, static_cast<bf16_t*>(out), hidden);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_normed_pair_mean(const void* a, int a_splits, const void* b, int b_splits, const void* bias_a,
                                     const void* bias_b, const void* wa, const void* wb, float eps, float factor, float factor_b,
                                     float* out, int n_rows, int hidden, int dtype, void* stream) {
    if (!a || !b || (wa == nullptr) != (wb == nullptr) || !out || n_rows < 0 || hidden <= 0 || a_splits < 0 || b_splits < 0 || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (hidden > 8192) return EGPT_UNSUPPORTED_SIZE;           // two rows lie in LDS
    if (n_rows == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t stride = static_cast<size_t>(n_rows) * hidden;
    const size_t lds = 2 * static_cast<size_t>(hidden) * sizeof(float);
    if (dtype == 0)
        normed_pair_mean_kernel<float><<<n_rows, 256, lds, s>>>(
            stream_view<float>(a, a_splits, stride), stream_view<float>(b, b_splits, stride), static_cast<const float*>(bias_a),
            static_cast<const float*>(bias_b), static_cast<const float*>(wa), static_cast<const float*>(wb), eps, factor, factor_b, out, hidden);
    else
        normed_pair_mean_kernel<bf16_t><<<n_rows, 256, lds, s>>>(
            stream_view<bf16_t>(a, a_splits, stride), stream_view<bf16_t>(b, b_splits, stride), static_cast<const bf16_t*>(bias_a),
            static_cast<const bf16_t*>(bias_b), static_cast<const bf16_t*>(wa), static_cast<const bf16_t*>(wb), eps, factor, factor_b, out, hidden);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_embed_positions(const int32_t* ids, const int32_t* positions, const void* table, const void* pos_table,
                                    float* out, int n_tokens, int hidden, int vocab, int max_pos, int dtype, void* stream) {
    if (!ids || !positions || !table || !pos_table || !out || n_tokens < 0 || hidden <= 0 || vocab <= 0 || max_pos <= 0 ||
        (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == 0)
        embed_positions_kernel<float><<<n_tokens, 256, 0, s>>>(ids, positions, static_cast<const float*>(table),
                                                               static_cast<const float*>(pos_table), out, hidden, vocab, max_pos);
    else
        embed_positions_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(ids, positions, static_cast<const bf16_t*>(table),
                                                                static_cast<const bf16_t*>(pos_table), out, hidden, vocab, max_pos);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_post_norm_add(const float* h, const void* y, int y_splits, const void* y2, int y2_splits, float fy, float fy2,
                                  const void* post_w, float eps, float mult,
                                  float* hist, int n_hist, const float* mix, float* h_out, const void* next_w, void* out,
                                  int n_rows, int hidden, int dtype, void* stream) {
    if (!h || !y || !post_w || !h_out || n_rows < 0 || hidden <= 0 || y_splits < 0 || y2_splits < 0 || n_hist < 0 || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if ((hist != nullptr) != (mix != nullptr) || (next_w != nullptr) != (out != nullptr)) return EGPT_BAD_ARGUMENT;
    if (hidden > 16384) return EGPT_UNSUPPORTED_SIZE;          // a row lies in LDS
    if (n_rows == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t stride = static_cast<size_t>(n_rows) * hidden;
    const size_t lds = static_cast<size_t>(hidden) * sizeof(float);
    if (dtype == 0)
        post_norm_add_kernel<float><<<n_rows, 256, lds, s>>>(h, stream_view<float>(y, y_splits, stride),
                                                             stream_view<float>(y2, y2 ? y2_splits : 0, stride), fy, fy2,
                                                             static_cast<const float*>(post_w), eps, mult, hist, n_hist, stride, mix,
                                                             h_out, static_cast<const float*>(next_w), static_cast<float*>(out), hidden);
    else
        post_norm_add_kernel<bf16_t><<<n_rows, 256, lds, s>>>(h, stream_view<bf16_t>(y, y_splits, stride),
                                                              stream_view<bf16_t>(y2, y2 ? y2_splits : 0, stride), fy, fy2,
                                                              static_cast<const bf16_t*>(post_w), eps, mult, hist, n_hist, stride, mix,
                                                              h_out, static_cast<const bf16_t*>(next_w), static_cast<bf16_t*>(out), hidden);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_tanh_cap(float* x, float scale, float cap, long long n, void* stream) {
    if (!x || n < 0 || !(cap >= 0.f)) return EGPT_BAD_ARGUMENT;           // cap 0: the factor alone
    if (n == 0) return EGPT_OK;
    const long long blocks = (n + 255) / 256;
    tanh_cap_kernel<<<static_cast<unsigned>(blocks > 4096 ? 4096 : blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(
        x, scale, cap, static_cast<size_t>(n));
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
