// What stands between a mixer's input product and its attention, head by head, for mixers that norm or rotate
// single heads: an embedding gather with its norm, per-head RMS norms of queries, keys and values with the store
// into cache pages, the preparation of latent attention (latent norm, interleaved rotation of the rotated parts,
// store of latent and rotated key), and a sigmoid gate.  Statistics, angles and the rotation are float32; values
// are rounded once, when they are written in the activation type.
//
// A product arrives as one tensor of the activation type or as float32 partial sums (ProductView in common.h).
// Keys lie in pages [page][kv head][offset][key size], values in pages [page][kv head][value size][offset].
#include "api.h"
#include "common.h"

namespace egpt {

// A product whose x operand was (h * norm weight) still lacks each row's factor 1 / sqrt(sum_s ss[s][row] / hidden + eps):
// the sums of squares arrive beside it (null: the product is complete).
struct RowFactor {
    const float* ss;
    int splits, n_rows, hidden;
    float eps;
    __device__ __forceinline__ float of(int row) const {
        if (ss == nullptr) return 1.0f;
        float total = 0.f;
        for (int s = 0; s < splits; ++s) total += ss[static_cast<size_t>(s) * n_rows + row];
        return inv_rms(total, 1.0f / static_cast<float>(hidden), eps);
    }
};

constexpr int kMaxHeadWidth = 1024;                   // the widest head (or latent) these kernels take
constexpr int kOwn = kMaxHeadWidth / kWave;           // values of it that a lane keeps

// x[t, :] = E[id_t, :] / sqrt(mean(E[id_t, :]^2) + eps) * w, written as the residual stream (float32 or fixed point).
template <typename T, typename R>
__global__ __launch_bounds__(256) void embed_rmsnorm_kernel(const int32_t* __restrict__ ids, const T* __restrict__ table,
                                                            const T* __restrict__ weight, float eps,
                                                            R* __restrict__ out, int hidden, int vocab) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    int id = ids[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);      // ids are range-checked on the host; never read outside
    const T* row = table + static_cast<size_t>(id) * hidden;
    float ss = 0.f;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        const float v = to_float(row[j]);
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    const float inv = inv_rms(ss, 1.0f / static_cast<float>(hidden), eps);
    R* o = out + static_cast<size_t>(t) * hidden;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) residual_store(o + j, to_float(row[j]) * inv * to_float(weight[j]));
}

// One wavefront per (token, head) of a product row [nq heads of dk | nkv heads of dk | nkv heads of dv | anything else]
// of row_width values: a query or key head is divided by its root mean square and multiplied by the weight that all
// heads share (a null weight: the head passes as it is, or with kNormPlain it is divided and no more), a value head
// is divided by its root mean square if kNormValues is set.  With kValuesAreKeys the row holds no value heads: value
// head g is key head g as it was projected (dv == dk).  Queries and keys are rotated when rot_dims > 0: the first
// rot_dims places of a head turn by the angles whose (cos, sin) stand in cos_sin [T][rot_dims / 2][2] (both times mag),
// place i with place i + rot_dims / 2, or with kInterleaved place 2i with place 2i + 1; behind the norm, or with
// kNormAfterRotation before it.  Queries go to q_out [T][nq * dk]; keys and values to the pages at slots[t] (slots
// null: nothing is stored).
constexpr int kNormValues = 1, kNormPlain = 2, kNormAfterRotation = 4, kValuesAreKeys = 8, kInterleaved = 16;

template <typename T>
__global__ __launch_bounds__(kWave) void head_norm_store_kernel(
    ProductView<T> proj, RowFactor factor, int row_width, T* __restrict__ q_out, const T* __restrict__ q_weight,
    const T* __restrict__ k_weight, float eps, int flags, const float* __restrict__ cos_sin, int rot_dims, float mag,
    const int32_t* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache, int nq, int nkv,
    int dk, int dv, int page_size) {
    const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
    const int kind = hh < nq ? 0 : (hh < nq + nkv ? 1 : 2);
    const int head = kind == 0 ? hh : (kind == 1 ? hh - nq : hh - nq - nkv);
    const int width = kind == 2 ? dv : dk;
    const bool own_keys = kind == 2 && (flags & kValuesAreKeys);
    const int in_off = kind == 0 ? head * dk : ((kind == 1 || own_keys) ? nq * dk + head * dk : (nq + nkv) * dk + head * dv);
    if (kind != 0 && slots == nullptr) return;
    const T* weight = kind == 0 ? q_weight : (kind == 1 ? k_weight : nullptr);
    const bool normed = kind == 2 ? (flags & kNormValues) != 0 : (weight != nullptr || (flags & kNormPlain));
    const int rot = kind == 2 ? 0 : rot_dims;
    const int half = rot / 2;
    const bool interleaved = (flags & kInterleaved) != 0;
    const bool norm_after = (flags & kNormAfterRotation) != 0;
    const size_t base = static_cast<size_t>(t) * row_width + in_off;
    const float* cs = cos_sin + static_cast<size_t>(t) * rot_dims;
    const float rf = factor.of(t);
    float v[kOwn], pv[kOwn];
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < kOwn; ++r) {
        const int d = lane + r * kWave;
        v[r] = d < width ? proj.at(base + d) * rf : 0.f;
        pv[r] = 0.f;
        if (d < rot) {                                    // the place this one turns with
            const int pd = interleaved ? (d ^ 1) : (d < half ? d + half : d - half);
            pv[r] = proj.at(base + pd) * rf;
        }
    }
    auto turn = [&](int d, float own, float other) {
        const int i = interleaved ? d / 2 : (d < half ? d : d - half);
        const bool first = interleaved ? (d & 1) == 0 : d < half;
        const float c = cs[2 * i] * mag, s = cs[2 * i + 1] * mag;
        return first ? __fmaf_rn(own, c, -__fmul_rn(other, s)) : __fmaf_rn(other, s, __fmul_rn(own, c));
    };
    if (norm_after) {
#pragma unroll
        for (int r = 0; r < kOwn; ++r) {
            const int d = lane + r * kWave;
            if (d < rot) v[r] = turn(d, v[r], pv[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < kOwn; ++r) ss = fmaf(v[r], v[r], ss);
    float inv = 1.0f;
    if (normed) inv = inv_rms(wave_sum(ss), 1.0f / static_cast<float>(width), eps);
    long page = 0;
    int off = 0;
    if (kind != 0) {
        page = slots[t] / page_size;
        off = slots[t] % page_size;
    }
#pragma unroll
    for (int r = 0; r < kOwn; ++r) {
        const int d = lane + r * kWave;
        if (d >= width) continue;
        float y = v[r] * inv;
        if (weight != nullptr) y *= to_float(weight[d]);
        if (d < rot && !norm_after) {
            const int pd = interleaved ? (d ^ 1) : (d < half ? d + half : d - half);
            float py = pv[r] * inv;
            if (weight != nullptr) py *= to_float(weight[pd]);
            y = turn(d, y, py);
        }
        if (kind == 0)
            q_out[static_cast<size_t>(t) * nq * dk + head * dk + d] = from_float<T>(y);
        else if (kind == 1)
            k_cache[((page * nkv + head) * page_size + off) * dk + d] = from_float<T>(y);
        else
            v_cache[((page * nkv + head) * dv + d) * page_size + off] = from_float<T>(y);
    }
}

// One wavefront per (token, query head) and one more per token for the latent, of a product row
// [nq heads of (dim unrotated | rot rotated) | rank latent | rot shared rotated key | anything else].
// With qsrc present the query heads are the rows [nq heads of (dim | rot)] of that product instead, and the latent begins
// at place `lead` of proj's row (behind whatever stands there in the queries' stead).
// A query head's unrotated part goes to q_plain [T][nq][dim], its rotated part, rotated, to q_full [T][nq][rank + rot]
// behind the first rank places (which the caller fills with the unrotated part carried into the latent space).
// The latent is divided by its root mean square and multiplied by c_weight; with the rotated shared key behind it
// it is the token's key [rank + rot] in the pages, and alone, transposed, its value [rank].
// Rotation: the pair (2i, 2i + 1) of the rotated part, i < rot_dims / 2, by the angle whose (cos, sin) stand in
// cos_sin [T][rot_dims / 2][2]; both are multiplied by mag; places from rot_dims on pass unchanged.
template <typename T>
__global__ __launch_bounds__(kWave) void latent_prep_kernel(
    ProductView<T> proj, RowFactor factor, int row_width, ProductView<T> qsrc, int lead, T* __restrict__ q_plain, T* __restrict__ q_full,
    const T* __restrict__ c_weight, float eps, const float* __restrict__ cos_sin, float mag, int rot_dims, const int32_t* __restrict__ slots,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int nq, int dim, int rot, int rank, int page_size) {
    const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
    const size_t row = static_cast<size_t>(t) * row_width;
    const float* cs = cos_sin + static_cast<size_t>(t) * rot_dims;      // (rot_dims / 2) pairs of (cos, sin)
    const int dk = rank + rot;
    const float rf = factor.of(t);
    if (hh < nq) {
        const bool own = qsrc.present();
        const ProductView<T>& src = own ? qsrc : proj;
        const float qf = own ? 1.0f : rf;
        const size_t base = (own ? static_cast<size_t>(t) * nq * (dim + rot) : row) + static_cast<size_t>(hh) * (dim + rot);
        for (int d = lane; d < dim; d += kWave)
            q_plain[(static_cast<size_t>(t) * nq + hh) * dim + d] = from_float<T>(src.at(base + d) * qf);
        T* dst = q_full + (static_cast<size_t>(t) * nq + hh) * dk + rank;
        for (int i = lane; i < rot / 2; i += kWave) {
            const float u = src.at(base + dim + 2 * i) * qf, w = src.at(base + dim + 2 * i + 1) * qf;
            float ru = u, rw = w;
            if (2 * i + 1 < rot_dims) rotate_pair(u, w, cs[2 * i] * mag, cs[2 * i + 1] * mag, ru, rw);
            dst[2 * i] = from_float<T>(ru);
            dst[2 * i + 1] = from_float<T>(rw);
        }
        if ((rot & 1) && lane == 0) dst[rot - 1] = from_float<T>(src.at(base + dim + rot - 1) * qf);
        return;
    }
    if (slots == nullptr) return;
    const size_t base = row + static_cast<size_t>(lead);
    float v[kOwn];
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < kOwn; ++r) {
        const int d = lane + r * kWave;
        v[r] = d < rank ? proj.at(base + d) * rf : 0.f;
        ss = fmaf(v[r], v[r], ss);
    }
    const float inv = inv_rms(wave_sum(ss), 1.0f / static_cast<float>(rank), eps);
    const long page = slots[t] / page_size;
    const int off = slots[t] % page_size;
    T* kdst = k_cache + (page * page_size + off) * dk;
    T* vdst = v_cache + page * rank * page_size + off;
#pragma unroll
    for (int r = 0; r < kOwn; ++r) {
        const int d = lane + r * kWave;
        if (d >= rank) continue;
        const T y = from_float<T>(v[r] * inv * to_float(c_weight[d]));
        kdst[d] = y;
        vdst[static_cast<long>(d) * page_size] = y;
    }
    for (int i = lane; i < rot / 2; i += kWave) {
        const float u = proj.at(base + rank + 2 * i) * rf, w = proj.at(base + rank + 2 * i + 1) * rf;
        float ru = u, rw = w;
        if (2 * i + 1 < rot_dims) rotate_pair(u, w, cs[2 * i] * mag, cs[2 * i + 1] * mag, ru, rw);
        kdst[rank + 2 * i] = from_float<T>(ru);
        kdst[rank + 2 * i + 1] = from_float<T>(rw);
    }
    if ((rot & 1) && lane == 0) kdst[rank + rot - 1] = from_float<T>(proj.at(base + rank + rot - 1) * rf);
}

// out[t][n] = x[t][n] * sigmoid(g[t][gate_off + n]); x lies [T][N], or with heads > 0 head by head [heads][T][N / heads]
// (what a product batched over heads leaves).  g: columns of a product row of width gate_width.
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(const T* __restrict__ x, int heads, ProductView<T> g,
                                                           RowFactor factor, int gate_width, int gate_off, T* __restrict__ out,
                                                           int n_tokens, int n) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= static_cast<size_t>(n_tokens) * n) return;
    const int t = static_cast<int>(idx / n), c = static_cast<int>(idx % n);
    size_t src = idx;
    if (heads > 0) {
        const int per = n / heads;
        src = (static_cast<size_t>(c / per) * n_tokens + t) * per + c % per;
    }
    const float gate = g.at(static_cast<size_t>(t) * gate_width + gate_off + c) * factor.of(t);
    out[idx] = from_float<T>(to_float(x[src]) * (1.0f / (1.0f + expf(-gate))));
}


// One workgroup per token of a product row [nq heads of dk | nkv heads of dk | nkv heads of dv | anything else]: the
// bias [nq * dk + nkv * dk + nkv * dv] is added, the queries are RMS-normed over all heads at once (one statistic
// over nq * dk values, a weight per value), and so are the keys (over nkv * dk); the queries are then multiplied by
// 1 + coef * ln(floor((p + 1) / every) + 1) at position p (every == 0: no such factor).  Queries go to q_out
// [T][nq * dk], keys and values to the pages at slots[t] (slots null: nothing is stored).
template <typename T>
__global__ __launch_bounds__(256) void whole_norm_store_kernel(
    ProductView<T> proj, int row_width, const T* __restrict__ bias, T* __restrict__ q_out, const T* __restrict__ q_weight,
    const T* __restrict__ k_weight, float eps, const int32_t* __restrict__ positions, float coef, int every,
    const int32_t* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache, int nq, int nkv, int dk, int dv,
    int page_size) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const size_t row = static_cast<size_t>(t) * row_width;
    const int qw = nq * dk, kw = nkv * dk, vw = nkv * dv;
    // a row of up to kKeep values per thread stays in registers between the statistics and the stores (all of a thread's
    // loads in flight together); wider rows are read twice
    constexpr int kKeep = 16;
    const bool kept = qw + kw + vw <= kKeep * static_cast<int>(blockDim.x);
    float val[kKeep];
    float ssq = 0.f, ssk = 0.f;
    if (kept) {
#pragma unroll
        for (int i = 0; i < kKeep; ++i) {
            const int j = threadIdx.x + i * blockDim.x;
            val[i] = 0.f;
            if (j < qw + kw + vw) {
                val[i] = proj.at(row + j);
                if (bias) val[i] += to_float(bias[j]);
            }
        }
#pragma unroll
        for (int i = 0; i < kKeep; ++i) {
            const int j = threadIdx.x + i * blockDim.x;
            if (j < qw) ssq = fmaf(val[i], val[i], ssq); else if (j < qw + kw) ssk = fmaf(val[i], val[i], ssk);
        }
    } else {
        for (int j = threadIdx.x; j < qw + kw; j += blockDim.x) {
            float v = proj.at(row + j);
            if (bias) v += to_float(bias[j]);
            if (j < qw) ssq = fmaf(v, v, ssq); else ssk = fmaf(v, v, ssk);
        }
    }
    float inv_q = 1.0f, inv_k = 1.0f;
    if (q_weight) inv_q = inv_rms(block_sum(ssq, scratch), 1.0f / static_cast<float>(qw), eps);
    if (k_weight) inv_k = inv_rms(block_sum(ssk, scratch), 1.0f / static_cast<float>(kw), eps);
    if (every > 0) inv_q *= 1.0f + coef * logf(static_cast<float>((positions[t] + 1) / every + 1));
    long page = 0;
    int off = 0;
    if (slots != nullptr) {
        page = slots[t] / page_size;
        off = slots[t] % page_size;
    }
    auto put = [&](int j, float v) {
        if (j < qw) {
            v *= inv_q;
            if (q_weight) v *= to_float(q_weight[j]);
            q_out[static_cast<size_t>(t) * qw + j] = from_float<T>(v);
        } else if (slots == nullptr) {
            return;
        } else if (j < qw + kw) {
            const int jj = j - qw;
            v *= inv_k;
            if (k_weight) v *= to_float(k_weight[jj]);
            k_cache[((page * nkv + jj / dk) * page_size + off) * dk + jj % dk] = from_float<T>(v);
        } else {
            const int jj = j - qw - kw;
            v_cache[((page * nkv + jj / dv) * dv + jj % dv) * page_size + off] = from_float<T>(v);
        }
    };
    if (kept) {
#pragma unroll
        for (int i = 0; i < kKeep; ++i) {
            const int j = threadIdx.x + i * blockDim.x;
            if (j < qw + kw + vw) put(j, val[i]);
        }
    } else {
        for (int j = threadIdx.x; j < qw + kw + vw; j += blockDim.x) {
            float v = proj.at(row + j);
            if (bias) v += to_float(bias[j]);
            put(j, v);
        }
    }
}

// out[t][h * dv + d] = x[t][h * dv + d] / rms(x[t][h * dv ..]) * weight[d] * act(g[t][gate_off + h * dv + d]): the
// RMS norm of every head's output with a weight that the heads share, and a gate from columns of a product row (no
// gate: the normed heads as they are).  x is float32 (one tensor, or partial sums that are added here) or, with xa
// present, a product in the activation type; its rows are x_width values wide and the heads begin at place 0.  The
// gate's activation: 0 silu, 1 sigmoid, 2 none (the columns hold the factor itself).  One wavefront per (token, head).
template <typename T>
__global__ __launch_bounds__(kWave) void head_norm_gate_kernel(ProductView<float> x, ProductView<T> xa, int x_width,
                                                               const T* __restrict__ weight, float eps, ProductView<T> g,
                                                               int gate_width, int gate_off, int gate_act, T* __restrict__ out,
                                                               int heads, int dv) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const size_t xr = static_cast<size_t>(t) * x_width + static_cast<size_t>(h) * dv;
    const bool act_typed = xa.present();
    float ss = 0.f;
    for (int d = lane; d < dv; d += kWave) {
        const float v = act_typed ? xa.at(xr + d) : x.at(xr + d);
        ss = fmaf(v, v, ss);
    }
    const float inv = inv_rms(wave_sum(ss), 1.0f / static_cast<float>(dv), eps);
    for (int d = lane; d < dv; d += kWave) {
        float y = (act_typed ? xa.at(xr + d) : x.at(xr + d)) * inv * to_float(weight[d]);
        if (g.present()) {
            const float gate = g.at(static_cast<size_t>(t) * gate_width + gate_off + h * dv + d);
            const float sig = 1.0f / (1.0f + expf(-gate));
            y *= gate_act == 0 ? gate * sig : (gate_act == 1 ? sig : gate);
        }
        out[(static_cast<size_t>(t) * heads + h) * dv + d] = from_float<T>(y);
    }
}

// The same for heads of many values: a workgroup of four wavefronts per (token, head), the statistics through LDS.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_wide_kernel(ProductView<float> x, ProductView<T> xa, int x_width,
                                                                    const T* __restrict__ weight, float eps, ProductView<T> g,
                                                                    int gate_width, int gate_off, int gate_act, T* __restrict__ out,
                                                                    int heads, int dv) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, h = blockIdx.y;
    const size_t xr = static_cast<size_t>(t) * x_width + static_cast<size_t>(h) * dv;
    const bool act_typed = xa.present();
    constexpr int kKeep = 8;                              // values of the head that a thread keeps between the two passes
    float v[kKeep];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
        const int d = threadIdx.x + i * 256;
        v[i] = d < dv ? (act_typed ? xa.at(xr + d) : x.at(xr + d)) : 0.f;
        ss = fmaf(v[i], v[i], ss);
    }
    for (int d = threadIdx.x + kKeep * 256; d < dv; d += 256) {
        const float u = act_typed ? xa.at(xr + d) : x.at(xr + d);
        ss = fmaf(u, u, ss);
    }
    const float inv = inv_rms(block_sum(ss, scratch), 1.0f / static_cast<float>(dv), eps);
    auto put = [&](int d, float value) {
        float y = value * inv * to_float(weight[d]);
        if (g.present()) {
            const float gate = g.at(static_cast<size_t>(t) * gate_width + gate_off + h * dv + d);
            const float sig = 1.0f / (1.0f + expf(-gate));
            y *= gate_act == 0 ? gate * sig : (gate_act == 1 ? sig : gate);
        }
        out[(static_cast<size_t>(t) * heads + h) * dv + d] = from_float<T>(y);
    };
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
        const int d = threadIdx.x + i * 256;
        if (d < dv) put(d, v[i]);
    }
    for (int d = threadIdx.x + kKeep * 256; d < dv; d += 256) put(d, act_typed ? xa.at(xr + d) : x.at(xr + d));
}

template <typename T>
static ProductView<T> view_of(const void* p, int n_splits, size_t split_stride) {
    ProductView<T> v;
    v.whole = n_splits == 0 ? static_cast<const T*>(p) : nullptr;
    v.partial = n_splits > 0 ? static_cast<const float*>(p) : nullptr;
    v.n_splits = n_splits;
    v.split_stride = split_stride;
    return v;
}

}  // namespace egpt

using namespace egpt;

extern "C" int egpt_embed_rmsnorm(const int32_t* ids, const void* table, const void* weight, float eps, void* out,
                                  int fixed, int n_tokens, int hidden, int vocab, int dtype, void* stream) {
    if (!ids || !table || !weight || !out || n_tokens < 0 || hidden <= 0 || vocab <= 0 || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == 0 && !fixed)
        embed_rmsnorm_kernel<<<n_tokens, 256, 0, s>>>(ids, static_cast<const float*>(table), static_cast<const float*>(weight),
                                                      eps, static_cast<float*>(out), hidden, vocab);
    else if (dtype == 0)
        embed_rmsnorm_kernel<<<n_tokens, 256, 0, s>>>(ids, static_cast<const float*>(table), static_cast<const float*>(weight),
                                                      eps, static_cast<fixed_t*>(out), hidden, vocab);
    else if (!fixed)
        embed_rmsnorm_kernel<<<n_tokens, 256, 0, s>>>(ids, static_cast<const bf16_t*>(table), static_cast<const bf16_t*>(weight),
                                                      eps, static_cast<float*>(out), hidden, vocab);
    else
        embed_rmsnorm_kernel<<<n_tokens, 256, 0, s>>>(ids, static_cast<const bf16_t*>(table), static_cast<const bf16_t*>(weight),
                                                      eps, static_cast<fixed_t*>(out), hidden, vocab);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_head_norm_store(const void* proj, int n_splits, const float* row_ss, int ss_splits, int hidden,
                                    float norm_eps, int row_width, void* q_out, const void* q_weight,
                                    const void* k_weight, float eps, int flags, const float* cos_sin, int rot_dims, float mag,
                                    const int32_t* slots, void* k_cache, void* v_cache, int n_tokens, int nq, int nkv, int dk,
                                    int dv, int page_size, int dtype, void* stream) {
    if (!proj || !q_out || n_splits < 0 || n_tokens < 0 || nq <= 0 || nkv <= 0 || dk <= 0 || dv <= 0 || page_size <= 0 ||
        (dtype != 0 && dtype != 1) || flags < 0 || flags >= 32)
        return EGPT_BAD_ARGUMENT;
    if (slots && (!k_cache || !v_cache)) return EGPT_BAD_ARGUMENT;
    if (rot_dims < 0 || rot_dims % 2 || rot_dims > dk || (rot_dims > 0 && !cos_sin)) return EGPT_BAD_ARGUMENT;
    if ((flags & kValuesAreKeys) && (dv != dk || (flags & kNormValues))) return EGPT_BAD_ARGUMENT;
    if (row_width < (nq + nkv) * dk + ((flags & kValuesAreKeys) ? 0 : nkv * dv)) return EGPT_BAD_ARGUMENT;
    if (dk > kMaxHeadWidth || dv > kMaxHeadWidth || nq + 2 * nkv > 65535) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (row_ss && (n_splits < 1 || ss_splits < 1 || hidden <= 0)) return EGPT_BAD_ARGUMENT;
    const RowFactor factor{row_ss, ss_splits, n_tokens, hidden, norm_eps};
    const size_t stride = static_cast<size_t>(n_tokens) * row_width;
    dim3 grid(n_tokens, nq + 2 * nkv);
    if (dtype == 0)
        head_norm_store_kernel<float><<<grid, kWave, 0, s>>>(
            view_of<float>(proj, n_splits, stride), factor, row_width, static_cast<float*>(q_out), static_cast<const float*>(q_weight),
            static_cast<const float*>(k_weight), eps, flags, cos_sin, rot_dims, mag, slots, static_cast<float*>(k_cache),
            static_cast<float*>(v_cache), nq, nkv, dk, dv, page_size);
    else
        head_norm_store_kernel<bf16_t><<<grid, kWave, 0, s>>>(
            view_of<bf16_t>(proj, n_splits, stride), factor, row_width, static_cast<bf16_t*>(q_out), static_cast<const bf16_t*>(q_weight),
            static_cast<const bf16_t*>(k_weight), eps, flags, cos_sin, rot_dims, mag, slots, static_cast<bf16_t*>(k_cache),
            static_cast<bf16_t*>(v_cache), nq, nkv, dk, dv, page_size);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_latent_prep(const void* proj, int n_splits, const float* row_ss, int ss_splits, int hidden,
                                float norm_eps, int row_width, const void* queries, int q_splits, int lead, void* q_plain,
                                void* q_full, const void* c_weight, float eps, const float* cos_sin, float mag, int rot_dims,
                                const int32_t* slots, void* k_cache, void* v_cache, int n_tokens, int nq, int dim,
                                int rot, int rank, int page_size, int dtype, void* stream) {
    if (!proj || !q_plain || !q_full || !c_weight || n_splits < 0 || n_tokens < 0 || nq <= 0 || dim <= 0 || rot < 0 ||
        rank <= 0 || page_size <= 0 || rot_dims < 0 || rot_dims > rot || rot_dims % 2 || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (rot_dims > 0 && !cos_sin) return EGPT_BAD_ARGUMENT;
    if (slots && (!k_cache || !v_cache)) return EGPT_BAD_ARGUMENT;
    if (!queries) lead = nq * (dim + rot);
    if (lead < 0 || q_splits < 0 || row_width < lead + rank + rot) return EGPT_BAD_ARGUMENT;
    if (rank > kMaxHeadWidth || nq + 1 > 65535) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (row_ss && (n_splits < 1 || ss_splits < 1 || hidden <= 0)) return EGPT_BAD_ARGUMENT;
    const RowFactor factor{row_ss, ss_splits, n_tokens, hidden, norm_eps};
    const size_t stride = static_cast<size_t>(n_tokens) * row_width;
    const size_t q_stride = static_cast<size_t>(n_tokens) * nq * (dim + rot);
    dim3 grid(n_tokens, nq + 1);
    if (dtype == 0)
        latent_prep_kernel<float><<<grid, kWave, 0, s>>>(
            view_of<float>(proj, n_splits, stride), factor, row_width, view_of<float>(queries, queries ? q_splits : 0, q_stride), lead,
            static_cast<float*>(q_plain), static_cast<float*>(q_full),
            static_cast<const float*>(c_weight), eps, cos_sin, mag, rot_dims, slots, static_cast<float*>(k_cache),
            static_cast<float*>(v_cache), nq, dim, rot, rank, page_size);
    else
        latent_prep_kernel<bf16_t><<<grid, kWave, 0, s>>>(
            view_of<bf16_t>(proj, n_splits, stride), factor, row_width, view_of<bf16_t>(queries, queries ? q_splits : 0, q_stride), lead,
            static_cast<bf16_t*>(q_plain), static_cast<bf16_t*>(q_full), static_cast<const bf16_t*>(c_weight), eps, cos_sin, mag, rot_dims, slots,
            static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), nq, dim, rot, rank, page_size);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_sigmoid_gate(const void* x, int heads, const void* gate, int gate_splits, const float* row_ss,
                                 int ss_splits, int hidden, float norm_eps, int gate_width,
                                 int gate_off, void* out, int n_tokens, int n, int dtype, void* stream) {
    if (!x || !gate || !out || n_tokens < 0 || n <= 0 || heads < 0 || (heads > 0 && n % heads) || gate_splits < 0 ||
        gate_off < 0 || gate_off + n > gate_width || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (row_ss && (gate_splits < 1 || ss_splits < 1 || hidden <= 0)) return EGPT_BAD_ARGUMENT;
    const RowFactor factor{row_ss, ss_splits, n_tokens, hidden, norm_eps};
    const size_t total = static_cast<size_t>(n_tokens) * n;
    const size_t stride = static_cast<size_t>(n_tokens) * gate_width;
    const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
    if (dtype == 0)
        sigmoid_gate_kernel<float><<<blocks, 256, 0, s>>>(static_cast<const float*>(x), heads,
                                                          view_of<float>(gate, gate_splits, stride), factor, gate_width, gate_off,
                                                          static_cast<float*>(out), n_tokens, n);
    else
        sigmoid_gate_kernel<bf16_t><<<blocks, 256, 0, s>>>(static_cast<const bf16_t*>(x), heads,
                                                           view_of<bf16_t>(gate, gate_splits, stride), factor, gate_width,
                                                           gate_off, static_cast<bf16_t*>(out), n_tokens, n);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_whole_norm_store(const void* proj, int n_splits, int row_width, const void* bias, void* q_out,
                                     const void* q_weight, const void* k_weight, float eps, const int32_t* positions,
                                     float coef, int every, const int32_t* slots, void* k_cache, void* v_cache,
                                     int n_tokens, int nq, int nkv, int dk, int dv, int page_size, int dtype, void* stream) {
    // nkv == 0: a row holds queries alone (a layer that reads keys and values that another layer stored); nothing is stored
    if (!proj || !q_out || n_splits < 0 || n_tokens < 0 || nq <= 0 || nkv < 0 || dk <= 0 || dv <= 0 || page_size <= 0 ||
        every < 0 || (dtype != 0 && dtype != 1) || (nkv == 0 && slots))
        return EGPT_BAD_ARGUMENT;
    if (row_width < (nq + nkv) * dk + nkv * dv) return EGPT_BAD_ARGUMENT;
    if (every > 0 && !positions) return EGPT_BAD_ARGUMENT;
    if (slots && (!k_cache || !v_cache)) return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t stride = static_cast<size_t>(n_tokens) * row_width;
    if (dtype == 0)
        whole_norm_store_kernel<float><<<n_tokens, 256, 0, s>>>(
            view_of<float>(proj, n_splits, stride), row_width, static_cast<const float*>(bias), static_cast<float*>(q_out),
            static_cast<const float*>(q_weight), static_cast<const float*>(k_weight), eps, positions, coef, every, slots,
            static_cast<float*>(k_cache), static_cast<float*>(v_cache), nq, nkv, dk, dv, page_size);
    else
        whole_norm_store_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(
            view_of<bf16_t>(proj, n_splits, stride), row_width, static_cast<const bf16_t*>(bias), static_cast<bf16_t*>(q_out),
            static_cast<const bf16_t*>(q_weight), static_cast<const bf16_t*>(k_weight), eps, positions, coef, every, slots,
            static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), nq, nkv, dk, dv, page_size);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_head_norm_gate(const void* x, int x_splits, int x_is_act, int x_width, const void* weight, float eps,
                                   const void* gate, int gate_splits, int gate_width, int gate_off, int gate_act, void* out,
                                   int n_tokens, int heads, int dv, int dtype, void* stream) {
    if (!x || x_splits < 0 || !weight || !out || n_tokens < 0 || heads <= 0 || dv <= 0 || gate_splits < 0 || (dtype != 0 && dtype != 1) ||
        gate_act < 0 || gate_act > 2 || x_width < heads * dv || (x_is_act && x_splits != 0))
        return EGPT_BAD_ARGUMENT;
    if (gate && (gate_off < 0 || gate_off + heads * dv > gate_width)) return EGPT_BAD_ARGUMENT;
    if (!gate) gate_splits = 0;
    if (heads > 65535) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t stride = static_cast<size_t>(n_tokens) * gate_width;
    dim3 grid(n_tokens, heads);
    // x float32 [n_tokens][x_width] (x_splits 0) or partial sums [x_splits][n_tokens][x_width]; or of the activation type
    ProductView<float> xv;
    xv.whole = (x_splits == 0 && !x_is_act) ? static_cast<const float*>(x) : nullptr;
    xv.partial = x_splits > 0 ? static_cast<const float*>(x) : nullptr;
    xv.n_splits = x_splits;
    xv.split_stride = static_cast<size_t>(n_tokens) * x_width;
    if (dv > 256) {                                       // heads of many values: four wavefronts a head
        if (dtype == 0)
            head_norm_gate_wide_kernel<float><<<grid, 256, 0, s>>>(xv, view_of<float>(x_is_act ? x : nullptr, 0, 0), x_width,
                                                                   static_cast<const float*>(weight), eps,
                                                                   view_of<float>(gate, gate_splits, stride), gate_width, gate_off,
                                                                   gate_act, static_cast<float*>(out), heads, dv);
        else
            head_norm_gate_wide_kernel<bf16_t><<<grid, 256, 0, s>>>(xv, view_of<bf16_t>(x_is_act ? x : nullptr, 0, 0), x_width,
                                                                    static_cast<const bf16_t*>(weight), eps,
                                                                    view_of<bf16_t>(gate, gate_splits, stride), gate_width, gate_off,
                                                                    gate_act, static_cast<bf16_t*>(out), heads, dv);
        EGPT_CHECK_LAUNCH();
        return EGPT_OK;
    }
    if (dtype == 0)
        head_norm_gate_kernel<float><<<grid, kWave, 0, s>>>(xv, view_of<float>(x_is_act ? x : nullptr, 0, 0), x_width,
                                                            static_cast<const float*>(weight), eps,
                                                            view_of<float>(gate, gate_splits, stride), gate_width, gate_off, gate_act,
                                                            static_cast<float*>(out), heads, dv);
    else
        head_norm_gate_kernel<bf16_t><<<grid, kWave, 0, s>>>(xv, view_of<bf16_t>(x_is_act ? x : nullptr, 0, 0), x_width,
                                                             static_cast<const bf16_t*>(weight), eps,
                                                             view_of<bf16_t>(gate, gate_splits, stride), gate_width, gate_off, gate_act,
                                                             static_cast<bf16_t*>(out), heads, dv);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
