// Linear attention with a matrix state per head that decays per key channel:
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   S [dk][dv] float32 per request and head.
// The state is carried from step to step in a record per request; a step walks its tokens in order, whatever the cut of
// the prompt: every element of the state sees the same operations in the same order in a prompt's portion as in single
// tokens, so the result does not depend on the cut at all.  Decays, the state and the output sum are float32.
//
// egpt_channel_decay makes the decays a = sigmoid(z)^(1/tau) from a low-rank projection (z = W low + b);
// egpt_bounded_gate makes decays with a learned lower bound, a = l + (1 - l) sigmoid(z + b), from columns of a product;
// egpt_decayed_state_scan runs the recurrence; its queries may pass through SiLU on their way in, and its keys may be
// tied to the decays, k = 1 - a (a forget gate that also sets what is written), instead of columns of the product.
#include "api.h"
#include "common.h"

namespace egpt {

namespace {
template <typename T>
ProductView<T> scan_view(const void* p, int n_splits, size_t stride) {
    ProductView<T> v;
    v.whole = n_splits == 0 ? static_cast<const T*>(p) : nullptr;
    v.partial = n_splits > 0 ? static_cast<const float*>(p) : nullptr;
    v.n_splits = n_splits;
    v.split_stride = stride;
    return v;
}
}  // namespace

constexpr int kMaxRank = 1024;

// One workgroup per token: the token's low-rank vector in LDS, a thread per channel.
// sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau), with softplus(-z) = max(-z, 0) + log1p(exp(-|z|)).
template <typename T>
__global__ __launch_bounds__(256) void channel_decay_kernel(ProductView<T> low, int low_width, int low_off, int rank,
                                                            const T* __restrict__ w, const T* __restrict__ bias, float inv_tau,
                                                            float* __restrict__ decay, int channels) {
    __shared__ float low_s[kMaxRank];
    const int t = blockIdx.x;
    for (int r = threadIdx.x; r < rank; r += blockDim.x) low_s[r] = low.at(static_cast<size_t>(t) * low_width + low_off + r);
    __syncthreads();
    for (int c = threadIdx.x; c < channels; c += blockDim.x) {
        float z = bias ? to_float(bias[c]) : 0.f;
        const T* wr = w + static_cast<size_t>(c) * rank;
        for (int r = 0; r < rank; ++r) z = fmaf(to_float(wr[r]), low_s[r], z);
        const float log_sigmoid = -(fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z))));
        decay[static_cast<size_t>(t) * channels + c] = expf(log_sigmoid * inv_tau);
    }
}

// a[t][c] = lower[c] + (1 - lower[c]) * sigmoid(z[t][c] + bias[c]), float32; z are columns z_off.. of a product row.
template <typename T>
__global__ __launch_bounds__(256) void bounded_gate_kernel(ProductView<T> z, int z_width, int z_off, const T* __restrict__ bias,
                                                           const T* __restrict__ lower, float* __restrict__ gate, int channels,
                                                           size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const size_t t = idx / channels;
    const int c = static_cast<int>(idx % channels);
    float v = z.at(t * z_width + z_off + c);
    if (bias) v += to_float(bias[c]);
    const float low = lower ? to_float(lower[c]) : 0.f;
    gate[idx] = low + (1.0f - low) * (1.0f / (1.0f + expf(-v)));
}

constexpr int kScanTokens = 32;     // tokens staged in LDS at a time
constexpr int kScanCols = 64;       // value channels per workgroup: a lane is a column of the state
constexpr int kScanKeys = 16;       // key channels per workgroup
constexpr int kScanWaves = 4;       // wavefronts per workgroup, kScanKeys / kScanWaves key channels each

// The recurrence has no term that mixes two key channels but the sum o_t = sum_r S[r][:] q[r], so the key channels are
// dealt over workgroups: one workgroup of four wavefronts per (request, head, 64 value channels, 16 key channels), whose
// part of o_t goes to out[split] (float32 [splits][tokens][heads * dv]) for the consumer to add in the order of the
// splits.  A lane is one column of the state; wavefront w keeps four of the workgroup's key channels of that column in
// registers.  The queries, keys and decays that a wavefront needs are the same for all its lanes (one address in LDS);
// what bounds a token is what LDS returns for them (every lane gets its copy), which is why a workgroup takes few key
// channels.  The wavefronts' parts go through LDS and are added in the order of the wavefronts, a batch of kScanTokens
// tokens at a time; the batch's operands are staged in LDS, the next batch's loads in flight in registers meanwhile.
template <typename T>
__global__ __launch_bounds__(64 * kScanWaves) void decayed_state_scan_kernel(
    ProductView<T> proj, int proj_width, int q_off, int k_off, int v_off, float q_scale, const float* __restrict__ decay,
    float* __restrict__ states, const int32_t* __restrict__ slots, const unsigned char* __restrict__ fresh,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, float* __restrict__ out, int n_tokens, int heads,
    int dk, int dv, int key_splits, int q_silu, int tied_keys) {
    constexpr int NS = kScanWaves, DKR = kScanKeys / kScanWaves, THREADS = 64 * NS, DKP = kScanKeys;
    constexpr int QKA = kScanTokens * DKP / THREADS;          // values of q (or k, or decays) of a batch per thread
    constexpr int VL = kScanTokens * kScanCols / THREADS;     // values of v, and outputs, of a batch per thread
    static_assert(DKR == 4 && QKA * THREADS == kScanTokens * DKP && VL * THREADS == kScanTokens * kScanCols, "a batch divides evenly");
    __shared__ __attribute__((aligned(16))) float q_s[kScanTokens * DKP];
    __shared__ __attribute__((aligned(16))) float k_s[kScanTokens * DKP];
    __shared__ __attribute__((aligned(16))) float a_s[kScanTokens * DKP];
    __shared__ float v_s[kScanTokens * kScanCols];
    __shared__ float part_s[kScanTokens * NS * kScanCols];
    const int b = blockIdx.x, h = blockIdx.y;
    const int split = blockIdx.z % key_splits, col0 = (blockIdx.z / key_splits) * kScanCols, key0 = split * kScanKeys;
    const int n = q_len[b];
    if (n <= 0) return;
    const int t0 = q_start[b];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int j = col0 + lane;
    const bool has_col = j < dv;
    float* state = states + (static_cast<size_t>(slots[b]) * heads + h) * dk * dv;
    float* o_split = out + static_cast<size_t>(split) * n_tokens * heads * dv;
    float s[DKR];
    const bool start_anew = fresh != nullptr && fresh[b] != 0;
#pragma unroll
    for (int i = 0; i < DKR; ++i) {
        const int r = key0 + wave * DKR + i;
        s[i] = (!start_anew && has_col && r < dk) ? state[static_cast<size_t>(r) * dv + j] : 0.f;
    }
    const int channels = heads * dk;
    float rq[QKA], rk[QKA], ra[QKA], rv[VL];
    auto fetch = [&](int base) {
        const int count = min(kScanTokens, n - base);
#pragma unroll
        for (int u = 0; u < QKA; ++u) {
            const int idx = tid + u * THREADS;
            const int tt = idx / DKP, r = key0 + idx % DKP;
            rq[u] = rk[u] = ra[u] = 0.f;
            if (tt < count && r < dk) {
                const size_t row = static_cast<size_t>(t0 + base + tt);
                rq[u] = proj.at(row * proj_width + q_off + h * dk + r);      // (scaled when it is staged: nothing here waits for a load)
                ra[u] = decay[row * channels + h * dk + r];
                if (!tied_keys) rk[u] = proj.at(row * proj_width + k_off + h * dk + r);
            }
        }
#pragma unroll
        for (int u = 0; u < VL; ++u) {
            const int idx = tid + u * THREADS;
            const int tt = idx / kScanCols, c = idx % kScanCols;
            rv[u] = 0.f;
            if (tt < count && col0 + c < dv)
                rv[u] = proj.at(static_cast<size_t>(t0 + base + tt) * proj_width + v_off + h * dv + col0 + c);
        }
    };
    fetch(0);
    for (int base = 0; base < n; base += kScanTokens) {
        const int count = min(kScanTokens, n - base);
        __syncthreads();                          // the batch before is read, its parts are added
#pragma unroll
        for (int u = 0; u < QKA; ++u) {
            // (a tied key is 1 - a; a place that holds no token or no channel has a = 0 and would get k = 1, which meets a
            // query of zero and a state row that is never stored)
            q_s[tid + u * THREADS] = (q_silu ? rq[u] / (1.0f + expf(-rq[u])) : rq[u]) * q_scale;
            k_s[tid + u * THREADS] = tied_keys ? 1.0f - ra[u] : rk[u];
            a_s[tid + u * THREADS] = ra[u];
        }
#pragma unroll
        for (int u = 0; u < VL; ++u) v_s[tid + u * THREADS] = rv[u];
        __syncthreads();
        if (base + kScanTokens < n) fetch(base + kScanTokens);
        for (int tt = 0; tt < count; ++tt) {
            const float vj = v_s[tt * kScanCols + lane];
            const float4 a = *reinterpret_cast<const float4*>(a_s + tt * DKP + wave * DKR);
            const float4 k = *reinterpret_cast<const float4*>(k_s + tt * DKP + wave * DKR);
            const float4 q = *reinterpret_cast<const float4*>(q_s + tt * DKP + wave * DKR);
            s[0] = fmaf(a.x, s[0], k.x * vj);
            s[1] = fmaf(a.y, s[1], k.y * vj);
            s[2] = fmaf(a.z, s[2], k.z * vj);
            s[3] = fmaf(a.w, s[3], k.w * vj);
            part_s[(tt * NS + wave) * kScanCols + lane] = (s[0] * q.x + s[1] * q.y) + (s[2] * q.z + s[3] * q.w);
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < VL; ++u) {
            const int idx = tid + u * THREADS;
            const int tt = idx / kScanCols, c = idx % kScanCols;
            if (tt < count && col0 + c < dv) {
                float o = 0.f;
#pragma unroll
                for (int w = 0; w < NS; ++w) o += part_s[(tt * NS + w) * kScanCols + c];
                o_split[(static_cast<size_t>(t0 + base + tt) * heads + h) * dv + col0 + c] = o;
            }
        }
    }
    if (has_col) {
#pragma unroll
        for (int i = 0; i < DKR; ++i) {
            const int r = key0 + wave * DKR + i;
            if (r < dk) state[static_cast<size_t>(r) * dv + j] = s[i];
        }
    }
}

}  // namespace egpt

using namespace egpt;

extern "C" int egpt_channel_decay(const void* low, int low_splits, int low_width, int low_off, int rank, const void* w,
                                  const void* bias, float tau, float* decay, int n_tokens, int channels, int dtype, void* stream) {
    if (!low || !w || !decay || low_splits < 0 || rank <= 0 || low_off < 0 || low_off + rank > low_width || n_tokens < 0 ||
        channels <= 0 || !(tau > 0.f) || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (rank > kMaxRank) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t stride = static_cast<size_t>(n_tokens) * low_width;
    if (dtype == 0)
        channel_decay_kernel<float><<<n_tokens, 256, 0, s>>>(scan_view<float>(low, low_splits, stride), low_width, low_off, rank,
                                                             static_cast<const float*>(w), static_cast<const float*>(bias),
                                                             1.0f / tau, decay, channels);
    else
        channel_decay_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(scan_view<bf16_t>(low, low_splits, stride), low_width, low_off, rank,
                                                              static_cast<const bf16_t*>(w), static_cast<const bf16_t*>(bias),
                                                              1.0f / tau, decay, channels);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_bounded_gate(const void* z, int z_splits, int z_width, int z_off, const void* bias, const void* lower,
                                 float* gate, int n_tokens, int channels, int dtype, void* stream) {
    if (!z || !gate || z_splits < 0 || z_off < 0 || channels <= 0 || z_off + channels > z_width || n_tokens < 0 ||
        (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t stride = static_cast<size_t>(n_tokens) * z_width, total = static_cast<size_t>(n_tokens) * channels;
    const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
    if (dtype == 0)
        bounded_gate_kernel<float><<<blocks, 256, 0, s>>>(scan_view<float>(z, z_splits, stride), z_width, z_off,
                                                          static_cast<const float*>(bias), static_cast<const float*>(lower), gate,
                                                          channels, total);
    else
        bounded_gate_kernel<bf16_t><<<blocks, 256, 0, s>>>(scan_view<bf16_t>(z, z_splits, stride), z_width, z_off,
                                                           static_cast<const bf16_t*>(bias), static_cast<const bf16_t*>(lower), gate,
                                                           channels, total);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

template <typename T>
static int launch_scan(const void* proj, int n_splits, int proj_width, int q_off, int k_off, int v_off, float q_scale,
                       const float* decay, float* states, const int32_t* slots, const unsigned char* fresh,
                       const int32_t* q_start, const int32_t* q_len, int n_seqs, int n_tokens, float* out, int heads, int dk,
                       int dv, int q_silu, int tied_keys, hipStream_t s) {
    const ProductView<T> view = scan_view<T>(proj, n_splits, static_cast<size_t>(n_tokens) * proj_width);
    const int key_splits = (dk + kScanKeys - 1) / kScanKeys;
    dim3 grid(n_seqs, heads, (dv + kScanCols - 1) / kScanCols * key_splits);
    decayed_state_scan_kernel<T><<<grid, 64 * kScanWaves, 0, s>>>(view, proj_width, q_off, k_off, v_off, q_scale, decay, states, slots,
                                                                  fresh, q_start, q_len, out, n_tokens, heads, dk, dv, key_splits,
                                                                  q_silu, tied_keys);
    return EGPT_OK;
}

extern "C" int egpt_scan_key_splits(int dk) { return dk > 0 ? (dk + kScanKeys - 1) / kScanKeys : 0; }

extern "C" int egpt_decayed_state_scan(const void* proj, int n_splits, int proj_width, int q_off, int k_off, int v_off,
                                       float q_scale, const float* decay, float* states, const int32_t* slots,
                                       const unsigned char* fresh, const int32_t* q_start, const int32_t* q_len, int n_seqs,
                                       int n_tokens, float* out, int heads, int dk, int dv, int q_silu, int tied_keys,
                                       int dtype, void* stream) {
    if (!proj || !decay || !states || !slots || !q_start || !q_len || !out || n_splits < 0 || n_seqs <= 0 || n_tokens < 0 ||
        heads <= 0 || dk <= 0 || dv <= 0 || q_off < 0 || (!tied_keys && k_off < 0) || v_off < 0 || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (q_off + heads * dk > proj_width || (!tied_keys && k_off + heads * dk > proj_width) || v_off + heads * dv > proj_width)
        return EGPT_BAD_ARGUMENT;
    if (heads > 65535 || static_cast<long long>((dv + kScanCols - 1) / kScanCols) * ((dk + kScanKeys - 1) / kScanKeys) > 65535)
        return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == 0)
        launch_scan<float>(proj, n_splits, proj_width, q_off, k_off, v_off, q_scale, decay, states, slots, fresh, q_start,
                           q_len, n_seqs, n_tokens, out, heads, dk, dv, q_silu, tied_keys, s);
    else
        launch_scan<bf16_t>(proj, n_splits, proj_width, q_off, k_off, v_off, q_scale, decay, states, slots, fresh, q_start,
                            q_len, n_seqs, n_tokens, out, heads, dk, dv, q_silu, tied_keys, s);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
