// Linear attention with a matrix state per head that decays per key channel:
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   S [dk][dv] float32 per request and head.
// The state is carried from step to step in a record per request; a step walks its tokens in order, whatever the cut of
// the prompt: every element of the state sees the same operations in the same order in a prompt's portion as in single
// tokens, so the result does not depend on the cut at all.  Decays, the state and the output sum are float32.
//
// egpt_channel_decay makes the decays a = sigmoid(z)^(1/tau) from a low-rank projection (z = W low + b);
// egpt_bounded_gate makes decays with a learned lower bound, a = l + (1 - l) sigmoid(z + b), from columns of a product;
// egpt_decayed_state_scan runs the recurrence; its queries, keys and values may each pass through SiLU on their way in,
// its keys may be tied to the decays, k = 1 - a (a forget gate that also sets what is written), instead of columns of
// the product, and its decay may be one constant per head.
//
// The delta rule, S <- diag(g_t) S; u_t = beta_t (v_t - S^T k_t); S <- S + k_t u_t^T; o_t = S^T q_t, mixes the key channels in
// every token (S^T k), so its scan keeps a head's whole key range in one workgroup: egpt_delta_rule_scan.  Its operands
// come from egpt_short_conv, which runs the short causal convolutions over time with their carried inputs, SiLU, and the
// unit norms of queries and keys.
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
// sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau), with softplus(-z) = max(-z, 0) + log1p(exp(-|z|)).  With rates the
// exponent is rates[c] per channel instead of 1/tau, and with negate z changes its sign first, which together give
// exp(-rate softplus(z)) = sigmoid(-z)^rate: a decay whose logarithm is a step size times a rate per channel.
template <typename T>
__global__ __launch_bounds__(256) void channel_decay_kernel(ProductView<T> low, int low_width, int low_off, int rank,
                                                            const T* __restrict__ w, const T* __restrict__ bias, float inv_tau,
                                                            const float* __restrict__ rates, int negate,
                                                            float* __restrict__ decay, int channels) {
    __shared__ float low_s[kMaxRank];
    const int t = blockIdx.x;
    for (int r = threadIdx.x; r < rank; r += blockDim.x) low_s[r] = low.at(static_cast<size_t>(t) * low_width + low_off + r);
    __syncthreads();
    for (int c = threadIdx.x; c < channels; c += blockDim.x) {
        float z = bias ? to_float(bias[c]) : 0.f;
        const T* wr = w + static_cast<size_t>(c) * rank;
        for (int r = 0; r < rank; ++r) z = fmaf(to_float(wr[r]), low_s[r], z);
        if (negate) z = -z;
        const float log_sigmoid = -(fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z))));
        decay[static_cast<size_t>(t) * channels + c] = expf(log_sigmoid * (rates ? rates[c] : inv_tau));
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
    int dk, int dv, int key_splits, int q_silu, int tied_keys, int k_silu, int v_silu, const float* __restrict__ head_decay) {
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
                ra[u] = head_decay ? head_decay[h] : decay[row * channels + h * dk + r];
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
            k_s[tid + u * THREADS] = tied_keys ? 1.0f - ra[u] : (k_silu ? rk[u] / (1.0f + expf(-rk[u])) : rk[u]);
            a_s[tid + u * THREADS] = ra[u];
        }
#pragma unroll
        for (int u = 0; u < VL; ++u) v_s[tid + u * THREADS] = v_silu ? rv[u] / (1.0f + expf(-rv[u])) : rv[u];
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
                                  const void* bias, float tau, const float* rates, int negate, float* decay, int n_tokens,
                                  int channels, int dtype, void* stream) {
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
                                                             1.0f / tau, rates, negate, decay, channels);
    else
        channel_decay_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(scan_view<bf16_t>(low, low_splits, stride), low_width, low_off, rank,
                                                              static_cast<const bf16_t*>(w), static_cast<const bf16_t*>(bias),
                                                              1.0f / tau, rates, negate, decay, channels);
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
                       int dv, int q_silu, int tied_keys, int k_silu, int v_silu, const float* head_decay, hipStream_t s) {
    const ProductView<T> view = scan_view<T>(proj, n_splits, static_cast<size_t>(n_tokens) * proj_width);
    const int key_splits = (dk + kScanKeys - 1) / kScanKeys;
    dim3 grid(n_seqs, heads, (dv + kScanCols - 1) / kScanCols * key_splits);
    decayed_state_scan_kernel<T><<<grid, 64 * kScanWaves, 0, s>>>(view, proj_width, q_off, k_off, v_off, q_scale, decay, states, slots,
                                                                  fresh, q_start, q_len, out, n_tokens, heads, dk, dv, key_splits,
                                                                  q_silu, tied_keys, k_silu, v_silu, head_decay);
    return EGPT_OK;
}

extern "C" int egpt_scan_key_splits(int dk) { return dk > 0 ? (dk + kScanKeys - 1) / kScanKeys : 0; }

extern "C" int egpt_decayed_state_scan(const void* proj, int n_splits, int proj_width, int q_off, int k_off, int v_off,
                                       float q_scale, const float* decay, float* states, const int32_t* slots,
                                       const unsigned char* fresh, const int32_t* q_start, const int32_t* q_len, int n_seqs,
                                       int n_tokens, float* out, int heads, int dk, int dv, int q_silu, int tied_keys,
                                       int k_silu, int v_silu, const float* head_decay, int dtype, void* stream) {
    // head_decay float32 [heads]: one constant decay per head in place of the decays per token and key channel
    if (!proj || (!decay && !head_decay) || (tied_keys && k_silu) || !states || !slots || !q_start || !q_len || !out || n_splits < 0 || n_seqs <= 0 || n_tokens < 0 ||
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
                           q_len, n_seqs, n_tokens, out, heads, dk, dv, q_silu, tied_keys, k_silu, v_silu, head_decay, s);
    else
        launch_scan<bf16_t>(proj, n_splits, proj_width, q_off, k_off, v_off, q_scale, decay, states, slots, fresh, q_start,
                            q_len, n_seqs, n_tokens, out, heads, dk, dv, q_silu, tied_keys, k_silu, v_silu, head_decay, s);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// Short causal convolutions over time, and the delta rule's scan.
namespace egpt {

constexpr int kMaxTaps = 16;

// One workgroup per token of a step (grid: requests x the step's longest portion).  The columns col0 .. col0 + channels
// of a product row are the inputs of `channels` independent convolutions over time: y_i = sum_j w[c][j] x_(i - taps + 1 + j)
// (the last tap is the current token's), with the inputs before the step's first token taken from the request's record
// hist [taps - 1][channels] (zeros for a request that starts anew).  y passes SiLU.  The first unit_heads * unit_dim
// channels are then made unit vectors head by head, y / sqrt(sum y^2 + unit_eps), the first scaled_heads of them also
// times `scale`.  Behind the channels the output row holds the sigmoid of the n_sig columns from sig_off on.  All float32.
template <typename T>
__global__ __launch_bounds__(1024) void short_conv_kernel(
    ProductView<T> proj, int proj_width, int col0, const T* __restrict__ conv_w, int taps, int channels, int unit_heads,
    int unit_dim, int scaled_heads, float scale, float unit_eps, int sig_off, int n_sig, const float* __restrict__ states,
    size_t state_stride, const int32_t* __restrict__ slots, const unsigned char* __restrict__ fresh,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, float* __restrict__ out, int out_width) {
    extern __shared__ float conv_s[];
    const int b = blockIdx.x;
    const int n = q_len[b];
    const int t0 = q_start[b];
    const float* hist = states + static_cast<size_t>(slots[b]) * state_stride;
    const bool anew = fresh != nullptr && fresh[b] != 0;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, n_waves = blockDim.x / kWave;
    for (int i = blockIdx.y; i < n; i += gridDim.y) {                   // (the grid has a workgroup per token of the longest portion, up to 65,535)
        const size_t t = static_cast<size_t>(t0 + i);
        __syncthreads();                                                 // the token before is written out
        for (int c = threadIdx.x; c < channels; c += blockDim.x) {
            float acc = 0.f;
            for (int j = 0; j < taps; ++j) {
                const int src = i - (taps - 1) + j;
                float x;
                if (src >= 0)
                    x = proj.at(static_cast<size_t>(t0 + src) * proj_width + col0 + c);
                else
                    x = anew ? 0.f : hist[static_cast<size_t>(src + taps - 1) * channels + c];
                acc = fmaf(x, to_float(conv_w[static_cast<size_t>(c) * taps + j]), acc);
            }
            conv_s[c] = acc / (1.0f + expf(-acc));
        }
        __syncthreads();
        float* orow = out + t * out_width;
        for (int hh = wave; hh < unit_heads; hh += n_waves) {
            const float* head = conv_s + hh * unit_dim;
            float ss = 0.f;
            for (int d = lane; d < unit_dim; d += kWave) ss = fmaf(head[d], head[d], ss);
            float f = 1.0f / sqrtf(wave_sum(ss) + unit_eps);
            if (hh < scaled_heads) f *= scale;
            for (int d = lane; d < unit_dim; d += kWave) orow[hh * unit_dim + d] = head[d] * f;
        }
        for (int c = unit_heads * unit_dim + threadIdx.x; c < channels; c += blockDim.x) orow[c] = conv_s[c];
        for (int c = threadIdx.x; c < n_sig; c += blockDim.x)
            orow[channels + c] = 1.0f / (1.0f + expf(-proj.at(t * proj_width + sig_off + c)));
    }
}

// After a step: a request's record takes the last taps - 1 inputs of its convolutions (those of this step, and, where the
// step brought fewer, what the record held, moved up).  Workgroups per request and 256 channels; a thread owns a channel's column.
template <typename T>
__global__ __launch_bounds__(256) void conv_carry_kernel(ProductView<T> proj, int proj_width, int col0, int taps, int channels,
                                                         float* __restrict__ states, size_t state_stride,
                                                         const int32_t* __restrict__ slots, const unsigned char* __restrict__ fresh,
                                                         const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len) {
    const int b = blockIdx.x;
    const int n = q_len[b];
    if (n <= 0) return;
    const int t0 = q_start[b];
    float* hist = states + static_cast<size_t>(slots[b]) * state_stride;
    const bool anew = fresh != nullptr && fresh[b] != 0;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
        float keep[kMaxTaps];
#pragma unroll
        for (int j = 0; j < kMaxTaps; ++j) {
            keep[j] = 0.f;
            if (j < taps - 1) {
                const int src = n - (taps - 1) + j;
                if (src >= 0)
                    keep[j] = proj.at(static_cast<size_t>(t0 + src) * proj_width + col0 + c);
                else if (!anew)
                    keep[j] = hist[static_cast<size_t>(src + taps - 1) * channels + c];
            }
        }
#pragma unroll
        for (int j = 0; j < kMaxTaps; ++j)
            if (j < taps - 1) hist[static_cast<size_t>(j) * channels + c] = keep[j];
    }
}

// The delta rule's scan.  A workgroup is one wavefront that owns 64 / SLICES columns of a head's state S [dk][dv]: its
// lanes are columns x SLICES ranges of R key channels (SLICES a power of two, SLICES * R >= dk), a lane keeps its range of
// its column in registers, and what has to be summed over the key channels (S^T k, S^T q and k . q) is summed over a
// lane's rows and then across the slices with lane exchanges: no barrier and no trip through memory stands between two
// tokens.  With S' = diag(g) S the token's output is S'^T q + (k . q) u, u = beta (v - S'^T k), so the sums are taken on
// the decayed state before it is written, and the write S <- S' + k u^T is off the path to the next token's sums.  The
// operands are staged in LDS a batch of TB tokens at a time (queries, keys and decays of the head, the wavefront's columns
// of the values, beta) while the next batch's loads are in flight in registers, all of them issued together, and a token's
// operands are read from LDS while the token before is computed; outputs leave through LDS, a batch at a time.  What
// bounds a token is the vector arithmetic of a lane's rows (four operations a row) and what LDS returns for them (every lane
// gets its copy of its slice's queries, keys and decays: one wavefront to a workgroup, so that wavefronts do not share a
// CU's LDS while there are CUs to spare).  Value head h reads the queries and keys of head h / (heads / kv_heads).  ops rows
// hold queries, keys, values and beta (float32); decay is [tokens][heads * dk].
// The sum of v over the N neighbouring lanes that hold the slices of one column (N a power of two, lanes N * i ..), in every
// one of them.  Within a row of 16 lanes the exchanges are operand modifiers of the additions themselves (pairs, quads,
// then the mirrored half row and the mirrored row, which hold equal values by then); beyond a row they go through the
// lane permute.
template <int CTRL>
__device__ __forceinline__ float lanes_add(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int N>
__device__ __forceinline__ float slices_sum(float v) {
    if (N >= 2) v = lanes_add<0xB1>(v);          // quad_perm [1, 0, 3, 2]
    if (N >= 4) v = lanes_add<0x4E>(v);          // quad_perm [2, 3, 0, 1]
    if (N >= 8) v = lanes_add<0x141>(v);         // row_half_mirror
    if (N >= 16) v = lanes_add<0x140>(v);        // row_mirror
    if (N >= 32) v += __shfl_xor(v, 16, kWave);
    if (N >= 64) v += __shfl_xor(v, 32, kWave);
    return v;
}

template <int SLICES, int R>
__global__ __launch_bounds__(64) void delta_rule_scan_kernel(
    const float* __restrict__ ops, int ops_width, int q_off, int k_off, int v_off, int beta_off, const float* __restrict__ decay,
    float* __restrict__ states, size_t state_stride, const int32_t* __restrict__ slots, const unsigned char* __restrict__ fresh,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, float* __restrict__ out, int heads, int kv_heads,
    int dk, int dv) {
    constexpr int THREADS = kWave, DKP = SLICES * R;
    constexpr int COLS = kWave / SLICES, WG_COLS = COLS;
    constexpr int WIDEST = DKP > WG_COLS ? DKP : WG_COLS;
    constexpr int TB = 512 / WIDEST < 16 ? (512 / WIDEST < 1 ? 1 : 512 / WIDEST) : 16;      // tokens to a batch: about 512 values of an operand
    constexpr int QKA = (TB * DKP + THREADS - 1) / THREADS;             // values of q (or k, or g) of a batch per thread
    constexpr int VL = (TB * WG_COLS + THREADS - 1) / THREADS;          // values of v, and outputs, of a batch per thread
    __shared__ __attribute__((aligned(16))) float q_s[TB * DKP];
    __shared__ __attribute__((aligned(16))) float k_s[TB * DKP];
    __shared__ __attribute__((aligned(16))) float g_s[TB * DKP];
    __shared__ float v_s[TB * WG_COLS];
    __shared__ float o_s[TB * WG_COLS];
    __shared__ float beta_s[TB];
    const int b = blockIdx.x, h = blockIdx.y, col0 = blockIdx.z * WG_COLS;
    const int n = q_len[b];
    if (n <= 0) return;
    const int t0 = q_start[b];
    const int tid = threadIdx.x, lane = tid;
    const int sl = lane % SLICES, c = lane / SLICES;                     // this lane's slice of the key channels, and its column
    const int j = col0 + c;
    const bool has_col = j < dv;
    const int kvh = h / (heads / kv_heads);
    float* state = states + static_cast<size_t>(slots[b]) * state_stride + static_cast<size_t>(h) * dk * dv;
    const bool anew = fresh != nullptr && fresh[b] != 0;
    float s[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int r = sl * R + i;
        s[i] = (!anew && has_col && r < dk) ? state[static_cast<size_t>(r) * dv + j] : 0.f;
    }
    float rq[QKA], rk[QKA], rg[QKA], rv[VL], rbeta = 0.f;
    auto fetch = [&](int base) {
        const int count = min(TB, n - base);
#pragma unroll
        for (int u = 0; u < QKA; ++u) {
            const int idx = tid + u * THREADS;
            const int tt = idx / DKP, r = idx % DKP;
            rq[u] = rk[u] = rg[u] = 0.f;
            if (tt < count && r < dk) {                                  // (tt < count <= TB bounds idx as well)
                const size_t row = static_cast<size_t>(t0 + base + tt);
                rq[u] = ops[row * ops_width + q_off + kvh * dk + r];
                rk[u] = ops[row * ops_width + k_off + kvh * dk + r];
                rg[u] = decay[row * heads * dk + static_cast<size_t>(h) * dk + r];
            }
        }
#pragma unroll
        for (int u = 0; u < VL; ++u) {
            const int idx = tid + u * THREADS;
            const int tt = idx / WG_COLS, cc = idx % WG_COLS;
            rv[u] = 0.f;
            if (tt < count && col0 + cc < dv)
                rv[u] = ops[static_cast<size_t>(t0 + base + tt) * ops_width + v_off + h * dv + col0 + cc];
        }
        rbeta = tid < count ? ops[static_cast<size_t>(t0 + base + tid) * ops_width + beta_off + h] : 0.f;      // (TB <= 16 < 64)
    };
    fetch(0);
    for (int base = 0; base < n; base += TB) {
        const int count = min(TB, n - base);
        __syncthreads();                              // the batch before is read
#pragma unroll
        for (int u = 0; u < QKA; ++u) {
            if (tid + u * THREADS < TB * DKP) {
                q_s[tid + u * THREADS] = rq[u];
                k_s[tid + u * THREADS] = rk[u];
                g_s[tid + u * THREADS] = rg[u];
            }
        }
#pragma unroll
        for (int u = 0; u < VL; ++u)
            if (tid + u * THREADS < TB * WG_COLS) v_s[tid + u * THREADS] = rv[u];
        if (tid < TB) beta_s[tid] = rbeta;
        __syncthreads();
        if (base + TB < n) fetch(base + TB);
        // (a token's operands are read from LDS while the token before is computed: two sets of registers in turn)
        float4 ga[R / 4], ka[R / 4], qa[R / 4], gb[R / 4], kb[R / 4], qb[R / 4];
        float va, ba, vb, bb;
        auto read = [&](int tt, float4* g, float4* k, float4* q, float& vj, float& beta) {
            const int at = tt < TB ? tt : TB - 1;                        // (behind the batch's last token: read and not used)
#pragma unroll
            for (int i = 0; i < R / 4; ++i) {
                g[i] = reinterpret_cast<const float4*>(g_s + at * DKP + sl * R)[i];
                k[i] = reinterpret_cast<const float4*>(k_s + at * DKP + sl * R)[i];
                q[i] = reinterpret_cast<const float4*>(q_s + at * DKP + sl * R)[i];
            }
            vj = v_s[at * WG_COLS + c];
            beta = beta_s[at];
        };
        auto token = [&](int tt, const float4* g, const float4* k, const float4* q, float vj, float beta) {
            float pk[4] = {0.f, 0.f, 0.f, 0.f}, pq[4] = {0.f, 0.f, 0.f, 0.f}, kq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < R / 4; ++i) {
                s[4 * i] *= g[i].x, s[4 * i + 1] *= g[i].y, s[4 * i + 2] *= g[i].z, s[4 * i + 3] *= g[i].w;
                pk[0] = fmaf(s[4 * i], k[i].x, pk[0]), pk[1] = fmaf(s[4 * i + 1], k[i].y, pk[1]);
                pk[2] = fmaf(s[4 * i + 2], k[i].z, pk[2]), pk[3] = fmaf(s[4 * i + 3], k[i].w, pk[3]);
                pq[0] = fmaf(s[4 * i], q[i].x, pq[0]), pq[1] = fmaf(s[4 * i + 1], q[i].y, pq[1]);
                pq[2] = fmaf(s[4 * i + 2], q[i].z, pq[2]), pq[3] = fmaf(s[4 * i + 3], q[i].w, pq[3]);
                kq[0] = fmaf(k[i].x, q[i].x, kq[0]), kq[1] = fmaf(k[i].y, q[i].y, kq[1]);
                kq[2] = fmaf(k[i].z, q[i].z, kq[2]), kq[3] = fmaf(k[i].w, q[i].w, kq[3]);
            }
            const float sk = slices_sum<SLICES>((pk[0] + pk[1]) + (pk[2] + pk[3]));
            const float sq = slices_sum<SLICES>((pq[0] + pq[1]) + (pq[2] + pq[3]));
            const float skq = slices_sum<SLICES>((kq[0] + kq[1]) + (kq[2] + kq[3]));
            const float u = beta * (vj - sk);
            if (sl == 0) o_s[tt * WG_COLS + c] = fmaf(skq, u, sq);
#pragma unroll
            for (int i = 0; i < R / 4; ++i) {
                s[4 * i] = fmaf(k[i].x, u, s[4 * i]), s[4 * i + 1] = fmaf(k[i].y, u, s[4 * i + 1]);
                s[4 * i + 2] = fmaf(k[i].z, u, s[4 * i + 2]), s[4 * i + 3] = fmaf(k[i].w, u, s[4 * i + 3]);
            }
        };
        read(0, ga, ka, qa, va, ba);
        for (int tt = 0; tt < count; tt += 2) {
            read(tt + 1, gb, kb, qb, vb, bb);
            token(tt, ga, ka, qa, va, ba);
            if (tt + 1 < count) {
                read(tt + 2, ga, ka, qa, va, ba);
                token(tt + 1, gb, kb, qb, vb, bb);
            }
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < VL; ++u) {
            const int idx = tid + u * THREADS;
            const int tt = idx / WG_COLS, cc = idx % WG_COLS;
            if (tt < count && col0 + cc < dv) out[(static_cast<size_t>(t0 + base + tt) * heads + h) * dv + col0 + cc] = o_s[idx];
        }
    }
    if (has_col) {
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int r = sl * R + i;
            if (r < dk) state[static_cast<size_t>(r) * dv + j] = s[i];
        }
    }
}

template <int SLICES, int R>
static void launch_delta(const float* ops, int ops_width, int q_off, int k_off, int v_off, int beta_off, const float* decay,
                         float* states, size_t state_stride, const int32_t* slots, const unsigned char* fresh,
                         const int32_t* q_start, const int32_t* q_len, int n_seqs, float* out, int heads, int kv_heads, int dk,
                         int dv, hipStream_t s) {
    constexpr int cols = kWave / SLICES;
    dim3 grid(n_seqs, heads, (dv + cols - 1) / cols);
    delta_rule_scan_kernel<SLICES, R><<<grid, kWave, 0, s>>>(ops, ops_width, q_off, k_off, v_off, beta_off, decay, states,
                                                            state_stride, slots, fresh, q_start, q_len, out, heads, kv_heads, dk, dv);
}

}  // namespace egpt

// out float32 [n_tokens][channels + n_sig]; states: the first record's convolution inputs [taps - 1][channels], a
// request's record lies state_stride floats further per slot.  The records are brought up to date behind the step's
// convolutions (a second launch on the same stream).
extern "C" int egpt_short_conv(const void* proj, int n_splits, int proj_width, int col0, const void* conv_w, int taps,
                               int channels, int unit_heads, int unit_dim, int scaled_heads, float scale, float unit_eps,
                               int sig_off, int n_sig, float* states, long long state_stride, const int32_t* slots,
                               const unsigned char* fresh, const int32_t* q_start, const int32_t* q_len, int n_seqs,
                               int max_q_len, int n_tokens, float* out, int dtype, void* stream) {
    if (!proj || !conv_w || !states || !slots || !q_start || !q_len || !out || n_splits < 0 || taps < 1 || channels <= 0 ||
        unit_heads < 0 || unit_dim < 0 || scaled_heads < 0 || scaled_heads > unit_heads || n_sig < 0 || col0 < 0 || n_seqs <= 0 ||
        max_q_len < 0 || n_tokens < 0 || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (static_cast<long long>(unit_heads) * unit_dim > channels || col0 + channels > proj_width ||
        (n_sig > 0 && (sig_off < 0 || sig_off + n_sig > proj_width)) || state_stride < static_cast<long long>(taps - 1) * channels)
        return EGPT_BAD_ARGUMENT;
    if (taps > kMaxTaps || channels > 15360) return EGPT_UNSUPPORTED_SIZE;     // a token's channels lie in LDS
    if (n_tokens == 0 || max_q_len == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t stride = static_cast<size_t>(n_tokens) * proj_width;
    const size_t lds = static_cast<size_t>(channels) * sizeof(float);
    const int out_width = channels + n_sig;
    dim3 grid(n_seqs, max_q_len > 65535 ? 65535 : max_q_len);
    dim3 carry_grid(n_seqs, (channels + 255) / 256);
    // (a token's channels are walked in rounds of the workgroup's width: wide workgroups where the channels are many and
    // the tokens few; a prompt's tokens fill the GPU with narrow ones: 34 us against 47 for 2,048 tokens of 1,792 channels)
    const int width = channels > 512 && static_cast<long long>(n_seqs) * max_q_len < 512 ? 1024 : 256;
    if (dtype == 0) {
        short_conv_kernel<float><<<grid, width, lds, s>>>(scan_view<float>(proj, n_splits, stride), proj_width, col0,
                                                        static_cast<const float*>(conv_w), taps, channels, unit_heads, unit_dim,
                                                        scaled_heads, scale, unit_eps, sig_off, n_sig, states,
                                                        static_cast<size_t>(state_stride), slots, fresh, q_start, q_len, out, out_width);
        if (taps > 1)
            conv_carry_kernel<float><<<carry_grid, 256, 0, s>>>(scan_view<float>(proj, n_splits, stride), proj_width, col0, taps, channels,
                                                            states, static_cast<size_t>(state_stride), slots, fresh, q_start, q_len);
    } else {
        short_conv_kernel<bf16_t><<<grid, width, lds, s>>>(scan_view<bf16_t>(proj, n_splits, stride), proj_width, col0,
                                                         static_cast<const bf16_t*>(conv_w), taps, channels, unit_heads, unit_dim,
                                                         scaled_heads, scale, unit_eps, sig_off, n_sig, states,
                                                         static_cast<size_t>(state_stride), slots, fresh, q_start, q_len, out, out_width);
        if (taps > 1)
            conv_carry_kernel<bf16_t><<<carry_grid, 256, 0, s>>>(scan_view<bf16_t>(proj, n_splits, stride), proj_width, col0, taps, channels,
                                                             states, static_cast<size_t>(state_stride), slots, fresh, q_start, q_len);
    }
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

// out float32 [n_tokens][heads * dv]; states: the first record's matrices [heads][dk][dv], a request's record lies
// state_stride floats further per slot.
extern "C" int egpt_delta_rule_scan(const float* ops, int ops_width, int q_off, int k_off, int v_off, int beta_off,
                                    const float* decay, float* states, long long state_stride, const int32_t* slots,
                                    const unsigned char* fresh, const int32_t* q_start, const int32_t* q_len, int n_seqs,
                                    int n_tokens, float* out, int heads, int kv_heads, int dk, int dv, void* stream) {
    if (!ops || !decay || !states || !slots || !q_start || !q_len || !out || n_seqs <= 0 || n_tokens < 0 || heads <= 0 ||
        kv_heads <= 0 || heads % kv_heads || dk <= 0 || dv <= 0 || q_off < 0 || k_off < 0 || v_off < 0 || beta_off < 0)
        return EGPT_BAD_ARGUMENT;
    if (q_off + kv_heads * dk > ops_width || k_off + kv_heads * dk > ops_width || v_off + heads * dv > ops_width ||
        beta_off + heads > ops_width || state_stride < static_cast<long long>(heads) * dk * dv)
        return EGPT_BAD_ARGUMENT;
    if (dk > 1024 || heads > 65535 || dv > 65535) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // A lane keeps 4, 8 or 16 key channels of a column: the fewest that ask for no more than 1,024 wavefronts (a prompt of
    // one request walks its tokens on as many wavefronts as the state has columns times slices, and a wavefront's time per
    // token is its instructions per token: fewer rows, more wavefronts, a shorter walk; a step of many requests fills the
    // GPU with 16 rows to a lane); as many slices of the key channels as cover dk, a power of two.
    int rows = 16, slices = 1;
    for (int r = 4; r <= 16; r *= 2) {
        int sl = 1;
        while (sl * r < dk) sl <<= 1;
        if (sl > 64) continue;
        const long long wavefronts = static_cast<long long>(n_seqs) * heads * ((dv + 64 / sl - 1) / (64 / sl));
        if (wavefronts <= 1024 || r == 16) {
            rows = r, slices = sl;
            break;
        }
    }
    const size_t stride = static_cast<size_t>(state_stride);
#define EGPT_DELTA(S)                                                                                                              \
    case S:                                                                                                                        \
        if (rows == 4)                                                                                                             \
            launch_delta<S, 4>(ops, ops_width, q_off, k_off, v_off, beta_off, decay, states, stride, slots, fresh, q_start, q_len, \
                               n_seqs, out, heads, kv_heads, dk, dv, s);                                                           \
        else if (rows == 8)                                                                                                        \
            launch_delta<S, 8>(ops, ops_width, q_off, k_off, v_off, beta_off, decay, states, stride, slots, fresh, q_start, q_len, \
                               n_seqs, out, heads, kv_heads, dk, dv, s);                                                           \
        else                                                                                                                       \
            launch_delta<S, 16>(ops, ops_width, q_off, k_off, v_off, beta_off, decay, states, stride, slots, fresh, q_start, q_len, \
                                n_seqs, out, heads, kv_heads, dk, dv, s);                                                          \
        break;
    switch (slices) {
        EGPT_DELTA(1) EGPT_DELTA(2) EGPT_DELTA(4) EGPT_DELTA(8) EGPT_DELTA(16) EGPT_DELTA(32) EGPT_DELTA(64)
        default: return EGPT_UNSUPPORTED_SIZE;
    }
#undef EGPT_DELTA
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
