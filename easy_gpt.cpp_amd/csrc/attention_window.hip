// Softmax attention over the paged cache with separate key and value sizes, a window that keeps the first tokens,
// a sink in the softmax, a learned bias per head and distance, keys visible only within the query's own block of
// positions, and a penalty per head that grows with the distance; ragged batches (prompt portions and single decoded tokens in one launch).
//
// Query i of request b stands at position p = kv_len[b] - q_len[b] + i and sees key j if j <= p and
// (window == 0 or p - j < window or j < keep_first).  score = (q . k) * scale over the key size dk; the softmax is
// over the visible keys, and with a sink its denominator also holds exp(sink[head]), which has no key and no value
// and is not scaled; with a distance bias [nq][far + 1] the score of key j gets bias[head][min(p - j, far)] added, unscaled;
// with block > 0 a key is seen only if floor(j / block) == floor(p / block) (blocks are counted from position 0 of the
// request, wherever a step cuts it); with slopes [nq] the score of key j loses slopes[head] * (p - j), unscaled;
// the output is the weighted sum of the values of size dv.  Query head h reads key/value head
// h / (nq / nkv).  Queries q [T][nq][dk]; keys in pages [page][kv head][offset][dk], values in pages
// [page][kv head][dv][offset]; nothing that is not visible is read, so pages need no clearing and pages that a window
// gave back are never touched.  Scores, softmax statistics and the output sum are float32.
#include "api.h"
#include "common.h"

namespace egpt {

constexpr int kWidest = 1024;          // the widest key or value
constexpr int kSimpleWaves = 4;

__device__ __forceinline__ int request_of(const int32_t* q_start, int n_seqs, int t) {
    int lo = 0, hi = n_seqs - 1;       // the last b with q_start[b] <= t
    while (lo < hi) {
        const int mid = (lo + hi + 1) / 2;
        if (q_start[mid] <= t) lo = mid; else hi = mid - 1;
    }
    return lo;
}

// the lowest key position that a query at position p sees, the kept first tokens aside
__device__ __forceinline__ int lowest_seen(int p, int window, int block) {
    int lo = window > 0 ? max(0, p - window + 1) : 0;
    if (block > 0) lo = max(lo, p / block * block);
    return lo;
}

__device__ __forceinline__ float lane_value(float v, int from) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), from));
}

__device__ __forceinline__ float dot_row(const float* q_s, const float* k, int n) {
    float dot = 0.f;
    int d = 0;
    if ((reinterpret_cast<uintptr_t>(k) & 15) == 0)
        for (; d + 4 <= n; d += 4) {
            const float4 a = *reinterpret_cast<const float4*>(k + d);
            dot = fmaf(q_s[d], a.x, dot);
            dot = fmaf(q_s[d + 1], a.y, dot);
            dot = fmaf(q_s[d + 2], a.z, dot);
            dot = fmaf(q_s[d + 3], a.w, dot);
        }
    for (; d < n; ++d) dot = fmaf(q_s[d], k[d], dot);
    return dot;
}
__device__ __forceinline__ float dot_row(const float* q_s, const bf16_t* k, int n) {
    float dot = 0.f;
    int d = 0;
    if ((reinterpret_cast<uintptr_t>(k) & 15) == 0)
        for (; d + 8 <= n; d += 8) {
            const uint4 a = *reinterpret_cast<const uint4*>(k + d);
            const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                dot = fmaf(q_s[d + 2 * e], __uint_as_float(w[e] << 16), dot);
                dot = fmaf(q_s[d + 2 * e + 1], __uint_as_float(w[e] & 0xffff0000u), dot);
            }
        }
    for (; d < n; ++d) dot = fmaf(q_s[d], to_float(k[d]), dot);
    return dot;
}

// One workgroup of kSimpleWaves wavefronts per (token, query head), any sizes.  The visible keys are numbered
// 0, 1, ... in the order of their positions (the kept first tokens, then the window) and taken 64 at a time, chunk c
// by wavefront c modulo kSimpleWaves: a lane scores one key, the wavefront agrees on the new maximum, then a lane owns
// the output's features lane, lane + 64, ...  The wavefronts' (maximum, sum, output) and the sink are merged in a fixed
// order, so a token's result depends on its position and its keys alone, never on the batch around it.
template <typename T>
__global__ __launch_bounds__(64 * kSimpleWaves) void window_attention_simple_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ kv_len, int n_seqs, int nq, int nkv, int dk, int dv,
    int page_size, float scale, int window, int keep_first, const float* __restrict__ sink,
    const float* __restrict__ dist_bias, int dist_far, int block, const float* __restrict__ slopes) {
    constexpr int kMaxOwn = kWidest / kWave;
    __shared__ __attribute__((aligned(16))) float q_s[kWidest];
    __shared__ float part_ml[kSimpleWaves][2];
    __shared__ float part_o[kSimpleWaves][kWidest];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int b = request_of(q_start, n_seqs, t);
    if (t - q_start[b] >= q_len[b]) return;                  // a row that belongs to no request
    const int p = kv_len[b] - q_len[b] + (t - q_start[b]);
    const int lo = lowest_seen(p, window, block);
    const int n_first = min(keep_first, lo);                 // kept first tokens that the window does not hold anyway
    const int n_visible = n_first + (p - lo + 1);
    const int kvh = h / (nq / nkv);
    const T* qp = q + (static_cast<size_t>(t) * nq + h) * dk;
    for (int d = threadIdx.x; d < dk; d += kWave * kSimpleWaves) q_s[d] = to_float(qp[d]);
    __syncthreads();
    const int32_t* table = block_table + static_cast<size_t>(b) * table_width;
    float acc[kMaxOwn] = {};
    float m_run = -INFINITY, l_run = 0.f;
    for (int c = wave * kWave; c < n_visible; c += kWave * kSimpleWaves) {
        const int vi = c + lane;
        float s = -INFINITY;
        if (vi < n_visible) {
            const int j = vi < n_first ? vi : lo + (vi - n_first);
            const long page = table[j / page_size];
            const T* kr = k_cache + ((page * nkv + kvh) * page_size + j % page_size) * dk;
            s = dot_row(q_s, kr, dk) * scale;
            if (dist_bias) s += dist_bias[static_cast<size_t>(h) * (dist_far + 1) + min(p - j, dist_far)];
            if (slopes) s -= slopes[h] * static_cast<float>(p - j);
        }
        const float m_new = fmaxf(m_run, wave_max(s));       // finite: the chunk's first key is visible
        const float pj = vi < n_visible ? expf(s - m_new) : 0.f;
        const float alpha = expf(m_run - m_new);             // exp(-inf) = 0 on the wavefront's first chunk
        l_run = l_run * alpha + wave_sum(pj);
        m_run = m_new;
#pragma unroll
        for (int r = 0; r < kMaxOwn; ++r) acc[r] *= alpha;
        const int n_valid = min(kWave, n_visible - c);
        for (int jj = 0; jj < n_valid; ++jj) {
            const float pw = lane_value(pj, jj);
            const int vj = c + jj;
            const int j = vj < n_first ? vj : lo + (vj - n_first);
            const long page = table[j / page_size];
            const T* vr = v_cache + (page * nkv + kvh) * dv * page_size + j % page_size;
#pragma unroll
            for (int r = 0; r < kMaxOwn; ++r) {
                const int d = lane + r * kWave;
                if (d < dv) acc[r] = fmaf(pw, to_float(vr[static_cast<long>(d) * page_size]), acc[r]);
            }
        }
    }
    if (lane == 0) {
        part_ml[wave][0] = m_run;
        part_ml[wave][1] = l_run;
    }
#pragma unroll
    for (int r = 0; r < kMaxOwn; ++r) {
        const int d = lane + r * kWave;
        if (d < dv) part_o[wave][d] = acc[r];
    }
    __syncthreads();
    if (wave != 0) return;
    // wavefront 0 holds the first chunk, so the overall maximum is finite; a wavefront without keys has maximum -inf
    // and weight exp(-inf) = 0
    float m_all = sink ? sink[h] : -INFINITY;
    for (int w = 0; w < kSimpleWaves; ++w) m_all = fmaxf(m_all, part_ml[w][0]);
    float l_all = sink ? expf(sink[h] - m_all) : 0.f;
    for (int w = 0; w < kSimpleWaves; ++w) l_all = fmaf(part_ml[w][1], expf(part_ml[w][0] - m_all), l_all);
    const float inv_l = 1.0f / l_all;
    T* o = out + (static_cast<size_t>(t) * nq + h) * dv;
#pragma unroll
    for (int r = 0; r < kMaxOwn; ++r) {
        const int d = lane + r * kWave;
        if (d < dv) {
            float a = 0.f;
            for (int w = 0; w < kSimpleWaves; ++w) a = fmaf(part_o[w][d], expf(part_ml[w][0] - m_all), a);
            o[d] = from_float<T>(a * inv_l);
        }
    }
}


// ---------------------------------------------------------------------------------------------- on the matrix cores
// The same attention for key sizes up to 256 that are multiples of 16 bytes' worth of elements, value sizes that are
// multiples of 16 up to 256, and page sizes that are multiples of 16.  Rows are (token, query head) pairs of one key/value
// head's group, 16 to a wavefront; the scores are computed transposed, S^T[key, row] = K[key, :] . Q[row, :], so that a
// lane holds scores of one row, the row's statistics are per-lane scalars and the probabilities are the second
// product's operand as they lie in registers: O^T[feature, row] += V^T[feature, key] . P^T[key, row].
//   bfloat16: v_mfma_f32_16x16x32_bf16, a lane's 16 bytes of an operand are 8 features (or 8 keys);
//   float32:  v_mfma_f32_16x16x4_f32 (float32 operands and accumulation), a lane's 16 bytes are 4 features (or 4 keys).
// A workgroup of RT wavefronts takes 16 * RW * RT rows of one request and key/value head (RW tiles of 16 rows to a
// wavefront, which then uses every key and value operand it reads from LDS RW times) and walks the chunks of KT keys
// that any of its rows can see: those that hold kept first tokens, then those of the window.  A chunk's keys and values
// are staged through LDS and shared by the wavefronts, the next chunk's loads in flight meanwhile; the queries lie in
// LDS too, so the key size is a run-time number (the value size, which sizes the accumulators, is a template
// parameter in steps).  With n_splits > 1 the
// chunks of a workgroup's rows are dealt over as many workgroups (grid z), which leave unnormalised results
// part_o [split][token][head][dv] and (maximum, sum) part_ml [split][token][head][2] that window_attention_fold_kernel
// combines; that kernel also adds the sink.  With one split the kernel finishes the rows itself.
typedef __attribute__((ext_vector_type(8))) __bf16 w_bf16x8;
typedef __attribute__((ext_vector_type(4))) float w_f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int w_u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int w_u32x2;

template <typename T>
__device__ __forceinline__ w_f32x4 matrix_piece(const w_u32x4& a, const w_u32x4& b, w_f32x4 acc) {
    if constexpr (sizeof(T) == 2) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(w_bf16x8, a), __builtin_bit_cast(w_bf16x8, b), acc,
                                                       0, 0, 0);
    } else {
        const w_f32x4 av = __builtin_bit_cast(w_f32x4, a), bv = __builtin_bit_cast(w_f32x4, b);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], bv[i], acc, 0, 0, 0);
        return acc;
    }
}

// Before accumulators are read behind a loop whose trip count is known only at run time: the wait between a matrix
// instruction and the read of its result is counted in instructions along the code, and sixteen idle cycles cover
// the longest instruction used here whatever path was taken.
__device__ __forceinline__ void matrix_results_ready() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15");
    __builtin_amdgcn_sched_barrier(0);
}

template <typename T>
__device__ __forceinline__ void store_four(T* dst, float a, float b, float c, float d) {
    if constexpr (sizeof(T) == 2) {
        uint2 packed;
        packed.x = f32_to_bf16_bits(a) | (static_cast<uint32_t>(f32_to_bf16_bits(b)) << 16);
        packed.y = f32_to_bf16_bits(c) | (static_cast<uint32_t>(f32_to_bf16_bits(d)) << 16);
        *reinterpret_cast<uint2*>(dst) = packed;
    } else {
        *reinterpret_cast<float4*>(dst) = float4{a, b, c, d};
    }
}

struct WindowArgs {
    const void* q;
    void* out;
    float* part_o;
    float* part_ml;
    const void* k_cache;
    const void* v_cache;
    const int32_t* block_table;
    const int32_t* q_start;
    const int32_t* q_len;
    const int32_t* kv_len;
    const float* sink;
    const float* dist_bias;  // [nq][dist_far + 1] or null
    int dist_far;
    const float* slopes;     // [nq] or null
    int block;               // keys are seen within the query's block of this many positions (0: no blocks)
    int table_width, n_seqs, n_tokens, nq, nkv, dk, dv, page_size, window, keep_first, n_splits;
    int page_shift;          // log2 of the page size if that is a power of two, else -1
    float scale;
};

__device__ __forceinline__ int page_index(int key, int page_size, int page_shift) {
    return page_shift >= 0 ? key >> page_shift : key / page_size;
}
__device__ __forceinline__ int place_in_page(int key, int page_size, int page_shift) {
    return page_shift >= 0 ? key & (page_size - 1) : key % page_size;
}

template <typename T, int DT, int RT, int RW>
__global__ __launch_bounds__(64 * RT, (DT * RW <= 8 ? 2 : 1)) void window_attention_tiled_kernel(WindowArgs a) {
    constexpr int E = 16 / sizeof(T);             // elements in 16 bytes
    constexpr int KT = sizeof(T) == 2 ? 64 : 32;  // keys per chunk
    constexpr int NKT = KT / 16;                  // tiles of 16 keys in a chunk
    constexpr int PF = 4 * E;                     // features (or keys) that one matrix_piece sums over
    constexpr int NP = KT / PF;                   // pieces of a chunk's keys
    constexpr int ROWS = 16 * RT * RW, THREADS = 64 * RT;     // a wavefront takes RW tiles of 16 rows
    constexpr int VROW = KT + E;                  // padded LDS row of values (elements)
    constexpr int U = 8;                          // loads that a thread has in flight while the queries are staged
    constexpr int KU = 8;                         // 16-byte pieces of a chunk's keys per thread: 64 keys of 256 features
    constexpr int VU = (DT * 16 * (KT / E) + THREADS - 1) / THREADS;      // and of its values
    extern __shared__ __attribute__((aligned(16))) unsigned char window_smem[];
    const T* __restrict__ q = static_cast<const T*>(a.q);
    const T* __restrict__ k_cache = static_cast<const T*>(a.k_cache);
    const T* __restrict__ v_cache = static_cast<const T*>(a.v_cache);
    const int dk = a.dk, dv = a.dv, nq = a.nq, nkv = a.nkv, page_size = a.page_size, window = a.window;
    const int page_shift = a.page_shift;
    const int n_pieces = (dk + PF - 1) / PF;
    const int krow = n_pieces * PF + E;           // padded LDS row of keys and of queries
    const int k_pieces = dk / E;                  // 16-byte pieces of a key
    T* q_s = reinterpret_cast<T*>(window_smem);
    T* k_s = q_s + ROWS * krow;
    T* v_s = k_s + KT * krow;

    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int lj = lane % 16, lg = lane / 16;
    const int kh = blockIdx.y;
    const int group_size = nq / nkv;

    int b = 0, grp = blockIdx.x;
    for (; b < a.n_seqs; ++b) {
        const int groups = (a.q_len[b] * group_size + ROWS - 1) / ROWS;
        if (grp < groups) break;
        grp -= groups;
    }
    if (b >= a.n_seqs) return;
    const int n = a.q_len[b], kv = a.kv_len[b], qs = a.q_start[b];
    const int rows = n * group_size;
    const int32_t* table = a.block_table + static_cast<size_t>(b) * a.table_width;

    // the workgroup's rows and the chunks of keys that they can see
    const int blk_first = grp * ROWS, blk_last = min(rows, blk_first + ROWS) - 1;
    const int p_max = kv - n + blk_last / group_size;
    const int p_min = kv - n + blk_first / group_size;
    const int lo_blk = lowest_seen(p_min, window, a.block);
    const int t_begin = lo_blk / KT, t_end = p_max / KT + 1;
    const int keep = (window > 0 || a.block > 0) ? min(a.keep_first, lo_blk) : 0;     // kept first tokens below the window
    const int kept_chunks = min((keep + KT - 1) / KT, t_begin);
    const int n_chunks = kept_chunks + (t_end - t_begin);
    const int per_split = (n_chunks + a.n_splits - 1) / a.n_splits;
    const int c_begin = blockIdx.z * per_split, c_end = min(n_chunks, c_begin + per_split);

    // this wavefront's tiles of 16 rows, this lane's row in each
    bool valid[RW];
    int tok[RW], head[RW], p_row[RW], lo_row[RW];
#pragma unroll
    for (int w = 0; w < RW; ++w) {
        const int r = blk_first + (wave * RW + w) * 16 + lj;
        valid[w] = r < rows;
        const int i_tok = valid[w] ? r / group_size : 0;
        tok[w] = qs + i_tok;
        head[w] = kh * group_size + (valid[w] ? r % group_size : 0);
        p_row[w] = valid[w] ? kv - n + i_tok : -1;
        lo_row[w] = valid[w] ? lowest_seen(p_row[w], window, a.block) : 0;
    }

    // the smallest position and the largest window start among a tile's rows (rows of no token aside)
    int tile_p_min[RW], tile_lo_max[RW];
#pragma unroll
    for (int w = 0; w < RW; ++w) {
        int pm = valid[w] ? p_row[w] : 0x7fffffff, lm = valid[w] ? lo_row[w] : 0;
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            pm = min(pm, __shfl_xor(pm, off, kWave));
            lm = max(lm, __shfl_xor(lm, off, kWave));
        }
        tile_p_min[w] = pm == 0x7fffffff ? -1 : pm;
        tile_lo_max[w] = lm;
    }

    // queries into LDS, zeros beyond the key size and in rows that belong to no token; the pads of the key rows and the
    // value rows beyond the value size are zeroed once, the chunks never write there
    {
        const int pieces = krow / E;
        for (int base = tid; base < ROWS * pieces; base += THREADS * U) {
            w_u32x4 regs[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int idx = base + u * THREADS;
                const int row = idx / pieces, c = idx % pieces;
                const int rr = blk_first + row;
                regs[u] = w_u32x4{0u, 0u, 0u, 0u};
                if (idx < ROWS * pieces && rr < rows && c * E < dk) {
                    const int t2 = qs + rr / group_size, h2 = kh * group_size + rr % group_size;
                    regs[u] = *reinterpret_cast<const w_u32x4*>(q + (static_cast<size_t>(t2) * nq + h2) * dk + c * E);
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int idx = base + u * THREADS;
                if (idx < ROWS * pieces) *reinterpret_cast<w_u32x4*>(q_s + (idx / pieces) * krow + (idx % pieces) * E) = regs[u];
            }
        }
        for (int idx = tid; idx < KT * (pieces - k_pieces); idx += THREADS)
            *reinterpret_cast<w_u32x4*>(k_s + (idx / (pieces - k_pieces)) * krow + (k_pieces + idx % (pieces - k_pieces)) * E) =
                w_u32x4{0u, 0u, 0u, 0u};
        constexpr int VPIECES = VROW / E;
        for (int idx = tid; idx < DT * 16 * VPIECES; idx += THREADS)
            if (idx / VPIECES >= dv) *reinterpret_cast<w_u32x4*>(v_s + (idx / VPIECES) * VROW + (idx % VPIECES) * E) = w_u32x4{0u, 0u, 0u, 0u};
    }

    w_f32x4 o[RW][DT];
    float m_run[RW], l_run[RW];
#pragma unroll
    for (int w = 0; w < RW; ++w) {
        m_run[w] = -INFINITY;
        l_run[w] = 0.f;
#pragma unroll
        for (int d = 0; d < DT; ++d) o[w][d] = w_f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const float scale = a.scale;
    constexpr float kLog2e = 1.4426950408889634f;
    const bool wave_active = blk_first + wave * RW * 16 < rows;      // a wavefront without rows only helps to stage

    // A chunk's keys [KT][dk] and values, transposed [dv][KT], travel through registers: the loads of the chunk after
    // this one are issued before this one's products and stored to LDS behind them.  What no row of the workgroup sees
    // is zeros.  A thread holds at most KU pieces of 16 bytes of keys (dk <= 256) and VU of values.
    constexpr int VKP = KT / E;   // 16-byte pieces of a value row
    w_u32x4 k_regs[KU], v_regs[VU];
    const int k_total = KT * k_pieces, v_total = dv * VKP;
    // which key of a chunk and which piece of it this thread's loads take, where they go in LDS and where they lie in a
    // page's block (the same in every chunk); a thread has ku_n pieces of keys to take, the same for all threads but
    // the last ones of the last round
    const int ku_n = (k_total + THREADS - 1) / THREADS;
    int k_row[KU], k_lds[KU], k_off[KU];
#pragma unroll
    for (int u = 0; u < KU; ++u) {
        const int idx = tid + u * THREADS;
        const bool used = idx < k_total;
        k_row[u] = used ? idx / k_pieces : -(1 << 28);          // (a key no chunk holds)
        k_lds[u] = used ? (idx / k_pieces) * krow + (idx % k_pieces) * E : 0;
        k_off[u] = kh * page_size * dk + (used ? (idx % k_pieces) * E : 0);
    }
    int v_key[VU], v_lds[VU];
    long v_off[VU];
#pragma unroll
    for (int u = 0; u < VU; ++u) {
        const int idx = tid + u * THREADS;
        const bool used = idx < v_total;
        const int f = idx / VKP, vk = (idx % VKP) * E;
        v_key[u] = used ? vk : -(1 << 28);
        v_off[u] = (static_cast<long>(kh) * dv + f) * page_size;
        // where the E keys go: as they are (float32), or in the order in which a lane takes them (bfloat16: within 32
        // keys by quarter of the wavefront, tile, key)
        v_lds[u] = f * VROW + (sizeof(T) == 4 ? vk : (vk / 32) * 32 + ((vk % 16) / 4) * 8 + ((vk % 32) / 16) * 4);
    }
    const long k_page_stride = static_cast<long>(nkv) * page_size * dk, v_page_stride = static_cast<long>(nkv) * dv * page_size;
    // page numbers are looked up a chunk ahead of the loads that need them, so that an iteration waits for one trip
    // to memory, not for two that depend on each other
    int k_page[KU], v_page[VU];
    auto lookup = [&](int c) {
        const int tile = c < kept_chunks ? c : t_begin + (c - kept_chunks);
        const int key0 = c < c_end ? tile * KT : (1 << 29);        // behind the last chunk: keys that nobody sees
#pragma unroll
        for (int u = 0; u < KU; ++u) {
            if (u >= ku_n) break;
            const int j = key0 + k_row[u];
            k_page[u] = -1;
            if (j >= 0 && j <= p_max && (j >= lo_blk || j < keep)) k_page[u] = table[page_index(j, page_size, page_shift)];
        }
#pragma unroll
        for (int u = 0; u < VU; ++u) {
            const int j = key0 + v_key[u];
            v_page[u] = -1;
            if (j >= 0 && j <= p_max && (j + E - 1 >= lo_blk || j < keep)) v_page[u] = table[page_index(j, page_size, page_shift)];
        }
    };
    auto fetch = [&](int c) {
        const int tile = c < kept_chunks ? c : t_begin + (c - kept_chunks);
        const int key0 = tile * KT;
#pragma unroll
        for (int u = 0; u < KU; ++u) {
            if (u >= ku_n) break;
            k_regs[u] = w_u32x4{0u, 0u, 0u, 0u};
            if (k_page[u] >= 0)
                k_regs[u] = *reinterpret_cast<const w_u32x4*>(
                    k_cache + k_page[u] * k_page_stride + (place_in_page(key0 + k_row[u], page_size, page_shift) * dk + k_off[u]));
        }
#pragma unroll
        for (int u = 0; u < VU; ++u) {
            const int j = key0 + v_key[u];
            w_u32x4 v = w_u32x4{0u, 0u, 0u, 0u};
            if (v_page[u] >= 0) {
                v = *reinterpret_cast<const w_u32x4*>(
                    v_cache + v_page[u] * v_page_stride + v_off[u] + place_in_page(j, page_size, page_shift));
                if (j + E > kv) {         // places of the page that no token has written yet may hold anything
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if constexpr (sizeof(T) == 4) {
                            if (j + e >= kv) v[e] = 0u;
                        } else {
                            if (j + 2 * e >= kv) v[e] = 0u;
                            else if (j + 2 * e + 1 >= kv) v[e] &= 0x0000ffffu;
                        }
                    }
                }
            }
            v_regs[u] = v;
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int u = 0; u < KU; ++u) {
            if (u >= ku_n) break;
            if (k_row[u] >= 0) *reinterpret_cast<w_u32x4*>(k_s + k_lds[u]) = k_regs[u];
        }
#pragma unroll
        for (int u = 0; u < VU; ++u) {
            if (v_key[u] < 0) continue;
            if constexpr (sizeof(T) == 4) {
                *reinterpret_cast<w_u32x4*>(v_s + v_lds[u]) = v_regs[u];
            } else {
                *reinterpret_cast<w_u32x2*>(v_s + v_lds[u]) = w_u32x2{v_regs[u].x, v_regs[u].y};
                *reinterpret_cast<w_u32x2*>(v_s + v_lds[u] + 8) = w_u32x2{v_regs[u].z, v_regs[u].w};
            }
        }
    };

    lookup(c_begin);
    fetch(c_begin);
    lookup(c_begin + 1);
    for (int c = c_begin; c < c_end; ++c) {
        const int tile = c < kept_chunks ? c : t_begin + (c - kept_chunks);
        const int key0 = tile * KT;
        __syncthreads();                  // the chunk before is read (and, the first time, the queries are written)
        stash();
        __syncthreads();
        fetch(c + 1);                     // in flight while this chunk is computed; behind the last chunk nothing is read
        lookup(c + 2);
        if (!wave_active) continue;
        // ---- scores of this wavefront's rows against the chunk's keys: a key operand serves all of its row tiles
        w_f32x4 acc[RW][NKT];
        const T* ks = k_s + lj * krow + lg * E;
        const T* qrow = q_s + (wave * RW * 16 + lj) * krow + lg * E;
#pragma unroll
        for (int w = 0; w < RW; ++w)
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) acc[w][kt] = w_f32x4{0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < n_pieces; ++j) {
            w_u32x4 qv[RW];
#pragma unroll
            for (int w = 0; w < RW; ++w) qv[w] = *reinterpret_cast<const w_u32x4*>(qrow + w * 16 * krow + j * PF);
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) {
                const w_u32x4 kvv = *reinterpret_cast<const w_u32x4*>(ks + kt * 16 * krow + j * PF);
#pragma unroll
                for (int w = 0; w < RW; ++w) acc[w][kt] = matrix_piece<T>(kvv, qv[w], acc[w][kt]);
            }
        }
        matrix_results_ready();
        // ---- mask, scale, one step of the online softmax (the lane's rows; a row's four lanes share the statistics)
        w_u32x4 p[RW][NP];
#pragma unroll
        for (int w = 0; w < RW; ++w) {
            float mx = -INFINITY;
            // a chunk that every row of the tile sees whole (below the diagonal and inside the window, or all kept
            // tokens) needs no mask
            const bool whole = key0 + KT - 1 <= tile_p_min[w] && (key0 >= tile_lo_max[w] || key0 + KT <= a.keep_first);
            if (a.dist_bias != nullptr) {
                // the bias of the row's head by distance; a chunk that lies `far` or more behind every row of the tile
                // gets the table's last entry throughout
                const float* brow = a.dist_bias + static_cast<size_t>(head[w]) * (a.dist_far + 1);
                const bool all_far = whole && tile_p_min[w] - (key0 + KT - 1) >= a.dist_far;
                const float b_far = brow[a.dist_far];
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int key = key0 + kt * 16 + lg * 4 + v;
                        const bool seen = key <= p_row[w] && (key >= lo_row[w] || key < a.keep_first);
                        float sc = -INFINITY;
                        if (all_far) sc = fmaf(acc[w][kt][v], scale, b_far);
                        else if (seen) sc = fmaf(acc[w][kt][v], scale, brow[min(p_row[w] - key, a.dist_far)]);
                        acc[w][kt][v] = sc;
                        mx = fmaxf(mx, sc);
                    }
            } else if (a.slopes != nullptr) {
                // the penalty of the row's head times the distance
                const float slope = a.slopes[head[w]];
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int key = key0 + kt * 16 + lg * 4 + v;
                        const bool seen = whole || (key <= p_row[w] && (key >= lo_row[w] || key < a.keep_first));
                        const float sc = seen ? fmaf(acc[w][kt][v], scale, -slope * static_cast<float>(p_row[w] - key)) : -INFINITY;
                        acc[w][kt][v] = sc;
                        mx = fmaxf(mx, sc);
                    }
            } else if (whole) {
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        acc[w][kt][v] *= scale;
                        mx = fmaxf(mx, acc[w][kt][v]);
                    }
            } else {
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int key = key0 + kt * 16 + lg * 4 + v;
                        const bool seen = key <= p_row[w] && (key >= lo_row[w] || key < a.keep_first);
                        const float sc = seen ? acc[w][kt][v] * scale : -INFINITY;
                        acc[w][kt][v] = sc;
                        mx = fmaxf(mx, sc);
                    }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
            mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
            const float m_new = fmaxf(m_run[w], mx);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;      // a row that has seen nothing yet: every exp below is 0
            if (__any(m_new != m_run[w])) {                             // (a factor of exactly 1 otherwise)
                const float alpha = __builtin_amdgcn_exp2f((m_run[w] - m_use) * kLog2e);
                l_run[w] *= alpha;
#pragma unroll
                for (int d = 0; d < DT; ++d) {
                    o[w][d][0] *= alpha; o[w][d][1] *= alpha; o[w][d][2] *= alpha; o[w][d][3] *= alpha;
                }
            }
            m_run[w] = m_new;
            float sum = 0.f;
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float pv = __builtin_amdgcn_exp2f((acc[w][kt][v] - m_use) * kLog2e);
                    sum += pv;
                    acc[w][kt][v] = pv;
                }
            l_run[w] += sum;
            // the probabilities as the second product's operand
            if constexpr (sizeof(T) == 2) {
#pragma unroll
                for (int j = 0; j < NP; ++j) {
                    w_bf16x8 pb;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        pb[v] = static_cast<__bf16>(acc[w][2 * j][v]);
                        pb[4 + v] = static_cast<__bf16>(acc[w][2 * j + 1][v]);
                    }
                    p[w][j] = __builtin_bit_cast(w_u32x4, pb);
                }
            } else {
#pragma unroll
                for (int j = 0; j < NP; ++j) p[w][j] = __builtin_bit_cast(w_u32x4, acc[w][j]);
            }
        }
        const T* vs = v_s + lj * VROW + lg * E;
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int j = 0; j < NP; ++j) {
                const w_u32x4 vv = *reinterpret_cast<const w_u32x4*>(vs + d * 16 * VROW + j * PF);
#pragma unroll
                for (int w = 0; w < RW; ++w) o[w][d] = matrix_piece<T>(vv, p[w][j], o[w][d]);
            }
    }
    matrix_results_ready();
#pragma unroll
    for (int w = 0; w < RW; ++w) {
        float l = l_run[w];
        l += __shfl_xor(l, 16, kWave);
        l += __shfl_xor(l, 32, kWave);
        if (!valid[w]) continue;
        if (a.n_splits > 1) {
            const size_t row_at = (static_cast<size_t>(blockIdx.z) * a.n_tokens + tok[w]) * nq + head[w];
            float* po = a.part_o + row_at * dv + lg * 4;
#pragma unroll
            for (int d = 0; d < DT; ++d)
                if (d * 16 < dv) *reinterpret_cast<float4*>(po + d * 16) = float4{o[w][d][0], o[w][d][1], o[w][d][2], o[w][d][3]};
            if (lg == 0) {
                a.part_ml[row_at * 2] = m_run[w];
                a.part_ml[row_at * 2 + 1] = l;
            }
            continue;
        }
        float weight = 1.0f;
        if (a.sink != nullptr) {
            const float sk = a.sink[head[w]];
            const float m_all = fmaxf(m_run[w], sk);
            weight = __builtin_amdgcn_exp2f((m_run[w] - m_all) * kLog2e);
            l = l * weight + __builtin_amdgcn_exp2f((sk - m_all) * kLog2e);
        }
        const float inv = weight / l;
        T* op = static_cast<T*>(a.out) + (static_cast<size_t>(tok[w]) * nq + head[w]) * dv + lg * 4;
#pragma unroll
        for (int d = 0; d < DT; ++d)
            if (d * 16 < dv)
                store_four<T>(op + d * 16, o[w][d][0] * inv, o[w][d][1] * inv, o[w][d][2] * inv, o[w][d][3] * inv);
    }
}

// The parts that the splits of a row's keys left, folded in the order of the splits, with the sink: one wavefront per
// (token, head).
template <typename T>
__global__ __launch_bounds__(kWave) void window_attention_fold_kernel(const float* __restrict__ part_o,
                                                                    const float* __restrict__ part_ml,
                                                                    const float* __restrict__ sink, T* __restrict__ out,
                                                                    int n_rows, int nq, int dv, int n_splits) {
    __shared__ float weights[kWave];           // at most 64 splits
    const int row = blockIdx.x, lane = threadIdx.x;
    float m = -INFINITY, l = 0.f;
    if (lane < n_splits) {
        const float* ml = part_ml + (static_cast<size_t>(lane) * n_rows + row) * 2;
        m = ml[0];
        l = ml[1];
    }
    float m_all = wave_max(m);
    if (sink) m_all = fmaxf(m_all, sink[row % nq]);
    const float w = lane < n_splits ? expf(m - m_all) : 0.f;     // exp(-inf) = 0 for a split that saw nothing
    float l_all = wave_sum(l * w);
    if (sink) l_all += expf(sink[row % nq] - m_all);
    weights[lane] = w;
    __syncthreads();
    const float inv = 1.0f / l_all;
    for (int d = lane; d < dv; d += kWave) {
        float acc = 0.f;
        for (int s = 0; s < n_splits; ++s)
            acc = fmaf(part_o[(static_cast<size_t>(s) * n_rows + row) * dv + d], weights[s], acc);
        out[static_cast<size_t>(row) * dv + d] = from_float<T>(acc * inv);
    }
}

template <typename T, int DT, int RT, int RW>
static int launch_tiled(const WindowArgs& a, int max_rows, hipStream_t s) {
    constexpr int E = 16 / sizeof(T), KT = sizeof(T) == 2 ? 64 : 32, PF = 4 * E, ROWS = 16 * RT * RW;
    const int krow = (a.dk + PF - 1) / PF * PF + E;
    const size_t lds = (static_cast<size_t>(ROWS + KT) * krow + static_cast<size_t>(DT) * 16 * (KT + E)) * sizeof(T);
    if (lds > 160 * 1024) return EGPT_UNSUPPORTED_SIZE;
    auto kernel = window_attention_tiled_kernel<T, DT, RT, RW>;
    if (lds > 48 * 1024) {
        static bool raised = false;       // per instance of this template: the limit is asked for once
        if (!raised) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    160 * 1024) != hipSuccess)
                return EGPT_LAUNCH_FAILED;
            raised = true;
        }
    }
    const int group_size = a.nq / a.nkv;
    const int blocks = (max_rows * group_size + ROWS - 1) / ROWS + a.n_seqs;
    dim3 grid(blocks, a.nkv, a.n_splits);
    kernel<<<grid, 64 * RT, lds, s>>>(a);
    return EGPT_OK;
}

// row_tiles: 4 (four wavefronts with 16 rows each) or 8 (with 32 rows each)
template <typename T, int DT>
static int launch_tiled_for_rows(const WindowArgs& a, int max_rows, int row_tiles, hipStream_t s) {
    if (row_tiles == 8) return launch_tiled<T, DT, 4, 2>(a, max_rows, s);
    return launch_tiled<T, DT, 4, 1>(a, max_rows, s);
}

template <typename T>
static int launch_tiled_for_dv(const WindowArgs& a, int max_rows, int row_tiles, hipStream_t s) {
    const int tiles = (a.dv + 15) / 16;
    if (tiles <= 2) return launch_tiled_for_rows<T, 2>(a, max_rows, row_tiles, s);
    if (tiles <= 4) return launch_tiled_for_rows<T, 4>(a, max_rows, row_tiles, s);
    if (tiles <= 6) return launch_tiled_for_rows<T, 6>(a, max_rows, row_tiles, s);
    if (tiles <= 8) return launch_tiled_for_rows<T, 8>(a, max_rows, row_tiles, s);
    if (tiles <= 12) return launch_tiled_for_rows<T, 12>(a, max_rows, row_tiles, s);
    if (tiles <= 16) return launch_tiled_for_rows<T, 16>(a, max_rows, row_tiles, s);
    return EGPT_UNSUPPORTED_SIZE;
}

}  // namespace egpt

using namespace egpt;

extern "C" int egpt_window_attention(const void* q, void* out, const void* k_cache, const void* v_cache,
                                     const int32_t* block_table, int table_width, const int32_t* q_start,
                                     const int32_t* q_len, const int32_t* kv_len, int n_seqs, int n_tokens, int nq,
                                     int nkv, int dk, int dv, int page_size, float scale, int window, int keep_first,
                                     const float* sink, const float* dist_bias, int dist_far, int block, const float* slopes,
                                     int dtype, void* stream) {
    if (!q || !out || !k_cache || !v_cache || !block_table || !q_start || !q_len || !kv_len) return EGPT_BAD_ARGUMENT;
    if (n_seqs <= 0 || n_tokens < 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || dk <= 0 || dv <= 0 || page_size <= 0 ||
        table_width <= 0 || window < 0 || keep_first < 0 || (dtype != 0 && dtype != 1) || (dist_bias && dist_far < 0) || block < 0)
        return EGPT_BAD_ARGUMENT;
    if (dk > kWidest || dv > kWidest || nq > 65535) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(n_tokens, nq);
    if (dtype == 0)
        window_attention_simple_kernel<float><<<grid, kWave * kSimpleWaves, 0, s>>>(
            static_cast<const float*>(q), static_cast<float*>(out), static_cast<const float*>(k_cache),
            static_cast<const float*>(v_cache), block_table, table_width, q_start, q_len, kv_len, n_seqs, nq, nkv, dk,
            dv, page_size, scale, window, keep_first, sink, dist_bias, dist_far, block, slopes);
    else
        window_attention_simple_kernel<bf16_t><<<grid, kWave * kSimpleWaves, 0, s>>>(
            static_cast<const bf16_t*>(q), static_cast<bf16_t*>(out), static_cast<const bf16_t*>(k_cache),
            static_cast<const bf16_t*>(v_cache), block_table, table_width, q_start, q_len, kv_len, n_seqs, nq, nkv, dk,
            dv, page_size, scale, window, keep_first, sink, dist_bias, dist_far, block, slopes);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_window_attention_tiled(const void* q, void* out, float* part_o, float* part_ml, const void* k_cache,
                                           const void* v_cache, const int32_t* block_table, int table_width,
                                           const int32_t* q_start, const int32_t* q_len, const int32_t* kv_len, int n_seqs,
                                           int n_tokens, int nq, int nkv, int dk, int dv, int page_size, float scale,
                                           int window, int keep_first, const float* sink, const float* dist_bias,
                                           int dist_far, int block, const float* slopes, int n_splits, int row_tiles, int dtype,
                                           void* stream) {
    if (!q || !out || !k_cache || !v_cache || !block_table || !q_start || !q_len || !kv_len) return EGPT_BAD_ARGUMENT;
    if (n_seqs <= 0 || n_tokens < 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || dk <= 0 || dv <= 0 || page_size <= 0 ||
        table_width <= 0 || window < 0 || keep_first < 0 || n_splits < 1 || (dtype != 0 && dtype != 1) ||
        (row_tiles != 4 && row_tiles != 8) || (dist_bias && dist_far < 0) || block < 0 || (dist_bias && slopes))
        return EGPT_BAD_ARGUMENT;
    if (n_splits > 1 && (!part_o || !part_ml)) return EGPT_BAD_ARGUMENT;
    const int e = dtype == 0 ? 4 : 8;
    if (dk % e || dk > 256 || dv % 16 || dv > 256 || page_size % 16 || nkv > 65535 || n_splits > 64) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    WindowArgs a;
    a.q = q; a.out = out; a.part_o = part_o; a.part_ml = part_ml; a.k_cache = k_cache; a.v_cache = v_cache;
    a.block_table = block_table; a.q_start = q_start; a.q_len = q_len; a.kv_len = kv_len; a.sink = sink;
    a.dist_bias = dist_bias; a.dist_far = dist_far; a.slopes = slopes; a.block = block;
    a.table_width = table_width; a.n_seqs = n_seqs; a.n_tokens = n_tokens; a.nq = nq; a.nkv = nkv; a.dk = dk; a.dv = dv;
    a.page_size = page_size; a.window = window; a.keep_first = keep_first; a.n_splits = n_splits; a.scale = scale;
    a.page_shift = -1;
    for (int sh = 0; sh < 30; ++sh)
        if ((1 << sh) == page_size) a.page_shift = sh;
    int code;
    if (dtype == 0)
        code = launch_tiled_for_dv<float>(a, n_tokens, row_tiles, s);
    else
        code = launch_tiled_for_dv<bf16_t>(a, n_tokens, row_tiles, s);
    if (code != EGPT_OK) return code;
    EGPT_CHECK_LAUNCH();
    if (n_splits > 1) {
        if (dtype == 0)
            window_attention_fold_kernel<float><<<n_tokens * nq, kWave, 0, s>>>(part_o, part_ml, sink, static_cast<float*>(out),
                                                                               n_tokens * nq, nq, dv, n_splits);
        else
            window_attention_fold_kernel<bf16_t><<<n_tokens * nq, kWave, 0, s>>>(part_o, part_ml, sink,
                                                                                static_cast<bf16_t*>(out), n_tokens * nq, nq,
                                                                                dv, n_splits);
        EGPT_CHECK_LAUNCH();
    }
    return EGPT_OK;
}
