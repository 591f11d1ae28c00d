// Softmax attention over the paged cache with separate key and value sizes, a window that keeps the first tokens,
// and a sink in the softmax; ragged batches (prompt portions and single decoded tokens in one launch).
//
// Query i of request b stands at position p = kv_len[b] - q_len[b] + i and sees key j if j <= p and
// (window == 0 or p - j < window or j < keep_first).  score = (q . k) * scale over the key size dk; the softmax is
// over the visible keys, and with a sink its denominator also holds exp(sink[head]), which has no key and no value
// and is not scaled; the output is the weighted sum of the values of size dv.  Query head h reads key/value head
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
    int page_size, float scale, int window, int keep_first, const float* __restrict__ sink) {
    constexpr int kMaxOwn = kWidest / kWave;
    __shared__ __attribute__((aligned(16))) float q_s[kWidest];
    __shared__ float part_ml[kSimpleWaves][2];
    __shared__ float part_o[kSimpleWaves][kWidest];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int b = request_of(q_start, n_seqs, t);
    if (t - q_start[b] >= q_len[b]) return;                  // a row that belongs to no request
    const int p = kv_len[b] - q_len[b] + (t - q_start[b]);
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
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

}  // namespace egpt

using namespace egpt;

extern "C" int egpt_window_attention(const void* q, void* out, const void* k_cache, const void* v_cache,
                                     const int32_t* block_table, int table_width, const int32_t* q_start,
                                     const int32_t* q_len, const int32_t* kv_len, int n_seqs, int n_tokens, int nq,
                                     int nkv, int dk, int dv, int page_size, float scale, int window, int keep_first,
                                     const float* sink, int dtype, void* stream) {
    if (!q || !out || !k_cache || !v_cache || !block_table || !q_start || !q_len || !kv_len) return EGPT_BAD_ARGUMENT;
    if (n_seqs <= 0 || n_tokens < 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || dk <= 0 || dv <= 0 || page_size <= 0 ||
        table_width <= 0 || window < 0 || keep_first < 0 || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (dk > kWidest || dv > kWidest || nq > 65535) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(n_tokens, nq);
    if (dtype == 0)
        window_attention_simple_kernel<float><<<grid, kWave * kSimpleWaves, 0, s>>>(
            static_cast<const float*>(q), static_cast<float*>(out), static_cast<const float*>(k_cache),
            static_cast<const float*>(v_cache), block_table, table_width, q_start, q_len, kv_len, n_seqs, nq, nkv, dk,
            dv, page_size, scale, window, keep_first, sink);
    else
        window_attention_simple_kernel<bf16_t><<<grid, kWave * kSimpleWaves, 0, s>>>(
            static_cast<const bf16_t*>(q), static_cast<bf16_t*>(out), static_cast<const bf16_t*>(k_cache),
            static_cast<const bf16_t*>(v_cache), block_table, table_width, q_start, q_len, kv_len, n_seqs, nq, nkv, dk,
            dv, page_size, scale, window, keep_first, sink);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
