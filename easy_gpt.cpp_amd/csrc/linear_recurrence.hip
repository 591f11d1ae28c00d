// Linear attention with a matrix state per head that decays per key channel:
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   S [dk][dv] float32 per request and head.
// The state is carried from step to step in a record per request; a step walks its tokens in order, whatever the cut of
// the prompt: every element of the state sees the same operations in the same order in a prompt's portion as in single
// tokens, so the result does not depend on the cut at all.  Decays, the state and the output sum are float32.
//
// egpt_channel_decay makes the decays a = sigmoid(z)^(1/tau) from a low-rank projection (z = W low + b);
// egpt_decayed_state_scan runs the recurrence.
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

constexpr int kScanTokens = 16;     // tokens staged in LDS at a time
constexpr int kScanCols = 64;       // value channels per workgroup

// One workgroup of four wavefronts per (request, head, 64 value channels).  A wavefront takes 16 value channels; its
// lanes are 4 slices of the key channels times 16 value channels, a lane keeps DKR key channels of one column of the
// state in registers, and the four slices' parts of o_t are added across the lanes in a fixed order.  Queries, keys,
// decays and values of kScanTokens tokens are staged in LDS (a slice's rows padded apart so that the four slices
// read different banks).
template <typename T, int DKR>
__global__ __launch_bounds__(256) void decayed_state_scan_kernel(
    ProductView<T> proj, int proj_width, int q_off, int k_off, int v_off, float q_scale, const float* __restrict__ decay,
    float* __restrict__ states, const int32_t* __restrict__ slots, const unsigned char* __restrict__ fresh,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, float* __restrict__ out, int heads, int dk, int dv) {
    constexpr int ROW = DKR + 4;                 // a slice's row in LDS
    constexpr int TOK = 4 * ROW;                 // a token's q (or k, or decay) in LDS
    __shared__ __attribute__((aligned(16))) float q_s[kScanTokens * TOK];
    __shared__ __attribute__((aligned(16))) float k_s[kScanTokens * TOK];
    __shared__ __attribute__((aligned(16))) float a_s[kScanTokens * TOK];
    __shared__ float v_s[kScanTokens * kScanCols];
    const int b = blockIdx.x, h = blockIdx.y, col0 = blockIdx.z * kScanCols;
    const int n = q_len[b];
    if (n <= 0) return;
    const int t0 = q_start[b];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int slice = lane / 16, col = wave * 16 + lane % 16;
    const int j = col0 + col;
    const bool has_col = j < dv;
    float* state = states + (static_cast<size_t>(slots[b]) * heads + h) * dk * dv;
    float s[DKR];
    const bool start_anew = fresh != nullptr && fresh[b] != 0;
#pragma unroll
    for (int i = 0; i < DKR; ++i) {
        const int r = slice * DKR + i;
        s[i] = (!start_anew && has_col && r < dk) ? state[static_cast<size_t>(r) * dv + j] : 0.f;
    }
    const int channels = heads * dk;
    // The next tokens' queries, keys, decays and values travel through registers: their loads are issued before this
    // batch of tokens is computed and stored to LDS behind it, so that a batch waits for memory once, not once per
    // array, and not at all while the recurrence runs long.
    constexpr int QKA = kScanTokens * 4 * DKR / 256, VL = kScanTokens * kScanCols / 256;
    float rq[QKA], rk[QKA], ra[QKA], rv[VL];
    auto fetch = [&](int base) {
        const int count = min(kScanTokens, n - base);
#pragma unroll
        for (int u = 0; u < QKA; ++u) {
            const int idx = tid + u * 256;
            const int tt = idx / (4 * DKR), r = idx % (4 * DKR);
            rq[u] = rk[u] = ra[u] = 0.f;
            if (tt < count && r < dk) {
                const size_t row = static_cast<size_t>(t0 + base + tt);
                rq[u] = proj.at(row * proj_width + q_off + h * dk + r) * q_scale;
                rk[u] = proj.at(row * proj_width + k_off + h * dk + r);
                ra[u] = decay[row * channels + h * dk + r];
            }
        }
#pragma unroll
        for (int u = 0; u < VL; ++u) {
            const int idx = tid + u * 256;
            const int tt = idx / kScanCols, c = idx % kScanCols;
            rv[u] = 0.f;
            if (tt < count && col0 + c < dv)
                rv[u] = proj.at(static_cast<size_t>(t0 + base + tt) * proj_width + v_off + h * dv + col0 + c);
        }
    };
    fetch(0);
    for (int base = 0; base < n; base += kScanTokens) {
        const int count = min(kScanTokens, n - base);
        __syncthreads();                          // the tokens before are read
#pragma unroll
        for (int u = 0; u < QKA; ++u) {
            const int idx = tid + u * 256;
            const int tt = idx / (4 * DKR), r = idx % (4 * DKR);
            const int at = tt * TOK + (r / DKR) * ROW + r % DKR;
            q_s[at] = rq[u];
            k_s[at] = rk[u];
            a_s[at] = ra[u];
        }
#pragma unroll
        for (int u = 0; u < VL; ++u) v_s[tid + u * 256] = rv[u];
        __syncthreads();
        if (base + kScanTokens < n) fetch(base + kScanTokens);
        for (int tt = 0; tt < count; ++tt) {
            const float vj = v_s[tt * kScanCols + col];
            const float4* a4 = reinterpret_cast<const float4*>(a_s + tt * TOK + slice * ROW);
            const float4* k4 = reinterpret_cast<const float4*>(k_s + tt * TOK + slice * ROW);
            const float4* q4 = reinterpret_cast<const float4*>(q_s + tt * TOK + slice * ROW);
            float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;       // four sums, so that no addition waits for the one before
#pragma unroll
            for (int i = 0; i < DKR / 4; ++i) {
                const float4 a = a4[i], k = k4[i], q = q4[i];
                s[4 * i] = fmaf(a.x, s[4 * i], k.x * vj);
                o0 = fmaf(s[4 * i], q.x, o0);
                s[4 * i + 1] = fmaf(a.y, s[4 * i + 1], k.y * vj);
                o1 = fmaf(s[4 * i + 1], q.y, o1);
                s[4 * i + 2] = fmaf(a.z, s[4 * i + 2], k.z * vj);
                o2 = fmaf(s[4 * i + 2], q.z, o2);
                s[4 * i + 3] = fmaf(a.w, s[4 * i + 3], k.w * vj);
                o3 = fmaf(s[4 * i + 3], q.w, o3);
            }
            float o = (o0 + o1) + (o2 + o3);
            o += __shfl_xor(o, 16, kWave);
            o += __shfl_xor(o, 32, kWave);
            if (slice == 0 && has_col) out[(static_cast<size_t>(t0 + base + tt) * heads + h) * dv + j] = o;
        }
    }
    if (has_col) {
#pragma unroll
        for (int i = 0; i < DKR; ++i) {
            const int r = slice * DKR + i;
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

template <typename T>
static int launch_scan(const void* proj, int n_splits, int proj_width, int q_off, int k_off, int v_off, float q_scale,
                       const float* decay, float* states, const int32_t* slots, const unsigned char* fresh,
                       const int32_t* q_start, const int32_t* q_len, int n_seqs, int n_tokens, float* out, int heads, int dk,
                       int dv, hipStream_t s) {
    const ProductView<T> view = scan_view<T>(proj, n_splits, static_cast<size_t>(n_tokens) * proj_width);
    dim3 grid(n_seqs, heads, (dv + kScanCols - 1) / kScanCols);
#define EGPT_SCAN(DKR_)                                                                                                   \
    decayed_state_scan_kernel<T, DKR_><<<grid, 256, 0, s>>>(view, proj_width, q_off, k_off, v_off, q_scale, decay, states, \
                                                            slots, fresh, q_start, q_len, out, heads, dk, dv)
    if (dk <= 32) EGPT_SCAN(8);
    else if (dk <= 64) EGPT_SCAN(16);
    else if (dk <= 128) EGPT_SCAN(32);
    else EGPT_SCAN(64);
#undef EGPT_SCAN
    return EGPT_OK;
}

extern "C" int egpt_decayed_state_scan(const void* proj, int n_splits, int proj_width, int q_off, int k_off, int v_off,
                                       float q_scale, const float* decay, float* states, const int32_t* slots,
                                       const unsigned char* fresh, const int32_t* q_start, const int32_t* q_len, int n_seqs,
                                       int n_tokens, float* out, int heads, int dk, int dv, int dtype, void* stream) {
    if (!proj || !decay || !states || !slots || !q_start || !q_len || !out || n_splits < 0 || n_seqs <= 0 || n_tokens < 0 ||
        heads <= 0 || dk <= 0 || dv <= 0 || q_off < 0 || k_off < 0 || v_off < 0 || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (q_off + heads * dk > proj_width || k_off + heads * dk > proj_width || v_off + heads * dv > proj_width)
        return EGPT_BAD_ARGUMENT;
    if (dk > 256 || heads > 65535 || (dv + kScanCols - 1) / kScanCols > 65535) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == 0)
        launch_scan<float>(proj, n_splits, proj_width, q_off, k_off, v_off, q_scale, decay, states, slots, fresh, q_start,
                           q_len, n_seqs, n_tokens, out, heads, dk, dv, s);
    else
        launch_scan<bf16_t>(proj, n_splits, proj_width, q_off, k_off, v_off, q_scale, decay, states, slots, fresh, q_start,
                            q_len, n_seqs, n_tokens, out, heads, dk, dv, s);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
