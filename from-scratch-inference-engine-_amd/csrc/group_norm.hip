// RMS norm in groups over the residual stream, fused with the residual sum of up to two pending deltas, and the
// short causal convolution that a layer may put in front of what its sublayers read.
//
// group_rmsnorm: one workgroup a row.  x = residual + delta_scale * (delta1 + delta2) goes to LDS (and back to the
// stream); the row is `groups` equal consecutive parts, a wave takes a part at a time and leaves
// 1 / sqrt(mean(part^2) + eps) in LDS; then every thread writes x * that * weight, for one or two weights.
//
// causal_conv: y[t] = x[t] + sum_j w[:, j] x[t - taps + 1 + j]; inputs before a portion's start come from the
// request's state (the last taps - 1 inputs, oldest first).  A second kernel stores the new last inputs after
// every row has been written, so no block reads a state that another has already replaced.
#include "common.h"
#include "api.h"

namespace {

constexpr int kThreads = 256;
constexpr int kMaxGroups = 256;

template <typename D>
__device__ __forceinline__ float delta_at(const D* d, int64_t i) { return d ? to_float(d[i]) : 0.f; }

__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
    const uint2 raw = *reinterpret_cast<const uint2*>(p);
    return float4{__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                  __uint_as_float(raw.y & 0xffff0000u)};
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, float4 v) {
    uint2 raw;
    raw.x = static_cast<uint32_t>(from_float<bf16_t>(v.x).bits) | static_cast<uint32_t>(from_float<bf16_t>(v.y).bits) << 16;
    raw.y = static_cast<uint32_t>(from_float<bf16_t>(v.z).bits) | static_cast<uint32_t>(from_float<bf16_t>(v.w).bits) << 16;
    *reinterpret_cast<uint2*>(p) = raw;
}

// VEC: rows of a multiple of four values behind aligned pointers: a thread takes four values at a time, and
// everything a round reads is asked for before anything is written.
template <typename T, typename D1, typename D2, bool VEC>
__global__ __launch_bounds__(kThreads) void group_rmsnorm_kernel(
    float* __restrict__ residual, const D1* __restrict__ delta1, const D2* __restrict__ delta2, float delta_scale,
    const float* __restrict__ weight1, const float* __restrict__ weight2, T* __restrict__ out1, T* __restrict__ out2,
    const int32_t* __restrict__ rows, int hidden, int groups, float eps, int write_back) {
    extern __shared__ float lds[];
    float* xs = lds;               // [hidden]
    float* inv = lds + hidden;     // [groups]
    const int r = blockIdx.x;
    const int64_t row = rows ? rows[r] : r;
    float* res = residual + row * hidden;
    const bool has_delta = delta1 || delta2;
    constexpr int V = VEC ? 4 : 1;
    for (int j = threadIdx.x * V; j < hidden; j += kThreads * V) {
        if constexpr (VEC) {
            float4 v = load4(res + j);
            if (has_delta) {
                // the two sublayers' outputs first, then the factor, then the stream: one order for every caller
                const float4 z = {0.f, 0.f, 0.f, 0.f};
                const float4 d1 = delta1 ? load4(delta1 + row * hidden + j) : z, d2 = delta2 ? load4(delta2 + row * hidden + j) : z;
                v.x = fmaf(delta_scale, d1.x + d2.x, v.x), v.y = fmaf(delta_scale, d1.y + d2.y, v.y);
                v.z = fmaf(delta_scale, d1.z + d2.z, v.z), v.w = fmaf(delta_scale, d1.w + d2.w, v.w);
                if (write_back) store4(res + j, v);
            }
            *reinterpret_cast<float4*>(xs + j) = v;
        } else {
            float v = res[j];
            if (has_delta) {
                const float d = delta_at(delta1, row * hidden + j) + delta_at(delta2, row * hidden + j);
                v = fmaf(delta_scale, d, v);
                if (write_back) res[j] = v;
            }
            xs[j] = v;
        }
    }
    __syncthreads();
    const int part = hidden / groups;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int g = wave; g < groups; g += kThreads / 64) {
        const float* p = xs + g * part;
        float sum = 0.f;
        for (int j = lane; j < part; j += 64) sum = fmaf(p[j], p[j], sum);
        sum = wave_sum(sum);
        if (lane == 0) inv[g] = 1.0f / sqrtf(sum / static_cast<float>(part) + eps);
    }
    __syncthreads();
    T* o1 = out1 + static_cast<int64_t>(r) * hidden;
    T* o2 = out2 ? out2 + static_cast<int64_t>(r) * hidden : nullptr;
    for (int j = threadIdx.x * V; j < hidden; j += kThreads * V) {
        if constexpr (VEC) {
            const float4 x = *reinterpret_cast<const float4*>(xs + j);
            const float4 n = {x.x * inv[j / part], x.y * inv[(j + 1) / part], x.z * inv[(j + 2) / part], x.w * inv[(j + 3) / part]};
            const float4 w1 = load4(weight1 + j);
            store4(o1 + j, float4{n.x * w1.x, n.y * w1.y, n.z * w1.z, n.w * w1.w});
            if (o2) {
                const float4 w2 = load4(weight2 + j);
                store4(o2 + j, float4{n.x * w2.x, n.y * w2.y, n.z * w2.z, n.w * w2.w});
            }
        } else {
            const float n = xs[j] * inv[j / part];
            o1[j] = from_float<T>(n * weight1[j]);
            if (o2) o2[j] = from_float<T>(n * weight2[j]);
        }
    }
}

// grid = (tokens, blocks of 256 channels, convolutions): a thread has one channel of one token, for one convolution or
// for one of a layer's two (x, w, y and the state of the second follow the first's: `second` floats into a slot's
// record).  A request that brings a single token has its state brought up to date here, by the thread that has just
// read it; longer portions leave that to the second kernel, which runs after every row has been written.
// TAPS: the number of taps if the kernel is built for it (everything a thread reads is asked for at once), 0: any.
template <typename T, int TAPS>
__global__ __launch_bounds__(kThreads) void causal_conv_kernel(const float* __restrict__ xa, const float* __restrict__ xb,
                                                               const float* __restrict__ wa, const float* __restrict__ wb,
                                                               T* __restrict__ ya, T* __restrict__ yb, float* __restrict__ state,
                                                               int64_t slot_stride, int64_t second, int n_slots,
                                                               const int32_t* __restrict__ q_starts,
                                                               const int32_t* __restrict__ seq_slots, int n_seqs, int hidden,
                                                               int taps) {
    __shared__ int s_info[3];
    const int t = blockIdx.x;
    // the request of this row: the one whose rows begin at or before it and end after it (every thread tries one)
    for (int s = threadIdx.x; s < n_seqs; s += kThreads) {
        const int lo = q_starts[s], hi = q_starts[s + 1];
        if (lo <= t && t < hi) {
            const int slot = seq_slots[s];
            s_info[0] = lo;
            s_info[1] = (slot >= 0 && slot < n_slots) ? slot : -1;
            s_info[2] = hi - lo;
        }
    }
    __syncthreads();
    const int c = blockIdx.y * kThreads + threadIdx.x;
    if (c >= hidden) return;
    const int first = s_info[0], slot = s_info[1];
    const int n_taps = TAPS ? TAPS : taps;
    const int keep = n_taps - 1;
    const bool store = s_info[2] == 1 && slot >= 0 && keep > 0;
    const int which = blockIdx.z;
    const float* x = which ? xb : xa;
    const float* w = (which ? wb : wa) + static_cast<int64_t>(c) * n_taps;
    T* y = which ? yb : ya;
    float* st = slot >= 0 ? state + slot * slot_stride + which * second + c : nullptr;
    const float here = x[static_cast<int64_t>(t) * hidden + c];
    float acc = here;
#pragma unroll
    for (int j = 0; j < n_taps - 1; ++j) {
        const int back = n_taps - 1 - j;  // how many tokens before this one
        const int src = t - back;
        float v;
        if (src >= first) v = x[static_cast<int64_t>(src) * hidden + c];
        else v = st ? st[static_cast<int64_t>(keep - (first - src)) * hidden] : 0.f;  // state row keep - k = k tokens before the portion
        acc = fmaf(w[j], v, acc);
    }
    acc = fmaf(w[n_taps - 1], here, acc);
    y[static_cast<int64_t>(t) * hidden + c] = from_float<T>(acc);
    if (store) {
        // a single token: every row moves one up (read before the row below it is written), the token's input is the last
#pragma unroll
        for (int i = 0; i < keep - 1; ++i) st[static_cast<int64_t>(i) * hidden] = st[static_cast<int64_t>(i + 1) * hidden];
        st[static_cast<int64_t>(keep - 1) * hidden] = here;
    }
}

// state'[i] for i in [0, taps - 1): the input (taps - 1 - i) tokens before the next portion's first token.
// grid = (requests, convolutions); a request of one token has been dealt with already.
__global__ __launch_bounds__(kThreads) void causal_conv_store_kernel(const float* __restrict__ xa, const float* __restrict__ xb,
                                                                     float* __restrict__ state, int64_t slot_stride,
                                                                     int64_t second, int n_slots,
                                                                     const int32_t* __restrict__ q_starts,
                                                                     const int32_t* __restrict__ seq_slots, int hidden,
                                                                     int taps) {
    const int s = blockIdx.x;
    const int slot = seq_slots[s];
    const int first = q_starts[s], n = q_starts[s + 1] - first;
    if (slot < 0 || slot >= n_slots || n <= 1) return;
    const float* x = blockIdx.y ? xb : xa;
    float* st = state + slot * slot_stride + blockIdx.y * second;
    const int keep = taps - 1;
    for (int c = threadIdx.x; c < hidden; c += kThreads) {
        // a thread owns its channel: old rows are read before they are overwritten (ascending i reads row i + n >= i)
        for (int i = 0; i < keep; ++i) {
            const int back = keep - i;  // tokens before the next portion's start
            float v;
            if (back <= n) v = x[static_cast<int64_t>(first + n - back) * hidden + c];
            else v = st[static_cast<int64_t>(i + n) * hidden + c];  // still an input of an earlier step: row i + n of the old state
            st[static_cast<int64_t>(i) * hidden + c] = v;
        }
    }
}

}  // namespace

extern "C" int fsie_group_rmsnorm(float* residual, const void* delta1, int delta1_dtype, const void* delta2, int delta2_dtype,
                                  float delta_scale, const float* weight1, const float* weight2, void* out1, void* out2,
                                  const int32_t* rows, int n_rows, int hidden, int groups, float eps, int out_dtype,
                                  int write_back, hipStream_t stream) {
    FSIE_REQUIRE(n_rows >= 0 && hidden > 0 && groups > 0 && groups <= kMaxGroups && hidden % groups == 0,
                 "group_rmsnorm: %d values do not make %d equal groups (at most %d)", hidden, groups, kMaxGroups);
    FSIE_REQUIRE(residual && weight1 && out1 && (!weight2) == (!out2), "group_rmsnorm: missing operand");
    FSIE_REQUIRE(out_dtype == FSIE_F32 || out_dtype == FSIE_BF16, "group_rmsnorm: unknown dtype %d", out_dtype);
    FSIE_REQUIRE((!delta1 || delta1_dtype == FSIE_F32 || delta1_dtype == FSIE_BF16) &&
                     (!delta2 || delta2_dtype == FSIE_F32 || delta2_dtype == FSIE_BF16), "group_rmsnorm: unknown delta dtype");
    FSIE_REQUIRE(!(rows && write_back), "group_rmsnorm: chosen rows are not written back");
    if (n_rows == 0) return 0;
    const size_t lds = sizeof(float) * (static_cast<size_t>(hidden) + groups);
    FSIE_REQUIRE(lds <= 64 * 1024, "group_rmsnorm: rows of %d values are more than the kernel holds", hidden);
    const auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool vec = hidden % 4 == 0 && aligned(residual) && aligned(delta1) && aligned(delta2) && aligned(weight1) &&
                     aligned(weight2) && aligned(out1) && aligned(out2);
#define FSIE_GN(T, D1, D2)                                                                                              \
    do {                                                                                                                \
        auto kernel = vec ? group_rmsnorm_kernel<T, D1, D2, true> : group_rmsnorm_kernel<T, D1, D2, false>;             \
        if (lds > 48 * 1024) {                                                                                          \
            const hipError_t ok = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),                            \
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
            FSIE_REQUIRE(ok == hipSuccess, "group_rmsnorm: %zu bytes of shared memory: %s", lds, hipGetErrorString(ok)); \
        }                                                                                                               \
        kernel<<<n_rows, kThreads, lds, stream>>>(residual, static_cast<const D1*>(delta1), static_cast<const D2*>(delta2), \
                                                  delta_scale, weight1, weight2, static_cast<T*>(out1),                 \
                                                  static_cast<T*>(out2), rows, hidden, groups, eps, write_back);        \
    } while (0)
#define FSIE_GN_D(T)                                                                       \
    if (delta1_dtype == FSIE_F32 && delta2_dtype == FSIE_F32) FSIE_GN(T, float, float);    \
    else if (delta1_dtype == FSIE_F32) FSIE_GN(T, float, bf16_t);                          \
    else if (delta2_dtype == FSIE_F32) FSIE_GN(T, bf16_t, float);                          \
    else FSIE_GN(T, bf16_t, bf16_t)
    if (!delta1) delta1_dtype = FSIE_F32;
    if (!delta2) delta2_dtype = FSIE_F32;
    if (out_dtype == FSIE_F32) { FSIE_GN_D(float); } else { FSIE_GN_D(bf16_t); }
#undef FSIE_GN_D
#undef FSIE_GN
    FSIE_CHECK_LAUNCH("group_rmsnorm");
    return 0;
}

// x2 (with w2, y2): a second convolution of the same sizes in the same launches; its state lies `second` floats into a
// slot's record.
extern "C" int fsie_causal_conv(const float* x, const float* w, void* y, const float* x2, const float* w2, void* y2,
                                float* state, int64_t slot_stride, int64_t second, int n_slots, const int32_t* q_starts,
                                const int32_t* seq_slots, int n_seqs, int n_tokens, int hidden, int taps, int dtype,
                                hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && n_seqs >= 0 && hidden > 0 && taps >= 1 && n_slots > 0,
                 "causal_conv: bad sizes T=%d requests=%d hidden=%d taps=%d", n_tokens, n_seqs, hidden, taps);
    FSIE_REQUIRE(x && w && y && q_starts && seq_slots && (taps == 1 || state), "causal_conv: missing operand");
    FSIE_REQUIRE((!x2) == (!w2) && (!x2) == (!y2), "causal_conv: a second convolution comes with its weights and its result");
    const int64_t one = static_cast<int64_t>(taps - 1) * hidden;
    FSIE_REQUIRE(slot_stride >= (x2 ? second + one : one) && (!x2 || second >= one), "causal_conv: slots closer than a state is long");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "causal_conv: unknown dtype %d", dtype);
    if (n_tokens == 0 || n_seqs == 0) return 0;
    const dim3 grid(n_tokens, static_cast<unsigned>(ceil_div64(hidden, kThreads)), x2 ? 2 : 1);
#define FSIE_CONV(T, TAPS)                                                                                               \
    causal_conv_kernel<T, TAPS><<<grid, kThreads, 0, stream>>>(x, x2, w, w2, static_cast<T*>(y), static_cast<T*>(y2), state,    \
                                                               slot_stride, second, n_slots, q_starts, seq_slots, n_seqs, hidden, \
                                                               taps)
#define FSIE_CONV_T(T)                  \
    if (taps == 4) FSIE_CONV(T, 4);     \
    else if (taps == 3) FSIE_CONV(T, 3); \
    else if (taps == 2) FSIE_CONV(T, 2); \
    else FSIE_CONV(T, 0)
    if (dtype == FSIE_F32) { FSIE_CONV_T(float); } else { FSIE_CONV_T(bf16_t); }
#undef FSIE_CONV_T
#undef FSIE_CONV
    FSIE_CHECK_LAUNCH("causal_conv");
    if (taps > 1 && n_tokens != n_seqs) {  // (as many tokens as requests: one each, or the kernel above would have no request for a row)
        causal_conv_store_kernel<<<dim3(n_seqs, x2 ? 2 : 1), kThreads, 0, stream>>>(x, x2, state, slot_stride, second, n_slots,
                                                                                   q_starts, seq_slots, hidden, taps);
        FSIE_CHECK_LAUNCH("causal_conv_store");
    }
    return 0;
}
