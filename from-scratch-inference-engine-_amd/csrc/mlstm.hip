// mLSTM: a matrix memory per head with exponential input and forget gates and a running maximum that keeps the
// exponentials in range.
//
//   i_t = cap tanh(gi_t / cap),  f_t = logsigmoid(cap tanh(gf_t / cap))            (log input gate, log forget gate)
//   m_t = max(f_t + m_(t-1), i_t),  keep_t = exp(f_t + m_(t-1) - m_t),  take_t = exp(i_t - m_t)
//   S_t = keep_t S_(t-1) + take_t k_t v_t^T,   n_t = keep_t n_(t-1) + take_t k_t
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
//
// S, n and m start at zero and live in the request's state record [heads][dim * vdim + dim + 4] (float32).  Both
// exponents are never positive.  Three kernels a step:
//   gates  one thread a (request, head): the activations of all its tokens, then the running maximum in order; it
//          carries m in the state and leaves (keep, take, exp(-m), m) per token and head
//   scan   a wave per (request, head, 16 value columns) walks the request's tokens in order; lane = (channel
//          quarter, column) holds a quarter of the key channels of its column of S in registers and the four quarters'
//          shares of S^T q meet through lane exchanges; one more wave per (request, head) carries n and leaves n . q
//   out    a wave per (token, head): the division, the head's unit RMS, the weight and the sigmoid gate
// Everything here is float32 whatever the projections' type.  The numbers of a token do not depend on how the
// request's tokens were cut into steps: the walk is token by token in both cases.
#include "common.h"
#include "api.h"

namespace {

constexpr int kCols = 16;        // value columns a wave
constexpr int kQuarters = 4;     // lane groups that split the key channels
constexpr int kMaxDim = 512;     // key channels a head

__device__ __forceinline__ float log_sigmoid(float z) {
    // -log(1 + exp(-z)), without overflow at either end
    return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
}

__global__ void mlstm_gates_kernel(const float* __restrict__ gates, float cap, float* __restrict__ state, int64_t record,
                                   int64_t m_at, int n_slots, const int32_t* __restrict__ q_starts,
                                   const int32_t* __restrict__ seq_slots, int n_seqs, int heads, float* __restrict__ coef) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_seqs * heads) return;
    const int s = idx / heads, h = idx - s * heads;
    const int slot = seq_slots[s];
    const int first = q_starts[s], last = q_starts[s + 1];
    float* m_state = (slot >= 0 && slot < n_slots) ? state + (static_cast<int64_t>(slot) * heads + h) * record + m_at : nullptr;
    float m = m_state ? *m_state : 0.f;
    for (int t = first; t < last; ++t) {
        const float gi = gates[static_cast<int64_t>(t) * 2 * heads + h];
        const float gf = gates[static_cast<int64_t>(t) * 2 * heads + heads + h];
        const float i = cap * tanhf(gi / cap);
        const float f = log_sigmoid(cap * tanhf(gf / cap));
        const float carried = f + m;
        const float m_new = fmaxf(carried, i);
        float4 c;
        c.x = expf(carried - m_new);
        c.y = expf(i - m_new);
        c.z = expf(-m_new);
        c.w = m_new;
        *reinterpret_cast<float4*>(coef + (static_cast<int64_t>(t) * heads + h) * 4) = c;
        m = m_new;
    }
    if (m_state && last > first) *m_state = m;
}

// NI: channels a lane holds (its quarter's share, rounded up); channel of register i: i * 4 + quarter
template <typename T, int NI>
__global__ __launch_bounds__(64) void mlstm_scan_kernel(const T* __restrict__ proj, int64_t stride, int q_off, int k_off,
                                                        int v_off, float q_scale, float* __restrict__ state, int64_t record,
                                                        int n_slots, const int32_t* __restrict__ q_starts,
                                                        const int32_t* __restrict__ seq_slots, int heads, int dim, int vdim,
                                                        const float* __restrict__ coef, float* __restrict__ num,
                                                        float* __restrict__ den, int col_tiles) {
    const int s = blockIdx.x, h = blockIdx.y, tile = blockIdx.z;
    const int lane = threadIdx.x;
    const int slot = seq_slots[s];
    const int first = q_starts[s], last = q_starts[s + 1];
    if (last <= first) return;
    float* rec = (slot >= 0 && slot < n_slots) ? state + (static_cast<int64_t>(slot) * heads + h) * record : nullptr;
    if (tile == col_tiles) {
        // the normaliser: lane l holds channels l, l + 64, ...
        constexpr int NN = (NI * kQuarters + 63) / 64;
        float n[NN];
        float* n_state = rec ? rec + static_cast<int64_t>(dim) * vdim : nullptr;
#pragma unroll
        for (int i = 0; i < NN; ++i) {
            const int c = i * 64 + lane;
            n[i] = (n_state && c < dim) ? n_state[c] : 0.f;
        }
        for (int t = first; t < last; ++t) {
            const T* row = proj + static_cast<int64_t>(t) * stride;
            const float4 cf = *reinterpret_cast<const float4*>(coef + (static_cast<int64_t>(t) * heads + h) * 4);
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < NN; ++i) {
                const int c = i * 64 + lane;
                const bool in = c < dim;
                const float k = in ? to_float(row[k_off + h * dim + c]) : 0.f;
                const float q = in ? to_float(row[q_off + h * dim + c]) * q_scale : 0.f;
                n[i] = fmaf(cf.x, n[i], cf.y * k);
                dot = fmaf(n[i], q, dot);
            }
            dot = wave_sum(dot);
            if (lane == 0) den[static_cast<int64_t>(t) * heads + h] = dot;
        }
        if (n_state) {
#pragma unroll
            for (int i = 0; i < NN; ++i) {
                const int c = i * 64 + lane;
                if (c < dim) n_state[c] = n[i];
            }
        }
        return;
    }
    const int quarter = lane >> 4, col = tile * kCols + (lane & 15);
    const bool col_in = col < vdim;
    float S[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int c = i * kQuarters + quarter;
        S[i] = (rec && col_in && c < dim) ? rec[static_cast<int64_t>(c) * vdim + col] : 0.f;
    }
    for (int t = first; t < last; ++t) {
        const T* row = proj + static_cast<int64_t>(t) * stride;
        const float4 cf = *reinterpret_cast<const float4*>(coef + (static_cast<int64_t>(t) * heads + h) * 4);
        const float v = col_in ? to_float(row[v_off + h * vdim + col]) * cf.y : 0.f;  // take * v
        float o = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int c = i * kQuarters + quarter;
            const bool in = c < dim;
            const float k = in ? to_float(row[k_off + h * dim + c]) : 0.f;
            const float q = in ? to_float(row[q_off + h * dim + c]) * q_scale : 0.f;
            S[i] = fmaf(cf.x, S[i], k * v);
            o = fmaf(S[i], q, o);
        }
        // the four quarters' shares, always in the same order
        o += __shfl_xor(o, 16, FSIE_WAVE);
        o += __shfl_xor(o, 32, FSIE_WAVE);
        if (quarter == 0 && col_in) num[(static_cast<int64_t>(t) * heads + h) * vdim + col] = o;
    }
    if (rec && col_in) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int c = i * kQuarters + quarter;
            if (c < dim) rec[static_cast<int64_t>(c) * vdim + col] = S[i];
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void mlstm_out_kernel(const float* __restrict__ num, const float* __restrict__ den,
                                                        const float* __restrict__ coef, const T* __restrict__ gate,
                                                        int64_t gate_stride, const float* __restrict__ weight,
                                                        T* __restrict__ y, int64_t n_units, int heads, int vdim, float eps) {
    const int64_t unit = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);  // token * heads + head
    if (unit >= n_units) return;
    const int lane = threadIdx.x & 63;
    const int64_t t = unit / heads;
    const int h = static_cast<int>(unit - t * heads);
    const float d = 1.0f / (fmaxf(fabsf(den[unit]), coef[unit * 4 + 2]) + 1e-6f);
    const float* o = num + unit * vdim;
    float sum = 0.f;
    for (int j = lane; j < vdim; j += 64) {
        const float v = o[j] * d;
        sum = fmaf(v, v, sum);
    }
    const float inv = 1.0f / sqrtf(wave_sum(sum) / static_cast<float>(vdim) + eps);
    const T* g = gate + t * gate_stride + h * vdim;
    T* out = y + unit * vdim;
    for (int j = lane; j < vdim; j += 64) {
        const float v = (o[j] * d) * inv * weight[h * vdim + j];
        out[j] = from_float<T>(v / (1.0f + expf(-to_float(g[j]))));
    }
}

}  // namespace

extern "C" int64_t fsie_mlstm_state_floats(int dim, int vdim) {
    return static_cast<int64_t>(dim) * vdim + dim + 4;
}

extern "C" int fsie_mlstm_scan(const void* proj, int64_t stride, int q_off, int k_off, int v_off, int dtype,
                               const float* gates, float gate_cap, float q_scale, float* state, int n_slots,
                               const int32_t* q_starts, const int32_t* seq_slots, int n_seqs, int n_tokens, int heads,
                               int dim, int vdim, float* coef, float* num, float* den, hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && n_seqs >= 0 && heads > 0 && dim > 0 && dim <= kMaxDim && vdim > 0 && n_slots > 0,
                 "mlstm_scan: bad sizes T=%d requests=%d heads=%d dim=%d (at most %d) vdim=%d", n_tokens, n_seqs, heads, dim,
                 kMaxDim, vdim);
    FSIE_REQUIRE(proj && gates && state && q_starts && seq_slots && coef && num && den, "mlstm_scan: missing operand");
    FSIE_REQUIRE(gate_cap > 0.f, "mlstm_scan: the gates' cap must be positive");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "mlstm_scan: unknown dtype %d", dtype);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(coef) % 16 == 0, "mlstm_scan: the coefficients must be 16-byte aligned");
    if (n_tokens == 0 || n_seqs == 0) return 0;
    const int64_t record = fsie_mlstm_state_floats(dim, vdim);
    const int64_t m_at = static_cast<int64_t>(dim) * vdim + dim;
    const int units = n_seqs * heads;
    mlstm_gates_kernel<<<(units + 63) / 64, 64, 0, stream>>>(gates, gate_cap, state, record, m_at, n_slots, q_starts, seq_slots,
                                                             n_seqs, heads, coef);
    FSIE_CHECK_LAUNCH("mlstm_gates");
    const int col_tiles = (vdim + kCols - 1) / kCols;
    const dim3 grid(n_seqs, heads, col_tiles + 1);
    const int per_lane = (dim + kQuarters - 1) / kQuarters;
#define FSIE_MLSTM(T, NI)                                                                                              \
    mlstm_scan_kernel<T, NI><<<grid, 64, 0, stream>>>(static_cast<const T*>(proj), stride, q_off, k_off, v_off, q_scale, state, \
                                                      record, n_slots, q_starts, seq_slots, heads, dim, vdim, coef, num, den, \
                                                      col_tiles)
#define FSIE_MLSTM_T(T)                         \
    if (per_lane <= 8) FSIE_MLSTM(T, 8);        \
    else if (per_lane <= 16) FSIE_MLSTM(T, 16); \
    else if (per_lane <= 32) FSIE_MLSTM(T, 32); \
    else if (per_lane <= 64) FSIE_MLSTM(T, 64); \
    else FSIE_MLSTM(T, 128)
    if (dtype == FSIE_F32) { FSIE_MLSTM_T(float); } else { FSIE_MLSTM_T(bf16_t); }
#undef FSIE_MLSTM_T
#undef FSIE_MLSTM
    FSIE_CHECK_LAUNCH("mlstm_scan");
    return 0;
}

extern "C" int fsie_mlstm_out(const float* num, const float* den, const float* coef, const void* gate, int64_t gate_stride,
                              const float* weight, void* y, int n_tokens, int heads, int vdim, float eps, int dtype,
                              hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && heads > 0 && vdim > 0, "mlstm_out: bad sizes");
    FSIE_REQUIRE(num && den && coef && gate && weight && y, "mlstm_out: missing operand");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "mlstm_out: unknown dtype %d", dtype);
    const int64_t units = static_cast<int64_t>(n_tokens) * heads;
    if (units == 0) return 0;
    const unsigned grid = static_cast<unsigned>((units + 3) / 4);
    if (dtype == FSIE_F32)
        mlstm_out_kernel<float><<<grid, 256, 0, stream>>>(num, den, coef, static_cast<const float*>(gate), gate_stride, weight,
                                                          static_cast<float*>(y), units, heads, vdim, eps);
    else
        mlstm_out_kernel<bf16_t><<<grid, 256, 0, stream>>>(num, den, coef, static_cast<const bf16_t*>(gate), gate_stride, weight,
                                                           static_cast<bf16_t*>(y), units, heads, vdim, eps);
    FSIE_CHECK_LAUNCH("mlstm_out");
    return 0;
}
