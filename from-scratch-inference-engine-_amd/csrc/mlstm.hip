// mLSTM: a matrix memory per head with exponential input and forget gates and a running maximum that keeps the
// exponentials in range.
//
//   i_t = cap tanh(gi_t / cap),  f_t = logsigmoid(cap tanh(gf_t / cap))            (log input gate, log forget gate)
//   m_t = max(f_t + m_(t-1), i_t),  keep_t = exp(f_t + m_(t-1) - m_t),  take_t = exp(i_t - m_t)
//   S_t = keep_t S_(t-1) + take_t k_t v_t^T,   n_t = keep_t n_(t-1) + take_t k_t
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
//
// S, n and m start at zero and live in the request's state record [heads][dim * vdim + dim + 4] (float32).  Both
// exponents are never positive.  The kernels of a step:
//   gates  a wave per (request, head): the activations of 64 tokens at a time, a token a lane, then the running
//          maximum in the tokens' order (the same few instructions in all lanes); it carries m in the state and
//          leaves (f, i, m before, m) per token and head
//   scan   portions below sixteen tokens, single decoded tokens among them: a wave per (request, head, 64 value
//          columns) walks the tokens in order with its columns of S in registers, a column a lane (heads of more
//          than 128 key channels: two or four lane groups split the channels, 32 or 16 columns a wave, and the
//          groups' shares of S^T q meet through lane exchanges); one more wave per (request, head) carries n and
//          leaves n . q
//   chunks longer portions go sixteen tokens at a time on the matrix cores.  With b_t the sum of f over the chunk's
//          tokens up to t and m_in the maximum that the chunk starts from,
//            S_t = exp(b_t + m_in - m_t) S_in + sum_{j <= t} exp(b_t - b_j + i_j - m_t) k_j v_j^T,
//          which is the recurrence with its factors multiplied out; m_t is at least every exponent's positive part, so
//          none is positive here either.  A first kernel lays out, per chunk and head, q_t exp(b_t + m_in - m_t),
//          k_j exp(b_last - b_j + i_j - m_last), the chunk's decay exp(b_last + m_in - m_last) and
//          A[t][j] = (q_t . k_j) exp(b_t - b_j + i_j - m_t); the walk over chunks that the recurrent mixers share
//          does the rest, with n as one more column of S whose values are all one.
//   out    a wave per (token, head): the division, the head's unit RMS, the weight and the sigmoid gate
// Everything here is float32 whatever the projections' type.  Which way a portion goes depends on its own length
// alone, and the two ways differ by rounding only.
#include "common.h"
#include "api.h"
#include "chunk_scan_impl.h"

namespace {

constexpr int kMaxDim = 512;     // key channels a head
constexpr int kMaxChunkDim = 256;  // ... of a head whose long portions go chunk by chunk
constexpr int kPrepThreads = 256;

__device__ __forceinline__ float log_sigmoid(float z) {
    // -log(1 + exp(-z)), without overflow at either end
    return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
}

// grid = requests * heads waves
__global__ __launch_bounds__(64) void mlstm_gates_kernel(const float* __restrict__ gates, float cap, float* __restrict__ state,
                                                         int64_t record, int64_t m_at, int n_slots,
                                                         const int32_t* __restrict__ q_starts,
                                                         const int32_t* __restrict__ seq_slots, int heads,
                                                         float* __restrict__ coef) {
    const int s = blockIdx.x / heads, h = blockIdx.x - s * heads;
    const int lane = threadIdx.x;
    const int slot = seq_slots[s];
    const int first = q_starts[s], last = q_starts[s + 1];
    if (last <= first) return;
    float* m_state = (slot >= 0 && slot < n_slots) ? state + (static_cast<int64_t>(slot) * heads + h) * record + m_at : nullptr;
    float m = m_state ? *m_state : 0.f;
    for (int t0 = first; t0 < last; t0 += 64) {
        const int t = t0 + lane;
        const int nt = min(64, last - t0);  // the same in all lanes
        float f = 0.f, i = 0.f;
        if (t < last) {
            const float gi = gates[static_cast<int64_t>(t) * 2 * heads + h];
            const float gf = gates[static_cast<int64_t>(t) * 2 * heads + heads + h];
            i = cap * tanhf(gi / cap);
            f = log_sigmoid(cap * tanhf(gf / cap));
        }
        float before = 0.f, mine = 0.f;
        if (nt == 64) {
            // a full round: nothing but the chain's add and maximum between two tokens
#pragma unroll
            for (int j = 0; j < 64; ++j) {
                const float fj = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, f), j));
                const float ij = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, i), j));
                const float m_new = fmaxf(fj + m, ij);
                if (lane == j) before = m, mine = m_new;
                m = m_new;
            }
        } else {
            for (int j = 0; j < nt; ++j) {
                const float fj = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, f), j));
                const float ij = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, i), j));
                const float m_new = fmaxf(fj + m, ij);
                if (lane == j) before = m, mine = m_new;
                m = m_new;
            }
        }
        if (t < last) *reinterpret_cast<float4*>(coef + (static_cast<int64_t>(t) * heads + h) * 4) = float4{f, i, before, mine};
    }
    if (m_state && lane == 0) *m_state = m;
}

// grid = (upper bound of the step's chunks, heads); the chunks of a step are numbered request by request.  Work array
// of a chunk and head as the walk over chunks wants it: qd [16][dp], kdT [dp][16], g [dp], A [16][16].
template <typename T>
__global__ __launch_bounds__(kPrepThreads) void mlstm_chunk_prep_kernel(
    const T* __restrict__ proj, int64_t proj_stride, int q_off, int k_off, const float* __restrict__ coef,
    float* __restrict__ work, const int32_t* __restrict__ q_starts, const int32_t* __restrict__ seq_slots, int n_seqs,
    int heads, int dim, int dp, float q_scale, int n_slots) {
    extern __shared__ float lds[];  // [2][16][dp + 4]: q, k
    __shared__ float s_dq[kGlaChunk], s_dk[kGlaChunk], s_b[kGlaChunk], s_i[kGlaChunk], s_m[kGlaChunk], s_g;
    const int ld = dp + 4;
    float* qs = lds;
    float* ks = qs + kGlaChunk * ld;
    const int h = blockIdx.y, tid = threadIdx.x;
    int first = 0, seq = -1;
    for (int s = 0; s < n_seqs; ++s) {
        const int n = gla_chunks_of(q_starts, seq_slots, s, n_slots);
        if (static_cast<int>(blockIdx.x) < first + n) { seq = s; break; }
        first += n;
    }
    if (seq < 0) return;  // the same for the whole workgroup
    const int t0 = q_starts[seq] + (static_cast<int>(blockIdx.x) - first) * kGlaChunk;
    const int nt = min(kGlaChunk, q_starts[seq + 1] - t0);
    float* w = work + (static_cast<int64_t>(blockIdx.x) * heads + h) * gla_chunk_floats(dp);
    float* qd = w;
    float* kdT = qd + kGlaChunk * dp;
    float* g = kdT + kGlaChunk * dp;
    float* A = g + dp;

    if (tid < kGlaChunk) {
        // b_t, in the tokens' order; the tokens past the portion's end stand still (f = 0, k = q = 0)
        const float4* cf = reinterpret_cast<const float4*>(coef) + static_cast<int64_t>(t0) * heads + h;
        const float m_in = cf[0].z;
        float b = 0.f, b_mine = 0.f, b_last = 0.f;
        for (int j = 0; j < nt; ++j) {
            b += cf[static_cast<int64_t>(j) * heads].x;
            if (j == tid) b_mine = b;
        }
        b_last = b;
        const float m_last = cf[static_cast<int64_t>(nt - 1) * heads].w;
        float dq = 0.f, dk = 0.f, i_mine = 0.f, m_mine = 0.f;
        if (tid < nt) {
            const float4 c = cf[static_cast<int64_t>(tid) * heads];
            dq = expf((b_mine + m_in) - c.w);
            dk = expf((b_last - b_mine) + (c.y - m_last));
            i_mine = c.y, m_mine = c.w;
        }
        s_dq[tid] = dq, s_dk[tid] = dk, s_b[tid] = b_mine, s_i[tid] = i_mine, s_m[tid] = m_mine;
        if (tid == 0) s_g = expf(b_last + m_in - m_last);
    }
    for (int e = tid; e < kGlaChunk * dp; e += kPrepThreads) {
        const int t = e / dp, c = e - t * dp;
        float q = 0.f, k = 0.f;
        if (t < nt && c < dim) {
            const T* row = proj + static_cast<int64_t>(t0 + t) * proj_stride + h * dim + c;
            q = to_float(row[q_off]) * q_scale;
            k = to_float(row[k_off]);
        }
        qs[t * ld + c] = q;
        ks[t * ld + c] = k;
    }
    __syncthreads();
    for (int e = tid; e < kGlaChunk * dp; e += kPrepThreads) {
        const int t = e / dp, c = e - t * dp;
        qd[e] = qs[t * ld + c] * s_dq[t];
    }
    for (int e = tid; e < dp * (kGlaChunk / 4); e += kPrepThreads) {
        const int c = e >> 2, t4 = (e & 3) * 4;
        floatx4 kd;
#pragma unroll
        for (int i = 0; i < 4; ++i) kd[i] = ks[(t4 + i) * ld + c] * s_dk[t4 + i];
        *reinterpret_cast<floatx4*>(kdT + c * kGlaChunk + t4) = kd;
    }
    for (int c = tid; c < dp; c += kPrepThreads) g[c] = s_g;
    // A: thread p < 136 has the pair number p of the rows (r, 15 - r) put side by side, r = p / 17
    if (tid < kGlaChunk * (kGlaChunk + 1) / 2) {
        const int r = tid / (kGlaChunk + 1), o = tid - r * (kGlaChunk + 1);
        const int i = o <= r ? r : kGlaChunk - 1 - r;
        const int j = o <= r ? o : o - r - 1;
        float a = 0.f;
        if (i < nt) {
            const float* qi = qs + i * ld;
            const float* kj = ks + j * ld;
            floatx4 a4 = {0.f, 0.f, 0.f, 0.f};
            for (int c = 0; c < dp; c += 4)  // (channels past dim: q = k = 0)
                a4 += *reinterpret_cast<const floatx4*>(qi + c) * *reinterpret_cast<const floatx4*>(kj + c);
            a = ((a4[0] + a4[1]) + (a4[2] + a4[3])) * expf((s_b[i] - s_b[j]) + (s_i[j] - s_m[i]));
        }
        A[i * kGlaChunk + j] = a;
    }
    // above the diagonal: zeros
    for (int e = tid; e < kGlaChunk * kGlaChunk; e += kPrepThreads) {
        if ((e & 15) > (e >> 4)) A[e] = 0.f;
    }
}

// Q lane groups split the key channels (one group for heads of up to 128 channels: a wave then reads and writes
// whole rows of 64 columns of S, 256 bytes side by side); NI: channels a lane holds (its group's share, rounded up);
// channel of register i: i * Q + group; a wave has 64 / Q value columns.
template <typename T, int NI, int Q>
__global__ __launch_bounds__(64) void mlstm_scan_kernel(const T* __restrict__ proj, int64_t stride, int q_off, int k_off,
                                                        int v_off, float q_scale, float* __restrict__ state, int64_t record,
                                                        int n_slots, const int32_t* __restrict__ q_starts,
                                                        const int32_t* __restrict__ seq_slots, int heads, int dim, int vdim,
                                                        const float* __restrict__ coef, float* __restrict__ num,
                                                        float* __restrict__ den, int col_tiles, int skip_from) {
    const int s = blockIdx.x, h = blockIdx.y, tile = blockIdx.z;
    const int lane = threadIdx.x;
    const int slot = seq_slots[s];
    const int first = q_starts[s], last = q_starts[s + 1];
    if (last <= first) return;
    float* rec = (slot >= 0 && slot < n_slots) ? state + (static_cast<int64_t>(slot) * heads + h) * record : nullptr;
    if (rec && last - first >= skip_from) return;  // the chunk kernels' portion
    if (tile == col_tiles) {
        // the normaliser: lane l holds channels l, l + 64, ...
        constexpr int NN = (NI * Q + 63) / 64;
        float n[NN];
        float* n_state = rec ? rec + static_cast<int64_t>(dim) * vdim : nullptr;
#pragma unroll
        for (int i = 0; i < NN; ++i) {
            const int c = i * 64 + lane;
            n[i] = (n_state && c < dim) ? n_state[c] : 0.f;
        }
        for (int t = first; t < last; ++t) {
            const T* row = proj + static_cast<int64_t>(t) * stride;
            const float4 gm = *reinterpret_cast<const float4*>(coef + (static_cast<int64_t>(t) * heads + h) * 4);
            const float2 cf = {expf(gm.x + gm.z - gm.w), expf(gm.y - gm.w)};  // keep, take
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
    constexpr int COLS = 64 / Q;
    const int quarter = lane / COLS, col = tile * COLS + lane % COLS;
    const bool col_in = col < vdim;
    float S[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int c = i * Q + quarter;
        S[i] = (rec && col_in && c < dim) ? rec[static_cast<int64_t>(c) * vdim + col] : 0.f;
    }
    for (int t = first; t < last; ++t) {
        const T* row = proj + static_cast<int64_t>(t) * stride;
        const float4 gm = *reinterpret_cast<const float4*>(coef + (static_cast<int64_t>(t) * heads + h) * 4);
            const float2 cf = {expf(gm.x + gm.z - gm.w), expf(gm.y - gm.w)};  // keep, take
        const float v = col_in ? to_float(row[v_off + h * vdim + col]) * cf.y : 0.f;  // take * v
        float o = 0.f;
        if constexpr (Q == 1) {
            // every lane needs every channel's k and q: a lane reads the channels lane, lane + 64, and each is handed
            // round from its lane
            constexpr int NR = (NI + 63) / 64;
            float kk[NR], qq[NR];
#pragma unroll
            for (int j = 0; j < NR; ++j) {
                const int c = j * 64 + lane;
                const bool in = c < dim;
                kk[j] = in ? to_float(row[k_off + h * dim + c]) : 0.f;
                qq[j] = in ? to_float(row[q_off + h * dim + c]) * q_scale : 0.f;
            }
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const float k = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, kk[i / 64]), i % 64));
                const float q = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, qq[i / 64]), i % 64));
                S[i] = fmaf(cf.x, S[i], k * v);
                o = fmaf(S[i], q, o);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int c = i * Q + quarter;
                const bool in = c < dim;
                const float k = in ? to_float(row[k_off + h * dim + c]) : 0.f;
                const float q = in ? to_float(row[q_off + h * dim + c]) * q_scale : 0.f;
                S[i] = fmaf(cf.x, S[i], k * v);
                o = fmaf(S[i], q, o);
            }
        }
        // the groups' shares, always in the same order
#pragma unroll
        for (int off = COLS; off < 64; off <<= 1) o += __shfl_xor(o, off, FSIE_WAVE);
        if (quarter == 0 && col_in) num[(static_cast<int64_t>(t) * heads + h) * vdim + col] = o;
    }
    if (rec && col_in) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int c = i * Q + quarter;
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
    const float d = 1.0f / (fmaxf(fabsf(den[unit]), expf(-coef[unit * 4 + 3])) + 1e-6f);
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

// Sizes of the chunk kernels' work array for a layer of these sizes: the tokens of a chunk, the shortest portion that
// goes chunk by chunk, and the floats of `chunk_work` a chunk (0: heads this wide are walked token by token only).  A
// step of n_tokens tokens in n_seqs requests has at most n_tokens / chunk_tokens + n_seqs chunks.
extern "C" int fsie_mlstm_scan_shape(int heads, int dim, int vdim, int* chunk_tokens, int* chunk_min, int64_t* chunk_floats) {
    FSIE_REQUIRE(heads > 0 && dim > 0 && dim <= kMaxDim && vdim > 0, "mlstm_scan_shape: bad sizes");
    int waves = 1;
    while (waves * 16 < dim) waves *= 2;
    *chunk_tokens = kGlaChunk;
    *chunk_min = kGlaChunkMin;
    *chunk_floats = dim <= kMaxChunkDim ? gla_chunk_floats(16 * waves) * heads : 0;
    return 0;
}

// chunk_work: room for max_chunks chunks, or null: with it, the portions of at least chunk_min tokens go chunk by
// chunk (max_chunks must be the bound that fsie_mlstm_scan_shape names, or more); without it every portion is walked
// token by token.  coef [n_tokens][heads][4] receives (f, i, m before the token, m).
extern "C" int fsie_mlstm_scan(const void* proj, int64_t stride, int q_off, int k_off, int v_off, int dtype,
                               const float* gates, float gate_cap, float q_scale, float* state, int n_slots,
                               const int32_t* q_starts, const int32_t* seq_slots, int n_seqs, int n_tokens, int heads,
                               int dim, int vdim, float* coef, float* num, float* den, float* chunk_work, int max_chunks,
                               hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && n_seqs >= 0 && heads > 0 && dim > 0 && dim <= kMaxDim && vdim > 0 && n_slots > 0,
                 "mlstm_scan: bad sizes T=%d requests=%d heads=%d dim=%d (at most %d) vdim=%d", n_tokens, n_seqs, heads, dim,
                 kMaxDim, vdim);
    FSIE_REQUIRE(proj && gates && state && q_starts && seq_slots && coef && num && den, "mlstm_scan: missing operand");
    FSIE_REQUIRE(gate_cap > 0.f, "mlstm_scan: the gates' cap must be positive");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "mlstm_scan: unknown dtype %d", dtype);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(coef) % 16 == 0, "mlstm_scan: the coefficients must be 16-byte aligned");
    FSIE_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + heads * dim <= stride && k_off + heads * dim <= stride &&
                     v_off + heads * vdim <= stride,
                 "mlstm_scan: the q, k and v columns do not fit a row of %lld", static_cast<long long>(stride));
    if (n_tokens == 0 || n_seqs == 0) return 0;
    const int64_t record = fsie_mlstm_state_floats(dim, vdim);
    const int64_t n_at = static_cast<int64_t>(dim) * vdim;
    const int64_t m_at = n_at + dim;
    // lane groups of the token-by-token walk: as few as the head's channels allow where that still leaves the chip four
    // waves a unit (whole rows of S a wave), else four (four times the waves, each with less to wait for)
    const bool wide = static_cast<int64_t>(n_seqs) * heads * ((vdim + 63) / 64) >= 1024;
    const int groups = dim > 256 || !wide ? 4 : dim > 128 ? 2 : 1;
    const int col_tiles = (vdim + 64 / groups - 1) / (64 / groups);
    const int chunk_tiles = (vdim + 15) / 16;
    FSIE_REQUIRE(heads <= 65535 && col_tiles + 1 <= 65535, "mlstm_scan: too many heads or columns");
    const bool chunks = chunk_work != nullptr && n_tokens >= kGlaChunkMin && dim <= kMaxChunkDim;
    if (chunks) {
        FSIE_REQUIRE(max_chunks >= n_tokens / kGlaChunk + n_seqs, "mlstm_scan: room for %d chunks, the step may have %d",
                     max_chunks, n_tokens / kGlaChunk + n_seqs);
        FSIE_REQUIRE(max_chunks <= 0x7fffffff / kGlaChunk, "mlstm_scan: too many chunks");
        FSIE_REQUIRE(stride <= 0x7fffffff / kGlaChunk && static_cast<int64_t>(heads) * vdim <= 0x7fffffff / kGlaChunk,
                     "mlstm_scan: rows too long for the chunk kernels' 32-bit offsets");
        FSIE_REQUIRE(reinterpret_cast<uintptr_t>(chunk_work) % 16 == 0, "mlstm_scan: the work array must be 16-byte aligned");
    }
    const int skip_from = chunks ? kGlaChunkMin : 0x7fffffff;
    mlstm_gates_kernel<<<n_seqs * heads, 64, 0, stream>>>(gates, gate_cap, state, record, m_at, n_slots, q_starts, seq_slots,
                                                          heads, coef);
    FSIE_CHECK_LAUNCH("mlstm_gates");
    const dim3 grid(n_seqs, heads, col_tiles + 1), chunk_grid(n_seqs, heads, chunk_tiles + 1);
    const int per_lane = (dim + groups - 1) / groups;
    int scan_waves = 1;  // a wave for every sixteen key channels, rounded up to a power of two: at most sixteen
    while (scan_waves * 16 < dim) scan_waves *= 2;
    const int dp = 16 * scan_waves;
    const dim3 prep_grid(chunks ? max_chunks : 1, heads);
    const size_t prep_lds = 2 * kGlaChunk * (dp + 4) * sizeof(float);
    const int64_t out_plane = static_cast<int64_t>(n_tokens) * heads * vdim;
#define FSIE_MLSTM(T, NI, Q)                                                                                              \
    mlstm_scan_kernel<T, NI, Q><<<grid, 64, 0, stream>>>(static_cast<const T*>(proj), stride, q_off, k_off, v_off, q_scale, state, \
                                                      record, n_slots, q_starts, seq_slots, heads, dim, vdim, coef, num, den, \
                                                      col_tiles, skip_from)
#define FSIE_MLSTM_CHUNKS(T, NW)                                                                                       \
    gla_chunk_scan_kernel<T, NW, true><<<chunk_grid, 64 * NW, 0, stream>>>(static_cast<const T*>(proj), stride, v_off, chunk_work,    \
                                                                     state, q_starts, seq_slots, num, out_plane, heads, dim,   \
                                                                     vdim, dp, 1, n_slots, record, n_at, den)
#define FSIE_MLSTM_T(T)                                                                                                \
    if (groups == 4 && per_lane <= 8) FSIE_MLSTM(T, 8, 4);                                                             \
    else if (groups == 4 && per_lane <= 16) FSIE_MLSTM(T, 16, 4);                                                      \
    else if (groups == 4 && per_lane <= 32) FSIE_MLSTM(T, 32, 4);                                                      \
    else if (groups == 4 && per_lane <= 64) FSIE_MLSTM(T, 64, 4);                                                      \
    else if (groups == 4) FSIE_MLSTM(T, 128, 4);                                                                       \
    else if (groups == 2) FSIE_MLSTM(T, 128, 2);                                                                       \
    else if (per_lane <= 32) FSIE_MLSTM(T, 32, 1);                                                                     \
    else if (per_lane <= 64) FSIE_MLSTM(T, 64, 1);                                                                     \
    else FSIE_MLSTM(T, 128, 1);                                                                                        \
    if (chunks) {                                                                                                      \
        mlstm_chunk_prep_kernel<T><<<prep_grid, kPrepThreads, prep_lds, stream>>>(                                      \
            static_cast<const T*>(proj), stride, q_off, k_off, coef, chunk_work, q_starts, seq_slots, n_seqs, heads, dim, dp,   \
            q_scale, n_slots);                                                                                         \
        if (scan_waves == 1) FSIE_MLSTM_CHUNKS(T, 1);                                                                  \
        else if (scan_waves == 2) FSIE_MLSTM_CHUNKS(T, 2);                                                             \
        else if (scan_waves == 4) FSIE_MLSTM_CHUNKS(T, 4);                                                             \
        else if (scan_waves == 8) FSIE_MLSTM_CHUNKS(T, 8);                                                             \
        else FSIE_MLSTM_CHUNKS(T, 16);                                                                                 \
    }
    if (dtype == FSIE_F32) { FSIE_MLSTM_T(float); } else { FSIE_MLSTM_T(bf16_t); }
#undef FSIE_MLSTM_T
#undef FSIE_MLSTM_CHUNKS
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
