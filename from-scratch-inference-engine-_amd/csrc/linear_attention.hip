// Gated linear attention: a recurrent state per request and head, S [dim][vdim] in float32,
//   S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
// with a decay per key channel alpha = sigmoid(z)^(1/tau).  One pair of kernels serves portions of prompts
// and single decoded tokens: the tokens of a request's portion are walked in order, from the state that the
// request's slot holds, and the state is left there for the next step.  Everything that enters the
// recurrence is float32 (decays, their logarithms, the state, the sums); q, k and v come in the
// activations' type as the projections left them.
//
// The walk is bound by arithmetic: every state element costs three instructions a token, on the vector
// units, in float32.  So the state of a head is spread over as many waves as the sizes give: a workgroup of
// sixteen waves holds [rows of one split][64 value columns], wave w a few consecutive key channels of it,
// lane = value column.  What a wave needs of a token besides v (its channels' decay, k and scaled q) is
// the same in all its lanes: a first kernel lays these out in float32 ([token][head][padded channel], the
// padding with decay 1 and k = q = 0), and the walk reads them with addresses that are uniform over the
// wave, which the compiler turns into scalar loads: no lane-wide traffic for them at all.
//
// A portion of kGlaChunkMin tokens or more does not walk token by token.  It is cut into chunks of sixteen
// tokens (counted from the portion's first token), and with B_t the sum of log alpha over the chunk's tokens
// up to and including t, per channel,
//   o_t   = (q_t * exp(B_t))^T S_in + sum_{j <= t} A[t][j] v_j,   A[t][j] = sum_c q_t[c] k_j[c] exp(B_t[c] - B_j[c]),
//   S_out = diag(exp(B_last)) S_in + sum_j (k_j * exp(B_last - B_j)) v_j^T,
// which is the same recurrence with its sums taken in another order: every exponent is a sum of logarithms of
// decays, none is positive, nothing can overflow whatever the decays are.  A first kernel computes the scaled
// q and k, the chunk's decay and A for every chunk and head at once (float32 on the vector units); the walk
// over chunks then is three small matrix products a chunk on the float32 matrix instruction
// (v_mfma_f32_16x16x4_f32, no rounding of operands), one wave per sixteen key channels and sixteen value
// columns with its tile of S in an accumulator; the waves of a head's columns meet every few chunks to add
// their shares of o.
#include "common.h"
#include "api.h"
#include "chunk_scan_impl.h"

#include <math.h>

namespace {

constexpr int kGlaWaves = 16;
constexpr int kGlaThreads = 64 * kGlaWaves;
constexpr int kGlaCols = 64;
constexpr int kGlaTokens = 8;  // tokens whose shares of o are added up at once
constexpr int kGlaChunkThreads = 256;


// log(sigmoid(z)) without overflow: min(z, 0) - log(1 + exp(-|z|))
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// Channel i of a head's q or k (x points at it), turned by the token's angles where a rotation is given: the first
// 2 * pairs channels of a head rotate, channel i with channel i + pairs, by cs[i mod pairs] = (cos, sin); float32.
template <typename T>
__device__ __forceinline__ float turned_channel(const T* __restrict__ x, int i, int pairs, const float2* __restrict__ cs) {
    const float a = to_float(x[0]);
    if (!cs || i >= 2 * pairs) return a;
    const bool low = i < pairs;
    const float b = to_float(low ? x[pairs] : x[-pairs]);
    const float2 t = cs[low ? i : i - pairs];
    return low ? fmaf(a, t.x, -(b * t.y)) : fmaf(a, t.x, b * t.y);
}

// prep [3][tokens][heads][dp]: scaled q, k, decay.  Grid: blocks of 256 elements over all tokens of the step,
// or (with short_only > 0) over the first tokens of every request (grid.y), and only for requests of at most
// short_only tokens: the others go chunk by chunk and need none of this.
template <typename T>
__global__ void gla_prep_kernel(const T* __restrict__ proj, int64_t proj_stride, int q_off, int k_off,
                                const float* __restrict__ z, float* __restrict__ prep, int64_t total, int heads, int dim,
                                int dp, float q_scale, float inv_tau, const int32_t* __restrict__ q_starts, int short_only,
                                const float* __restrict__ head_decay, const float2* __restrict__ cos_sin, int pairs) {
    int64_t e = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (short_only > 0) {
        const int lo = q_starts[blockIdx.y], len = q_starts[blockIdx.y + 1] - lo;
        if (len > short_only || e >= static_cast<int64_t>(len) * heads * dp) return;
        e += static_cast<int64_t>(lo) * heads * dp;
    }
    if (e >= total) return;
    const int i = static_cast<int>(e % dp);
    const int64_t th = e / dp;
    const int h = static_cast<int>(th % heads);
    const int64_t t = th / heads;
    float q = 0.f, k = 0.f, a = 1.f;
    if (i < dim) {
        const T* row = proj + t * proj_stride + h * dim + i;
        const float2* cs = cos_sin ? cos_sin + t * pairs : nullptr;
        q = turned_channel(row + q_off, i, pairs, cs) * q_scale;
        k = turned_channel(row + k_off, i, pairs, cs);
        a = head_decay ? head_decay[h] : expf(inv_tau * log_sigmoid(z[(t * heads + h) * dim + i]));
    }
    prep[e] = q;
    prep[total + e] = k;
    prep[2 * total + e] = a;
}

// grid = (requests of the step, heads, column blocks * row splits).  out [row splits][tokens][heads * vdim]:
// every split's share of o, for the consumer to add in order.
template <typename T, int ROWS>
__global__ __launch_bounds__(kGlaThreads) void gla_scan_kernel(
    const T* __restrict__ proj, int64_t proj_stride, int v_off, const float* __restrict__ prep, int64_t prep_plane,
    float* __restrict__ state, const int32_t* __restrict__ q_starts, const int32_t* __restrict__ seq_slots,
    float* __restrict__ out, int64_t out_plane, int heads, int dim, int vdim, int dp, int row_splits, int n_slots,
    int skip_from) {
    constexpr int TT = kGlaTokens;
    __shared__ float part[kGlaWaves][TT][kGlaCols];
    const int seq = blockIdx.x, h = blockIdx.y;
    const int split = blockIdx.z % row_splits, col_block = blockIdx.z / row_splits;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same in all lanes: what depends on it alone is scalar
    const int col = col_block * kGlaCols + lane;
    const int lo = q_starts[seq], hi = q_starts[seq + 1];
    const int slot = seq_slots[seq];
    if (hi <= lo || slot < 0 || slot >= n_slots) return;  // the same for the whole workgroup
    if (hi - lo >= skip_from) return;                     // the chunk kernels' portion
    const bool col_ok = col < vdim;
    const int row0 = (split * kGlaWaves + wave) * ROWS;  // this wave's first key channel

    float* my_state = state + ((static_cast<int64_t>(slot) * heads + h) * dim) * vdim + col;
    float S[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) S[r] = (col_ok && row0 + r < dim) ? my_state[static_cast<int64_t>(row0 + r) * vdim] : 0.f;

    const float* qp = prep + static_cast<int64_t>(h) * dp + row0;
    const float* kp = qp + prep_plane;
    const float* ap = kp + prep_plane;
    const int64_t token_stride = static_cast<int64_t>(heads) * dp;
    float* mine = out + split * out_plane;

    for (int t0 = lo; t0 < hi; t0 += TT) {
        const int nt = min(TT, hi - t0);
        float v[TT];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            v[tt] = (tt < nt && col_ok)
                        ? to_float(proj[static_cast<int64_t>(t0 + tt) * proj_stride + v_off + h * vdim + col]) : 0.f;
        }
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            if (tt < nt) {  // the same for the whole workgroup
                const int64_t at = static_cast<int64_t>(t0 + tt) * token_stride;
                float o = 0.f;
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    S[r] = fmaf(ap[at + r], S[r], kp[at + r] * v[tt]);
                    o = fmaf(S[r], qp[at + r], o);
                }
                part[wave][tt][lane] = o;
            }
        }
        lds_barrier();
        for (int e = tid; e < nt * kGlaCols; e += kGlaThreads) {
            const int tt = e >> 6, c = e & 63;
            const int cc = col_block * kGlaCols + c;
            if (cc < vdim) {
                float o = part[0][tt][c];
#pragma unroll
                for (int w = 1; w < kGlaWaves; ++w) o += part[w][tt][c];
                mine[(static_cast<int64_t>(t0 + tt) * heads + h) * vdim + cc] = o;
            }
        }
        lds_barrier();  // the shares have been read: the next tile may overwrite them
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        if (col_ok && row0 + r < dim) my_state[static_cast<int64_t>(row0 + r) * vdim] = S[r];
    }
}

// The chunks of a step are numbered request by request, in the order of the requests; a request whose portion
// is shorter than kGlaChunkMin, or that has no slot, has none.  (A handful of scalar loads per workgroup.)
// grid = (upper bound of the step's chunks, heads).  The logarithms are kept to the base two (the hardware's
// exponential is 2^x).  Every (token, channel) of the chunk is one thread's in the loads and in the stores; only
// the running sums over the chunk's tokens are a thread a channel.  A's pairs (j <= i) are dealt to the first
// 136 threads, row i together with row 15 - i, so that no wave carries the empty half of the square.
template <typename T>
__global__ __launch_bounds__(kGlaChunkThreads) void gla_chunk_prep_kernel(
    const T* __restrict__ proj, int64_t proj_stride, int q_off, int k_off, const float* __restrict__ z,
    float* __restrict__ work, const int32_t* __restrict__ q_starts, const int32_t* __restrict__ seq_slots, int n_seqs,
    int heads, int dim, int dp, float q_scale, float inv_tau, int n_slots, const float* __restrict__ head_decay,
    const float2* __restrict__ cos_sin, int pairs) {
    extern __shared__ float lds[];  // [3][16][dp + 4]: q, k, B
    const int ld = dp + 4;
    float* qs = lds;
    float* ks = qs + kGlaChunk * ld;
    float* bs = ks + kGlaChunk * ld;
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
    const float to_log2 = inv_tau * 1.44269504088896340736f;

    for (int e = tid; e < kGlaChunk * dp; e += kGlaChunkThreads) {
        const int t = e / dp, c = e - t * dp;
        float q = 0.f, k = 0.f, la = 0.f;
        if (t < nt && c < dim) {
            const T* row = proj + static_cast<int64_t>(t0 + t) * proj_stride + h * dim + c;
            const float2* cs = cos_sin ? cos_sin + static_cast<int64_t>(t0 + t) * pairs : nullptr;
            q = turned_channel(row + q_off, c, pairs, cs) * q_scale;
            k = turned_channel(row + k_off, c, pairs, cs);
            la = head_decay ? log2f(head_decay[h])
                            : to_log2 * log_sigmoid(z[(static_cast<int64_t>(t0 + t) * heads + h) * dim + c]);
        }
        qs[t * ld + c] = q;
        ks[t * ld + c] = k;
        bs[t * ld + c] = la;
    }
    __syncthreads();
    for (int c = tid; c < dp; c += kGlaChunkThreads) {
        float sum = 0.f;
#pragma unroll
        for (int t = 0; t < kGlaChunk; ++t) {
            sum += bs[t * ld + c];
            bs[t * ld + c] = sum;
        }
        float whole = __builtin_amdgcn_exp2f(sum);
        if (head_decay && c < dim) {
            // a fixed decay: the chunk's decay is its power, by multiplications (it is what the state carries from
            // chunk to chunk, so its rounding adds up over a long prompt)
            whole = 1.f;
            for (int t = 0; t < nt; ++t) whole *= head_decay[h];
        }
        g[c] = whole;
    }
    __syncthreads();
    for (int e = tid; e < kGlaChunk * dp; e += kGlaChunkThreads) {
        const int t = e / dp, c = e - t * dp;
        qd[e] = qs[t * ld + c] * __builtin_amdgcn_exp2f(bs[t * ld + c]);
    }
    for (int e = tid; e < dp * (kGlaChunk / 4); e += kGlaChunkThreads) {
        const int c = e >> 2, t4 = (e & 3) * 4;
        const float last = bs[(kGlaChunk - 1) * ld + c];
        floatx4 kd;
#pragma unroll
        for (int i = 0; i < 4; ++i) kd[i] = ks[(t4 + i) * ld + c] * __builtin_amdgcn_exp2f(last - bs[(t4 + i) * ld + c]);
        *reinterpret_cast<floatx4*>(kdT + c * kGlaChunk + t4) = kd;
    }
    // A: thread p < 136 has the pair number p of the rows (r, 15 - r) put side by side, r = p / 17
    if (tid < kGlaChunk * (kGlaChunk + 1) / 2) {
        const int r = tid / (kGlaChunk + 1), o = tid - r * (kGlaChunk + 1);
        const int i = o <= r ? r : kGlaChunk - 1 - r;
        const int j = o <= r ? o : o - r - 1;
        float a = 0.f;
        if (i < nt) {
            const float* qi = qs + i * ld;
            const float* kj = ks + j * ld;
            const float* bi = bs + i * ld;
            const float* bj = bs + j * ld;
            for (int c = 0; c < dp; c += 4) {  // (channels past dim: q = k = 0)
                const floatx4 q4 = *reinterpret_cast<const floatx4*>(qi + c), k4 = *reinterpret_cast<const floatx4*>(kj + c);
                const floatx4 x4 = *reinterpret_cast<const floatx4*>(bi + c) - *reinterpret_cast<const floatx4*>(bj + c);
#pragma unroll
                for (int u = 0; u < 4; ++u) a = fmaf(q4[u] * k4[u], __builtin_amdgcn_exp2f(x4[u]), a);
            }
        }
        A[i * kGlaChunk + j] = a;
    }
    // above the diagonal: zeros
    for (int e = tid; e < kGlaChunk * kGlaChunk; e += kGlaChunkThreads) {
        if ((e & 15) > (e >> 4)) A[e] = 0.f;
    }
}

// Key channels a wave holds and the splits of a head's channels over workgroups: as many splits (1, 2, 4)
// as still leave a wave four channels, while the workgroups of one request number fewer than 128.  A
// function of the layer's sizes alone, never of the step.
void gla_shape(int heads, int dim, int vdim, int* rows, int* splits) {
    const int col_blocks = (vdim + kGlaCols - 1) / kGlaCols;
    int s = 1;
    while (s < 4 && dim >= kGlaWaves * 2 * s * 4 && heads * col_blocks * s < 128) s *= 2;
    const int per_wave = (dim + kGlaWaves * s - 1) / (kGlaWaves * s);
    int r = 1;
    while (r < per_wave) r *= 2;
    *rows = r;
    *splits = s;
}

}  // namespace

// Sizes of the work arrays of fsie_gla_scan for a layer of these sizes: floats of `prep` a token, the planes
// of `out` (row splits), and for the portions that go chunk by chunk the tokens of a chunk, the shortest such
// portion and the floats of `chunk_work` a chunk.  A step of n_tokens tokens in n_seqs requests has at most
// n_tokens / chunk_tokens + n_seqs chunks, and none if n_tokens < chunk_min.
extern "C" int fsie_gla_scan_shape(int heads, int dim, int vdim, int* prep_floats_per_token, int* out_planes,
                                   int* chunk_tokens, int* chunk_min, int64_t* chunk_floats) {
    FSIE_REQUIRE(heads > 0 && dim > 0 && dim <= 256 && vdim > 0, "gla_scan_shape: bad sizes");
    int rows, splits;
    gla_shape(heads, dim, vdim, &rows, &splits);
    *prep_floats_per_token = 3 * heads * kGlaWaves * splits * rows;
    *out_planes = splits;
    *chunk_tokens = kGlaChunk;
    *chunk_min = kGlaChunkMin;
    *chunk_floats = gla_chunk_floats(kGlaWaves * splits * rows) * heads;
    return 0;
}

// proj [n_tokens][proj_stride]: of every token the q heads (heads x dim) from column q_off, the k heads
// from k_off, the v heads (heads x vdim) from v_off.  z [n_tokens][heads * dim] float32: the decays before
// the sigmoid.  state [n_slots][heads][dim][vdim] float32.  Request s of the step owns the tokens
// q_starts[s] .. q_starts[s + 1] and the slot seq_slots[s] (a slot outside the table: the request is
// skipped).  q is multiplied by q_scale; alpha = sigmoid(z)^inv_tau.  prep: work array of n_tokens *
// prep_floats_per_token floats; out: out_planes arrays [n_tokens][heads * vdim] float32 whose sum, in order,
// is o (fsie_gla_scan_shape gives both numbers).  chunk_work: room for max_chunks chunks, or null: with it, the
// portions of at least chunk_min tokens go chunk by chunk (max_chunks must be the bound that fsie_gla_scan_shape
// names, or more); without it every portion is walked token by token.  Which way a portion goes depends on
// its own length alone, and the two ways differ by rounding only.
extern "C" int fsie_gla_scan(const void* proj, int64_t proj_stride, int q_off, int k_off, int v_off, const float* z,
                             float* state, const int32_t* q_starts, const int32_t* seq_slots, int n_seqs, int n_tokens,
                             float* prep, float* out, float* chunk_work, int max_chunks, int heads, int dim, int vdim,
                             float q_scale, float inv_tau, int n_slots, int dtype, const float* head_decay,
                             const void* qk, int64_t qk_stride, const float* cos_sin, int rot_pairs, hipStream_t stream) {
    FSIE_REQUIRE(rot_pairs >= 0 && 2 * rot_pairs <= dim && (rot_pairs == 0 || cos_sin), "gla_scan: %d rotated pairs in heads of %d",
                 rot_pairs, dim);
    const float2* turn = rot_pairs > 0 ? reinterpret_cast<const float2*>(cos_sin) : nullptr;
    // q and k may live in rows of their own (qk, rows qk_stride apart, the same column offsets): a caller that has
    // turned them by the positions without touching the projection
    const void* qk_rows = qk ? qk : proj;
    const int64_t qk_step = qk ? qk_stride : proj_stride;
    FSIE_REQUIRE(!qk || (q_off + heads * dim <= qk_stride && k_off + heads * dim <= qk_stride),
                 "gla_scan: the q and k columns do not fit a row of %lld", static_cast<long long>(qk_stride));
    FSIE_REQUIRE(n_seqs >= 0 && n_tokens >= 0 && heads > 0 && dim > 0 && vdim > 0 && n_slots > 0, "gla_scan: bad sizes");
    FSIE_REQUIRE(dim <= 256, "gla_scan: %d key channels a head are more than the kernel takes (256)", dim);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "gla_scan: unknown dtype %d", dtype);
    FSIE_REQUIRE(proj && (z || head_decay) && state && q_starts && seq_slots && out && prep, "gla_scan: missing operand");
    FSIE_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && (qk || (q_off + heads * dim <= proj_stride &&
                     k_off + heads * dim <= proj_stride)) && v_off + heads * vdim <= proj_stride,
                 "gla_scan: the q, k and v columns do not fit a row of %lld", static_cast<long long>(proj_stride));
    if (n_seqs == 0 || n_tokens == 0) return 0;
    int rows, splits;
    gla_shape(heads, dim, vdim, &rows, &splits);
    const int dp = kGlaWaves * splits * rows;
    const int col_blocks = (vdim + kGlaCols - 1) / kGlaCols;
    FSIE_REQUIRE(heads <= 65535 && col_blocks * splits <= 65535 && (vdim + 15) / 16 <= 65535, "gla_scan: too many heads or columns");
    const int64_t plane = static_cast<int64_t>(n_tokens) * heads * dp;
    const int64_t out_plane = static_cast<int64_t>(n_tokens) * heads * vdim;
    const dim3 grid(n_seqs, heads, col_blocks * splits);
    const bool chunks = chunk_work != nullptr && n_tokens >= kGlaChunkMin;
    if (chunks) {
        FSIE_REQUIRE(max_chunks >= n_tokens / kGlaChunk + n_seqs, "gla_scan: room for %d chunks, the step may have %d",
                     max_chunks, n_tokens / kGlaChunk + n_seqs);
        FSIE_REQUIRE(max_chunks <= 0x7fffffff / kGlaChunk, "gla_scan: too many chunks");
        FSIE_REQUIRE(proj_stride <= 0x7fffffff / kGlaChunk && qk_step <= 0x7fffffff / kGlaChunk && static_cast<int64_t>(heads) * vdim <= 0x7fffffff / kGlaChunk,
                     "gla_scan: rows too long for the chunk kernels' 32-bit offsets");
    }
    const int skip_from = chunks ? kGlaChunkMin : 0x7fffffff;
    // with the chunk kernels at work only portions below their length are walked: their first tokens, request by request
    const int short_only = chunks ? kGlaChunkMin - 1 : 0;
    const dim3 prep_grid(static_cast<unsigned>(chunks ? ceil_div64(static_cast<int64_t>(short_only) * heads * dp, 256)
                                                      : ceil_div64(plane, 256)),
                         chunks ? n_seqs : 1);
    FSIE_REQUIRE(n_seqs <= 65535 || !chunks, "gla_scan: too many requests");
    const dim3 chunk_grid(chunks ? max_chunks : 1, heads);
    const size_t chunk_lds = 3 * kGlaChunk * (dp + 4) * sizeof(float);
    const dim3 scan_grid(n_seqs, heads, (vdim + 15) / 16);
    int scan_waves = 1;  // a wave for every sixteen key channels, rounded up to a power of two: at most sixteen
    while (scan_waves * 16 < dim) scan_waves *= 2;
#define FSIE_GLA_CHUNKS(T, NW)                                                                                        \
    gla_chunk_scan_kernel<T, NW, false><<<scan_grid, 64 * NW, 0, stream>>>(static_cast<const T*>(proj), proj_stride, v_off,    \
                                                                    chunk_work, state, q_starts, seq_slots, out,        \
                                                                    out_plane, heads, dim, vdim, dp, splits, n_slots,           \
                                                                    static_cast<int64_t>(dim) * vdim, 0, nullptr)
#define FSIE_GLA_LAUNCH(T, ROWS)                                                                                       \
    gla_scan_kernel<T, ROWS><<<grid, kGlaThreads, 0, stream>>>(static_cast<const T*>(proj), proj_stride, v_off, prep, plane, \
                                                               state, q_starts, seq_slots, out, out_plane, heads, dim, vdim, \
                                                               dp, splits, n_slots, skip_from)
#define FSIE_GLA_BY_ROWS(T)                                                                                          \
    gla_prep_kernel<T><<<prep_grid, 256, 0, stream>>>(static_cast<const T*>(qk_rows), qk_step, q_off, k_off, z, prep, \
                                                      plane, heads, dim, dp, q_scale, inv_tau, q_starts, short_only, head_decay,  \
                                                      turn, rot_pairs);                                              \
    if (rows == 1) FSIE_GLA_LAUNCH(T, 1);                                                                            \
    else if (rows == 2) FSIE_GLA_LAUNCH(T, 2);                                                                       \
    else if (rows == 4) FSIE_GLA_LAUNCH(T, 4);                                                                       \
    else if (rows == 8) FSIE_GLA_LAUNCH(T, 8);                                                                       \
    else FSIE_GLA_LAUNCH(T, 16);                                                                                     \
    if (chunks) {                                                                                                    \
        gla_chunk_prep_kernel<T><<<chunk_grid, kGlaChunkThreads, chunk_lds, stream>>>(                                \
            static_cast<const T*>(qk_rows), qk_step, q_off, k_off, z, chunk_work, q_starts, seq_slots, n_seqs, heads, dim, \
            dp, q_scale, inv_tau, n_slots, head_decay, turn, rot_pairs);                                             \
        if (scan_waves == 1) FSIE_GLA_CHUNKS(T, 1);                                                                  \
        else if (scan_waves == 2) FSIE_GLA_CHUNKS(T, 2);                                                             \
        else if (scan_waves == 4) FSIE_GLA_CHUNKS(T, 4);                                                             \
        else if (scan_waves == 8) FSIE_GLA_CHUNKS(T, 8);                                                             \
        else FSIE_GLA_CHUNKS(T, 16);                                                                                 \
    }
    if (dtype == FSIE_F32) {
        FSIE_GLA_BY_ROWS(float);
    } else {
        FSIE_GLA_BY_ROWS(bf16_t);
    }
#undef FSIE_GLA_BY_ROWS
#undef FSIE_GLA_LAUNCH
#undef FSIE_GLA_CHUNKS
    FSIE_CHECK_LAUNCH("gla_scan");
    return 0;
}
