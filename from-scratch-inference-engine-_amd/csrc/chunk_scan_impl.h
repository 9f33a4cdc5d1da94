// The walk over chunks of sixteen tokens that the recurrent mixers share: a state S [dim][vdim] per request and
// head that every chunk multiplies by a decay per key channel and adds a product of sixteen keys and values to,
//   o_t   = qd_t^T S_in + sum_{j <= t} A[t][j] v_j,      S_out = diag(g) S_in + sum_j kd_j v_j^T,
// from a work array that the mixer's own kernel has filled for every chunk and head: qd [16][dp], kd transposed
// [dp][16], g [dp] and A [16][16] (zero above the diagonal), all float32.  What qd, kd, g and A are made of (decays
// per channel, one decay a head, gates) is the mixer's business.
#pragma once

#include "common.h"

namespace {

constexpr int kGlaChunk = 16;     // tokens of a chunk: one tile of the matrix instruction
constexpr int kGlaChunkMin = 16;  // portions of at least this many tokens go chunk by chunk

typedef float floatx4 __attribute__((ext_vector_type(4)));

// A workgroup barrier that waits for this wave's shared-memory traffic only.  __syncthreads also waits for
// the wave's loads and stores of global memory, and the walk has both in flight at every barrier (the next
// tokens' v on their way in, the last tokens' o on their way out): with it every tile of tokens paid two
// trips to memory, ten times its arithmetic.  What the waves exchange here goes through shared memory alone.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ int gla_chunks_of(const int32_t* q_starts, const int32_t* seq_slots, int s, int n_slots) {
    const int len = q_starts[s + 1] - q_starts[s];
    const int slot = seq_slots[s];
    return (len >= kGlaChunkMin && slot >= 0 && slot < n_slots) ? (len + kGlaChunk - 1) / kGlaChunk : 0;
}

// Work array of one chunk and head: qd [16][dp] (q * exp(B_t)), kdT [dp][16] (k * exp(B_last - B_t), channel
// major), g [dp] (exp(B_last)), A [16][16] (zero above the diagonal).  Tokens past the portion's end and
// channels past dim count as decay 1 with q = k = 0.
__host__ __device__ inline int64_t gla_chunk_floats(int dp) { return static_cast<int64_t>(2 * kGlaChunk + 1) * dp + kGlaChunk * kGlaChunk; }

// grid = (requests of the step, heads, tiles of sixteen value columns); a workgroup has a wave for every
// sixteen key channels of the head (NW: their number, rounded up to a power of two), and wave w holds the tile S[16 w .. 16 w + 15][its columns] in an
// accumulator: lane l has the channels 4 (l / 16) .. + 3 of it at the column l % 16.  That is also the layout of
// the instruction's second operand over four steps, if step i takes the channels 4 g + i (g = 0..3) as its four
// inner indices; a sum does not mind the order, so S is multiplied from the left as it lies.  The same
// renumbering of the inner index (the tokens 4 g + m at step m) lets v, kdT and A be read in vectors of four.
// A wave's chain per chunk is nine matrix instructions; the waves' shares of the chunks' o (and the four steps
// of A v, dealt to the waves in turn) meet in shared memory, a barrier every few chunks, and are added in the
// order of the waves.  The shares of o that the token-by-token kernel would leave in further planes of `out` are zero here.
//
// ONES: the grid has one more tile of columns after the head's last, and that tile carries a single further column
// of S whose values v are all one: a normaliser n_t = diag(g) n_(t-1) + k_t, with o = q . n.  It lies at
// `ones_at` floats into the head's record, its channels side by side, and its o goes to ones_out [tokens][heads].
template <typename T, int NW, bool ONES>
__global__ __launch_bounds__(64 * NW) void gla_chunk_scan_kernel(
    const T* __restrict__ proj, int64_t proj_stride, int v_off, const float* __restrict__ work,
    float* __restrict__ state, const int32_t* __restrict__ q_starts, const int32_t* __restrict__ seq_slots,
    float* __restrict__ out, int64_t out_plane, int heads, int dim, int vdim, int dp, int planes, int n_slots,
    int64_t state_head_stride, int64_t ones_at, float* __restrict__ ones_out) {
    constexpr int G = NW <= 8 ? 4 : 2;  // chunks between two barriers: their shares of o lie in LDS side by side
    __shared__ float part[2][G][NW][4][64];
    const int seq = blockIdx.x, h = blockIdx.y;
    const int n_chunks = gla_chunks_of(q_starts, seq_slots, seq, n_slots);
    if (n_chunks == 0) return;  // the same for the whole workgroup
    int first = 0;
    for (int s = 0; s < seq; ++s) first += gla_chunks_of(q_starts, seq_slots, s, n_slots);
    const int lo = q_starts[seq], hi = q_starts[seq + 1], slot = seq_slots[seq];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g4 = lane >> 4;
    const bool ones_tile = ONES && blockIdx.z == gridDim.z - 1;  // the same for the whole workgroup
    const int col = blockIdx.z * 16 + n;
    const bool col_ok = ones_tile ? n == 0 : col < vdim;
    const int64_t row_stride = ones_tile ? 1 : vdim;
    const int ch0 = wave * 16;  // this wave's first key channel

    // (a head's S [dim][vdim] starts every state_head_stride floats: the mixer may keep more than S in a head's record)
    float* my_state = state + (static_cast<int64_t>(slot) * heads + h) * state_head_stride + (ones_tile ? ones_at : col);
    floatx4 S;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = ch0 + 4 * g4 + i;
        S[i] = (col_ok && row < dim) ? my_state[static_cast<int64_t>(row) * row_stride] : 0.f;
    }
    const int64_t per_chunk = gla_chunk_floats(dp) * heads;
    const float* w = work + (static_cast<int64_t>(first) * heads + h) * gla_chunk_floats(dp);
    const T* vp = proj + v_off + h * vdim;
    const int64_t out_stride = static_cast<int64_t>(heads) * vdim;

    // The operands of the next D - 1 chunks are on their way while a chunk is multiplied: a ring of D sets of
    // registers, the walk unrolled D times so that every set has a fixed place.
    constexpr int D = 4;
    floatx4 q4[D], k4[D], g4v[D], a4[D];
    float v[D][4];
    // A chunk's addresses are a base that is the same in all lanes plus a lane's share that never changes.
    const int q_at = n * dp + ch0 + 4 * g4;
    const int k_at = kGlaChunk * dp + (ch0 + n) * kGlaChunk + 4 * g4;
    const int g_at = 2 * kGlaChunk * dp + ch0 + 4 * g4;
    const int a_at = (2 * kGlaChunk + 1) * dp + n * kGlaChunk + 4 * g4;
    const int v_col = min(col, vdim - 1);  // (columns past the head's last: a number, unused)
    int v_at[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) v_at[m] = (4 * g4 + m) * static_cast<int>(proj_stride) + v_col;
    auto fetch = [&](const int slot_, int ci) {
        ci = min(ci, n_chunks - 1);  // past the end: the last chunk once more, never used
        const float* wc = w + ci * per_chunk;
        const int t0 = lo + ci * kGlaChunk;
        const T* vc = vp + static_cast<int64_t>(t0) * proj_stride;
        // (a token past the portion's end has q = k = 0 and a zero row and column of A: the v of the portion's
        // last token stands in for it, a number that is multiplied by zero)
        if (ones_tile) {
#pragma unroll
            for (int m = 0; m < 4; ++m) v[slot_][m] = 1.f;
        } else if (t0 + kGlaChunk <= hi) {  // the same in all lanes
#pragma unroll
            for (int m = 0; m < 4; ++m) v[slot_][m] = to_float(vc[v_at[m]]);
        } else {
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                v[slot_][m] = to_float(vc[static_cast<int64_t>(min(4 * g4 + m, hi - 1 - t0)) * proj_stride + v_col]);
            }
        }
        q4[slot_] = *reinterpret_cast<const floatx4*>(wc + q_at);
        k4[slot_] = *reinterpret_cast<const floatx4*>(wc + k_at);
        g4v[slot_] = *reinterpret_cast<const floatx4*>(wc + g_at);
        a4[slot_] = *reinterpret_cast<const floatx4*>(wc + a_at);
    };
    // o of the `count` chunks of group gi (G chunks between two barriers) from the waves' shares, added in the
    // order of the waves, a value a thread and round.  Further planes of `out`: zeros.
    auto finish = [&](int gi, int count, bool really) {
        const int t0 = lo + gi * G * kGlaChunk;
        float* oc = ones_tile ? ones_out + static_cast<int64_t>(t0) * heads + h
                              : out + static_cast<int64_t>(t0) * out_stride + h * vdim + blockIdx.z * 16;
        const int o_stride = ones_tile ? heads : static_cast<int>(out_stride);
#pragma unroll
        for (int e0 = 0; e0 < 256 * G; e0 += 64 * NW) {
            const int e = e0 + tid;
            const int j = e >> 8, i = (e >> 6) & 3, l = e & 63;
            if (j < count) {
                float sum = part[gi & 1][j][0][i][l];
#pragma unroll
                for (int ww = 1; ww < NW; ++ww) sum += part[gi & 1][j][ww][i][l];
                const int tok = j * kGlaChunk + 4 * (l >> 4) + i, c = l & 15;
                if (really && t0 + tok < hi && (ones_tile ? c == 0 : blockIdx.z * 16 + c < vdim)) {
                    float* dst = oc + tok * o_stride + c;
                    *dst = sum;
                    if (!ones_tile)
                        for (int pl = 1; pl < planes; ++pl) dst[pl * out_plane] = 0.f;
                }
            }
        }
    };
#pragma unroll
    for (int u = 0; u < D - 1; ++u) fetch(u, u);
    for (int base = 0; base < n_chunks; base += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            const int ci = base + u;
            if (ci < n_chunks) {  // the same for the whole workgroup
                fetch((u + D - 1) % D, ci + D - 1);
                const int t0 = lo + ci * kGlaChunk;
                // o in two sums that do not wait for each other
                const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                floatx4 o[2];
                o[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(q4[u][0], S[0], zero, 0, 0, 0);
                o[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(q4[u][1], S[1], zero, 0, 0, 0);
                o[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(q4[u][2], S[2], o[0], 0, 0, 0);
                o[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(q4[u][3], S[3], o[1], 0, 0, 0);
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    if (m % NW == wave) o[m & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[u][m], v[u][m], o[m & 1], 0, 0, 0);
                }
                S *= g4v[u];
#pragma unroll
                for (int m = 0; m < 4; ++m) S = __builtin_amdgcn_mfma_f32_16x16x4f32(k4[u][m], v[u][m], S, 0, 0, 0);
                // the group before this one: its shares lie in the other half of `part` since the last barrier;
                // adding them up and storing o goes on while the matrix instructions above are at work
                const int gi = ci / G;
                if (u % G == 0) finish(gi - 1, G, gi > 0);
                const floatx4 mine = o[0] + o[1];
#pragma unroll
                for (int i = 0; i < 4; ++i) part[gi & 1][u % G][wave][i][lane] = mine[i];
                // at a group's end everyone has written its half and has read the other: the next group may
                // overwrite that
                if (u % G == G - 1 || ci == n_chunks - 1) lds_barrier();
            }
        }
    }
    finish((n_chunks - 1) / G, n_chunks - (n_chunks - 1) / G * G, true);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = ch0 + 4 * g4 + i;
        if (col_ok && row < dim) my_state[static_cast<int64_t>(row) * row_stride] = S[i];
    }
}

}  // namespace
