// Routed experts: the router, the grouping of (token, choice) pairs by expert, one product per expert over tiles
// of its rows, and the weighted sum of a token's chosen experts.
//
//   route    a wave a token: float32 logits against every expert's row, sigmoid, the `top` largest of
//            score + correction (ties to the lower index), weights = chosen scores / their sum * scale
//   group    one workgroup: counts per expert, starts, a slot for every pair (pairs of one expert keep the order
//            of the pairs), and the table of row tiles (expert, first slot, slots) that never cross an expert
//   gemm     a workgroup per tile of 16, 32, 64 or 128 slots of one expert on the matrix cores: bfloat16 operands
//            (mfma 16x16x32) or true float32 ones (mfma 16x16x4); both operands run along K in memory, which is
//            the order the instruction wants; rows are gathered through the order table; the epilogue is the exact
//            GELU (up) or the pair's routing weight (down, float32 result)
//   combine  a token's rows added in the order of its choices, float32
// Nothing here waits for the host: the tile table has a fixed worst-case length and unused tiles are empty.
#include "common.h"
#include "api.h"
#include "wave_dots.h"

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kMaxExperts = 256;
constexpr int kMaxTop = 16;

// kind 0: scores are sigmoids of the logits; 1: their softmax over all experts.  groups > 1: the experts form that many
// equal groups of neighbours, a group's score is its largest score (+ correction), and only experts of the `keep` best
// groups can be chosen.  renorm: the chosen scores are divided by their sum.
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ x, const T* __restrict__ router,
                                                        const float* __restrict__ correction, int32_t* __restrict__ ids,
                                                        float* __restrict__ weights, int n_tokens, int hidden, int experts,
                                                        int top, float scale, int kind, int groups, int keep, int renorm) {
    __shared__ float s_score[4][kMaxExperts], s_choice[4][kMaxExperts];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + wave;
    const bool live = t < n_tokens;
    const T* row = x + static_cast<int64_t>(live ? t : 0) * hidden;
    float* score = s_score[wave];
    float* choice = s_choice[wave];
    const bool vec = wave_dots_vec(x, router, hidden);
    for (int e0 = 0; e0 < experts && live; e0 += kWaveDots) {
        float z[kWaveDots];
        wave_dots(row, router, hidden, e0, experts, vec, lane, z);
        // lane i keeps expert e0 + i: its score, and what the choice goes by
        float mine = 0.f;
#pragma unroll
        for (int i = 0; i < kWaveDots; ++i)
            if (lane == i) mine = z[i];
        if (lane < kWaveDots && e0 + lane < experts) {
            const float sc = kind == 1 ? mine : 1.0f / (1.0f + expf(-mine));  // (softmax: the logit for now)
            score[e0 + lane] = sc;
            choice[e0 + lane] = sc + (correction ? correction[e0 + lane] : 0.f);
        }
    }
    __syncthreads();
    if (kind == 1 && live) {
        // every lane reads all logits (the same walk in every lane), then each writes the experts it owns
        float m = -INFINITY, sum = 0.f;
        for (int e = 0; e < experts; ++e) m = fmaxf(m, score[e]);
        for (int e = 0; e < experts; ++e) sum += expf(score[e] - m);
        float mine[kMaxExperts / 64];
#pragma unroll
        for (int i = 0; i < kMaxExperts / 64; ++i) mine[i] = lane + 64 * i < experts ? expf(score[lane + 64 * i] - m) / sum : 0.f;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < kMaxExperts / 64; ++i) {
            const int e = lane + 64 * i;
            if (e < experts) {
                score[e] = mine[i];
                choice[e] = mine[i] + (correction ? correction[e] : 0.f);
            }
        }
    }
    __syncthreads();
    if (!live) return;
    // every lane walks the same choice (a few experts, a few picks): no exchange needed
    unsigned long long kept[kMaxExperts / 64];
#pragma unroll
    for (int i = 0; i < kMaxExperts / 64; ++i) kept[i] = ~0ull;
    const int per_group = groups > 1 ? experts / groups : experts;
    if (groups > 1 && keep < groups) {
#pragma unroll
        for (int i = 0; i < kMaxExperts / 64; ++i) kept[i] = 0ull;
        for (int c = 0; c < keep; ++c) {
            int best = -1;
            float best_v = -INFINITY;
            for (int g = 0; g < groups; ++g) {
                if ((kept[g >> 6] >> (g & 63)) & 1ull) continue;
                float v = -INFINITY;
                for (int e = g * per_group; e < (g + 1) * per_group; ++e) v = fmaxf(v, choice[e]);
                if (best < 0 || v > best_v) best = g, best_v = v;
            }
            kept[best >> 6] |= 1ull << (best & 63);
        }
    }
    int picked[kMaxTop];
    float chosen[kMaxTop];
    float total = 0.f;
    for (int c = 0; c < top; ++c) {
        int best = -1;
        float best_v = -INFINITY;
        for (int e = 0; e < experts; ++e) {
            bool taken = false;
            for (int p = 0; p < c; ++p) taken = taken || picked[p] == e;
            const int g = e / per_group;
            const bool allowed = groups <= 1 || ((kept[g >> 6] >> (g & 63)) & 1ull);
            const float v = allowed ? choice[e] : -INFINITY;
            if (!taken && (best < 0 || v > best_v)) best = e, best_v = v;
        }
        picked[c] = best;
        chosen[c] = score[best];
        total += chosen[c];
    }
    if (lane < top) {
        float mine = 0.f;
        int id = 0;
        for (int c = 0; c < top; ++c)
            if (c == lane) mine = chosen[c], id = picked[c];
        ids[static_cast<int64_t>(t) * top + lane] = id;
        weights[static_cast<int64_t>(t) * top + lane] = renorm ? mine / (total + 1e-20f) * scale : mine * scale;
    }
}

// one workgroup of 1024 threads
__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t* __restrict__ ids, int n_pairs, int experts,
                                                         int tile_rows, int32_t* __restrict__ order,
                                                         int32_t* __restrict__ slot_of, int32_t* __restrict__ tiles,
                                                         int max_tiles) {
    __shared__ int s_count[kMaxExperts];
    __shared__ int s_start[kMaxExperts + 1];
    __shared__ int s_tile0[kMaxExperts + 1];
    const int tid = threadIdx.x;
    for (int e = tid; e < experts; e += blockDim.x) s_count[e] = 0;
    __syncthreads();
    // thread i takes the pairs [i * chunk, (i + 1) * chunk): a pair's place among its expert's pairs is the pairs of
    // that expert before it, so the grouping is the same whatever the hardware does first
    const int chunk = (n_pairs + blockDim.x - 1) / blockDim.x;
    const int lo = min(n_pairs, tid * chunk), hi = min(n_pairs, lo + chunk);
    // pass 1: counts (an expert id outside the table is counted as expert 0; the router never makes one)
    for (int p = lo; p < hi; ++p) {
        int e = ids[p];
        e = (e < 0 || e >= experts) ? 0 : e;
        atomicAdd(&s_count[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int at = 0, tile = 0;
        for (int e = 0; e < experts; ++e) {
            s_start[e] = at;
            s_tile0[e] = tile;
            at += s_count[e];
            tile += (s_count[e] + tile_rows - 1) / tile_rows;
        }
        s_start[experts] = at;
        s_tile0[experts] = tile;
    }
    __syncthreads();
    // the tile table
    for (int i = tid; i < max_tiles; i += blockDim.x) {
        int e = 0;
        while (e < experts && s_tile0[e + 1] <= i) ++e;
        int32_t* tl = tiles + 3 * i;
        if (e >= experts) {
            tl[0] = 0, tl[1] = 0, tl[2] = 0;
        } else {
            const int first = s_start[e] + (i - s_tile0[e]) * tile_rows;
            tl[0] = e, tl[1] = first, tl[2] = min(tile_rows, s_start[e + 1] - first);
        }
    }
    __shared__ int s_scan[1024];
    if (n_pairs <= static_cast<int>(blockDim.x)) {
        // a pair a thread at most (every decode step): the pairs of its expert before it are counted one by one, all
        // threads reading the same id at a time
        int mine = -1;
        if (tid < n_pairs) {
            mine = ids[tid];
            mine = (mine < 0 || mine >= experts) ? 0 : mine;
        }
        s_scan[tid] = mine;
        __syncthreads();
        if (tid < n_pairs) {
            int before = 0;
            for (int p = 0; p < tid; ++p) before += s_scan[p] == mine;
            const int at = s_start[mine] + before;
            order[at] = tid;
            slot_of[tid] = at;
        }
        return;
    }
    // pass 2: a pair's slot = its expert's start + the pairs of that expert before it.  An expert at a time: the
    // threads' counts of it, an exclusive scan over the threads (in LDS), then the slots.
    for (int e = 0; e < experts; ++e) {
        if (s_count[e] == 0) continue;  // (the same for all threads)
        int mine = 0;
        for (int p = lo; p < hi; ++p) {
            int id = ids[p];
            id = (id < 0 || id >= experts) ? 0 : id;
            mine += id == e;
        }
        s_scan[tid] = mine;
        __syncthreads();
        for (int off = 1; off < static_cast<int>(blockDim.x); off <<= 1) {
            const int add = tid >= off ? s_scan[tid - off] : 0;
            __syncthreads();
            s_scan[tid] += add;
            __syncthreads();
        }
        int at = s_start[e] + s_scan[tid] - mine;
        for (int p = lo; p < hi; ++p) {
            int id = ids[p];
            id = (id < 0 || id >= experts) ? 0 : id;
            if (id == e) {
                order[at] = p;
                slot_of[p] = at;
                ++at;
            }
        }
        __syncthreads();
    }
}

__device__ __forceinline__ float gelu_erf(float z) { return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f)); }

// Workgroups go to the chip's eight dies in turn, and a die has its own L2.  Die d takes the tiles
// [d per_die, (d + 1) per_die) of the table (neighbouring tiles are mostly one expert's: a die reads an eighth of the
// experts' weights, not all of them) and walks them for one block of outputs before it goes to the next block, so
// that its tiles' rows stay in its L2 meanwhile.
__device__ __forceinline__ bool die_tile(int max_tiles, int n_blocks, int* tile, int* n_block) {
    const int per_die = (max_tiles + 7) / 8;
    const int die = blockIdx.x & 7, mine = blockIdx.x >> 3;
    *n_block = mine / per_die;
    *tile = die * per_die + (mine - *n_block * per_die);
    return *tile < max_tiles && *n_block < n_blocks;
}

// A workgroup of four waves and a tile of 16 MT slots of one expert.  A wave has MT x NB accumulators of 16 x 16 that
// share the rows' and the weights' fragments: lane l supplies, for the rows' operand, row l % 16 of each of its MT
// blocks and the values of K that its lane group (l / 16) owns, and the same of NB weight rows for the other operand;
// accumulator register r of lane l is (row 4 (l / 16) + r, column l % 16).
//   KSPLIT false (many rows an expert): the waves take 16 NB outputs each, side by side, and all of K.
//   KSPLIT true (few rows an expert: the product is bound by the read of the weights): the waves share 16 NB outputs
//   and take every fourth step of K each; their shares meet in LDS and are added in the order of the waves.
// A slot's sums depend on the variant, never on the other slots of its tile.
template <typename T, int MT, int NB, bool KSPLIT>
__global__ __launch_bounds__(256) void moe_gemm_kernel(const T* __restrict__ a, const T* __restrict__ w, void* __restrict__ out,
                                                       const int32_t* __restrict__ tiles, const int32_t* __restrict__ order,
                                                       int gather_div, const float* __restrict__ pair_weight, int N, int K,
                                                       int epilogue, int max_tiles) {
    __shared__ float red[KSPLIT ? 3 * MT * NB * 4 * 64 : 1];
    int tile, n_block;
    constexpr int kOutputs = KSPLIT ? 16 * NB : 64 * NB;  // outputs a workgroup
    if constexpr (KSPLIT) {
        // a handful of tiles, every weight read once: neighbouring workgroups take different tiles, so that every die
        // has its share of every expert's read
        tile = blockIdx.x % max_tiles, n_block = blockIdx.x / max_tiles;
    } else if (!die_tile(max_tiles, (N + kOutputs - 1) / kOutputs, &tile, &n_block)) {
        return;
    }
    const int32_t* tl = tiles + 3 * tile;
    const int expert = tl[0], slot0 = tl[1], n_rows = tl[2];
    if (n_rows <= 0) return;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int n0 = (KSPLIT ? n_block : n_block * 4 + wave) * 16 * NB;
    if (n0 >= N) return;  // (KSPLIT: the same for the whole workgroup)
    const int r = lane & 15, g = lane >> 4;
    const T* arow[MT];
    bool row_in[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        row_in[i] = 16 * i + r < n_rows;
        int64_t src = slot0 + 16 * i + r;
        if (row_in[i] && gather_div > 0) src = order[src] / gather_div;
        arow[i] = a + (row_in[i] ? src : 0) * K;
    }
    const T* wbase = w + static_cast<int64_t>(expert) * N * K;
    const T* wrow[NB];
    bool col_in[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int n = n0 + 16 * j + r;
        col_in[j] = n < N;
        wrow[j] = wbase + static_cast<int64_t>(col_in[j] ? n : 0) * K;
    }
    floatx4 acc[MT][NB];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    if constexpr (sizeof(T) == 2) {
        const bool vec = (K & 7) == 0 && (reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0;
        union Frag { uint4 raw; bf16x8 v; uint16_t h[8]; };
        if (vec) {
            // KSPLIT: a wave takes two steps side by side (a whole 128-byte line of every row) of every eight, and
            // asks for both before it multiplies
            constexpr int PAIR = KSPLIT ? 2 : 1;
#pragma unroll 2
            for (int kb = KSPLIT ? wave * 64 : 0; kb < K; kb += KSPLIT ? 256 : 32) {
                Frag fa[PAIR][MT], fb[PAIR][NB];
#pragma unroll
                for (int st = 0; st < PAIR; ++st) {
                    const int k = kb + 32 * st + 8 * g;
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        fa[st][i].raw = uint4{0, 0, 0, 0};
                        if (row_in[i] && k < K) fa[st][i].raw = *reinterpret_cast<const uint4*>(arow[i] + k);
                    }
#pragma unroll
                    for (int j = 0; j < NB; ++j) {
                        fb[st][j].raw = uint4{0, 0, 0, 0};
                        if (col_in[j] && k < K) fb[st][j].raw = *reinterpret_cast<const uint4*>(wrow[j] + k);
                    }
                }
#pragma unroll
                for (int st = 0; st < PAIR; ++st)
#pragma unroll
                    for (int i = 0; i < MT; ++i)
#pragma unroll
                        for (int j = 0; j < NB; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[st][i].v, fb[st][j].v, acc[i][j], 0, 0, 0);
            }
        } else {
            for (int k0 = KSPLIT ? wave * 32 : 0; k0 < K; k0 += KSPLIT ? 128 : 32) {
                const int k = k0 + 8 * g;
                Frag fa[MT], fb[NB];
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int u = 0; u < 8; ++u) fa[i].h[u] = (row_in[i] && k + u < K) ? arow[i][k + u].bits : 0;
#pragma unroll
                for (int j = 0; j < NB; ++j)
#pragma unroll
                    for (int u = 0; u < 8; ++u) fb[j].h[u] = (col_in[j] && k + u < K) ? wrow[j][k + u].bits : 0;
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int j = 0; j < NB; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i].v, fb[j].v, acc[i][j], 0, 0, 0);
            }
        }
    } else {
        // true float32 on the matrix cores: an instruction takes four values of K, one a lane group
#pragma unroll 2
        for (int k0 = KSPLIT ? wave * 4 : 0; k0 < K; k0 += KSPLIT ? 16 : 4) {
            const int k = k0 + g;
            float fa[MT], fb[NB];
#pragma unroll
            for (int i = 0; i < MT; ++i) fa[i] = (row_in[i] && k < K) ? to_float(arow[i][k]) : 0.f;
#pragma unroll
            for (int j = 0; j < NB; ++j) fb[j] = (col_in[j] && k < K) ? to_float(wrow[j][k]) : 0.f;
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    }
    if constexpr (KSPLIT) {
        if (wave > 0) {
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j)
#pragma unroll
                    for (int u = 0; u < 4; ++u) red[((((wave - 1) * MT + i) * NB + j) * 4 + u) * 64 + lane] = acc[i][j][u];
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int ww = 0; ww < 3; ++ww)
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j)
#pragma unroll
                    for (int u = 0; u < 4; ++u) acc[i][j][u] += red[(((ww * MT + i) * NB + j) * 4 + u) * 64 + lane];
    }
    // accumulator register u of block i: slot row 16 i + 4 g + u, output n0 + 16 j + r
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int row = 16 * i + 4 * g + u;
            if (row >= n_rows) continue;
            const int64_t slot = slot0 + row;
            const float scale = epilogue == 1 ? pair_weight[order[slot]] : 1.f;
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const int n = n0 + 16 * j + r;
                if (n >= N) continue;
                const float v = acc[i][j][u];
                if (epilogue == 1) {
                    static_cast<float*>(out)[slot * N + n] = v * scale;
                } else if (epilogue >= 2) {
                    // gate and up rows in turn: the even output's neighbour lane holds its up value
                    const float up = __shfl_xor(v, 1, FSIE_WAVE);
                    if (!(n & 1)) static_cast<T*>(out)[slot * (N / 2) + n / 2] = from_float<T>(gate_act(v, epilogue - 2) * up);
                } else {
                    static_cast<T*>(out)[slot * N + n] = from_float<T>(gelu_erf(v));
                }
            }
        }
    }
}

// grid = (tokens, blocks of 1024 values); VEC: four values a thread
template <bool VEC>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ rows, const int32_t* __restrict__ slot_of,
                                                          float* __restrict__ y, int top, int hidden) {
    const int t = blockIdx.x;
    int slots[kMaxTop];
#pragma unroll
    for (int c = 0; c < kMaxTop; ++c) slots[c] = c < top ? slot_of[t * top + c] : 0;
    constexpr int V = VEC ? 4 : 1;
    const int j = (blockIdx.y * 256 + threadIdx.x) * V;
    if (j >= hidden) return;
    float sum[V];
#pragma unroll
    for (int u = 0; u < V; ++u) sum[u] = 0.f;
#pragma unroll
    for (int c = 0; c < kMaxTop; ++c) {
        if (c < top) {
            const float* src = rows + static_cast<int64_t>(slots[c]) * hidden + j;
            if constexpr (VEC) {
                const float4 v = *reinterpret_cast<const float4*>(src);
                sum[0] += v.x, sum[1] += v.y, sum[2] += v.z, sum[3] += v.w;
            } else {
                sum[0] += src[0];
            }
        }
    }
    float* dst = y + static_cast<int64_t>(t) * hidden + j;
    if constexpr (VEC) *reinterpret_cast<float4*>(dst) = float4{sum[0], sum[1], sum[2], sum[3]};
    else dst[0] = sum[0];
}

}  // namespace

extern "C" int fsie_moe_route(const void* x, const void* router, const float* correction, int dtype, int32_t* ids,
                              float* weights, int n_tokens, int hidden, int experts, int top, float scale, int kind,
                              int groups, int keep, int renorm, hipStream_t stream) {
    FSIE_REQUIRE(kind == 0 || kind == 1, "moe_route: unknown kind of scores %d", kind);
    FSIE_REQUIRE(groups >= 1 && experts % groups == 0 && keep >= 1 && keep <= groups &&
                     (groups == 1 || top <= keep * (experts / groups)),
                 "moe_route: %d experts in %d groups of which %d are kept do not give %d choices", experts, groups, keep, top);
    FSIE_REQUIRE(n_tokens >= 0 && hidden > 0 && experts > 0 && experts <= kMaxExperts && top > 0 && top <= experts &&
                     top <= kMaxTop, "moe_route: bad sizes T=%d hidden=%d experts=%d (at most %d) top=%d (at most %d)",
                 n_tokens, hidden, experts, kMaxExperts, top, kMaxTop);
    FSIE_REQUIRE(x && router && ids && weights, "moe_route: missing operand");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "moe_route: unknown dtype %d", dtype);
    if (n_tokens == 0) return 0;
    const unsigned grid = static_cast<unsigned>((n_tokens + 3) / 4);
    if (dtype == FSIE_F32)
        moe_route_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(x), static_cast<const float*>(router),
                                                          correction, ids, weights, n_tokens, hidden, experts, top, scale, kind,
                                                          groups, keep, renorm);
    else
        moe_route_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(router),
                                                           correction, ids, weights, n_tokens, hidden, experts, top, scale, kind,
                                                          groups, keep, renorm);
    FSIE_CHECK_LAUNCH("moe_route");
    return 0;
}

extern "C" int fsie_moe_group(const int32_t* ids, int n_pairs, int experts, int tile_rows, int32_t* order, int32_t* slot_of,
                              int32_t* tiles, int max_tiles, hipStream_t stream) {
    FSIE_REQUIRE(n_pairs >= 0 && experts > 0 && experts <= kMaxExperts && tile_rows > 0,
                 "moe_group: bad sizes pairs=%d experts=%d tile=%d", n_pairs, experts, tile_rows);
    FSIE_REQUIRE(max_tiles >= (n_pairs + tile_rows - 1) / tile_rows + experts, "moe_group: the tile table is too short");
    FSIE_REQUIRE(ids && order && slot_of && tiles, "moe_group: missing operand");
    if (n_pairs == 0) return 0;
    moe_group_kernel<<<1, 1024, 0, stream>>>(ids, n_pairs, experts, tile_rows, order, slot_of, tiles, max_tiles);
    FSIE_CHECK_LAUNCH("moe_group");
    return 0;
}

// Rows of a tile that the products are best run with for this many (token, choice) pairs over this many experts: 16
// or 32 (the weights' read bounds the product: the waves split K, and an expert's rows should fit one tile so that
// its weights are read once), 64 or 128 (a weight fragment serves four or eight blocks of rows).  fsie_moe_group and
// fsie_moe_gemm take any of the four.
extern "C" int fsie_moe_tile_rows(int n_pairs, int experts) {
    const int per_expert = n_pairs / (experts > 0 ? experts : 1);
    return per_expert >= 256 ? 128 : per_expert >= 48 ? 64 : per_expert > 8 ? 32 : 16;
}

extern "C" int fsie_moe_gemm(const void* a, const void* w, void* out, const int32_t* tiles, int max_tiles,
                             const int32_t* order, int gather_div, const float* pair_weight, int N, int K, int epilogue,
                             int dtype, int tile_rows, hipStream_t stream) {
    FSIE_REQUIRE(max_tiles >= 0 && N > 0 && K > 0 && gather_div >= 0, "moe_gemm: bad sizes tiles=%d N=%d K=%d", max_tiles, N, K);
    FSIE_REQUIRE(tile_rows == 16 || tile_rows == 32 || tile_rows == 64 || tile_rows == 128,
                 "moe_gemm: tiles of %d rows (the kernels take 16, 32, 64, 128)", tile_rows);
    FSIE_REQUIRE(a && w && out && tiles && order, "moe_gemm: missing operand");
    FSIE_REQUIRE(epilogue == 0 || (epilogue == 1 && pair_weight) || (epilogue >= 2 && FSIE_ACT_KNOWN(epilogue - 2) && N % 2 == 0),
                 "moe_gemm: unknown epilogue %d", epilogue);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "moe_gemm: unknown dtype %d", dtype);
    if (max_tiles == 0) return 0;
    const int64_t per_die = ceil_div64(max_tiles, 8);
    FSIE_REQUIRE(per_die * 8 * ceil_div64(N, 16) <= 0x7fffffff, "moe_gemm: too many tiles");
#define FSIE_MOE_GEMM(T, MT, NB, KSPLIT)                                                                                 \
    moe_gemm_kernel<T, MT, NB, KSPLIT><<<static_cast<unsigned>((KSPLIT ? max_tiles : per_die * 8) *                        \
                                                               ceil_div64(N, KSPLIT ? 16 * NB : 64 * NB)),                  \
                                         256, 0, stream>>>(static_cast<const T*>(a), static_cast<const T*>(w), out, tiles, order, \
                                                           gather_div, pair_weight, N, K, epilogue, max_tiles)
#define FSIE_MOE_GEMM_T(T)                                      \
    if (tile_rows == 16) FSIE_MOE_GEMM(T, 1, 2, true);          \
    else if (tile_rows == 32) FSIE_MOE_GEMM(T, 2, 2, true);     \
    else if (tile_rows == 64) FSIE_MOE_GEMM(T, 4, 4, false);    \
    else FSIE_MOE_GEMM(T, 8, 4, false)
    if (dtype == FSIE_F32) { FSIE_MOE_GEMM_T(float); } else { FSIE_MOE_GEMM_T(bf16_t); }
#undef FSIE_MOE_GEMM_T
#undef FSIE_MOE_GEMM
    FSIE_CHECK_LAUNCH("moe_gemm");
    return 0;
}

extern "C" int fsie_moe_combine(const float* rows, const int32_t* slot_of, float* y, int n_tokens, int top, int hidden,
                                hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && top > 0 && hidden > 0, "moe_combine: bad sizes");
    FSIE_REQUIRE(rows && slot_of && y, "moe_combine: missing operand");
    if (n_tokens == 0) return 0;
    FSIE_REQUIRE(top <= kMaxTop, "moe_combine: top %d (at most %d)", top, kMaxTop);
    const bool vec = hidden % 4 == 0 && (reinterpret_cast<uintptr_t>(rows) & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    const dim3 grid(n_tokens, static_cast<unsigned>(ceil_div64(hidden, vec ? 1024 : 256)));
    if (vec) moe_combine_kernel<true><<<grid, 256, 0, stream>>>(rows, slot_of, y, top, hidden);
    else moe_combine_kernel<false><<<grid, 256, 0, stream>>>(rows, slot_of, y, top, hidden);
    FSIE_CHECK_LAUNCH("moe_combine");
    return 0;
}
