// What stands between the fused projection and attention when the heads are normalised, only partly rotated,
// or have values of another size than their keys: one kernel a step and layer.
//
// proj [tokens][stride] holds of every token q (heads * dim from q_off), k (kv_heads * dim from k_off),
// v (kv_heads * vdim from v_off) and, optionally, one gate logit a head (from g_off).  Per token:
//   q, k heads: RMS norm over dim with a weight shared by the heads (q_weight / k_weight, or none; the query heads'
//               weights may also differ: head h then takes q_weight + h * q_weight_stride), then the
//               first 2 * pairs values turned, value i with value i + pairs, by the step's cosines and sines
//               cos_sin [tokens][pairs][2]; all of it float32
//   v:          (1 - mix) v + mix * v_other where another layer's values of the same token are given; with v_unit_norm
//               every head's values are then divided by sqrt(mean(v^2) + v_eps)
//   gate:       sigmoid of the logits, float32 [tokens][heads]
// q goes to q_out [tokens][heads * D] and k, v into the pools at slots[t], heads of D >= max(dim, vdim) values,
// zeros behind the dim (or vdim) that are used: the attention kernels take one head size for keys and values.
// A second kernel brings attention's result [tokens][heads * D] back to [tokens][heads * vdim], times the gate.
#include "common.h"
#include "api.h"

namespace {

constexpr int kThreads = 256;
// steps of this many tokens and more are taken to be portions of prompts (consecutive slots), fewer a decode batch
constexpr int kPortionTokens = 256;

// value j of a head's run x[0 .. dim) after norm (factor `scale`, weight w or none) and rotation
template <typename T>
__device__ __forceinline__ float normed_turned(const T* __restrict__ x, int j, float scale, const float* __restrict__ w,
                                               int pairs, const float2* __restrict__ cs) {
    const float a = w ? (to_float(x[j]) * scale) * w[j] : to_float(x[j]);
    if (j >= 2 * pairs) return a;
    const int jp = j < pairs ? j + pairs : j - pairs;
    const float b = w ? (to_float(x[jp]) * scale) * w[jp] : to_float(x[jp]);
    const float2 t = cs[j < pairs ? j : j - pairs];
    return j < pairs ? fmaf(a, t.x, -(b * t.y)) : fmaf(a, t.x, b * t.y);
}

// four consecutive values as floats / from floats: one 16-byte (float32) or 8-byte (bfloat16) access
__device__ __forceinline__ void load4(const float* p, float (&f)[4]) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    f[0] = v.x, f[1] = v.y, f[2] = v.z, f[3] = v.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float (&f)[4]) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    f[0] = __uint_as_float(v.x << 16), f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16), f[3] = __uint_as_float(v.y & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, const float (&f)[4]) {
    *reinterpret_cast<float4*>(p) = float4{f[0], f[1], f[2], f[3]};
}
__device__ __forceinline__ void store4(bf16_t* p, const float (&f)[4]) {
    uint2 w;
    w.x = pack2_bf16(f[0], f[1]);
    w.y = pack2_bf16(f[2], f[3]);
    *reinterpret_cast<uint2*>(p) = w;
}

// VEC: every size, offset and stride is a multiple of 4, heads are at most 256 values and the arrays are 16-byte
// aligned: a lane takes four neighbouring values with one access.  HPW: units of work a wave takes one after the
// other (a query head, a key head, a kv head's values, or all gates, in this order); with several, everything they
// need from memory is asked for before the first reduction, so that a wave's one wait for memory serves them all
// (portions of prompts: the kernel is made of that wait).
// With VEC a head takes L = 16, 32 or 64 lanes (four values a lane, L the smallest that holds D), so a wave's pass
// takes 64 / L heads side by side and its accesses stay wide for small heads.  The workgroups after the first
// `head_blocks` take the values and the gates, a wave a unit.
template <typename T, bool VEC, int HPW>
__global__ __launch_bounds__(kThreads) void attention_prep_kernel(
    const T* __restrict__ proj, int64_t stride, int q_off, int k_off, int v_off, int g_off, int heads, int kv_heads, int dim,
    int vdim, int D, const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps, int pairs,
    const float2* __restrict__ cos_sin, const T* __restrict__ v_other, int64_t v_other_stride, const float* __restrict__ mix,
    T* __restrict__ q_out, float* __restrict__ gate, const int32_t* __restrict__ slots, T* __restrict__ k_pool,
    T* __restrict__ v_pool, int page_size, int64_t pool_slots, int values_elsewhere, int L, int head_blocks,
    int q_weight_stride, int v_unit_norm, float v_eps) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int side = 64 / L;  // heads side by side in a pass
    const bool tail = static_cast<int>(blockIdx.y) >= head_blocks;
    const int unit0 = (blockIdx.y * (kThreads / 64) + (threadIdx.x >> 6)) * HPW * side;
    const T* row = proj + static_cast<int64_t>(t) * stride;
    const int64_t slot = slots ? slots[t] : -1;
    const bool store = k_pool && slot >= 0 && slot < pool_slots;
    const int64_t page = store ? slot / page_size : 0;
    const int off = store ? static_cast<int>(slot - page * page_size) : 0;
    const float2* cs = cos_sin + static_cast<int64_t>(t) * pairs;
    const int n_heads_all = heads + kv_heads;
    // where head `unit` is read from, which weight it takes and where it goes (null: nowhere)
    auto source = [&](int unit) { return row + (unit < heads ? q_off + unit * dim : k_off + (unit - heads) * dim); };
    auto weight = [&](int unit) { return unit < heads ? (q_weight ? q_weight + unit * q_weight_stride : nullptr) : k_weight; };
    auto target = [&](int unit) -> T* {
        if (unit < heads) return q_out + (static_cast<int64_t>(t) * heads + unit) * D;
        return store ? k_pool + ((page * kv_heads + (unit - heads)) * page_size + off) * D : nullptr;
    };
    if constexpr (VEC) {
        // The partner values of the rotation come from the lane that holds them, already normed, through a lane exchange.
        const int l = lane & (L - 1), mine = lane / L;
        const int j = 4 * l;
        const bool in = j < dim, turned = j < 2 * pairs, low = j < pairs;
        float a[HPW][4], ww[HPW][4], c4[4] = {1.f, 1.f, 1.f, 1.f}, s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < HPW; ++u) {
            const int unit = unit0 + u * side + mine;
            const bool live = !tail && unit < n_heads_all && in;
            const float* w = unit < n_heads_all ? weight(unit) : nullptr;
#pragma unroll
            for (int i = 0; i < 4; ++i) a[u][i] = 0.f, ww[u][i] = 1.f;
            if (live) load4(source(unit) + j, a[u]);
            if (live && w) load4(w + j, ww[u]);
        }
        if (turned && !tail && unit0 < n_heads_all) {
            const float2* tp = cs + (low ? j : j - pairs);
#pragma unroll
            for (int i = 0; i < 4; ++i) c4[i] = tp[i].x, s4[i] = tp[i].y;
        }
        const int partner = (lane & ~(L - 1)) | ((low ? l + (pairs >> 2) : l - (pairs >> 2)) & (L - 1));
#pragma unroll
        for (int u = 0; u < HPW; ++u) {
            if (tail || unit0 + u * side >= n_heads_all) break;  // (the same for the whole wave)
            const int unit = unit0 + u * side + mine;
            const bool head = unit < n_heads_all;
            const bool normed = head && weight(unit) != nullptr;
            float scale = 1.f;
            if (q_weight || k_weight) {  // (the same for the whole wave; a head without a weight drops the result)
                float sum = fmaf(a[u][0], a[u][0], fmaf(a[u][1], a[u][1], fmaf(a[u][2], a[u][2], a[u][3] * a[u][3])));
                for (int o = L >> 1; o > 0; o >>= 1) sum += __shfl_xor(sum, o, FSIE_WAVE);
                scale = 1.0f / sqrtf(sum / static_cast<float>(dim) + eps);
            }
            float b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                a[u][i] = normed ? (a[u][i] * scale) * ww[u][i] : a[u][i];
                b[i] = __shfl(a[u][i], partner, FSIE_WAVE);
            }
            if (turned) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    a[u][i] = low ? fmaf(a[u][i], c4[i], -(b[i] * s4[i])) : fmaf(a[u][i], c4[i], b[i] * s4[i]);
            }
            T* o = head ? target(unit) : nullptr;
            if (o && j < D) store4(o + j, a[u]);
        }
    } else {
        for (int u = 0; u < HPW && !tail; ++u) {
            const int unit = unit0 + u;
            if (unit >= n_heads_all) break;
            T* o = target(unit);
            if (!o) continue;
            const T* x = source(unit);
            const float* w = weight(unit);
            float scale = 1.f;
            if (w) {
                float sum = 0.f;
                for (int j = lane; j < dim; j += 64) sum = fmaf(to_float(x[j]), to_float(x[j]), sum);
                scale = 1.0f / sqrtf(wave_sum(sum) / static_cast<float>(dim) + eps);
            }
            for (int j = lane; j < D; j += 64) o[j] = from_float<T>(j < dim ? normed_turned(x, j, scale, w, pairs, cs) : 0.f);
        }
    }
    if (tail) {
        const int unit = n_heads_all + (blockIdx.y - head_blocks) * (kThreads / 64) + (threadIdx.x >> 6);
        if (unit < heads + 2 * kv_heads) {
            if (!store || values_elsewhere) return;
            const int g = unit - n_heads_all;
            const float lam = (v_other && mix) ? mix[0] : 0.f;
            auto value = [&](int j) {
                float v = to_float(row[v_off + g * vdim + j]);
                if (v_other) v = fmaf(lam, to_float(v_other[static_cast<int64_t>(t) * v_other_stride + g * vdim + j]), (1.0f - lam) * v);
                return v;
            };
            float unit = 1.f;
            if (v_unit_norm) {  // the head's values divided by their root mean square, as they are cached
                float sum = 0.f;
                for (int j = lane; j < vdim; j += 64) {
                    const float v = value(j);
                    sum = fmaf(v, v, sum);
                }
                unit = 1.0f / sqrtf(wave_sum(sum) / static_cast<float>(vdim) + v_eps);
            }
            for (int j = lane; j < D; j += 64)
                v_pool[((page * kv_heads + g) * D + j) * page_size + off] = from_float<T>(j < vdim ? value(j) * unit : 0.f);
        } else if (unit == heads + 2 * kv_heads && gate) {
            for (int h = lane; h < heads; h += 64)
                gate[static_cast<int64_t>(t) * heads + h] = 1.0f / (1.0f + expf(-to_float(row[g_off + h])));
        }
    }
}

// The values of many tokens (a portion of a prompt): a block takes eight consecutive tokens of one kv head, a thread
// a dimension.  A page of values lies as [dimension][slot], so a token's values are 2-byte pieces a page apart;
// where the eight tokens fill eight consecutive slots from a multiple of eight (the usual case inside a portion)
// a thread writes them as one 16-byte piece per dimension.  bfloat16 only (the float32 path writes value by value).
__global__ __launch_bounds__(kThreads) void attention_prep_values_kernel(
    const bf16_t* __restrict__ proj, int64_t stride, int v_off, int kv_heads, int vdim, int D,
    const bf16_t* __restrict__ v_other, int64_t v_other_stride, const float* __restrict__ mix,
    const int32_t* __restrict__ slots, bf16_t* __restrict__ v_pool, int page_size, int64_t pool_slots, int n_tokens) {
    const int t0 = blockIdx.x * 8, g = blockIdx.y;
    const int n = min(8, n_tokens - t0);
    int64_t slot[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) slot[i] = i < n ? slots[t0 + i] : -1;
    bool run = n == 8 && slot[0] >= 0 && slot[0] + 7 < pool_slots && (slot[0] & 7) == 0 && (page_size & 7) == 0;
#pragma unroll
    for (int i = 1; i < 8; ++i) run = run && slot[i] == slot[0] + i;
    const float lam = (v_other && mix) ? mix[0] : 0.f;
    for (int j = threadIdx.x; j < D; j += blockDim.x) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            v[i] = 0.f;
            if (i < n && j < vdim) {
                v[i] = to_float(proj[static_cast<int64_t>(t0 + i) * stride + v_off + g * vdim + j]);
                if (v_other) v[i] = fmaf(lam, to_float(v_other[static_cast<int64_t>(t0 + i) * v_other_stride + g * vdim + j]), (1.0f - lam) * v[i]);
            }
        }
        if (run) {
            const int64_t page = slot[0] / page_size;
            const int off = static_cast<int>(slot[0] - page * page_size);
            *reinterpret_cast<uint4*>(v_pool + ((page * kv_heads + g) * D + j) * page_size + off) =
                uint4{pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]), pack2_bf16(v[4], v[5]), pack2_bf16(v[6], v[7])};
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (i < n && slot[i] >= 0 && slot[i] < pool_slots) {
                    const int64_t page = slot[i] / page_size;
                    const int off = static_cast<int>(slot[i] - page * page_size);
                    v_pool[((page * kv_heads + g) * D + j) * page_size + off] = from_float<bf16_t>(v[i]);
                }
            }
        }
    }
}

// VEC: vdim and D are multiples of 4 and the arrays 16-byte aligned: a thread takes four values of a head
template <typename T, bool VEC>
__global__ __launch_bounds__(kThreads) void gate_heads_kernel(const T* __restrict__ x, int D, const float* __restrict__ gate,
                                                              T* __restrict__ y, int heads, int vdim, int64_t total,
                                                              int64_t y_stride, float y_scale) {
    constexpr int N = VEC ? 4 : 1;
    const int64_t e = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * N;
    if (e >= total) return;
    const int64_t th = e / vdim;  // token * heads + head
    const int j = static_cast<int>(e - th * vdim);
    const float g = (gate ? gate[th] : 1.f) * y_scale;
    const int64_t t = th / heads;
    T* to = y + t * y_stride + (th - t * heads) * vdim + j;  // (rows of y may be columns of wider rows)
    if constexpr (VEC) {
        float a[4];
        load4(x + th * D + j, a);
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] *= g;
        store4(to, a);
    } else {
        *to = from_float<T>(to_float(x[th * D + j]) * g);
    }
}

}  // namespace

extern "C" int fsie_attention_prep(const void* proj, int64_t stride, int q_off, int k_off, int v_off, int g_off, int heads,
                                   int kv_heads, int dim, int vdim, int D, const float* q_weight, const float* k_weight,
                                   float eps, int pairs, const float* cos_sin, const void* v_other, int64_t v_other_stride,
                                   const float* mix, void* q_out, float* gate, const int32_t* slots, void* k_pool,
                                   void* v_pool, int page_size, int64_t pool_slots, int n_tokens, int dtype,
                                   int q_weight_stride, int v_unit_norm, float v_eps, hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0 && D >= dim && D >= vdim,
                 "attention_prep: bad sizes heads=%d kv=%d dim=%d vdim=%d D=%d", heads, kv_heads, dim, vdim, D);
    FSIE_REQUIRE(pairs >= 0 && 2 * pairs <= dim && (pairs == 0 || cos_sin), "attention_prep: %d rotated pairs in heads of %d",
                 pairs, dim);
    FSIE_REQUIRE(proj && q_out, "attention_prep: missing operand");
    FSIE_REQUIRE(!k_pool || (v_pool && slots && page_size > 0 && pool_slots > 0), "attention_prep: bad page geometry");
    FSIE_REQUIRE(!v_other || mix, "attention_prep: values to mix in come with their weight");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "attention_prep: unknown dtype %d", dtype);
    if (n_tokens == 0) return 0;
    const auto mult4 = [](int64_t v) { return (v & 3) == 0; };
    const auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    FSIE_REQUIRE(q_weight_stride >= 0, "attention_prep: bad stride of the query heads' weights");
    const bool vec = D <= 256 && mult4(q_weight_stride) && mult4(stride) && mult4(q_off) && mult4(k_off) && mult4(dim) && mult4(D) && mult4(pairs) && al16(proj) &&
                     al16(q_out) && al16(k_pool) && al16(q_weight) && al16(k_weight) && al16(cos_sin);
    // portions of prompts in bfloat16: the values go through the kernel that writes eight slots at once
    // (not where the values are normed: that takes a head's values together)
    const int values_elsewhere = (k_pool && dtype == FSIE_BF16 && n_tokens >= kPortionTokens && al16(v_pool) && !v_unit_norm) ? 1 : 0;
    // many tokens: four units a wave (see the kernel); few: one, so that a decode step has waves enough
    const int hpw = n_tokens >= kPortionTokens ? 4 : 1;
    const int lanes = vec ? (D <= 64 ? 16 : (D <= 128 ? 32 : 64)) : 64;  // lanes a head
    const int per_block = (kThreads / 64) * hpw * (64 / lanes);
    const int head_blocks = (heads + kv_heads + per_block - 1) / per_block;
    // behind the heads: a unit a kv head's values, then one for the gates (with the values written elsewhere and
    // gates to make, the values' waves leave at once)
    const int tail_units = gate ? kv_heads + 1 : (values_elsewhere || !k_pool ? 0 : kv_heads);
    const int tail_blocks = (tail_units + kThreads / 64 - 1) / (kThreads / 64);
    const dim3 grid(static_cast<unsigned>(n_tokens), static_cast<unsigned>(head_blocks + tail_blocks));
#define FSIE_PREP_H(T, V, H)                                                                                             \
    attention_prep_kernel<T, V, H><<<grid, kThreads, 0, stream>>>(                                                       \
        static_cast<const T*>(proj), stride, q_off, k_off, v_off, g_off, heads, kv_heads, dim, vdim, D, q_weight, k_weight, \
        eps, pairs, reinterpret_cast<const float2*>(cos_sin), static_cast<const T*>(v_other), v_other_stride, mix,       \
        static_cast<T*>(q_out), gate, slots, static_cast<T*>(k_pool), static_cast<T*>(v_pool), page_size, pool_slots,   \
        values_elsewhere, lanes, head_blocks, q_weight_stride, v_unit_norm, v_eps)
#define FSIE_PREP_V(T, V) \
    if (hpw == 4) FSIE_PREP_H(T, V, 4); else FSIE_PREP_H(T, V, 1)
#define FSIE_PREP(T) \
    if (vec) { FSIE_PREP_V(T, true); } else { FSIE_PREP_V(T, false); }
    if (dtype == FSIE_F32) { FSIE_PREP(float) } else { FSIE_PREP(bf16_t) }
#undef FSIE_PREP
#undef FSIE_PREP_V
#undef FSIE_PREP_H
    FSIE_CHECK_LAUNCH("attention_prep");
    if (values_elsewhere) {
        const dim3 vgrid(static_cast<unsigned>((n_tokens + 7) / 8), static_cast<unsigned>(kv_heads));
        attention_prep_values_kernel<<<vgrid, D <= 64 ? 64 : (D <= 128 ? 128 : kThreads), 0, stream>>>(
            static_cast<const bf16_t*>(proj), stride, v_off, kv_heads, vdim, D, static_cast<const bf16_t*>(v_other),
            v_other_stride, mix, slots, static_cast<bf16_t*>(v_pool), page_size, pool_slots, n_tokens);
        FSIE_CHECK_LAUNCH("attention_prep_values");
    }
    return 0;
}

// y[t][h][0 .. vdim) = x[t][h][0 .. vdim) * gate[t][h] (gate null: 1) * y_scale, x's heads D values apart, y's rows y_stride
extern "C" int fsie_gate_heads(const void* x, int D, const float* gate, void* y, int n_tokens, int heads, int vdim, int dtype,
                               int64_t y_stride, float y_scale, hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && heads > 0 && vdim > 0 && D >= vdim && y_stride >= static_cast<int64_t>(heads) * vdim,
                 "gate_heads: bad sizes");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "gate_heads: unknown dtype %d", dtype);
    const int64_t total = static_cast<int64_t>(n_tokens) * heads * vdim;
    if (total == 0) return 0;
    const bool vec = vdim % 4 == 0 && D % 4 == 0 && y_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    const unsigned grid = static_cast<unsigned>(ceil_div64(vec ? total / 4 : total, kThreads));
#define FSIE_GATE(T, V) \
    gate_heads_kernel<T, V><<<grid, kThreads, 0, stream>>>(static_cast<const T*>(x), D, gate, static_cast<T*>(y), heads, vdim, total, \
                                                   y_stride, y_scale)
    if (dtype == FSIE_F32) {
        if (vec) FSIE_GATE(float, true); else FSIE_GATE(float, false);
    } else {
        if (vec) FSIE_GATE(bf16_t, true); else FSIE_GATE(bf16_t, false);
    }
#undef FSIE_GATE
    FSIE_CHECK_LAUNCH("gate_heads");
    return 0;
}
