// Norms and activations beyond the plain pre-norm layer: the norm of a sublayer's output fused with
// the residual sum and the next norm (a layer with a norm before and after every sublayer), the norm
// of every head of a mixer's output fused with its gate, and the soft cap of the logits.
// All arithmetic is float32; T is the type of activations (float or bfloat16).
#include "common.h"
#include "api.h"

namespace {

constexpr int kThreads = 256;

// One block per output row r; source row = rows ? rows[r] : r.
//   y = delta[row]                          (one array of T, or the sum in order of n_parts float32 arrays)
//   d = y * rsqrt(mean(y^2) + post_eps) * post_weight
//   v = residual[row] + d;                  if write_back: residual[row] = v
//   out[r] = v * rsqrt(mean(v^2) + eps) * weight
// The row is kept in LDS between the passes (hidden floats).
template <typename T>
__global__ __launch_bounds__(kThreads) void sandwich_norm_kernel(
    float* __restrict__ residual, const T* __restrict__ delta, const float* __restrict__ post_weight, float post_eps,
    const float* __restrict__ weight, float eps, T* __restrict__ out, const int32_t* __restrict__ rows, int hidden,
    int write_back, int n_parts, int64_t part_stride) {
    extern __shared__ float row_buf[];
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int64_t row = rows ? rows[r] : r;
    float* res = residual + row * hidden;
    const T* del = n_parts ? nullptr : delta + row * hidden;
    const float* parts = n_parts ? reinterpret_cast<const float*>(delta) + row * hidden : nullptr;
    float sum_sq = 0.f;
    for (int j = threadIdx.x; j < hidden; j += kThreads) {
        float y;
        if (del) {
            y = to_float(del[j]);
        } else {
            y = 0.f;
            for (int s = 0; s < n_parts; ++s) y += parts[s * part_stride + j];
        }
        row_buf[j] = y;
        sum_sq += y * y;
    }
    const float post_scale = 1.0f / sqrtf(block_sum(sum_sq, scratch) / static_cast<float>(hidden) + post_eps);
    sum_sq = 0.f;
    for (int j = threadIdx.x; j < hidden; j += kThreads) {
        const float v = res[j] + (row_buf[j] * post_scale) * post_weight[j];
        row_buf[j] = v;
        if (write_back) res[j] = v;
        sum_sq += v * v;
    }
    const float scale = 1.0f / sqrtf(block_sum(sum_sq, scratch) / static_cast<float>(hidden) + eps);
    T* dst = out + static_cast<int64_t>(r) * hidden;
    for (int j = threadIdx.x; j < hidden; j += kThreads)
        dst[j] = from_float<T>(weight ? (row_buf[j] * scale) * weight[j] : row_buf[j]);  // (no weight: the stream itself)
}

// Four consecutive elements: one 16-byte (float32) or 8-byte (bfloat16) access.
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    return float4{__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16),
                  __uint_as_float(w.y & 0xffff0000u)};
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, float4 v) {
    uint2 w;
    w.x = pack2_bf16(v.x, v.y);
    w.y = pack2_bf16(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = w;
}

// The same for hidden % 4 == 0 and hidden <= 4 * THREADS * ITERS: a thread keeps its quads of the row in
// registers, and every load of the row (stream, delta or partial sums, both weights) goes out before
// anything waits.  Places past the end read the last quad again and are masked out of sums and stores.
template <typename T, int ITERS, int THREADS>
__global__ __launch_bounds__(THREADS) void sandwich_norm_vec_kernel(
    float* __restrict__ residual, const T* __restrict__ delta, const float* __restrict__ post_weight, float post_eps,
    const float* __restrict__ weight, float eps, T* __restrict__ out, const int32_t* __restrict__ rows, int hidden,
    int write_back, int n_parts, int64_t part_stride) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int64_t row = rows ? rows[r] : r;
    float* res = residual + row * hidden;
    const T* del = n_parts ? nullptr : delta + row * hidden;
    const float* parts = n_parts ? reinterpret_cast<const float*>(delta) + row * hidden : nullptr;
    float4 y[ITERS], v[ITERS], wp[ITERS], w[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = min((it * THREADS + static_cast<int>(threadIdx.x)) * 4, hidden - 4);
        v[it] = load4(res + j);
        wp[it] = load4(post_weight + j);
        w[it] = weight ? load4(weight + j) : float4{1.f, 1.f, 1.f, 1.f};
        if (del) {
            y[it] = load4(del + j);
        } else {
            float4 a = load4(parts + j);
#pragma unroll 4
            for (int s = 1; s < n_parts; ++s) {
                const float4 p = load4(parts + s * part_stride + j);
                a.x += p.x, a.y += p.y, a.z += p.z, a.w += p.w;
            }
            y[it] = a;
        }
    }
    float sum_sq = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        if ((it * THREADS + static_cast<int>(threadIdx.x)) * 4 < hidden)
            sum_sq += y[it].x * y[it].x + y[it].y * y[it].y + y[it].z * y[it].z + y[it].w * y[it].w;
    }
    const float post_scale = 1.0f / sqrtf(block_sum(sum_sq, scratch) / static_cast<float>(hidden) + post_eps);
    sum_sq = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = (it * THREADS + static_cast<int>(threadIdx.x)) * 4;
        v[it].x += (y[it].x * post_scale) * wp[it].x;
        v[it].y += (y[it].y * post_scale) * wp[it].y;
        v[it].z += (y[it].z * post_scale) * wp[it].z;
        v[it].w += (y[it].w * post_scale) * wp[it].w;
        if (j < hidden) {
            if (write_back) store4(res + j, v[it]);
            sum_sq += v[it].x * v[it].x + v[it].y * v[it].y + v[it].z * v[it].z + v[it].w * v[it].w;
        }
    }
    // without a weight the stream itself is the result (a layer whose sublayers read the stream as it is)
    const float scale = weight ? 1.0f / sqrtf(block_sum(sum_sq, scratch) / static_cast<float>(hidden) + eps) : 1.f;
    T* dst = out + static_cast<int64_t>(r) * hidden;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = (it * THREADS + static_cast<int>(threadIdx.x)) * 4;
        if (j < hidden)
            store4(dst + j, float4{(v[it].x * scale) * w[it].x, (v[it].y * scale) * w[it].y, (v[it].z * scale) * w[it].z,
                                   (v[it].w * scale) * w[it].w});
    }
}

// One wave per (token, head): o [tokens][heads * width] float32 is normalised over the `width` values of
// the head (plain weight [width], shared by the heads) and multiplied by act(gate) of the same place;
// gate [tokens][gate_stride] of T (the columns of the head start at h * width).
template <typename T>
__global__ __launch_bounds__(kThreads) void gated_headnorm_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                                  int64_t gate_stride, const float* __restrict__ weight,
                                                                  T* __restrict__ out, int64_t n_runs, int heads, int width,
                                                                  float eps, int act, int n_planes, int64_t plane,
                                                                  int64_t out_stride, float out_scale) {
    const int lane = threadIdx.x & (FSIE_WAVE - 1);
    const int64_t run = static_cast<int64_t>(blockIdx.x) * (kThreads / FSIE_WAVE) + threadIdx.x / FSIE_WAVE;
    if (run >= n_runs) return;
    const int64_t t = run / heads;
    const int h = static_cast<int>(run - t * heads);
    const float* src = o + (t * heads + h) * width;
    const T* g = gate + t * gate_stride + static_cast<int64_t>(h) * width;
    T* dst = out + t * out_stride + static_cast<int64_t>(h) * width;  // (rows of out may be columns of wider rows)
    // o comes as n_planes arrays a `plane` apart, added in order (the shares of a state kernel's row splits)
    auto value = [&](int i) {
        float x = src[i];
        for (int p = 1; p < n_planes; ++p) x += src[p * plane + i];
        return x;
    };
    float sum = 0.f;
    for (int i = lane; i < width; i += FSIE_WAVE) {
        const float x = value(i);
        sum += x * x;
    }
    sum = wave_sum(sum);
    const float scale = 1.0f / sqrtf(sum / static_cast<float>(width) + eps);
    for (int i = lane; i < width; i += FSIE_WAVE)
        dst[i] = from_float<T>((((value(i) * scale) * weight[i]) * gate_act(to_float(g[i]), act)) * out_scale);
}

__global__ void softcap_kernel(float* __restrict__ x, int64_t n, float cap, float inv_cap) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) x[i] = cap * tanhf(x[i] * inv_cap);
}

}  // namespace

// The norm of a sublayer's output, the residual sum and the next norm in one pass (see the kernel).
// delta: [total_rows][hidden] of the activations' type, or with n_parts > 0 that many float32 arrays
// [total_rows][hidden] one after the other.  rows (or null): the n_rows source rows to work on.
extern "C" int fsie_sandwich_norm(float* residual, const void* delta, const float* post_weight, float post_eps,
                                  const float* weight, float eps, void* out, const int32_t* rows, int n_rows, int hidden,
                                  int dtype, int write_back, int n_parts, int total_rows, hipStream_t stream) {
    FSIE_REQUIRE(n_rows >= 0 && hidden > 0 && hidden <= 16384, "sandwich_norm: bad sizes rows=%d hidden=%d (at most 16384)",
                 n_rows, hidden);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "sandwich_norm: unknown dtype %d", dtype);
    FSIE_REQUIRE(residual && delta && post_weight && out, "sandwich_norm: missing operand");
    FSIE_REQUIRE(n_parts >= 0 && n_parts <= FSIE_GEMM_MAX_SPLITS, "sandwich_norm: 0 to %d partial sums, got %d",
                 FSIE_GEMM_MAX_SPLITS, n_parts);
    FSIE_REQUIRE(!(write_back && rows), "sandwich_norm: chosen rows are read, not written back");
    if (n_rows == 0) return 0;
    const int64_t part_stride = static_cast<int64_t>(total_rows) * hidden;
    const bool aligned = hidden % 4 == 0 && reinterpret_cast<uintptr_t>(residual) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(delta) % 16 == 0 && reinterpret_cast<uintptr_t>(post_weight) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(weight) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    if (aligned && hidden <= 8192) {
#define FSIE_SANDWICH(T, ITERS, THREADS)                                                                             \
    sandwich_norm_vec_kernel<T, ITERS, THREADS><<<n_rows, THREADS, 0, stream>>>(                                     \
        residual, static_cast<const T*>(delta), post_weight, post_eps, weight, eps, static_cast<T*>(out), rows, hidden, \
        write_back, n_parts, part_stride)
#define FSIE_SANDWICH_BY_SIZE(T)                                                      \
    if (n_rows <= 128 && hidden > 1024) {  /* few rows: more waves a row */           \
        if (hidden <= 4096) FSIE_SANDWICH(T, 1, 1024); else FSIE_SANDWICH(T, 2, 1024); \
    } else if (hidden <= 1024) FSIE_SANDWICH(T, 1, 256);                              \
    else if (hidden <= 2048) FSIE_SANDWICH(T, 2, 256);                                \
    else if (hidden <= 4096) FSIE_SANDWICH(T, 4, 256);                                \
    else FSIE_SANDWICH(T, 8, 256)
        if (dtype == FSIE_F32) {
            FSIE_SANDWICH_BY_SIZE(float);
        } else {
            FSIE_SANDWICH_BY_SIZE(bf16_t);
        }
#undef FSIE_SANDWICH_BY_SIZE
#undef FSIE_SANDWICH
        FSIE_CHECK_LAUNCH("sandwich_norm");
        return 0;
    }
    const size_t lds = sizeof(float) * hidden;
    if (dtype == FSIE_F32) {
        sandwich_norm_kernel<float><<<n_rows, kThreads, lds, stream>>>(residual, static_cast<const float*>(delta), post_weight,
                                                                     post_eps, weight, eps, static_cast<float*>(out), rows,
                                                                     hidden, write_back, n_parts, part_stride);
    } else {
        sandwich_norm_kernel<bf16_t><<<n_rows, kThreads, lds, stream>>>(residual, static_cast<const bf16_t*>(delta), post_weight,
                                                                      post_eps, weight, eps, static_cast<bf16_t*>(out), rows,
                                                                      hidden, write_back, n_parts, part_stride);
    }
    FSIE_CHECK_LAUNCH("sandwich_norm");
    return 0;
}

extern "C" int fsie_gated_headnorm(const float* o, int n_planes, const void* gate, int64_t gate_stride, const float* weight,
                                   void* out, int n_tokens, int heads, int width, float eps, int act, int dtype,
                                   int64_t out_stride, float out_scale, hipStream_t stream) {
    FSIE_REQUIRE(n_planes >= 1, "gated_headnorm: at least one plane of o");
    FSIE_REQUIRE(out_stride >= static_cast<int64_t>(heads) * width, "gated_headnorm: rows of out shorter than the heads");
    const int64_t plane = static_cast<int64_t>(n_tokens) * heads * width;
    FSIE_REQUIRE(n_tokens >= 0 && heads > 0 && width > 0, "gated_headnorm: bad sizes T=%d heads=%d width=%d", n_tokens, heads,
                 width);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "gated_headnorm: unknown dtype %d", dtype);
    FSIE_REQUIRE(FSIE_ACT_KNOWN(act), "gated_headnorm: unknown activation %d", act);
    FSIE_REQUIRE(o && gate && weight && out && gate_stride >= static_cast<int64_t>(heads) * width,
                 "gated_headnorm: missing operand or a gate row shorter than the heads");
    if (n_tokens == 0) return 0;
    const int64_t runs = static_cast<int64_t>(n_tokens) * heads;
    const unsigned grid = static_cast<unsigned>(ceil_div64(runs, kThreads / FSIE_WAVE));
    if (dtype == FSIE_F32) {
        gated_headnorm_kernel<float><<<grid, kThreads, 0, stream>>>(o, static_cast<const float*>(gate), gate_stride, weight,
                                                                  static_cast<float*>(out), runs, heads, width, eps, act, n_planes, plane,
                                                                  out_stride, out_scale);
    } else {
        gated_headnorm_kernel<bf16_t><<<grid, kThreads, 0, stream>>>(o, static_cast<const bf16_t*>(gate), gate_stride, weight,
                                                                   static_cast<bf16_t*>(out), runs, heads, width, eps, act, n_planes, plane,
                                                                   out_stride, out_scale);
    }
    FSIE_CHECK_LAUNCH("gated_headnorm");
    return 0;
}

// x <- cap * tanh(x / cap), in place, float32.
extern "C" int fsie_softcap(float* x, int64_t n, float cap, hipStream_t stream) {
    FSIE_REQUIRE(n >= 0 && cap > 0.f, "softcap: bad arguments n=%lld cap=%f", static_cast<long long>(n), cap);
    if (n == 0) return 0;
    softcap_kernel<<<static_cast<unsigned>(ceil_div64(n, kThreads)), kThreads, 0, stream>>>(x, n, cap, 1.0f / cap);
    FSIE_CHECK_LAUNCH("softcap");
    return 0;
}
