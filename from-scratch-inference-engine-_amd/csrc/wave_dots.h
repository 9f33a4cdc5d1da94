// Dot products of one row x with a few rows of a matrix, a wave at work: float32 sums from operands of any type.
#pragma once

#include "common.h"

namespace {

constexpr int kWaveDots = 8;  // rows of the matrix a pass

// z[i] = x . w[min(r0 + i, n_rows - 1)] for i < kWaveDots, the same in every lane.  A lane takes 16 bytes of x and of
// every row per round (all of a round's loads are asked for before any is used), sums its share in the order of the
// rounds, and the lanes' shares meet in the wave's fixed order.  Rows that are not a whole number of 16 bytes, or
// not aligned (vec false), are read value by value, with the same sums a lane.
template <typename T>
__device__ __forceinline__ void wave_dots(const T* __restrict__ x, const T* __restrict__ w, int hidden, int r0, int n_rows,
                                          bool vec, int lane, float* z) {
    constexpr int V = 16 / sizeof(T);
#pragma unroll
    for (int i = 0; i < kWaveDots; ++i) z[i] = 0.f;
    for (int j = lane * V; j < hidden; j += 64 * V) {
        union { uint4 raw; T v[V]; } xv, wv[kWaveDots];
        if (vec) {
            xv.raw = *reinterpret_cast<const uint4*>(x + j);
#pragma unroll
            for (int i = 0; i < kWaveDots; ++i) {
                const int r = min(r0 + i, n_rows - 1);  // (past the last: the last once more, for the caller to drop)
                wv[i].raw = *reinterpret_cast<const uint4*>(w + static_cast<int64_t>(r) * hidden + j);
            }
        } else {
#pragma unroll
            for (int u = 0; u < V; ++u) xv.v[u] = j + u < hidden ? x[j + u] : from_float<T>(0.f);
#pragma unroll
            for (int i = 0; i < kWaveDots; ++i) {
                const int r = min(r0 + i, n_rows - 1);
#pragma unroll
                for (int u = 0; u < V; ++u) wv[i].v[u] = j + u < hidden ? w[static_cast<int64_t>(r) * hidden + j + u] : from_float<T>(0.f);
            }
        }
#pragma unroll
        for (int i = 0; i < kWaveDots; ++i)
#pragma unroll
            for (int u = 0; u < V; ++u) z[i] = fmaf(to_float(xv.v[u]), to_float(wv[i].v[u]), z[i]);
    }
#pragma unroll
    for (int i = 0; i < kWaveDots; ++i) z[i] = wave_sum(z[i]);
}

template <typename T>
__device__ __forceinline__ bool wave_dots_vec(const T* x, const T* w, int hidden) {
    return hidden % (16 / static_cast<int>(sizeof(T))) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
           (reinterpret_cast<uintptr_t>(w) & 15) == 0;
}

}  // namespace
