// Helpers around the GEMM-scatter: the inverse routing table (which picks land on which
// token, in a fixed order), the fixed-order row reduction of the deterministic mode, and
// the zero-fill / down-convert passes of the atomic mode.
#pragma once
#include "egs_device.h"

namespace egs {

constexpr int kCsrLdsTokens = 16384;     // token counters kept in LDS up to this T (64 KB)

// token counters live in LDS or, for very long sequences, in global memory; agent-scope
// relaxed atomics keep one lane's update visible to the other lanes' later reads either way
__device__ __forceinline__ int32_t cnt_load(int32_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void cnt_store(int32_t *p, int32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane)
{
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        int o = __shfl_up(v, d, kWave);
        if (lane >= d) v += o;
    }
    return v;
}

// One wavefront per batch builds, for its [E*K] picks, a stable counting sort by token:
//   seg_off[b][t] .. seg_off[b][t+1]  = positions in perm[b] of the picks that selected t
//   perm[b][pos]                      = pick number q = e*K + k, increasing inside a segment
// Stability (picks of one token stay in increasing q) is what fixes the summation order of
// the deterministic scatter.  Ranks inside a 64-pick chunk come from ballots over the bits of
// the token id, not from atomics, so the result does not depend on hardware ordering.
__global__ __launch_bounds__(kWave) void csr_build_kernel(const void *Ind, int32_t ind_dtype, int32_t T, int32_t N,
                                                          int32_t *seg_off, int32_t *perm, int32_t *cnt_global)
{
    extern __shared__ int32_t cnt_lds[];
    const int lane = (int)threadIdx.x, b = (int)blockIdx.x;
    int32_t *cnt = (T <= kCsrLdsTokens) ? cnt_lds : cnt_global + (size_t)b * T;
    const int64_t base_pick = (int64_t)b * N;

    for (int t = lane; t < T; t += kWave) cnt_store(&cnt[t], 0);
    __syncthreads();
    for (int q0 = 0; q0 < N; q0 += kWave) {
        int q = q0 + lane;
        int32_t t = q < N ? load_token(Ind, ind_dtype, base_pick + q, T) : -1;
        if (t >= 0) atomicAdd(&cnt[t], 1);          // integer counts: order does not matter
    }
    __syncthreads();
    int running = 0;
    for (int t0 = 0; t0 < T; t0 += kWave) {
        int t = t0 + lane;
        int c = t < T ? cnt_load(&cnt[t]) : 0;
        int incl = wave_inclusive_scan(c, lane);
        int excl = running + incl - c;
        if (t < T) {
            seg_off[(size_t)b * (T + 1) + t] = excl;
            cnt_store(&cnt[t], excl);               // becomes the write cursor of token t
        }
        running += __shfl(incl, kWave - 1, kWave);
    }
    if (lane == 0) seg_off[(size_t)b * (T + 1) + T] = running;
    __syncthreads();

    const int nbits = T > 1 ? 32 - __clz(T - 1) : 0;
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    for (int q0 = 0; q0 < N; q0 += kWave) {
        int q = q0 + lane;
        int32_t t = q < N ? load_token(Ind, ind_dtype, base_pick + q, T) : -1;
        uint64_t same = __ballot(t >= 0);
        for (int bit = 0; bit < nbits; ++bit) {
            bool one = (t >> bit) & 1;
            uint64_t bal = __ballot(one);
            same &= one ? bal : ~bal;
        }
        if (t >= 0) {
            int rank = __popcll(same & lt_mask);
            int group = __popcll(same);
            int start = cnt_load(&cnt[t]);
            perm[base_pick + start + rank] = q;
            if (rank == group - 1) cnt_store(&cnt[t], start + group);
        }
        __syncthreads();                             // cursor update visible to the next chunk
    }
}

// out[b,t,:] = sum over the picks of token t, in perm order, of the fp32 rows P[b, pick, :];
// every row of out is written exactly once (tokens nobody picked become zero).
template <class TT, int VW>
__global__ __launch_bounds__(kThreads) void segment_sum_kernel(const float *P, const int32_t *seg_off,
                                                               const int32_t *perm, char *out, int32_t B, int32_t T,
                                                               int32_t N, int32_t I)
{
    const int IV = (I + VW - 1) / VW;
    const size_t items = (size_t)B * T * IV;
    for (size_t item = (size_t)blockIdx.x * kThreads + threadIdx.x; item < items;
         item += (size_t)gridDim.x * kThreads) {
        size_t row = item / IV;
        int iv = (int)(item - row * IV);
        int b = (int)(row / T), t = (int)(row - (size_t)b * T);
        int s0 = seg_off[(size_t)b * (T + 1) + t], s1 = seg_off[(size_t)b * (T + 1) + t + 1];
        float acc[VW];
#pragma unroll
        for (int x = 0; x < VW; ++x) acc[x] = 0.f;
        for (int s = s0; s < s1; ++s) {
            int q = perm[(size_t)b * N + s];
            const float *src = P + ((size_t)b * N + q) * I + (size_t)iv * VW;
            if constexpr (VW == 4) {
                f32x4 v = *reinterpret_cast<const f32x4 *>(src);
#pragma unroll
                for (int x = 0; x < 4; ++x) acc[x] += v[x];
            } else {
                acc[0] += src[0];
            }
        }
        size_t at = row * I + (size_t)iv * VW;
        if constexpr (TT::ES == 4) {
            float *dst = reinterpret_cast<float *>(out) + at;
            if constexpr (VW == 4) *reinterpret_cast<f32x4 *>(dst) = f32x4{acc[0], acc[1], acc[2], acc[3]};
            else dst[0] = acc[0];
        } else {
            uint16_t *dst = reinterpret_cast<uint16_t *>(out) + at;
            if constexpr (VW == 4) {
                u32x2 w;
                w[0] = f32_to_elem_bits<TT>(acc[0]) | (f32_to_elem_bits<TT>(acc[1]) << 16);
                w[1] = f32_to_elem_bits<TT>(acc[2]) | (f32_to_elem_bits<TT>(acc[3]) << 16);
                *reinterpret_cast<u32x2 *>(dst) = w;
            } else {
                dst[0] = (uint16_t)f32_to_elem_bits<TT>(acc[0]);
            }
        }
    }
}

// zero n floats (the atomic mode's accumulator).  A kernel rather than a memset so that the
// call sequence can be captured into a graph.  `vec` = dst is 16-byte aligned.
__global__ __launch_bounds__(kThreads) void fill_zero_f32_kernel(float *dst, size_t n, int vec)
{
    const size_t n4 = vec ? n / 4 : 0;
    const size_t gid = (size_t)blockIdx.x * kThreads + threadIdx.x, stride = (size_t)gridDim.x * kThreads;
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    for (size_t i = gid; i < n4; i += stride) reinterpret_cast<f32x4 *>(dst)[i] = z;
    for (size_t i = n4 * 4 + gid; i < n; i += stride) dst[i] = 0.f;
}

// fp32 accumulator -> 16-bit output element type, n elements.  `vec` = dst is 8-byte aligned
// (src is a 256-byte aligned workspace).
template <class TT>
__global__ __launch_bounds__(kThreads) void downconvert_kernel(const float *src, uint16_t *dst, size_t n, int vec)
{
    const size_t n4 = vec ? n / 4 : 0;
    const size_t gid = (size_t)blockIdx.x * kThreads + threadIdx.x, stride = (size_t)gridDim.x * kThreads;
    for (size_t i = gid; i < n4; i += stride) {
        f32x4 v = reinterpret_cast<const f32x4 *>(src)[i];
        u32x2 w;
        w[0] = f32_to_elem_bits<TT>(v[0]) | (f32_to_elem_bits<TT>(v[1]) << 16);
        w[1] = f32_to_elem_bits<TT>(v[2]) | (f32_to_elem_bits<TT>(v[3]) << 16);
        reinterpret_cast<u32x2 *>(dst)[i] = w;
    }
    for (size_t i = n4 * 4 + gid; i < n; i += stride) dst[i] = (uint16_t)f32_to_elem_bits<TT>(src[i]);
}

__global__ __launch_bounds__(kThreads) void validate_indices_kernel(const void *Ind, int32_t ind_dtype, int64_t n,
                                                                    int32_t T, int32_t *bad)
{
    int local = 0;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
        int64_t t = load_index_raw(Ind, ind_dtype, i);
        local += (t < 0 || t >= (int64_t)T) ? 1 : 0;
    }
    if (local) atomicAdd(bad, local);
}

}  // namespace egs
