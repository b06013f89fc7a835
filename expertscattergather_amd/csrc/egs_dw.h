// Weight gradient of one expert as a split reduction over its picks:
//
//   dW(e, i, j) = sum_{m in split s} Xs[b, Ind[m], i] * Ys[m, j]
//
// Both operands arrive "reduction-strided" (the reduction index m selects a row, the output
// index runs along the row), so each thread fetches VEC x VEC blocks, transposes them in
// registers and stores reduction-contiguous 16-byte chunks into the swizzled LDS tiles that
// feed the MFMAs.  Row addresses of the next slabs are decoded from Ind one slab ahead.
// Each workgroup owns a BI x BJ tile of dW(e) for one split of the picks; splits are summed
// afterwards in a fixed order (dw_reduce_kernel), so the result is bitwise reproducible.
//
// Replaces the reference's expert_gather_scatter_dW_kernel (egs/triton_kernels.py:261-356),
// which reduces over the batch for one (e,k) and then accumulates K ways with atomics.
#pragma once
#include "egs_device.h"

namespace egs {

struct DwParams {
    const char *Xs;         // [B,T,I] strided source (gathered through Ind)
    const char *Ys;         // [B,E,K,J] dense
    const void *Ind;
    float *part;            // [S,E,I,J] fp32 partial sums (S > 1)
    char *dW;               // final output when S == 1
    int32_t B, T, E, K, I, J;
    int64_t ldx_b, ldx_t;
    int32_t ind_dtype;
    int32_t x_vec, y_vec, o_vec;
    int32_t i_tiles, j_tiles;
    int32_t S, rows_per_split;     // rows_per_split is a multiple of the slab depth
    int32_t out_dtype, dw_layout;  // used when S == 1
};

template <class TT, int BI, int BJ, int BK>
__global__ __launch_bounds__(kThreads) void dw_kernel(DwParams p)
{
    constexpr int ES = TT::ES, VEC = TT::VEC;
    constexpr int CH = BK / VEC, KSTEPS = CH / 4;
    constexpr int TI = BI / 4 / 16, TJ = BJ / 16;          // 4 waves along i, each BI/4 x BJ
    constexpr int KB = BK / VEC;
    constexpr int NBX = KB * (BI / VEC), NBY = KB * (BJ / VEC);
    constexpr int NLX = (NBX + kThreads - 1) / kThreads, NLY = (NBY + kThreads - 1) / kThreads;
    static_assert(BK <= kThreads, "slab row decode uses one thread per row");

    __shared__ __attribute__((aligned(16))) char smem_i[BI * BK * ES];
    __shared__ __attribute__((aligned(16))) char smem_j[BJ * BK * ES];
    __shared__ int64_t x_off[2][BK];
    __shared__ int64_t y_off[2][BK];

    int e, tile;
    const int tiles_per_e = p.i_tiles * p.j_tiles * p.S;
    if (!decode_expert_tile((int)blockIdx.x, tiles_per_e, p.E, e, tile)) return;
    const int s = tile / (p.i_tiles * p.j_tiles);
    const int ij = tile - s * (p.i_tiles * p.j_tiles);
    const int it = ij / p.j_tiles, jt = ij - it * p.j_tiles;
    const int i0 = it * BI, j0 = jt * BJ;
    const int tid = (int)threadIdx.x;
    const int Me = p.B * p.K;
    const int row_begin = s * p.rows_per_split;
    const int row_end = min(Me, row_begin + p.rows_per_split);
    const int nslab = row_end > row_begin ? (row_end - row_begin + BK - 1) / BK : 0;
    const bool x_vec = p.x_vec != 0, y_vec = p.y_vec != 0;

    auto stage_rows = [&](int slab, int buf) {
        if (tid < BK) {
            int m = row_begin + slab * BK + tid;
            int64_t xo = -1, yo = -1;
            if (m < row_end) {
                int b = m / p.K, k = m - b * p.K;
                int64_t pick = ((int64_t)b * p.E + e) * p.K + k;
                int32_t t = load_token(p.Ind, p.ind_dtype, pick, p.T);
                if (t >= 0) {
                    xo = (int64_t)b * p.ldx_b + (int64_t)t * p.ldx_t;
                    yo = pick * p.J;
                }
            }
            x_off[buf][tid] = xo;
            y_off[buf][tid] = yo;
        }
    };

    u32x4 xreg[NLX * VEC], yreg[NLY * VEC];
    auto issue = [&](int buf) {
#pragma unroll
        for (int n = 0; n < NLX; ++n) {
            int blk = tid + n * kThreads;
            int kb = blk / (BI / VEC), cb = blk % (BI / VEC);
#pragma unroll
            for (int r = 0; r < VEC; ++r) {
                int64_t xo = (blk < NBX) ? x_off[buf][kb * VEC + r] : -1;
                const char *ptr = xo < 0 ? nullptr : p.Xs + xo * ES;
                xreg[n * VEC + r] = load_chunk<ES>(ptr, i0 + cb * VEC, p.I, x_vec);
            }
        }
#pragma unroll
        for (int n = 0; n < NLY; ++n) {
            int blk = (kThreads - 1 - tid) + n * kThreads;     // idle threads of the X side go first
            int kb = blk / (BJ / VEC), cb = blk % (BJ / VEC);
#pragma unroll
            for (int r = 0; r < VEC; ++r) {
                int64_t yo = (blk < NBY) ? y_off[buf][kb * VEC + r] : -1;
                const char *ptr = yo < 0 ? nullptr : p.Ys + yo * ES;
                yreg[n * VEC + r] = load_chunk<ES>(ptr, j0 + cb * VEC, p.J, y_vec);
            }
        }
    };
    auto commit = [&]() {
        u32x4 *tile_i = reinterpret_cast<u32x4 *>(smem_i);
        u32x4 *tile_j = reinterpret_cast<u32x4 *>(smem_j);
#pragma unroll
        for (int n = 0; n < NLX; ++n) {
            int blk = tid + n * kThreads;
            int kb = blk / (BI / VEC), cb = blk % (BI / VEC);
            if (blk < NBX) {
                u32x4 in[VEC], out[VEC];
#pragma unroll
                for (int r = 0; r < VEC; ++r) in[r] = xreg[n * VEC + r];
                if constexpr (VEC == 8) transpose8x8_16b(in, out); else transpose4x4_32b(in, out);
#pragma unroll
                for (int c = 0; c < VEC; ++c) tile_i[tile_chunk_index<CH>(cb * VEC + c, kb)] = out[c];
            }
        }
#pragma unroll
        for (int n = 0; n < NLY; ++n) {
            int blk = (kThreads - 1 - tid) + n * kThreads;
            int kb = blk / (BJ / VEC), cb = blk % (BJ / VEC);
            if (blk < NBY) {
                u32x4 in[VEC], out[VEC];
#pragma unroll
                for (int r = 0; r < VEC; ++r) in[r] = yreg[n * VEC + r];
                if constexpr (VEC == 8) transpose8x8_16b(in, out); else transpose4x4_32b(in, out);
#pragma unroll
                for (int c = 0; c < VEC; ++c) tile_j[tile_chunk_index<CH>(cb * VEC + c, kb)] = out[c];
            }
        }
    };

    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);    // uniform: what derives from it is scalar work
    const int a = lane & 15, g = lane >> 4;
    const int wave_i0 = wave * (BI / 4);
    f32x4 acc[TI][TJ];
#pragma unroll
    for (int x = 0; x < TI; ++x)
#pragma unroll
        for (int y = 0; y < TJ; ++y) acc[x][y] = f32x4{0.f, 0.f, 0.f, 0.f};
    int irow_l[TI], jrow_l[TJ];
#pragma unroll
    for (int x = 0; x < TI; ++x) irow_l[x] = wave_i0 + x * 16 + a;
#pragma unroll
    for (int y = 0; y < TJ; ++y) jrow_l[y] = (a >> 2) * (4 * TJ) + y * 4 + (a & 3);   // relabelled: 4*TJ consecutive j per lane

    if (nslab > 0) {
        stage_rows(0, 0);
        __syncthreads();
        issue(0);
        if (nslab > 1) stage_rows(1, 1);
    }
    for (int sl = 0; sl < nslab; ++sl) {
        commit();
        __syncthreads();                                  // tiles of slab sl and row offsets of slab sl+1 visible
        if (sl + 1 < nslab) issue((sl + 1) & 1);
        if (sl + 2 < nslab) stage_rows(sl + 2, sl & 1);   // buffer sl&1 was last read before the barrier above
        const u32x4 *tile_i = reinterpret_cast<const u32x4 *>(smem_i);
        const u32x4 *tile_j = reinterpret_cast<const u32x4 *>(smem_j);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            u32x4 fi[TI], fj[TJ];
#pragma unroll
            for (int x = 0; x < TI; ++x) fi[x] = tile_i[tile_chunk_index<CH>(irow_l[x], ks * 4 + g)];
#pragma unroll
            for (int y = 0; y < TJ; ++y) fj[y] = tile_j[tile_chunk_index<CH>(jrow_l[y], ks * 4 + g)];
#pragma unroll
            for (int x = 0; x < TI; ++x)
#pragma unroll
                for (int y = 0; y < TJ; ++y) mma_chunk<TT>(acc[x][y], fj[y], fi[x]);
        }
        __syncthreads();
    }

    // ---------------- epilogue: lane holds, for row i, the 4*TJ consecutive columns j0 + g*4*TJ ...
    const bool direct = (p.S == 1);
    const bool o_vec = p.o_vec != 0;
#pragma unroll
    for (int x = 0; x < TI; ++x) {
        int i = i0 + wave_i0 + x * 16 + a;
        if (i >= p.I) continue;
#pragma unroll
        for (int y = 0; y < TJ; ++y) {
            int j = j0 + g * (4 * TJ) + y * 4;
            if (j >= p.J) continue;
            f32x4 v = acc[x][y];
            if (!direct) {
                float *dst = p.part + (((size_t)s * p.E + e) * p.I + i) * p.J + j;
                if ((p.J & 3) == 0) {
                    *reinterpret_cast<f32x4 *>(dst) = v;     // workspace base is 256-byte aligned
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) if (j + r < p.J) dst[r] = v[r];
                }
            } else if (p.dw_layout == 0) {                  // [E,I,J]
                size_t at = ((size_t)e * p.I + i) * p.J + j;
                if (p.out_dtype == 0) {
                    float *dst = reinterpret_cast<float *>(p.dW) + at;
                    if (o_vec && j + 4 <= p.J) *reinterpret_cast<f32x4 *>(dst) = v;
                    else {
#pragma unroll
                        for (int r = 0; r < 4; ++r) if (j + r < p.J) dst[r] = v[r];
                    }
                } else {
                    uint16_t *dst = reinterpret_cast<uint16_t *>(p.dW) + at;
                    uint32_t h[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) h[r] = p.out_dtype == 1 ? f32_to_f16_bits(v[r]) : f32_to_bf16_bits(v[r]);
                    if (o_vec && j + 4 <= p.J) {
                        u32x2 w; w[0] = h[0] | (h[1] << 16); w[1] = h[2] | (h[3] << 16);
                        *reinterpret_cast<u32x2 *>(dst) = w;
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r) if (j + r < p.J) dst[r] = (uint16_t)h[r];
                    }
                }
            } else {                                        // [E,J,I]: i is the contiguous axis
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (j + r >= p.J) continue;
                    size_t at = ((size_t)e * p.J + (j + r)) * p.I + i;
                    if (p.out_dtype == 0) reinterpret_cast<float *>(p.dW)[at] = v[r];
                    else reinterpret_cast<uint16_t *>(p.dW)[at] =
                        (uint16_t)(p.out_dtype == 1 ? f32_to_f16_bits(v[r]) : f32_to_bf16_bits(v[r]));
                }
            }
        }
    }
}

// dW(e,i,j) = sum_s part[s][e][i][j] in increasing s, rounded once to the output type and
// written in the requested layout.
static __global__ __launch_bounds__(kThreads) void dw_reduce_kernel(const float *part, char *dW, int32_t S, int32_t E,
                                                             int32_t I, int32_t J, int32_t out_dtype, int32_t dw_layout)
{
    const size_t total = (size_t)E * I * J;
    for (size_t o = (size_t)blockIdx.x * kThreads + threadIdx.x; o < total; o += (size_t)gridDim.x * kThreads) {
        size_t src = o;
        if (dw_layout != 0) {       // o = (e*J + j)*I + i  ->  src = (e*I + i)*J + j
            size_t i = o % I, ej = o / I;
            size_t j = ej % J, e = ej / J;
            src = (e * I + i) * J + j;
        }
        float sum = 0.f;
        for (int s = 0; s < S; ++s) sum += part[(size_t)s * total + src];
        if (out_dtype == 0) reinterpret_cast<float *>(dW)[o] = sum;
        else reinterpret_cast<uint16_t *>(dW)[o] = (uint16_t)(out_dtype == 1 ? f32_to_f16_bits(sum) : f32_to_bf16_bits(sum));
    }
}

}  // namespace egs
