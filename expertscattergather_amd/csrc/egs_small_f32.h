// Gather-GEMM for small experts in fp32: Y[b,e,k,:] = X[b, Ind[b,e,k], :] . W(e), reduction length 32/64/128, 16..64
// output columns (the reference's default shape in its own precision: B64 T256 E32 K32 I128 J64 fp32).
//
// The fp32 matrix instruction (16x16x4) is the roof here (AI 40 FLOP/B against a ridge of 20), so the kernel is
// arranged to keep it fed: W(e) - 32 KB at the default shape, too much for registers next to 64 picks - is brought
// into LDS once per workgroup in [column][reduction] order, so that a lane's four reduction-consecutive weights are
// one 16-byte LDS read shared by the row tiles of its wavefront; the gathered rows go global -> registers ->
// operand order (coalesced 64-byte runs per row, then the 4 x 16 lane transposition) a few 16-deep slabs ahead of
// the MFMAs.  One wavefront = 32 (or 64) picks of one expert, a workgroup 256; one barrier (W(e) in place).
//
// Replaces the reference's expert_gather_kernel (egs/triton_kernels.py:49-143) on these shapes.
#pragma once
#include "egs_small.h"

namespace egs {

__host__ __device__ constexpr size_t rows_small_f32_lds(int R, int N) { return (size_t)N * (R + 4) * 4; }

// Requirements (checked by the launcher): fp32, R == 16 * KS in {32, 64, 128}, N == 16 * TN <= 64, rows of A, W and C
// 16-byte aligned, every tensor below 4 GiB.  W is [E,R,N] (W_NMAJOR) or [E,N,R].
// TQ = 16-pick row tiles per wavefront (4, or 2 with twice the wavefronts: a workgroup covers 256 picks either way)
template <bool W_NMAJOR, int KS, int TN, int TQ = 4>
__global__ __launch_bounds__(64 * (16 / TQ)) void rows_small_f32_kernel(SmallRowsParams p)
{
    constexpr int R = 16 * KS, N = 16 * TN, LDW = R + 4;        // LDW: padded so that the 16 lanes of a read spread over the banks
    constexpr int PW = 16 * TQ, NTHREADS = 64 * (256 / PW);     // picks per wavefront, threads per workgroup
    constexpr int PF = KS < 4 ? KS : 4;                                 // slabs of gathered rows in flight
    extern __shared__ __attribute__((aligned(16))) float w_lds[];      // [N][LDW]
    int e, tile;
    int bid = (int)blockIdx.x;
    // routing-table build of a later scatter riding along (csr_blocks = B, or 0): one workgroup per batch element, first in line
    if (bid < p.csr_blocks) {
        csr_count_body(reinterpret_cast<int32_t *>(w_lds), bid, bid, (int)threadIdx.x, NTHREADS, p.Ind, p.ind_dtype, p.T,
                       p.E * p.K, p.seg_off, p.perm, nullptr, nullptr);
        return;
    }
    bid -= p.csr_blocks;
    if (p.rows_share_xcd ? !decode_tile_expert(bid, p.tiles_per_e, p.E, e, tile)
                         : !decode_expert_tile(bid, p.tiles_per_e, p.E, e, tile)) return;       // uniform per workgroup
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int a = lane & 15, g = lane >> 4;
    const int Me = p.B * p.K;
    const int m0 = (tile * (256 / PW) + wave) * PW;
    const bool live_wave = m0 < Me;

    // the index load goes first: the chain index -> row is the long one (lanes beyond the wavefront's picks repeat them
    // and own nothing)
    const int m_lane = m0 + lane % PW;
    const int mm_lane = min(m_lane, Me - 1);
    const int b_lane = mm_lane / p.K;
    const int64_t pick = ((int64_t)b_lane * p.E + e) * p.K + (mm_lane - b_lane * p.K);
    uint64_t t_word = 0;
    if (live_wave) t_word = load_index_word(p.Ind, p.ind_dtype, pick);

    // W(e) -> registers (all loads in flight behind the index load), LDS as [column][reduction] further down
    const char *We = p.W + (size_t)e * R * N * 4;
    constexpr int W_CHUNKS = R * N / 4, W_IT = (W_CHUNKS + NTHREADS - 1) / NTHREADS;
    u32x4 wv[W_IT];
#pragma unroll
    for (int i = 0; i < W_IT; ++i) {
        const int c = min(tid + i * NTHREADS, W_CHUNKS - 1);
        wv[i] = *reinterpret_cast<const u32x4 *>(We + (size_t)c * 16);      // both layouts are read as they lie
    }

    uint32_t aoff = 0, coff = 0;
    int state = 0;                      // 0: nothing to store, 1: store the product, 2: store zeros (bad index)
    if (live_wave) {
        const int64_t t_raw = decode_index_word(t_word, p.Ind, p.ind_dtype, pick);
        const int32_t t = (t_raw < 0 || t_raw >= (int64_t)p.T) ? -1 : (int32_t)t_raw;
        if (t >= 0) aoff = (uint32_t)(((int64_t)b_lane * p.lda_b + (int64_t)t * p.lda_t) * 4);
        coff = (uint32_t)(pick * N * 4);
        state = (m_lane < Me && lane < PW) ? (t >= 0 ? 1 : 2) : 0;
    }
    // gathered rows: lanes 4r .. 4r+3 fetch the four 16-byte chunks of a 16-deep slab of row 16 tq + r
    uint32_t xo[TQ];
#pragma unroll
    for (int tq = 0; tq < TQ; ++tq) xo[tq] = (uint32_t)__shfl((int)aoff, tq * 16 + (lane >> 2), kWave) + (uint32_t)((lane & 3) * 16);
    u32x4 xr[PF][TQ];
    if (live_wave) {
#pragma unroll
        for (int s = 0; s < PF; ++s)
#pragma unroll
            for (int tq = 0; tq < TQ; ++tq) xr[s][tq] = *reinterpret_cast<const u32x4 *>(p.A + xo[tq] + s * 64);
    }
#pragma unroll
    for (int i = 0; i < W_IT; ++i) {
        const int c = tid + i * NTHREADS;
        if (c < W_CHUNKS) {
            if constexpr (!W_NMAJOR) {      // stored [N][R]: rows copied as they are
                const int n = c / (R / 4), k4 = c - n * (R / 4);
                *reinterpret_cast<u32x4 *>(w_lds + n * LDW + 4 * k4) = wv[i];
            } else {                        // stored [R][N]: four columns of one reduction row per thread, written transposed
                const int r = c / (N / 4), n4 = c - r * (N / 4);
#pragma unroll
                for (int x = 0; x < 4; ++x) w_lds[(4 * n4 + x) * LDW + r] = bits_f32(wv[i][x]);
            }
        }
    }
    __syncthreads();                    // W(e) is in place
    if (!live_wave) return;

    f32x4 acc[TQ][TN];
#pragma unroll
    for (int tq = 0; tq < TQ; ++tq)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) acc[tq][tn] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int s = 0; s < KS; ++s) {
        u32x4 xf[TQ];
#pragma unroll
        for (int tq = 0; tq < TQ; ++tq) xf[tq] = lanes_4a_g_to_16g_a(xr[s % PF][tq], lane);
        if (s + PF < KS) {
#pragma unroll
            for (int tq = 0; tq < TQ; ++tq) xr[s % PF][tq] = *reinterpret_cast<const u32x4 *>(p.A + xo[tq] + (s + PF) * 64);
        }
        // lane (a, g): weights of column 16 tn + a at reduction 16 s + 4 g .. + 3
        u32x4 wf[TN];
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) wf[tn] = *reinterpret_cast<const u32x4 *>(w_lds + (tn * 16 + a) * LDW + s * 16 + g * 4);
        // the four reduction elements of a lane outermost: consecutive matrix instructions then go to different
        // accumulators and none waits for the one before it
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int tq = 0; tq < TQ; ++tq)
                    acc[tq][tn] = __builtin_amdgcn_mfma_f32_16x16x4f32(bits_f32(wf[tn][c]), bits_f32(xf[tq][c]), acc[tq][tn], 0, 0, 0);
    }

    // lane (a, g) holds, for pick 16 tq + a, columns 16 tn + 4 g .. + 3: the four lanes g of a pick write 64 contiguous bytes
#pragma unroll
    for (int tq = 0; tq < TQ; ++tq) {
        const int st = __shfl(state, tq * 16 + a, kWave);
        const uint32_t co = (uint32_t)__shfl((int)coff, tq * 16 + a, kWave);
        if (st == 0) continue;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const f32x4 v = st == 2 ? f32x4{0.f, 0.f, 0.f, 0.f} : acc[tq][tn];
            *reinterpret_cast<f32x4 *>(p.C + co + (tn * 16 + g * 4) * 4) = v;
        }
    }
}

}  // namespace egs
