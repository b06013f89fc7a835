// Gather-GEMM for small experts in fp32: Y[b,e,k,:] = X[b, Ind[b,e,k], :] . W(e), reduction length 32/64/128, 16..64
// output columns (the reference's default shape in its own precision: B64 T256 E32 K32 I128 J64 fp32).
//
// The fp32 matrix instruction (16x16x4) is the roof here (AI 40 FLOP/B against a ridge of 20), so the kernel is
// arranged to keep it fed: W(e) - 32 KB at the default shape, too much for registers next to 64 picks - is brought
// into LDS once per workgroup in [column][reduction] order, so that a lane's four reduction-consecutive weights are
// one 16-byte LDS read; the gathered rows go global -> registers -> operand order (coalesced 64-byte runs per row,
// then the 4 x 16 lane transposition).  One wavefront = 32 (or 64) picks of one expert, a workgroup 256; one barrier
// (W(e) in place).  A wavefront multiplies and stores its 16-pick row tiles one after the other, the first tile's rows
// requested before the barrier and the others after it.
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
    extern __shared__ __attribute__((aligned(16))) float w_lds[];      // [N][LDW]
    int e, tile;
    int bid = (int)blockIdx.x;
    // routing-table build of a later scatter riding along (csr_blocks = B, or 0): one workgroup per batch element, first in line
    if (bid < p.csr_blocks) {
        if (p.csr_split)
            csr_count_half_body(reinterpret_cast<int32_t *>(w_lds), bid >> 1, bid & 1, (int)threadIdx.x, NTHREADS, p.Ind,
                                p.ind_dtype, p.T, p.E * p.K, p.seg_off, p.perm);
        else
            csr_count_body(reinterpret_cast<int32_t *>(w_lds), bid, bid, (int)threadIdx.x, NTHREADS, p.Ind, p.ind_dtype, p.T,
                           p.E * p.K, p.seg_off, p.perm, nullptr, nullptr);
        return;
    }
    bid -= p.csr_blocks;
    if (!decode_rows_block(bid, p.rows_share_xcd, p.tiles_per_e, p.E, e, tile)) return;       // uniform per workgroup
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
    // (no branch around any load of the prologue, also where a wavefront has no picks left - its clamped addresses are valid:
    // behind a branch the compiler loses track of the order of the outstanding loads and makes the first matrix instruction
    // wait for all of them, the rows of the last slab included)
    const uint64_t t_word = load_index_word(p.Ind, p.ind_dtype, pick);

    // W(e) -> registers (all loads in flight behind the index load), LDS as [column][reduction] further down
    const char *We = p.W + (size_t)e * R * N * 4;
    constexpr int W_CHUNKS = R * N / 4, W_IT = (W_CHUNKS + NTHREADS - 1) / NTHREADS;
    // Which 16-byte chunk a thread takes.  [N][R] (rows copied as they lie): consecutive threads, consecutive chunks.
    // [R][N] (written to LDS transposed, four single floats per chunk): a wavefront takes 16 reduction rows x 16 columns per
    // load, lanes 4 q .. 4 q + 3 the four chunks of row q's 64 bytes - as many L1 accesses as consecutive chunks make, and
    // the 64 floats of one transposed write (columns 16 apart in steps of 4 lanes, rows q = 0..15) fall on 64 different
    // banks; with consecutive chunks they fell on 16, four lanes deep.
    auto w_chunk = [&](int i) -> int {
        if constexpr (!W_NMAJOR) {
            const int c = tid + i * NTHREADS;
            return c < W_CHUNKS ? c : -1;
        } else {
            const int u = wave + i * (NTHREADS / 64);                       // (16-row block, 16-column group) of this load
            if ((KS * TN) % (NTHREADS / 64) != 0 && u >= KS * TN) return -1;
            const int r = (u / TN) * 16 + (lane >> 2), n4 = (u % TN) * 4 + (lane & 3);
            return r * (N / 4) + n4;
        }
    };
    u32x4 wv[W_IT];
#pragma unroll
    for (int i = 0; i < W_IT; ++i) {
        const int c = w_chunk(i);
        wv[i] = *reinterpret_cast<const u32x4 *>(We + (size_t)max(c, 0) * 16);
    }

    const int64_t t_raw = decode_index_word(t_word, p.Ind, p.ind_dtype, pick);
    const int32_t t = (t_raw < 0 || t_raw >= (int64_t)p.T) ? -1 : (int32_t)t_raw;
    const uint32_t aoff = t >= 0 ? (uint32_t)(((int64_t)b_lane * p.lda_b + (int64_t)t * p.lda_t) * 4) : 0u;
    const uint32_t coff = (uint32_t)(pick * N * 4);
    const int state = (m_lane < Me && lane < PW) ? (t >= 0 ? 1 : 2) : 0;  // 0: nothing to store, 1: store the product, 2: store zeros (bad index)
    // gathered rows: lanes 4r .. 4r+3 fetch the four 16-byte chunks of a 16-deep slab of row 16 tq + r
    uint32_t xo[TQ];
#pragma unroll
    for (int tq = 0; tq < TQ; ++tq) xo[tq] = (uint32_t)__shfl((int)aoff, tq * 16 + (lane >> 2), kWave) + (uint32_t)((lane & 3) * 16);
    // every 16-deep slab of every row tile goes in flight now, the first row tile's first
    // The first row tile's slabs are requested now, the others after the barrier: a CU's eight wavefronts push 160 KB
    // through its one address path in this prologue (2560 cycles at 64 bytes a cycle), a wavefront cannot go on to
    // its LDS writes before its requests are accepted, and the barrier waits for the last of them - with every slab
    // requested here the first matrix instruction started 4700 cycles after the indices had arrived.
    u32x4 xr[TQ][KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) xr[0][s] = *reinterpret_cast<const u32x4 *>(p.A + xo[0] + s * 64);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < W_IT; ++i) {
        const int c = w_chunk(i);
        if (W_CHUNKS % NTHREADS == 0 || c >= 0) {
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
#pragma unroll
    for (int tq = 1; tq < TQ; ++tq)
#pragma unroll
        for (int s = 0; s < KS; ++s) xr[tq][s] = *reinterpret_cast<const u32x4 *>(p.A + xo[tq] + s * 64);
    __builtin_amdgcn_sched_barrier(0);

    // Row tiles are multiplied and stored one after the other (TG = 1), so that the stores of one run under the matrix
    // instructions of the next instead of all at the kernel's end - as long as a tile alone keeps four accumulators
    // busy (consecutive matrix instructions on one accumulator would wait for each other); narrower outputs take the
    // row tiles of the wavefront together (TG = TQ).
    constexpr int TG = TN >= 4 ? 1 : TQ;
#pragma unroll
    for (int t0 = 0; t0 < TQ; t0 += TG) {
        f32x4 acc[TG][TN];
#pragma unroll
        for (int t = 0; t < TG; ++t)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) acc[t][tn] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            u32x4 xf[TG];
#pragma unroll
            for (int t = 0; t < TG; ++t) xf[t] = lanes_4a_g_to_16g_a(xr[t0 + t][s], lane);
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
                    for (int t = 0; t < TG; ++t)
                        acc[t][tn] = __builtin_amdgcn_mfma_f32_16x16x4f32(bits_f32(wf[tn][c]), bits_f32(xf[t][c]), acc[t][tn], 0, 0, 0);
        }
        // lane (a, g) holds, for pick 16 tq + a, columns 16 tn + 4 g .. + 3: the four lanes g of a pick write 64 contiguous bytes
#pragma unroll
        for (int t = 0; t < TG; ++t) {
            const int tq = t0 + t;
            const int st = __shfl(state, tq * 16 + a, kWave);
            const uint32_t co = (uint32_t)__shfl((int)coff, tq * 16 + a, kWave);
            if (st == 0) continue;
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                const f32x4 v = st == 2 ? f32x4{0.f, 0.f, 0.f, 0.f} : acc[t][tn];
                *reinterpret_cast<f32x4 *>(p.C + co + (tn * 16 + g * 4) * 4) = v;
            }
        }
    }
}

}  // namespace egs
