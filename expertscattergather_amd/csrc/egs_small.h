// Rows x weight product for small experts (16-bit elements, reduction length 32/64/128,
// at most 128 output columns, W[e] of a few KiB): the regime of the reference's default shape
// (B64 T256 E32 K32 I128 J64), where every kernel moves ~13 MB and must finish in a few
// microseconds.  At that size the staged pipeline of the general kernel (LDS tiles, barriers
// per slab) and even the instruction count per wavefront cost more than the memory traffic,
// so this kernel is written to issue few instructions: every load is unconditional (addresses
// are clamped, never guarded), addresses are 32-bit offsets from a uniform base, rounding uses
// the packed hardware conversion, and there is no LDS and no barrier.
//
// One wavefront owns 64 picks of one expert.  W[e] lives in registers as MFMA operand
// fragments for the whole kernel; the rows are loaded straight from global memory into operand
// registers (a row's 16-byte chunks are exactly what an MFMA lane consumes).
//   GATHER   rows come from [B,T,R] through Ind, results go to the dense [B,E,K,N] rows
//            (gather forward; dY of the scatter)
//   !GATHER  rows are the dense [B,E,K,R] rows, results go to dense [B,E,K,N] product rows, fp32
//            or 16-bit (first phase of the scatter and of dX).  The first `csr_blocks`
//            workgroups of such a launch build the routing table instead, so that the sort
//            runs in the shadow of the product and costs no launch of its own.
//
// MFMA operand trick: the hardware wants, per lane, 8 reduction-consecutive elements of one
// row.  When the weight is stored with the output index contiguous instead, a lane loads an
// 8(reduction) x 4 or 8(output) block and transposes it in registers; the block's output
// indices become that lane's row in 4 or 8 different MFMA tiles, which only permutes where
// results end up (each lane still ends with a run of consecutive output columns).
#pragma once
#include "egs_device.h"
#include "egs_scatter_aux.h"
#include "egs_dw_tile.h"

namespace egs {

struct SmallRowsParams {
    const char *A;          // GATHER: [B,T,R] rows, strides (lda_b, lda_t, 1) elements;  else [B,E,K,R] dense
    const char *W;          // [E,R,N] (W_NMAJOR) or [E,N,R]
    const void *Ind;
    char *C;                // [B,E,K,N] rows: elements, or fp32 when OUT_F32
    int32_t B, T, E, K, N;
    int64_t lda_b, lda_t;
    int32_t ind_dtype;
    int32_t tiles_per_e;    // workgroups (256 picks each) per expert
    int32_t rows_share_xcd; // workgroup -> (expert, row tile) map, see decode_rows_block: 0 experts map to XCDs, 1 / 2 / 4 row tiles do (source rows reused across experts)
    // routing-table build riding along (csr_blocks = B, or 0): see csr_count_body; csr_split: two workgroups per batch
    // element (csr_blocks = 2 B), see csr_count_half_body
    int32_t csr_blocks, csr_split;
    int32_t *seg_off, *perm, *rank_tmp, *long_tab;
};

// Requirements (checked by the launcher): 2-byte elements, R == 32*KS, N % 8 == 0,
// 8 <= N <= 16*TN, A rows / W / C 16-byte aligned, every tensor smaller than 4 GiB.
// WPB = wavefronts per workgroup (a workgroup covers 64 * WPB picks of one expert; tiles_per_e counts such workgroups)
template <class TT, bool W_NMAJOR, int KS, int TN, bool GATHER, bool OUT_F32, int WPB = 4>
__device__ __forceinline__ void rows_small_body(const SmallRowsParams &p, const int block, int32_t *sh_cnt_small)
{
    constexpr int TQ = 4;                       // 4 row tiles = 64 picks per wave
    constexpr int R = 32 * KS;
    constexpr int OES = OUT_F32 ? 4 : 2;        // output element size
    static_assert(!(GATHER && OUT_F32), "gather results are stored in the element type");
    if (block < p.csr_blocks) {             // uniform per workgroup; 0 unless a routing table rides along
        if (p.csr_split)
            csr_count_half_body(sh_cnt_small, block >> 1, block & 1, (int)threadIdx.x, 64 * WPB, p.Ind, p.ind_dtype, p.T,
                                p.E * p.K, p.seg_off, p.perm);
        else
            csr_count_body(sh_cnt_small, block, block, (int)threadIdx.x, 64 * WPB, p.Ind, p.ind_dtype, p.T,
                           p.E * p.K, p.seg_off, p.perm, p.rank_tmp, p.long_tab);
        return;
    }
    int e, tile;
    const int bid = block - p.csr_blocks;
    if (!decode_rows_block(bid, p.rows_share_xcd, p.tiles_per_e, p.E, e, tile)) return;       // uniform per workgroup
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: scalar address work
    const int a = lane & 15, g = lane >> 4;
    const int Me = p.B * p.K;
    const int m0 = (tile * WPB + wave) * 64;
    if (m0 >= Me) return;                       // no barriers below: a wave may leave alone
    const int N = p.N;

    // Order of the loads.  Loads return in order, and the long chain is index -> row.  So the index load goes
    // first, the weight loads follow in the shadow of its latency, and the row loads are issued as soon as the
    // index is there (the wait names the index load alone); the weight blocks are transposed only after that.
    // this lane's pick (row m0 + lane): byte offsets of its source row and of its result row
    const int m_lane = m0 + lane;
    const int mm_lane = min(m_lane, Me - 1);
    const int b_lane = mm_lane / p.K;
    const int64_t pick = ((int64_t)b_lane * p.E + e) * p.K + (mm_lane - b_lane * p.K);
    uint64_t t_word = 0;
    if constexpr (GATHER) t_word = load_index_word(p.Ind, p.ind_dtype, pick);

    // Which output column does accumulator row a' = 4g+r of MFMA tile tn hold?  Chosen so that
    // in every store instruction the four lanes g = 0..3 of one result row write one contiguous
    // 64-byte run (16 bytes each); the weight fragments are loaded to match.
    //   K-major weight (any row may be fetched):  fp32 out  n = 16*tn + a'
    //                                             16-bit    n = 32*(tn/2) + 8*(a'/4) + 4*(tn%2) + a'%4
    //   N-major weight (a lane fetches 4- or 8-column blocks, tile = column inside the block):
    //       fp32 out            block v (4 cols): starts at 64*v + 16*(a'%4) + 4*(a'/4)
    //       16-bit, TN == 4     one 4-col block:  starts at 32*((a'/2)%2) + 8*(a'/4) + 4*(a'%2)
    //       16-bit, TN == 8     one 8-col block:  starts at 32*(a'%4) + 8*(a'/4)
    const char *We = p.W + (size_t)e * R * N * 2;
    constexpr bool W_BLK8 = W_NMAJOR && OES == 2 && TN == 8;    // 8 x 8 blocks (16-byte loads), else 8 x 4 blocks
    constexpr int NBLK = TN / 4;
    u32x4 wf[KS][TN];                           // K-major weights and 8 x 8 blocks are loaded into place
    u32x2 wraw[W_NMAJOR && !W_BLK8 ? NBLK : 1][KS][8];
    if constexpr (W_NMAJOR) {
        if constexpr (W_BLK8) {
            const uint32_t col = (uint32_t)min((a & 3) * 32 + (a >> 2) * 8, N - 8);   // lanes past N recompute a valid block; never stored
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int x = 0; x < 8; ++x)
                    wf[ks][x] = *reinterpret_cast<const u32x4 *>(We + ((uint32_t)(ks * 32 + g * 8 + x) * (uint32_t)N + col) * 2u);
        } else {
#pragma unroll
            for (int v = 0; v < NBLK; ++v) {
                const int start = OES == 4 ? v * 64 + (a & 3) * 16 + (a >> 2) * 4
                                           : ((a >> 1) & 1) * 32 + (a >> 2) * 8 + (a & 1) * 4;
                const uint32_t col = (uint32_t)min(start, N - 4);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int x = 0; x < 8; ++x)
                        wraw[v][ks][x] = *reinterpret_cast<const u32x2 *>(We + ((uint32_t)(ks * 32 + g * 8 + x) * (uint32_t)N + col) * 2u);
            }
        }
    } else {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const int row = OES == 4 ? tn * 16 + a : (tn >> 1) * 32 + (a >> 2) * 8 + (tn & 1) * 4 + (a & 3);
            const uint32_t n = (uint32_t)min(row, N - 1);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                wf[ks][tn] = *reinterpret_cast<const u32x4 *>(We + (n * (uint32_t)R + (uint32_t)(ks * 32 + g * 8)) * 2u);
        }
    }

    __builtin_amdgcn_sched_barrier(0);          // index and weight loads are issued; nothing below moves above them

    uint32_t aoff = 0, coff = 0;
    int state = 0;                              // 0: nothing to store, 1: store the product, 2: store zeros (bad index)
    if constexpr (GATHER) {
        const int64_t t_raw = decode_index_word(t_word, p.Ind, p.ind_dtype, pick);
        const int32_t t = (t_raw < 0 || t_raw >= (int64_t)p.T) ? -1 : (int32_t)t_raw;
        if (t >= 0) aoff = (uint32_t)(((int64_t)b_lane * p.lda_b + (int64_t)t * p.lda_t) * 2);
        coff = (uint32_t)(pick * N * OES);
        state = m_lane < Me ? (t >= 0 ? 1 : 2) : 0;
    } else {
        aoff = (uint32_t)(pick * R * 2);
        coff = (uint32_t)(pick * N * OES);
        state = m_lane < Me ? 1 : 0;
    }

    // row fragments: lane (a, g) of row tile tq supplies elements [32*ks + 8*g, +8) of row 16*tq + a.  They are
    // fetched coalesced (lanes 4r .. 4r+3 take four consecutive 16-byte chunks of row 16*tq + r: one 64-byte
    // access per row instead of four scattered 16-byte ones) and moved to operand order across lanes.
    u32x4 xf[TQ][KS];
#pragma unroll
    for (int tq = 0; tq < TQ; ++tq) {
        const uint32_t xo = (uint32_t)__shfl((int)aoff, tq * 16 + (lane >> 2), kWave) + (uint32_t)((lane & 3) * 16);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) xf[tq][ks] = *reinterpret_cast<const u32x4 *>(p.A + xo + ks * 64);
    }
    __builtin_amdgcn_sched_barrier(0);          // the row loads are issued before anything waits for weights or rows

    // the weight blocks become operand fragments (register transposes)
    if constexpr (W_BLK8) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 blk[8];
#pragma unroll
            for (int x = 0; x < 8; ++x) blk[x] = wf[ks][x];
            transpose8x8_16b(blk, wf[ks]);
        }
    } else if constexpr (W_NMAJOR) {
#pragma unroll
        for (int v = 0; v < NBLK; ++v)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                u32x4 out4[4];
                transpose8x4_16b(wraw[v][ks], out4);
#pragma unroll
                for (int c = 0; c < 4; ++c) wf[ks][v * 4 + c] = out4[c];
            }
    }
#pragma unroll
    for (int tq = 0; tq < TQ; ++tq)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) xf[tq][ks] = lanes_4a_g_to_16g_a(xf[tq][ks], lane);

#pragma unroll
    for (int tq = 0; tq < TQ; ++tq) {
        f32x4 acc[TN];
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) acc[tn] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) mma_chunk<TT>(acc[tn], wf[ks][tn], xf[tq][ks]);
        const int st = __shfl(state, tq * 16 + a, kWave);
        const uint32_t co = (uint32_t)__shfl((int)coff, tq * 16 + a, kWave);
        if (st == 2) {
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) acc[tn] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        if (st != 0) {
            if constexpr (OES == 4) {
                // one 16-byte piece (4 columns) per instruction
#pragma unroll
                for (int u = 0; u < TN; ++u) {
                    int col;
                    f32x4 v;
                    if constexpr (W_NMAJOR) {                   // u = 4*v + r; values are the 4 tiles of block v
                        const int vb = u >> 2, r = u & 3;
                        col = vb * 64 + r * 16 + g * 4;
                        v = f32x4{acc[vb * 4 + 0][r], acc[vb * 4 + 1][r], acc[vb * 4 + 2][r], acc[vb * 4 + 3][r]};
                    } else {                                    // u = tile; values are its 4 rows
                        col = u * 16 + g * 4;
                        v = acc[u];
                    }
                    if (col + 4 <= N) *reinterpret_cast<f32x4 *>(p.C + co + col * 4) = v;
                }
            } else {
                // one 16-byte piece (8 columns) per instruction
#pragma unroll
                for (int u = 0; u < TN / 2; ++u) {
                    int col;
                    float v[8];
                    if constexpr (!W_NMAJOR) {                  // tiles 2u and 2u+1, 4 rows each
                        col = u * 32 + g * 8;
#pragma unroll
                        for (int r = 0; r < 4; ++r) { v[r] = acc[2 * u][r]; v[4 + r] = acc[2 * u + 1][r]; }
                    } else if constexpr (TN == 4) {             // rows 2u and 2u+1 of the 4 tiles
                        col = u * 32 + g * 8;
#pragma unroll
                        for (int c = 0; c < 4; ++c) { v[c] = acc[c][2 * u]; v[4 + c] = acc[c][2 * u + 1]; }
                    } else {                                    // TN == 8: row u of the 8 tiles
                        col = u * 32 + g * 8;
#pragma unroll
                        for (int c = 0; c < 8; ++c) v[c] = acc[c][u];
                    }
                    if (col + 8 <= N) {
                        u32x4 w = {pack2<TT>(v[0], v[1]), pack2<TT>(v[2], v[3]), pack2<TT>(v[4], v[5]), pack2<TT>(v[6], v[7])};
                        *reinterpret_cast<u32x4 *>(p.C + co + col * 2) = w;
                    }
                }
            }
        }
    }
}

template <class TT, bool W_NMAJOR, int KS, int TN, bool GATHER, bool OUT_F32>
__global__ __launch_bounds__(kThreads) void rows_small_kernel(SmallRowsParams p)
{
    extern __shared__ int32_t sh_dyn_small[];
    rows_small_body<TT, W_NMAJOR, KS, TN, GATHER, OUT_F32>(p, (int)blockIdx.x, sh_dyn_small);
}

}  // namespace egs

namespace egs {

// ------------------------------------------------------------------------------------------
// Weight gradient for small experts: dW(e, i, j) = sum_m Xs[b, Ind[m], i] * Ys[m, j].
// One workgroup owns a 64 x 64 tile of dW(e) for one split of the expert's picks; its four
// wavefronts take interleaved 32-pick steps, each accumulating the whole tile in registers,
// and are summed through LDS in wavefront order (fixed order -> reproducible).  Both operands
// are "reduction-strided" (a pick selects a row, the output index runs along it): each lane
// loads 8(picks) x 4(columns) blocks of both with 8-byte loads straight from global memory
// and transposes them in registers into MFMA fragments; no operand staging in LDS.
struct SmallDwParams {
    const char *Xs;         // [B,T,I] rows, strides (ldx_b, ldx_t, 1) elements; span < 4 GiB
    const char *Ys;         // [B,E,K,J] dense; < 4 GiB
    const void *Ind;
    float *part;            // [S,E,I,J] fp32 partial sums (S > 1)
    char *dW;               // final output when S == 1
    int32_t B, T, E, K, I, J;
    int64_t ldx_b, ldx_t;
    int32_t ind_dtype;
    int32_t i_tiles, j_tiles;
    int32_t S, rows_per_split;      // rows_per_split is a multiple of 128
    int32_t out_dtype, dw_layout;
};

constexpr int kDwSmallMaxRows = 1024;   // picks of one workgroup (row offsets staged in LDS)
constexpr int kDwSmallLdsBytes = 4 * 64 * 64 * 4;

// Requirements: 2-byte elements, I % 8 == 0, J % 8 == 0, rows 16-byte aligned, spans < 4 GiB,
// rows_per_split <= kDwSmallMaxRows.
template <class TT, int NW = 4>
__device__ __forceinline__ void dw_small_body(const SmallDwParams &p, const int block, float *red)
{
    // NW wavefronts; red: NW * 16 KB of 16-byte aligned LDS (kDwSmallLdsBytes for four), one 64 x 64 tile per wavefront
    constexpr int NT = NW * 64;
    uint32_t *xoff_lds = reinterpret_cast<uint32_t *>(red);              // reused before the reduction:
    uint32_t *yoff_lds = xoff_lds + kDwSmallMaxRows;                      //   row byte offsets, 0xFFFFFFFF = no row

    int e, tile;
    const int tiles_per_e = p.i_tiles * p.j_tiles * p.S;
    if (!decode_expert_tile(block, tiles_per_e, p.E, e, tile)) return;
    const int s = tile / (p.i_tiles * p.j_tiles);
    const int ij = tile - s * (p.i_tiles * p.j_tiles);
    const int it = ij / p.j_tiles, jt = ij - it * p.j_tiles;
    const int i0 = it * 64, j0 = jt * 64;
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: scalar address work
    const int a = lane & 15, g = lane >> 4;
    const int Me = p.B * p.K;
    const int row_begin = s * p.rows_per_split;
    const int nrows = max(0, min(Me, row_begin + p.rows_per_split) - row_begin);

    for (int r = tid; r < p.rows_per_split; r += NT) {
        uint32_t xo = 0xFFFFFFFFu, yo = 0;
        if (r < nrows) {
            const int m = row_begin + r;
            const int b = m / p.K, k = m - b * p.K;
            const int64_t pick = ((int64_t)b * p.E + e) * p.K + k;
            const int32_t t = load_token(p.Ind, p.ind_dtype, pick, p.T);
            if (t >= 0) xo = (uint32_t)(((int64_t)b * p.ldx_b + (int64_t)t * p.ldx_t) * 2);
            yo = (uint32_t)(pick * p.J * 2);
        }
        xoff_lds[r] = xo;
        yoff_lds[r] = yo;
    }
    __syncthreads();

    // block columns of this lane: X block at i0 + 4a (tile ci = column 4a + ci), Y block at j0 + 4a (tile cj):
    // adjacent lanes fetch adjacent 8-byte pieces of a row, and after the MFMA lane (a, g) holds, for row
    // i = i0 + 4a + ci, the four consecutive columns j0 + 16g + 4r + cj
    const uint32_t xcol = (uint32_t)min(i0 + a * 4, p.I - 4) * 2u;
    const uint32_t ycol = (uint32_t)min(j0 + a * 4, p.J - 4) * 2u;

    f32x4 acc[4][4];            // [ci][cj]
#pragma unroll
    for (int ci = 0; ci < 4; ++ci)
#pragma unroll
        for (int cj = 0; cj < 4; ++cj) acc[ci][cj] = f32x4{0.f, 0.f, 0.f, 0.f};

    struct Stage { u32x2 x[8], y[8]; };
    auto load_stage = [&](int step, Stage &st) {       // step = 32 picks; this lane's 8 picks: 8g .. 8g+7
        const int r0 = step * 32 + g * 8;
        const u32x4 xa = *reinterpret_cast<const u32x4 *>(xoff_lds + r0), xb = *reinterpret_cast<const u32x4 *>(xoff_lds + r0 + 4);
        const u32x4 ya = *reinterpret_cast<const u32x4 *>(yoff_lds + r0), yb = *reinterpret_cast<const u32x4 *>(yoff_lds + r0 + 4);
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            const uint32_t xo = x < 4 ? xa[x] : xb[x - 4], yo = x < 4 ? ya[x] : yb[x - 4];
            const bool live = xo != 0xFFFFFFFFu;
            u32x2 xv = *reinterpret_cast<const u32x2 *>(p.Xs + (live ? xo : 0u) + xcol);
            u32x2 yv = *reinterpret_cast<const u32x2 *>(p.Ys + yo + ycol);
            if (!live) { xv = u32x2{0u, 0u}; yv = xv; }   // a missing pick contributes nothing
            st.x[x] = xv;
            st.y[x] = yv;
        }
    };
    auto consume = [&](const Stage &st) {
        u32x4 xf[4], yf[4];
        transpose8x4_16b(st.x, xf);
        transpose8x4_16b(st.y, yf);
#pragma unroll
        for (int ci = 0; ci < 4; ++ci)
#pragma unroll
            for (int cj = 0; cj < 4; ++cj) mma_chunk<TT>(acc[ci][cj], yf[cj], xf[ci]);
    };

    const int nsteps = (nrows + 31) / 32;               // rows past nrows carry the "no row" offset
    if (wave < nsteps) {
        Stage cur, nxt;
        load_stage(wave, cur);
        for (int step = wave; step < nsteps; step += NW) {
            if (step + NW < nsteps) load_stage(step + NW, nxt);
            consume(cur);
            cur = nxt;
        }
    }
    __syncthreads();                                    // row offsets no longer needed: LDS becomes the reduction buffer

    // wave tile -> LDS [wave][i 0..63][j 0..63], 16-byte chunks XOR-swizzled by the row group
    float *mine = red + wave * 4096;
#pragma unroll
    for (int ci = 0; ci < 4; ++ci)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i = a * 4 + ci, chunk = (g * 4 + r) ^ a;
            *reinterpret_cast<f32x4 *>(mine + i * 64 + chunk * 4) =
                f32x4{acc[ci][0][r], acc[ci][1][r], acc[ci][2][r], acc[ci][3][r]};
        }
    __syncthreads();

    // sum the four wavefront tiles in wavefront order and write 4 consecutive elements of the
    // requested layout per thread: [.,I,J] rows of j, or [.,J,I] rows of i (read transposed from LDS).
    // Partial sums (S > 1) use the same layout as the final tensor, so the second pass is a plain
    // element-wise sum.
    const bool direct = (p.S == 1);
    const bool eji = p.dw_layout != 0;
    for (int item = tid; item < 64 * 16; item += NT) {
        const int major = item >> 4, minor4 = (item & 15) * 4;      // major: i (EIJ) or j (EJI); minor: 4 x j or 4 x i
        f32x4 v;
        if (!eji) {
            const int phys = ((minor4 >> 2) ^ (major >> 2)) * 4;
            v = *reinterpret_cast<const f32x4 *>(red + major * 64 + phys);
#pragma unroll
            for (int w = 1; w < NW; ++w) {
                const f32x4 u = *reinterpret_cast<const f32x4 *>(red + w * 4096 + major * 64 + phys);
                v[0] += u[0]; v[1] += u[1]; v[2] += u[2]; v[3] += u[3];
            }
        } else {
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int i = minor4 + x;
                const int at = i * 64 + (((major >> 2) ^ (i >> 2)) * 4) + (major & 3);
                float acc1 = red[at];
#pragma unroll
                for (int w = 1; w < NW; ++w) acc1 += red[w * 4096 + at];
                v[x] = acc1;
            }
        }
        const int gi = i0 + (eji ? minor4 : major), gj = j0 + (eji ? major : minor4);
        if (gi >= p.I || gj >= p.J) continue;           // I % 4 == 0 and J % 4 == 0: a group of 4 is inside or outside
        const size_t at = eji ? ((size_t)e * p.J + gj) * p.I + gi : ((size_t)e * p.I + gi) * p.J + gj;
        if (!direct) {
            *reinterpret_cast<f32x4 *>(p.part + (size_t)s * p.E * p.I * p.J + at) = v;
        } else if (p.out_dtype == 0) {
            *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(p.dW) + at) = v;
        } else {
            u32x2 w2;
            w2[0] = p.out_dtype == 1 ? pack2<ElemF16>(v[0], v[1]) : pack2<ElemBF16>(v[0], v[1]);
            w2[1] = p.out_dtype == 1 ? pack2<ElemF16>(v[2], v[3]) : pack2<ElemBF16>(v[2], v[3]);
            *reinterpret_cast<u32x2 *>(reinterpret_cast<uint16_t *>(p.dW) + at) = w2;
        }
    }
}

template <class TT>
__global__ __launch_bounds__(kThreads) void dw_small_kernel(SmallDwParams p)
{
    __shared__ __attribute__((aligned(16))) float red[kDwSmallLdsBytes / 4];
    dw_small_body<TT>(p, (int)blockIdx.x, red);
}

// dW = sum_s part[s] in increasing s, rounded once; partials already have the output's layout.
// 4 elements per thread (total % 4 == 0, 16-byte aligned); `block` of `nblocks` workgroups.
__device__ __forceinline__ void dw_reduce4_body(const float *part, char *dW, int32_t S, size_t total4, int32_t out_dtype,
                                                const int block, const int nblocks)
{
    for (size_t o = (size_t)block * kThreads + threadIdx.x; o < total4; o += (size_t)nblocks * kThreads) {
        f32x4 v = reinterpret_cast<const f32x4 *>(part)[o];
        for (int s = 1; s < S; ++s) {
            const f32x4 u = reinterpret_cast<const f32x4 *>(part)[(size_t)s * total4 + o];
            v[0] += u[0]; v[1] += u[1]; v[2] += u[2]; v[3] += u[3];
        }
        if (out_dtype == 0) {
            reinterpret_cast<f32x4 *>(dW)[o] = v;
        } else {
            u32x2 w2;
            w2[0] = out_dtype == 1 ? pack2<ElemF16>(v[0], v[1]) : pack2<ElemBF16>(v[0], v[1]);
            w2[1] = out_dtype == 1 ? pack2<ElemF16>(v[2], v[3]) : pack2<ElemBF16>(v[2], v[3]);
            reinterpret_cast<u32x2 *>(dW)[o] = w2;
        }
    }
}


static __global__ __launch_bounds__(kThreads) void dw_reduce4_kernel(const float *part, char *dW, int32_t S, size_t total4,
                                                              int32_t out_dtype)
{
    dw_reduce4_body(part, dW, S, total4, out_dtype, (int)blockIdx.x, (int)gridDim.x);
}

// ------------------------------------------------------------------------------------------
// Heterogeneous launches: independent pieces of one backward call share a launch, so that the
// call pays one launch ramp and the pieces overlap.  Workgroups [0, rows_blocks) run the rows
// product (and, for the scatter, the routing table), the rest the weight gradient.
template <class TT, bool W_NMAJOR, int KS, int TN, bool GATHER, bool OUT_F32>
__global__ __launch_bounds__(kThreads) void rows_dw_small_kernel(SmallRowsParams p, SmallDwParams q, int rows_blocks)
{
    extern __shared__ int32_t sh_dyn_fused[];
    __shared__ __attribute__((aligned(16))) float red[kDwSmallLdsBytes / 4];
    if ((int)blockIdx.x < rows_blocks) rows_small_body<TT, W_NMAJOR, KS, TN, GATHER, OUT_F32>(p, (int)blockIdx.x, sh_dyn_fused);
    else dw_small_body<TT>(q, (int)blockIdx.x - rows_blocks, red);
}

// A gather and the one-pass weight gradient (egs_dw_tile.h, 32 x 64 tiles) of the same backward call in one launch.
// Both kinds of workgroup have 8 wavefronts and the kernel's register and LDS footprint admits one workgroup per
// CU: when the launcher chooses this kernel the two kinds together have no more workgroups than the device has
// CUs, so every workgroup gets a CU of its own and the two kinds do not compete for a CU's path to the L2 (which
// is what bounds the weight gradient; sharing CUs made the pair as slow as running one after the other).
template <class TT, bool W_NMAJOR, int KS, int TN>
__global__ __launch_bounds__(kDwWideThreads) void rows_dw_tile_kernel(SmallRowsParams p, DwTileParams q, int rows_blocks)
{
    extern __shared__ __attribute__((aligned(16))) char sh_dyn_rows_tile[];
    // the weight gradient's workgroups (the longer ones) come first in launch order
    const int dw_blocks = (int)gridDim.x - rows_blocks;
    if ((int)blockIdx.x < dw_blocks) dw_tile_body<TT, kDwWideThreads / 64, 64>(q, (int)blockIdx.x, sh_dyn_rows_tile);
    else rows_small_body<TT, W_NMAJOR, KS, TN, true, false, kDwWideThreads / 64>(p, (int)blockIdx.x - dw_blocks,
                                                                                  reinterpret_cast<int32_t *>(sh_dyn_rows_tile));
}

// segment sums of a scatter and the second pass of a weight gradient in one launch:
// workgroups [0, seg_blocks) reduce product rows per token (ordinary and long segments), the rest sum dW partials
template <class TT, class PT, int VW>
__global__ __launch_bounds__(kThreads) void segsum_dwreduce_kernel(SegSumParams sp, int seg_blocks, const float *part,
                                                                   char *dW, int32_t S, size_t total4, int32_t out_dtype)
{
    const int block = (int)blockIdx.x;
    if (block < seg_blocks) segment_sum_dispatch<TT, PT, VW>(sp, block);
    else dw_reduce4_body(part, dW, S, total4, out_dtype, block - seg_blocks, (int)gridDim.x - seg_blocks);
}

}  // namespace egs
