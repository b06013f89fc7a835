// Weight gradient for large 16-bit shapes on the direct-to-LDS pipeline of egs_rows_gemm_dl.h:
//
//   dW(e, i, j) = sum_{m in split s} Xs[b, Ind[m], i] * Ys[m, j]
//
// Both operands are [reduction][column] in memory, and they stay that way in LDS: each BK-row
// slab of gathered Xs rows (256 columns) and of Ys rows (BQ columns) is fetched with direct
// 16-byte loads whose per-row byte offsets come from a table decoded from Ind, and the MFMA
// fragments are produced by LDS transpose reads.  256 x BQ output tile, 8 wavefronts (2 x 4),
// one barrier per slab.  Stages: NST = 2 (64-row slabs) keeps one slab in flight under the
// multiplication of another and decodes the offsets two slabs ahead inside the loop.  NST = 3
// (128 columns, 48 KB stages of 64 rows) and NST = 4 (256 columns, 32 KB stages of 32 rows)
// keep NST - 1 slabs in flight; the offsets of 1024 reduction rows at a time are decoded before
// their first slab is requested, so that no index load sits between the direct loads and the
// wait for a slab can leave exactly the later slabs' loads outstanding.  Rows that do not exist
// (rejected picks, the ragged end of a split) get an offset outside the buffer descriptor and
// arrive as zeros.
//
// Preconditions (checked by the host, which otherwise uses dw_kernel): 16-bit elements,
// I % 8 == 0, J % 8 == 0, 16-byte aligned rows, operands below 2 GiB.
//
// Replaces the reference's expert_gather_scatter_dW_kernel (egs/triton_kernels.py:261-356) on
// these shapes.
#pragma once
#include "egs_dw.h"
#include "egs_rows_gemm_dl.h"
#include "egs_small.h"

namespace egs {

constexpr int kDlThreads = 512;      // 8 wavefronts
constexpr int kDwChunkRows = 1024;   // three-stage form: reduction rows whose offsets are staged in LDS at a time

struct DwDlParams {
    DwParams d;               // i_tiles / j_tiles count 256-row and BQ-column tiles here
    uint32_t x_bytes, y_bytes;
};

template <class TT, int BQ, int NST = 2, int BK = 64>
__global__ __launch_bounds__(kDlThreads) void dw_dl_kernel(DwDlParams pp)
{
    static_assert(TT::ES == 2, "16-bit element types");
    static_assert(BQ == 256 || BQ == 128, "column tile");
    static_assert(BK == 64 || BK == 32, "slab depth");
    static_assert(NST >= 2 && NST <= 4 && (NST > 2 || BK == 64), "stages");
    constexpr int BP = 256;
    constexpr int KS = BK / 32;                          // matrix-instruction steps per slab
    constexpr int TP = 8, TQ = BQ / 64;                  // 16 x 16 tiles per wavefront: 128 x BQ/4
    constexpr int P_BYTES = BK * BP * 2, Q_BYTES = BK * BQ * 2, STAGE = P_BYTES + Q_BYTES;
    constexpr int PL = BK / 16;                          // P loads per wavefront per slab (1 KB = two rows each)
    constexpr int QL = BK * BQ / 4096;                   // Q loads per wavefront per slab
    constexpr int QCR = BQ / 8;                          // 16-byte chunks per Q row
    static_assert(NST * STAGE + (NST > 2 ? 8 * kDwChunkRows : 0) <= 160 * 1024, "LDS of a CU");

    constexpr int TAB = NST == 2 ? 2 * BK : kDwChunkRows;  // two slabs' offsets, or a whole chunk's
    __shared__ __attribute__((aligned(1024))) char smem[NST * STAGE];
    __shared__ uint32_t x_voff[TAB];
    __shared__ uint32_t y_voff[TAB];

    const DwParams &p = pp.d;
    int e, tile;
    const int tiles_per_e = p.i_tiles * p.j_tiles * p.S;
    if (!decode_expert_tile((int)blockIdx.x, tiles_per_e, p.E, e, tile)) return;
    const int s = tile / (p.i_tiles * p.j_tiles);
    const int ij = tile - s * (p.i_tiles * p.j_tiles);
    const int it = ij / p.j_tiles, jt = ij - it * p.j_tiles;
    const int i0 = it * BP, j0 = jt * BQ;
    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int Me = p.B * p.K;
    const int row_begin = s * p.rows_per_split;
    const int row_end = min(Me, row_begin + p.rows_per_split);
    const int nslab = row_end > row_begin ? (row_end - row_begin + BK - 1) / BK : 0;

    const u32x4 rs_x = make_rsrc(p.Xs, pp.x_bytes);
    const u32x4 rs_y = make_rsrc(p.Ys, pp.y_bytes);

    // ---------------- row offset tables: thread r < 64 owns reduction row r of a slab
    auto pick_of = [&](int slab, int64_t &pick, int &b) -> bool {
        int m = row_begin + slab * BK + tid;
        if (tid >= BK || m >= row_end) return false;
        b = m / p.K;
        pick = ((int64_t)b * p.E + e) * p.K + (m - b * p.K);
        return true;
    };
    auto table_store = [&](int buf, bool ok, int64_t pick, int b, int32_t t) {
        if (tid < BK) {
            const bool live = ok && t >= 0;
            x_voff[buf * BK + tid] = live ? (uint32_t)(((int64_t)b * p.ldx_b + (int64_t)t * p.ldx_t) * 2) : kVoffInvalid;
            y_voff[buf * BK + tid] = live ? (uint32_t)(pick * p.J * 2) : kVoffInvalid;
        }
    };

    // ---------------- loaders.  P tile [64][256]: load j covers rows 2j, 2j+1 (lane l: row 2j + l/32,
    // physical chunk l%32).  Q tile [64][BQ]: 64/QCR rows per load.
    int p_row[PL], p_col[PL], q_row[QL], q_col[QL];    // tile row a load lands on, byte offset of its column chunk (-1: outside)
#pragma unroll
    for (int jj = 0; jj < PL; ++jj) {
        int row = (wave * PL + jj) * 2 + (lane >> 5);
        int pc = lane & 31;
        int lchunk = ((((pc >> 1) ^ tr_swizzle(row)) << 1) | (pc & 1));
        p_row[jj] = row;
        p_col[jj] = i0 + lchunk * 8 < p.I ? (i0 + lchunk * 8) * 2 : -1;
    }
#pragma unroll
    for (int jj = 0; jj < QL; ++jj) {
        int row = (wave * QL + jj) * (64 / QCR) + lane / QCR;
        int pc = lane % QCR;
        int lchunk = ((((pc >> 1) ^ tr_swizzle(row)) << 1) | (pc & 1));
        q_row[jj] = row;
        q_col[jj] = j0 + lchunk * 8 < p.J ? (j0 + lchunk * 8) * 2 : -1;
    }
    // tab0: where the slab's 64 rows start in the offset tables
    auto issue = [&](int tab0, int stage) {
        char *base = smem + stage * STAGE;
#pragma unroll
        for (int jj = 0; jj < PL; ++jj) {
            uint32_t ro = x_voff[tab0 + p_row[jj]];
            uint32_t vo = (ro == kVoffInvalid || p_col[jj] < 0) ? kVoffInvalid : ro + (uint32_t)p_col[jj];
            direct_load16(rs_x, vo, 0, base + (wave * PL + jj) * 1024);
        }
#pragma unroll
        for (int jj = 0; jj < QL; ++jj) {
            uint32_t ro = y_voff[tab0 + q_row[jj]];
            uint32_t vo = (ro == kVoffInvalid || q_col[jj] < 0) ? kVoffInvalid : ro + (uint32_t)q_col[jj];
            direct_load16(rs_y, vo, 0, base + P_BYTES + (wave * QL + jj) * 1024);
        }
    };

    // ---------------- fragment addresses: a lane supplies row 32 ks + 8 g + 4 h + a/4 and four columns
    // 16 t + 4 (a%4) of tile t, and receives column 16 t + a of rows 8 g + 4 h .. + 3
    const int a = lane & 15, g = lane >> 4;
    const int wave_p0 = (wave >> 2) * 128, wave_q0 = (wave & 3) * (BQ / 4);
    int p_at[KS][2], q_at[KS][2];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            int row = ks * 32 + g * 8 + h * 4 + (a >> 2);
            p_at[ks][h] = row * (BP * 2) + (((wave_p0 >> 4) ^ tr_swizzle(row)) << 5) + (a & 3) * 8;
            q_at[ks][h] = row * (BQ * 2) + (((wave_q0 >> 4) ^ tr_swizzle(row)) << 5) + (a & 3) * 8;
        }

    f32x4 acc[TP][TQ];
#pragma unroll
    for (int x = 0; x < TP; ++x)
#pragma unroll
        for (int y = 0; y < TQ; ++y) acc[x][y] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto multiply = [&](int stage) {
        const char *tile_p = smem + stage * STAGE;
        const char *tile_q = tile_p + P_BYTES;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 pf[TP], qf[TQ];
#pragma unroll
            for (int x = 0; x < TP; ++x) {
                u32x2 lo = lds_read_tr16(tile_p + (p_at[ks][0] ^ (x << 5)));
                u32x2 hi = lds_read_tr16(tile_p + (p_at[ks][1] ^ (x << 5)));
                pf[x] = u32x4{lo[0], lo[1], hi[0], hi[1]};
            }
#pragma unroll
            for (int y = 0; y < TQ; ++y) {
                u32x2 lo = lds_read_tr16(tile_q + (q_at[ks][0] ^ (y << 5)));
                u32x2 hi = lds_read_tr16(tile_q + (q_at[ks][1] ^ (y << 5)));
                qf[y] = u32x4{lo[0], lo[1], hi[0], hi[1]};
            }
#pragma unroll
            for (int x = 0; x < TP; ++x)
#pragma unroll
                for (int y = 0; y < TQ; ++y) mma_chunk<TT>(acc[x][y], qf[y], pf[x]);
        }
    };

    if constexpr (NST == 2) {
    static_assert(NST > 2 || (PL == 4 && BK == 64), "the two-stage form is written for 64-row slabs");
    // ---------------- prologue: tables of slabs 0 and 1, loads of slab 0, index of slab 2 in flight
    {
        int64_t pick = 0; int b = 0;
        bool ok = pick_of(0, pick, b);
        int32_t t = ok ? load_token(p.Ind, p.ind_dtype, pick, p.T) : -1;
        table_store(0, ok, pick, b, t);
        ok = nslab > 1 && pick_of(1, pick, b);
        t = ok ? load_token(p.Ind, p.ind_dtype, pick, p.T) : -1;
        table_store(1, ok, pick, b, t);
    }
    __syncthreads();
    if (nslab > 0) issue(0, 0);
    int64_t nx_pick = 0; int nx_b = 0; int32_t nx_t = -1;
    bool nx_ok = nslab > 2 && pick_of(2, nx_pick, nx_b);
    if (nx_ok) nx_t = load_token(p.Ind, p.ind_dtype, nx_pick, p.T);

    for (int sl = 0; sl < nslab; ++sl) {
        wait_vmem<0>();
        __syncthreads();            // slab sl landed; table of slab sl+1 visible; stage and table of slab sl-1 free
        if (sl + 1 < nslab) issue(((sl + 1) & 1) * BK, (sl + 1) & 1);
        if (sl + 2 < nslab) table_store(sl & 1, nx_ok, nx_pick, nx_b, nx_t);     // read again after the next barrier
        nx_ok = sl + 3 < nslab && pick_of(sl + 3, nx_pick, nx_b);
        nx_t = -1;
        if (nx_ok) nx_t = load_token(p.Ind, p.ind_dtype, nx_pick, p.T);
        multiply(sl & 1);
    }
    } else {
    // ---------------- three or four stages, all but one in flight.  The row offsets of a whole chunk of reduction rows are
    // decoded from Ind before the chunk's first slab is requested, so that no index load sits between the
    // direct loads of the pipeline: the wait for slab sl leaves exactly the loads of slab sl + 1 outstanding.
    int stage = 0;
    for (int chunk0 = row_begin; chunk0 < row_end; chunk0 += kDwChunkRows) {
        const int chunk_rows = min(kDwChunkRows, row_end - chunk0);
        const int nsl = (chunk_rows + BK - 1) / BK;
        __syncthreads();            // the previous chunk's offsets and stages are no longer being read
        for (int r = tid; r < nsl * BK; r += kDlThreads) {
            const int m = chunk0 + r;
            uint32_t xo = kVoffInvalid, yo = kVoffInvalid;
            if (r < chunk_rows) {
                const int b = m / p.K;
                const int64_t pick = ((int64_t)b * p.E + e) * p.K + (m - b * p.K);
                const int32_t t = load_token(p.Ind, p.ind_dtype, pick, p.T);
                if (t >= 0) {
                    xo = (uint32_t)(((int64_t)b * p.ldx_b + (int64_t)t * p.ldx_t) * 2);
                    yo = (uint32_t)(pick * p.J * 2);
                }
            }
            x_voff[r] = xo;
            y_voff[r] = yo;
        }
        __syncthreads();
#pragma unroll
        for (int st = 0; st < NST - 1; ++st)
            if (st < nsl) issue(st * BK, stage + st < NST ? stage + st : stage + st - NST);
        for (int sl = 0; sl < nsl; ++sl) {
            // slab sl has landed once only the slabs requested after it (at most NST - 2) are outstanding
            const int later = min(nsl - 1 - sl, NST - 2);
            if (NST >= 4 && later >= 2) wait_vmem<(NST >= 4 ? 2 : 0) * (PL + QL)>();
            else if (later >= 1) wait_vmem<PL + QL>();
            else wait_vmem<0>();
            __syncthreads();        // slab sl landed everywhere; the stage of slab sl - 1 is free
            if (sl + NST - 1 < nsl) issue((sl + NST - 1) * BK, stage + NST - 1 < NST ? stage + NST - 1 : stage - 1);
            multiply(stage);
            if (++stage == NST) stage = 0;
        }
    }
    }

    // ---------------- epilogue: lane holds row i = i0 + wave_p0 + 16 x + a, columns j0 + wave_q0 + 16 y + 4 g .. + 3
    const bool direct = (p.S == 1);
#pragma unroll
    for (int x = 0; x < TP; ++x) {
        int i = i0 + wave_p0 + x * 16 + a;
        if (i >= p.I) continue;
#pragma unroll
        for (int y = 0; y < TQ; ++y) {
            int j = j0 + wave_q0 + y * 16 + g * 4;
            if (j >= p.J) continue;                 // J % 8 == 0: the four columns are all in or all out
            f32x4 v = acc[x][y];
            if (!direct) {
                // partial sums already in the layout of the output, so that the second pass is a plain sum
                if (p.dw_layout == 0) {
                    float *dst = p.part + (((size_t)s * p.E + e) * p.I + i) * p.J + j;
                    *reinterpret_cast<f32x4 *>(dst) = v;        // workspace base is 256-byte aligned, J % 4 == 0
                } else {                                        // [E,J,I]: 16 lanes cover 16 consecutive i
#pragma unroll
                    for (int r = 0; r < 4; ++r) p.part[(((size_t)s * p.E + e) * p.J + (j + r)) * p.I + i] = v[r];
                }
            } else if (p.dw_layout == 0) {                      // [E,I,J]
                size_t at = ((size_t)e * p.I + i) * p.J + j;
                if (p.out_dtype == 0) {
                    *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(p.dW) + at) = v;
                } else {
                    u32x2 w;
                    if (p.out_dtype == 1) {
                        w[0] = f32_to_f16_bits(v[0]) | (f32_to_f16_bits(v[1]) << 16);
                        w[1] = f32_to_f16_bits(v[2]) | (f32_to_f16_bits(v[3]) << 16);
                    } else {
                        w[0] = pack2<ElemBF16>(v[0], v[1]);
                        w[1] = pack2<ElemBF16>(v[2], v[3]);
                    }
                    *reinterpret_cast<u32x2 *>(reinterpret_cast<uint16_t *>(p.dW) + at) = w;
                }
            } else {                                            // [E,J,I]: 16 lanes cover 16 consecutive i
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    size_t at = ((size_t)e * p.J + (j + r)) * p.I + i;
                    if (p.out_dtype == 0) reinterpret_cast<float *>(p.dW)[at] = v[r];
                    else reinterpret_cast<uint16_t *>(p.dW)[at] =
                        (uint16_t)(p.out_dtype == 1 ? f32_to_f16_bits(v[r]) : f32_to_bf16_bits(v[r]));
                }
            }
        }
    }
}

}  // namespace egs
