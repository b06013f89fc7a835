// The rows x weight product of egs_rows_gemm.h for large, well-formed 16-bit shapes, built around
// what gfx950 adds for this: 16-byte direct global->LDS loads and LDS transpose reads.
//
//   * 256 x 256 output tile, 64-deep slabs, 8 wavefronts (2 x 4), each 128 x 64 of the tile.
//   * Both operand slabs travel HBM/L2 -> LDS without touching registers (one buffer load per
//     1 KB of a slab), two slabs in flight: the loads of slab k+1 are issued right after the
//     barrier that publishes slab k and land while its 64 MFMAs per wavefront run.  One barrier
//     per slab.
//   * Rows that are fetched through Ind are just per-lane byte offsets into the buffer
//     descriptor; rows that do not exist get an offset outside it and arrive as zeros.
//   * K-major operands ([row][reduction]) are read back with 16-byte LDS reads (XOR swizzle set
//     up by choosing which global chunk each lane fetches); a weight stored [reduction][column]
//     stays that way in LDS and is read with the transpose read, so no register transposes.
//
// Preconditions (checked by the host, which otherwise uses rows_gemm_kernel): 16-bit elements,
// R % 64 == 0, N % 8 == 0, 16-byte aligned rows, operands below 2 GiB.  fp8 (e4m3) weights in the
// [reduction][column] layout are supported with bf16 activations (N % 16 == 0): the bytes go to LDS as
// they are, the 8-bit transpose read hands each lane eight reduction-consecutive values and those are
// widened to bf16 (exactly) in registers.
//
// Replaces the reference's expert_gather_kernel (egs/triton_kernels.py:49-143) and the product
// part of expert_scatter_kernel (:156-247) on these shapes.
#pragma once
#include "egs_rows_gemm.h"
#include "egs_scatter_aux.h"

namespace egs {

constexpr int kDlBM = 256, kDlBN = 256, kDlBK = 64, kDlThreads = 512;
constexpr int kDlTileBytes = 256 * 64 * 2;              // one operand slab
constexpr int kDlStageBytes = 2 * kDlTileBytes;
constexpr int kDlSmemBytes = 2 * kDlStageBytes + kDlBM * 4 + kDlBM * 8;
constexpr int kDlSmemBytesScatter = 150 * 1024;

// swizzle of the [reduction][column] tile: 32-byte units of a row are XORed with bits {0,1,3} of
// the row number, which spreads the 16 rows one transpose read touches over all banks
__device__ __forceinline__ int tr_swizzle(int row) { return (row & 3) | (((row >> 3) & 1) << 2); }
// swizzle keys of the K-major tiles (XORed into the 16-byte chunk index of a 128-byte row).  The
// row side reads 16 consecutive rows per 16 lanes; the weight side reads the relabelled rows
// 16 c + 4 j + d (c, d = 0..3), whose distinguishing bits are 1, 4 and 5.
__device__ __forceinline__ int kmajor_key_rows(int row) { return row & 7; }
__device__ __forceinline__ int kmajor_key_relabelled(int row) { return (((row >> 4) & 3) << 1) | ((row >> 1) & 1); }

template <class TT, int WES, bool GATHER, bool W_TRANS, int EPI>
__global__ __launch_bounds__(kDlThreads) void rows_gemm_dl_kernel(RowsGemmParams p)
{
    static_assert(TT::ES == 2, "16-bit element types");
    static_assert(WES == 2 || (WES == 1 && W_TRANS && TT::ID == 2), "fp8 weights: [reduction][column] layout, widened to bf16");
    constexpr bool W_FP8 = (WES == 1);
    static_assert(EPI == EPI_STORE || EPI == EPI_STORE_F32, "plain stores only");
    constexpr int BM = kDlBM, BN = kDlBN, BK = kDlBK;
    constexpr int TM = 8, TN = 4;                        // 16 x 16 tiles per wavefront: 128 x 64

    // two slab stages, then the row tables; the scatter variants reserve more so that the routing-table
    // workgroups riding along have room for eight wavefronts' histograms at T = 4096
    __shared__ __attribute__((aligned(1024))) char smem[GATHER ? kDlSmemBytes : kDlSmemBytesScatter];
    uint32_t *a_voff = reinterpret_cast<uint32_t *>(smem + 2 * kDlStageBytes);
    int64_t *c_off = reinterpret_cast<int64_t *>(smem + 2 * kDlStageBytes + BM * 4);

    const int tid = (int)threadIdx.x;
    int block = (int)blockIdx.x;
    if constexpr (!GATHER) {
        // the scatter's routing table does not depend on the product: one workgroup per batch element
        // builds it here (csr_threads of the workgroup, histograms in the slab buffers) instead of in a launch of its own
        if (block < p.csr_blocks) {
            if (tid >= p.csr_threads) return;
            csr_count_body(reinterpret_cast<int32_t *>(smem), block, tid, p.csr_threads, p.Ind, p.ind_dtype, p.T, p.E * p.K,
                           p.seg_off, p.perm, p.rank_tmp, p.long_tab);
            return;
        }
        block -= p.csr_blocks;
    }
    int e, tile;
    if (!decode_expert_tile(block, p.m_tiles * p.n_tiles, p.E, e, tile)) return;
    const int mt = tile / p.n_tiles, nt = tile - mt * p.n_tiles;
    const int m0 = mt * BM, n0 = nt * BN;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int R = p.R, N = p.N;
    const int Me = p.B * p.K;

    // ---------------- per-row bookkeeping: byte offset each tile row reads from, element offset it writes to
    if (tid < BM) {
        int m = m0 + tid;
        uint32_t ao = kVoffInvalid;
        int64_t co = -1;
        if (m < Me) {
            int b = m / p.K, k = m - b * p.K;
            int64_t pick = ((int64_t)b * p.E + e) * p.K + k;
            if constexpr (GATHER) {
                int32_t t = load_token(p.Ind, p.ind_dtype, pick, p.T);
                if (t >= 0) ao = (uint32_t)(((int64_t)b * p.lda_b + (int64_t)t * p.lda_t) * 2);
            } else {
                ao = (uint32_t)(pick * R * 2);
            }
            co = pick * N;
        }
        a_voff[tid] = ao;
        c_off[tid] = co;
    }
    __syncthreads();

    const u32x4 rs_a = make_rsrc(p.A, p.a_bytes);
    const u32x4 rs_w = make_rsrc(p.W + (size_t)e * R * N * WES, (uint32_t)((size_t)R * N * WES));

    // ---------------- loader set-up: each wavefront issues 4 loads per operand per slab
    // K-major tile [256 rows][8 chunks]: load j covers rows 8j..8j+7; lane l lands on row 8j + l/8,
    // physical chunk l%8, and therefore fetches logical chunk (l%8) ^ (l/8).
    uint32_t pv[4], qv[4];
    {
        const int lc = (lane & 7) ^ (lane >> 3);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            uint32_t ao = a_voff[(wave * 4 + jj) * 8 + (lane >> 3)];
            pv[jj] = ao == kVoffInvalid ? kVoffInvalid : ao + lc * 16;
            if constexpr (!W_TRANS) {
                int row = (wave * 4 + jj) * 8 + (lane >> 3);
                int n = n0 + row;
                qv[jj] = n < N ? (uint32_t)n * (uint32_t)R * 2 + ((lane & 7) ^ kmajor_key_relabelled(row)) * 16 : kVoffInvalid;
            } else if constexpr (W_FP8) {
                // bytes, [64 reduction rows][16 chunks]: load j (two per wavefront) covers rows 4j..4j+3; lane l lands
                // on row 4j + l/16, physical chunk l%16; chunks are XORed with the low four bits of the row so that
                // the 32 rows one transpose read touches spread over all banks
                int row = (wave * 2 + (jj & 1)) * 4 + (lane >> 4);
                int lchunk = (lane & 15) ^ (row & 15);
                int n = n0 + lchunk * 16;
                qv[jj] = (jj < 2 && n < N) ? (uint32_t)row * (uint32_t)N + n : kVoffInvalid;
            } else {
                // [64 reduction rows][32 chunks]: load j covers rows 2j, 2j+1; lane l lands on row 2j + l/32,
                // physical chunk l%32
                int row = (wave * 4 + jj) * 2 + (lane >> 5);
                int pc = lane & 31;
                int lchunk = ((((pc >> 1) ^ tr_swizzle(row)) << 1) | (pc & 1));
                int n = n0 + lchunk * 8;
                qv[jj] = n < N ? ((uint32_t)row * (uint32_t)N + n) * 2 : kVoffInvalid;
            }
        }
    }
    auto issue = [&](int kt, int stage) {
        char *base = smem + stage * kDlStageBytes + wave * 4096;
        const uint32_t so_a = (uint32_t)kt * (BK * 2);
        const uint32_t so_w = W_TRANS ? (uint32_t)kt * BK * (uint32_t)N * WES : (uint32_t)kt * (BK * 2);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) direct_load16(rs_a, pv[jj], so_a, base + jj * 1024);
        if constexpr (W_FP8) {
            char *qbase = smem + stage * kDlStageBytes + kDlTileBytes + wave * 2048;
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) direct_load16(rs_w, qv[jj], so_w, qbase + jj * 1024);
        } else {
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) direct_load16(rs_w, qv[jj], so_w, base + kDlTileBytes + jj * 1024);
        }
    };

    // ---------------- fragment addresses
    const int a = lane & 15, g = lane >> 4;
    const int wave_m0 = (wave >> 2) * 128, wave_n0 = (wave & 3) * 64;
    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // row-side: row = wave_m0 + 16 i + a, physical chunk (4 ks + g) ^ (a & 7)
    int m_at[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) m_at[ks] = (wave_m0 + a) * 128 + (((ks * 4 + g) ^ (a & 7)) << 4);
    // weight-side, K-major: rows relabelled so that a lane ends up with 16 consecutive output columns
    //   row(j) = wave_n0 + 16 (a/4) + 4 j + a%4
    // weight-side, [reduction][column]: lane supplies row 32 ks + 8 g + 4 h + a/4 and columns
    //   wave_n0 + 16 j + 4 (a%4) .. +3, so it receives column wave_n0 + 16 j + a
    int n_at[2][2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            if constexpr (!W_TRANS) {
                int row = wave_n0 + (a >> 2) * 16 + x * 4 + (a & 3);          // j = x (mod 2); + 8 rows per j/2
                n_at[ks][x] = row * 128 + (((ks * 4 + g) ^ kmajor_key_relabelled(row)) << 4);
            } else if constexpr (W_FP8) {
                int row = ks * 32 + g * 8 + (a >> 1);                         // one read per fragment; x unused
                n_at[ks][x] = row * 256 + (((wave_n0 >> 4) ^ (row & 15)) << 4) + (a & 1) * 8;
            } else {
                int row = ks * 32 + g * 8 + x * 4 + (a >> 2);                 // x = h
                n_at[ks][x] = row * 512 + (((wave_n0 >> 4) ^ tr_swizzle(row)) << 5) + (a & 3) * 8;
            }
        }

    const int nk = R / BK;
    issue(0, 0);
    for (int kt = 0; kt < nk; ++kt) {
        wait_vmem<0>();
        __syncthreads();            // slab kt visible to all; everyone is done reading the other stage
        if (kt + 1 < nk) issue(kt + 1, (kt + 1) & 1);
        const char *tile_m = smem + (kt & 1) * kDlStageBytes;
        const char *tile_n = tile_m + kDlTileBytes;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            u32x4 mf[TM], nf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) mf[i] = *reinterpret_cast<const u32x4 *>(tile_m + m_at[ks] + i * 2048);
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (!W_TRANS) {
                    nf[j] = *reinterpret_cast<const u32x4 *>(tile_n + n_at[ks][j & 1] + (j >> 1) * 1024);
                } else if constexpr (W_FP8) {
                    u32x2 q8 = lds_read_tr8(tile_n + (n_at[ks][0] ^ (j << 4)));      // chunk wave_n0/16 + j, j < 4
                    nf[j] = fp8x8_to_bf16_chunk(q8[0], q8[1]);
                } else {
                    // unit index wave_n0/16 + j: XOR with the swizzle commutes with adding j only bitwise,
                    // so fold j in by XOR on the unit field (wave_n0/16 is a multiple of 4, j < 4)
                    u32x2 lo = lds_read_tr16(tile_n + (n_at[ks][0] ^ (j << 5)));
                    u32x2 hi = lds_read_tr16(tile_n + (n_at[ks][1] ^ (j << 5)));
                    nf[j] = u32x4{lo[0], lo[1], hi[0], hi[1]};
                }
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) mma_chunk<TT>(acc[i][j], nf[j], mf[i]);
        }
    }

    // ---------------- epilogue: 4 (transposed weights) or 16 (K-major weights) consecutive columns per lane and row
    constexpr int OES = (EPI == EPI_STORE_F32) ? 4 : 2;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        int64_t co = c_off[wave_m0 + i * 16 + a];
        if (co < 0) continue;
        char *crow = p.C + co * OES;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            int n = n0 + wave_n0 + (W_TRANS ? j * 16 + g * 4 : g * 16 + j * 4);
            if (n >= N) continue;              // N % 8 == 0 and n % 4 == 0: the 4 columns are all in or all out
            f32x4 v = acc[i][j];
            if (p.w_scale != nullptr) {
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] *= p.w_scale[(size_t)e * N + n + r];
            }
            if constexpr (OES == 4) {
                *reinterpret_cast<f32x4 *>(crow + (size_t)n * 4) = v;
            } else {
                u32x2 w;
                w[0] = pack2<TT>(v[0], v[1]);
                w[1] = pack2<TT>(v[2], v[3]);
                *reinterpret_cast<u32x2 *>(crow + (size_t)n * 2) = w;
            }
        }
    }
}

}  // namespace egs
