// The rows x weight product of egs_rows_gemm.h for large, well-formed 16-bit shapes, built around
// what gfx950 adds for this: 16-byte direct global->LDS loads and LDS transpose reads.
//
//   * BM x BN output tile (BM = 128 or 256, BN = 256, or 128 for outputs narrower than 192 columns),
//     BK-deep slabs (32 or 64), BM/128 x BN/64 wavefronts, each 128 x 64 of the tile.
//   * Both operand slabs travel HBM/L2 -> LDS without touching registers (one buffer load per
//     1 KB of a slab), NSTAGE - 1 slabs in flight: the loads of slab k + NSTAGE - 1 are issued
//     right after the barrier that publishes slab k and land while the MFMAs run.  One barrier
//     per slab.  The shape in use is 256 x 256 x 64 with two stages (one 134 KB workgroup per CU, fewest
//     bytes moved per flop); 128 x 256 x 32 with two or three stages (two or three workgroups per
//     CU) and 256 x 256 x 32 with four stages compile as well but measured slower on every benchmark
//     configuration (the loads are bound by bandwidth beyond the L2, not by latency, and 32-deep slabs
//     pay twice the barriers).
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

// LDS bytes of one workgroup: slab stages (rows in 16-bit elements, weights in WES-byte elements), then the row tables
// (4 + 8 bytes per tile row)
__host__ __device__ constexpr int dl_stage_bytes(int BM, int BN, int BK, int WES = 2) { return (BM * 2 + BN * WES) * BK; }
__host__ __device__ constexpr int dl_smem_bytes(int BM, int BN, int BK, int NSTAGE, int WES = 2)
{
    return NSTAGE * dl_stage_bytes(BM, BN, BK, WES) + BM * 12;
}
// the scatter variants of the one-workgroup-per-CU shape reserve more, so that the routing-table
// workgroups riding along have room for eight wavefronts' histograms at T = 4096
__host__ __device__ constexpr int dl_smem_bytes_scatter(int BM, int BN, int BK, int NSTAGE)
{
    return BM == 256 && BN == 256 ? 150 * 1024 : dl_smem_bytes(BM, BN, BK, NSTAGE);
}
__host__ __device__ constexpr int dl_threads(int BM, int BN) { return (BM / 128) * (BN / 64) * 64; }

// swizzle of the [reduction][column] tile: 32-byte units of a row are XORed with bits {0,1,3} of
// the row number, which spreads the 16 rows one transpose read touches over all banks
__device__ __forceinline__ int tr_swizzle(int row) { return (row & 3) | (((row >> 3) & 1) << 2); }
// swizzle key of the K-major tiles (XORed into the 16-byte chunk index of a row of CR chunks), chosen so
// that the 16 lanes of one fragment read (16 consecutive rows) hit 16 different 16-byte bank groups.
template <int CR> __device__ __forceinline__ int kmajor_key_rows(int row) { return CR == 8 ? (row & 7) : ((row >> 2) & 3); }

template <class TT, int WES, int BM, int BN, int BK, int NSTAGE, bool GATHER, bool W_TRANS, int EPI>
// (four-wavefront workgroups on 32-deep slabs are meant to run two to a CU: at most 256 registers per wavefront)
__global__ __launch_bounds__(dl_threads(BM, BN), (BK == 32 && dl_threads(BM, BN) == 256) ? 2 : 1) void rows_gemm_dl_kernel(RowsGemmParams p)
{
    static_assert(TT::ES == 2, "16-bit element types");
    static_assert(EPI == EPI_STORE || EPI == EPI_STORE_F32, "plain stores only");
    static_assert(WES == 2 || (WES == 1 && W_TRANS && TT::ID == 2), "fp8 weights: [reduction][column] layout, widened to bf16");
    static_assert((BM == 128 || BM == 256) && (BN == 128 || BN == 256) && (BK == 32 || BK == 64) &&
                  (NSTAGE >= 2 && NSTAGE <= 4), "tile shapes");
    constexpr bool W_FP8 = (WES == 1);
    static_assert(!W_FP8 || BN == 256, "the fp8 tile layout is written for 256-byte rows");
    constexpr int WN = BN / 64;                          // wavefront columns
    constexpr int NT = dl_threads(BM, BN), NW = NT / 64; // BM/128 x BN/64 wavefronts
    constexpr int TM = 8, TN = 4;                        // 16 x 16 tiles per wavefront: 128 x 64
    constexpr int KSTEPS = BK / 32;
    constexpr int CR = BK / 8;                           // 16-byte chunks per K-major row
    constexpr int P_BYTES = BM * BK * 2, STAGE = dl_stage_bytes(BM, BN, BK, WES);
    constexpr int PL = BM * CR / 64 / NW;                // loads per wavefront and slab: row side,
    constexpr int WROW = BN * 2;                         // bytes of a [reduction][column] tile row (16-bit)
    constexpr int QL = W_FP8 ? BK / 4 / NW : (W_TRANS ? BK * WROW / 1024 / NW : BN * CR / 64 / NW);   // weight side
    static_assert(PL >= 1 && QL >= 1 && PL + QL < 16, "loads per slab");

    __shared__ __attribute__((aligned(1024))) char smem[GATHER ? dl_smem_bytes(BM, BN, BK, NSTAGE, WES)
                                                               : dl_smem_bytes_scatter(BM, BN, BK, NSTAGE)];
    uint32_t *a_voff = reinterpret_cast<uint32_t *>(smem + NSTAGE * STAGE);
    int64_t *c_off = reinterpret_cast<int64_t *>(smem + NSTAGE * STAGE + BM * 4);

    const int tid = (int)threadIdx.x;
    int block = (int)blockIdx.x;
    if constexpr (!GATHER) {
        // the scatter's routing table does not depend on the product: one workgroup per batch element
        // builds it here (csr_threads of the workgroup, histograms in the slab buffers) instead of in a launch of its own
        if (block < p.csr_blocks) {
            if (tid >= p.csr_threads) return;
            const int cb = block / p.csr_parts;
            csr_count_body(reinterpret_cast<int32_t *>(smem), cb, cb, tid, p.csr_threads, p.Ind, p.ind_dtype, p.T, p.E * p.K,
                           p.seg_off, p.perm, p.rank_tmp, p.long_tab, NoPrefetch(), block - cb * p.csr_parts, p.csr_parts);
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

    // ---------------- loader set-up.  One load covers 1 KB of a tile = 64 / CR rows of a K-major tile;
    // lane l lands on row (64 / CR) j + l / CR, physical chunk l % CR, and therefore fetches the logical
    // chunk (l % CR) ^ key(row).
    uint32_t pv[PL], qv[QL];
#pragma unroll
    for (int jj = 0; jj < PL; ++jj) {
        const int row = (wave * PL + jj) * (64 / CR) + lane / CR;
        const uint32_t ao = a_voff[row];
        pv[jj] = ao == kVoffInvalid ? kVoffInvalid : ao + (((lane % CR) ^ kmajor_key_rows<CR>(row)) << 4);
    }
#pragma unroll
    for (int jj = 0; jj < QL; ++jj) {
        if constexpr (!W_TRANS) {
            const int row = (wave * QL + jj) * (64 / CR) + lane / CR;
            const int n = n0 + row;
            qv[jj] = n < N ? (uint32_t)n * (uint32_t)R * 2 + (((lane % CR) ^ kmajor_key_rows<CR>(row)) << 4) : kVoffInvalid;
        } else if constexpr (W_FP8) {
            // bytes, [BK reduction rows][16 chunks]: a load covers 4 rows; lane l lands on row 4j + l/16, physical
            // chunk l%16; chunks are XORed with the low four bits of the row so that the 32 rows one transpose
            // read touches spread over all banks
            const int row = (wave * QL + jj) * 4 + (lane >> 4);
            const int n = n0 + ((lane & 15) ^ (row & 15)) * 16;
            qv[jj] = n < N ? (uint32_t)row * (uint32_t)N + n : kVoffInvalid;
        } else {
            // [BK reduction rows][BN/8 chunks]: a load covers 2 (4) rows of 32 (16) chunks; lane l lands on
            // row 2j + l/32 (4j + l/16), physical chunk l%32 (l%16)
            constexpr int LPR = WROW / 16;               // lanes (chunks) per row
            const int row = (wave * QL + jj) * (64 / LPR) + lane / LPR;
            const int pc = lane % LPR;
            const int n = n0 + ((((pc >> 1) ^ tr_swizzle(row)) << 1) | (pc & 1)) * 8;
            qv[jj] = n < N ? ((uint32_t)row * (uint32_t)N + n) * 2 : kVoffInvalid;
        }
    }
    auto issue = [&](int kt, int stage) {
        char *pbase = smem + stage * STAGE + wave * (PL * 1024);
        char *qbase = smem + stage * STAGE + P_BYTES + wave * (QL * 1024);
        const uint32_t so_a = (uint32_t)kt * (BK * 2);
        const uint32_t so_w = W_TRANS ? (uint32_t)kt * BK * (uint32_t)N * WES : (uint32_t)kt * (BK * 2);
#pragma unroll
        for (int jj = 0; jj < PL; ++jj) direct_load16(rs_a, pv[jj], so_a, pbase + jj * 1024);
#pragma unroll
        for (int jj = 0; jj < QL; ++jj) direct_load16(rs_w, qv[jj], so_w, qbase + jj * 1024);
    };

    // ---------------- fragment addresses
    const int a = lane & 15, g = lane >> 4;
    const int wave_m0 = (wave / WN) * 128, wave_n0 = (wave % WN) * 64;
    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // row side: row = wave_m0 + 16 i + a (key does not depend on i), physical chunk (4 ks + g) ^ key
    int m_at[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
        m_at[ks] = (wave_m0 + a) * (BK * 2) + (((ks * 4 + g) ^ kmajor_key_rows<CR>(wave_m0 + a)) << 4);
    // weight side, K-major: row(j) = wave_n0 + 16 j + a, read like the row side
    // weight side, [reduction][column]: lane supplies row 32 ks + 8 g + 4 h + a/4 and columns
    //   wave_n0 + 16 j + 4 (a%4) .. +3, so it receives column wave_n0 + 16 j + a   (fp8: row 32 ks + 8 g + a/2,
    //   bytes 8 (a%2) .. +7 of the 16-byte chunk of tile j)
    int n_at[KSTEPS][2];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if constexpr (!W_TRANS) {
                const int row = wave_n0 + a;                    // + 16 j: the key does not depend on j
                n_at[ks][h] = row * (BK * 2) + (((ks * 4 + g) ^ kmajor_key_rows<CR>(row)) << 4);
            } else if constexpr (W_FP8) {
                const int row = ks * 32 + g * 8 + (a >> 1);
                n_at[ks][h] = row * 256 + (((wave_n0 >> 4) ^ (row & 15)) << 4) + (a & 1) * 8;
            } else {
                const int row = ks * 32 + g * 8 + h * 4 + (a >> 2);
                n_at[ks][h] = row * WROW + (((wave_n0 >> 4) ^ tr_swizzle(row)) << 5) + (a & 3) * 8;
            }
        }

    const int nk = R / BK;
#pragma unroll
    for (int st = 0; st < NSTAGE - 1; ++st)
        if (st < nk) issue(st, st);
    int stage = 0;
    for (int kt = 0; kt < nk; ++kt) {
        // slab kt has landed once at most the loads of the slabs issued after it are outstanding
        {
            const int later = min(nk - 1 - kt, NSTAGE - 2);     // slabs requested after slab kt that may stay in flight
            if (NSTAGE >= 4 && later >= 2) wait_vmem<(NSTAGE >= 4 ? 2 * (PL + QL) : 0)>();
            else if (NSTAGE >= 3 && later >= 1) wait_vmem<(NSTAGE >= 3 ? PL + QL : 0)>();
            else wait_vmem<0>();
        }
        __syncthreads();            // slab kt visible to all; everyone is done reading the stage refilled next
        if (kt + NSTAGE - 1 < nk) {
            int fill = stage + NSTAGE - 1;
            if (fill >= NSTAGE) fill -= NSTAGE;
            issue(kt + NSTAGE - 1, fill);
        }
        const char *tile_m = smem + stage * STAGE;
        const char *tile_n = tile_m + P_BYTES;
        // Fragment reads run one step ahead of the MFMAs that use them: the row fragments of the next pair
        // of 16-row tiles (and, at the end of a reduction step, the weight fragments of the next step) are
        // requested before the eight MFMAs of the current pair are issued, so a wavefront's LDS latency is
        // covered by its own MFMAs instead of stalling them.
        auto read_n = [&](int ks, u32x4 (&nr)[TN]) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (!W_TRANS) {
                    nr[j] = *reinterpret_cast<const u32x4 *>(tile_n + n_at[ks][0] + j * (16 * BK * 2));
                } else if constexpr (W_FP8) {
                    const u32x2 q8 = lds_read_tr8(tile_n + (n_at[ks][0] ^ (j << 4)));       // chunk wave_n0/16 + j, j < 4
                    nr[j] = u32x4{q8[0], q8[1], 0u, 0u};                                    // widened at first use
                } else {
                    // unit wave_n0/16 + j: wave_n0/16 is a multiple of 4 and j < 4, so j folds in by XOR
                    const u32x2 lo = lds_read_tr16(tile_n + (n_at[ks][0] ^ (j << 5)));
                    const u32x2 hi = lds_read_tr16(tile_n + (n_at[ks][1] ^ (j << 5)));
                    nr[j] = u32x4{lo[0], lo[1], hi[0], hi[1]};
                }
            }
        };
        auto read_m2 = [&](int ks, int ip, u32x4 (&mr)[2]) {
            mr[0] = *reinterpret_cast<const u32x4 *>(tile_m + m_at[ks] + (2 * ip) * (16 * BK * 2));
            mr[1] = *reinterpret_cast<const u32x4 *>(tile_m + m_at[ks] + (2 * ip + 1) * (16 * BK * 2));
        };
        constexpr int PAIRS = TM / 2;
        u32x4 nraw[2][TN], mf[2][2];
        read_n(0, nraw[0]);
        read_m2(0, 0, mf[0]);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            u32x4 nf[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (W_FP8) nf[j] = fp8x8_to_bf16_chunk(nraw[ks & 1][j][0], nraw[ks & 1][j][1]);
                else nf[j] = nraw[ks & 1][j];
            }
#pragma unroll
            for (int ip = 0; ip < PAIRS; ++ip) {
                const int cur = (ks * PAIRS + ip) & 1;
                if (ip + 1 < PAIRS) {
                    read_m2(ks, ip + 1, mf[cur ^ 1]);
                } else if (ks + 1 < KSTEPS) {
                    read_n(ks + 1, nraw[(ks + 1) & 1]);
                    read_m2(ks + 1, 0, mf[cur ^ 1]);
                }
                __builtin_amdgcn_sched_barrier(0);      // the requests above stay ahead of the MFMAs below
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int j = 0; j < TN; ++j) mma_chunk<TT>(acc[2 * ip + h][j], nf[j], mf[cur][h]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (++stage == NSTAGE) stage = 0;
    }

    constexpr int OES = (EPI == EPI_STORE_F32) ? 4 : 2;
    if constexpr (OES == 4) {
        // fp32 product rows: measured slightly faster straight from registers than through LDS
        // ---------------- epilogue.  After the MFMAs lane (a, g) holds, for row 16 i + a, the four columns
        // 16 j + 4 g .. + 3.  The values are regrouped across lanes first (lane 4 r + c takes piece c of row r),
        // so that the four pieces of a row, 64 contiguous bytes of fp32 or 32 of a 16-bit type, leave from
        // adjacent lanes as one access.
        const int srow = lane >> 2, sg = lane & 3;
    #pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int64_t co = c_off[wave_m0 + i * 16 + srow];
            char *crow = p.C + co * OES;
    #pragma unroll
            for (int j = 0; j < TN; ++j) {
                f32x4 v = acc[i][j];
                if (p.w_scale != nullptr) {
                    const int nn = n0 + wave_n0 + j * 16 + g * 4;
    #pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] *= nn + r < N ? p.w_scale[(size_t)e * N + nn + r] : 0.f;
                }
                const int n = n0 + wave_n0 + j * 16 + sg * 4;      // N % 8 == 0 and n % 4 == 0: the 4 columns are all in or all out
                if constexpr (OES == 4) {
                    const u32x4 w = lanes_16g_a_to_4a_g(__builtin_bit_cast(u32x4, v), lane);
                    if (co >= 0 && n < N) *reinterpret_cast<u32x4 *>(crow + (size_t)n * 4) = w;
                } else {
                    u32x4 w = {pack2<TT>(v[0], v[1]), pack2<TT>(v[2], v[3]), 0u, 0u};
                    w = lanes_16g_a_to_4a_g(w, lane);
                    if (co >= 0 && n < N) *reinterpret_cast<u32x2 *>(crow + (size_t)n * 2) = u32x2{w[0], w[1]};
                }
            }
        }
    } else {
        // ---------------- epilogue.  After the MFMAs lane (a, g) holds, for row 16 i + a, the four columns
        // 16 j + 4 g .. + 3: pieces of 16 rows per store.  The tile goes through LDS instead (the slab stages are
        // free now), 128 rows of fp32 (or all 256 rows of a 16-bit type) at a time, and leaves as whole row
        // segments: one store instruction writes 1 KB of one row (fp32) or 512 bytes of each of two rows, which
        // is what the write path wants (product rows are the largest stream of the scatter: 1 GB at C3).
        // LDS row = BN columns; its 16-byte chunks are XORed with the low four row bits so that the 16 lanes
        // of a fragment (16 rows, same chunk) spread over the banks.
        constexpr int ROW_BYTES = BN * OES;                 // 1024 or 512
        constexpr int HALVES = (BM * ROW_BYTES) / (NSTAGE * STAGE) > 1 ? 2 : ((BM * ROW_BYTES > NSTAGE * STAGE) ? 2 : 1);
        constexpr int ROWS_PER_PASS = BM / HALVES;
        static_assert(ROWS_PER_PASS * ROW_BYTES <= NSTAGE * STAGE, "staging tile fits the slab stages");
        static_assert(HALVES == 1 || BM == 256, "two passes split the two wavefront rows of a 256-row tile");
        constexpr int CPR = ROW_BYTES / 16;                  // chunks per staged row: 64 or 32
    #pragma unroll 1
        for (int half = 0; half < HALVES; ++half) {
            __syncthreads();                                // stages (or the previous pass) no longer being read
            if (HALVES == 1 || (wave / WN) == half) {
                const int row0 = (HALVES == 1 ? wave_m0 : 0) + a;
    #pragma unroll
                for (int i = 0; i < TM; ++i) {
                    const int row = row0 + i * 16;
    #pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        f32x4 v = acc[i][j];
                        const int col = wave_n0 + j * 16 + g * 4;
                        if (p.w_scale != nullptr) {
    #pragma unroll
                            for (int r = 0; r < 4; ++r) v[r] *= n0 + col + r < N ? p.w_scale[(size_t)e * N + n0 + col + r] : 0.f;
                        }
                        if constexpr (OES == 4) {
                            const int chunk = (col >> 2) ^ (row & 15);
                            *reinterpret_cast<f32x4 *>(smem + row * ROW_BYTES + chunk * 16) = v;
                        } else {
                            const int chunk = (col >> 3) ^ (row & 15);
                            u32x2 w = {pack2<TT>(v[0], v[1]), pack2<TT>(v[2], v[3])};
                            *reinterpret_cast<u32x2 *>(smem + row * ROW_BYTES + chunk * 16 + (col & 4) * 2) = w;
                        }
                    }
                }
            }
            __syncthreads();
            // every wavefront writes out its share of the staged rows, whole row segments per instruction
            constexpr int LANES_PER_ROW = CPR;               // 64 (one row per instruction) or 32 (two rows)
            constexpr int ROWS_PER_INSTR = 64 / LANES_PER_ROW;
            const int lrow = lane / LANES_PER_ROW, lchunk = lane % LANES_PER_ROW;
            const int n_here = n0 + lchunk * (16 / OES);
            for (int r0 = wave * ROWS_PER_INSTR; r0 < ROWS_PER_PASS; r0 += NW * ROWS_PER_INSTR) {
                const int row = r0 + lrow;
                const int64_t co = c_off[half * ROWS_PER_PASS + row];
                const u32x4 v = *reinterpret_cast<const u32x4 *>(smem + row * ROW_BYTES + ((lchunk ^ (row & 15)) << 4));
                if (co >= 0 && n_here < N) *reinterpret_cast<u32x4 *>(p.C + co * OES + (size_t)n_here * OES) = v;
            }
        }
    }
}

}  // namespace egs
