// Per-expert "rows x weight" product with an index on one side:
//
//   gather   C[m, n] = sum_r A[b, Ind[m], r] * Wt(n, r)     rows of A fetched through Ind, C dense
//   scatter  C[b, Ind[m], n] += sum_r A[m, r] * Wt(n, r)    A dense, rows of C addressed through Ind
//
// where m = b*K + k enumerates the picks of one expert e.  One workgroup owns a BM x BN tile
// of one expert's product, stages BK-wide slabs of both operands in K-major swizzled LDS
// tiles (register prefetch of the next slab overlaps the MFMAs of the current one) and runs
// 16x16 MFMA tiles on WM x WN wavefronts (4 for the 128-wide tiles, 8 for the 256 x 256 tile
// whose higher reuse matters once both operands stream through L2).
//
// Replaces the reference's expert_gather_kernel (egs/triton_kernels.py:49-143) and
// expert_scatter_kernel (:156-247).  Unlike those, the M dimension of a tile is the picks of
// one expert (not batch rows of one (e,k)), so W[e] is read once per tile instead of once
// per pick.
#pragma once
#include "egs_device.h"

namespace egs {

enum : int { EPI_STORE = 0, EPI_STORE_F32 = 1, EPI_ATOMIC_F32 = 2 };

struct RowsGemmParams {
    const char *A;          // gather: [B,T,R] source;  scatter: [B,E,K,R] dense rows
    const char *W;          // [E,R,N] (W_TRANS) or [E,N,R]
    const void *Ind;        // [B,E,K]
    char *C;                // gather: [B,E,K,N];  scatter: fp32 [B,E,K,N] rows or fp32 [B,T,N] accumulator
    const float *w_scale;   // [E,N] or nullptr
    int32_t B, T, E, K;
    int32_t R, N;           // reduction length, output columns
    int64_t lda_b, lda_t;   // element strides of the [B,T,R] source (gather)
    int32_t ind_dtype;
    int32_t a_vec, w_vec, c_vec;   // 1 when 16-byte accesses are safe on that tensor
    int32_t m_tiles, n_tiles;
    uint32_t a_bytes;       // extent of A in bytes when it is below 2 GiB, else 0 (direct-load kernel only)
    // routing table of the scatter built by the first csr_blocks (= B) workgroups of the product launch
    // (direct-load kernel only; csr_done reports that the launch took it along)
    // csr_parts workgroups share a batch element's table (csr_blocks = B * csr_parts; set by the launcher)
    int32_t csr_blocks, csr_done, csr_threads, csr_parts;
    int32_t *seg_off, *perm, *rank_tmp, *long_tab;
};

template <class TT, int WES, int BM, int BN, int BK, int WM, int WN, bool GATHER, bool W_TRANS, int EPI>
__global__ __launch_bounds__(WM * WN * kWave) void rows_gemm_kernel(RowsGemmParams p)
{
    constexpr int NT = WM * WN * kWave;          // threads per workgroup: one wavefront per (WM, WN) cell
    constexpr int ES = TT::ES, VEC = TT::VEC;
    constexpr int CH = BK / VEC;                 // chunks per LDS row
    constexpr int KSTEPS = CH / 4;               // MFMA chunk steps per slab
    constexpr bool SWAP = (EPI == EPI_ATOMIC_F32);   // atomics want consecutive n across lanes
    constexpr int TM = BM / WM / 16, TN = BN / WN / 16;
    constexpr bool W_FP8 = (WES == 1);
    static_assert(BM <= NT, "row bookkeeping uses one thread per tile row");
    static_assert((BM * CH) % NT == 0 && NT % CH == 0, "M loader mapping");
    static_assert(!W_FP8 || TT::ES == 2, "fp8 weights are widened to bf16");

    __shared__ __attribute__((aligned(16))) char smem_m[BM * BK * ES];
    __shared__ __attribute__((aligned(16))) char smem_n[BN * BK * ES];
    __shared__ int64_t a_off[BM];
    __shared__ int64_t c_off[BM];

    int e, tile;
    if (!decode_expert_tile((int)blockIdx.x, p.m_tiles * p.n_tiles, p.E, e, tile)) return;
    const int mt = tile / p.n_tiles, nt = tile - mt * p.n_tiles;
    const int m0 = mt * BM, n0 = nt * BN;
    const int tid = (int)threadIdx.x;
    const int R = p.R, N = p.N;
    const char *We = p.W + (size_t)e * R * N * WES;
    const bool w_vec = p.w_vec != 0, a_vec = p.a_vec != 0;

    // ---------------- weight-side loader
    constexpr int NVN = (BN * CH + NT - 1) / NT;            // K-major: chunks per thread
    // transposed: blocks of VEC reduction rows x BW output columns (16-bit: 8 x 4 so that every
    // thread gets one block and holds 16 registers of it; fp32: 4 x 4)
    constexpr int BW = 4;
    constexpr int KB = BK / VEC, NBK = BN / BW;
    constexpr int NBL = (KB * NBK + NT - 1) / NT;
    u32x4 nreg[W_TRANS ? (VEC == 8 ? NBL * 4 : NBL * VEC) : NVN];     // 16-bit blocks: 8 x u32x2 packed in 4 x u32x4

    auto issue_n = [&](int kt) {
        if constexpr (!W_TRANS) {
#pragma unroll
            for (int i = 0; i < NVN; ++i) {
                int v = tid + i * NT;
                int row = v / CH, c = v % CH;
                int n = n0 + row;
                const char *ptr = (v < BN * CH && n < N) ? We + (size_t)n * R * WES : nullptr;
                if constexpr (W_FP8) nreg[i] = load_chunk_fp8_as_bf16(ptr, kt * BK + c * VEC, R, w_vec);
                else nreg[i] = load_chunk<ES>(ptr, kt * BK + c * VEC, R, w_vec);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NBL; ++i) {
                int blk = tid + i * NT;
                int kb = blk / NBK, nb = blk % NBK;
#pragma unroll
                for (int r = 0; r < VEC; ++r) {
                    int rr = kt * BK + kb * VEC + r;
                    const char *ptr = (blk < KB * NBK && rr < R) ? We + (size_t)rr * N * WES : nullptr;
                    if constexpr (VEC == 8) {
                        u32x2 h;
                        if constexpr (W_FP8) h = load_half_chunk_fp8_as_bf16(ptr, n0 + nb * BW, N, w_vec);
                        else h = load_half_chunk16(ptr, n0 + nb * BW, N, w_vec);
                        nreg[i * 4 + (r >> 1)][(r & 1) * 2] = h[0];
                        nreg[i * 4 + (r >> 1)][(r & 1) * 2 + 1] = h[1];
                    } else {
                        nreg[i * VEC + r] = load_chunk<ES>(ptr, n0 + nb * BW, N, w_vec);
                    }
                }
            }
        }
    };
    auto commit_n = [&]() {
        u32x4 *tile_n = reinterpret_cast<u32x4 *>(smem_n);
        if constexpr (!W_TRANS) {
#pragma unroll
            for (int i = 0; i < NVN; ++i) {
                int v = tid + i * NT;
                if (v < BN * CH) tile_n[tile_chunk_index<CH>(v / CH, v % CH)] = nreg[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < NBL; ++i) {
                int blk = tid + i * NT;
                int kb = blk / NBK, nb = blk % NBK;
                if (blk < KB * NBK) {
                    u32x4 out[4];
                    if constexpr (VEC == 8) {
                        u32x2 in[8];
#pragma unroll
                        for (int r = 0; r < 8; ++r)
                            in[r] = u32x2{nreg[i * 4 + (r >> 1)][(r & 1) * 2], nreg[i * 4 + (r >> 1)][(r & 1) * 2 + 1]};
                        transpose8x4_16b(in, out);
                    } else {
                        u32x4 in[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) in[r] = nreg[i * VEC + r];
                        transpose4x4_32b(in, out);
                    }
#pragma unroll
                    for (int c = 0; c < BW; ++c) tile_n[tile_chunk_index<CH>(nb * BW + c, kb)] = out[c];
                }
            }
        }
    };

    issue_n(0);     // does not depend on Ind: overlap with the index fetch below

    // ---------------- per-row bookkeeping: where each tile row reads from / writes to
    // (atomic epilogue: whether two rows of the tile land on the same token is found here, with a bitmap over
    // (batch element, token) mod kDupBits in the not yet used slab buffer - exact for the rows of one batch element
    // while T <= kDupBits, on the safe side otherwise)
    constexpr int kDupBits = 16384;
    static_assert(EPI != EPI_ATOMIC_F32 || BM * BK * ES >= kDupBits / 8, "bitmap fits the slab buffer");
    int dup_row = 0;
    if constexpr (EPI == EPI_ATOMIC_F32) {
        uint32_t *bitmap = reinterpret_cast<uint32_t *>(smem_m);
        for (int i = tid; i < kDupBits / 32; i += NT) bitmap[i] = 0u;
        __syncthreads();
    }
    const int Me = p.B * p.K;
    if (tid < BM) {
        int m = m0 + tid;
        int64_t ao = -1, co = -1;
        if (m < Me) {
            int b = m / p.K, k = m - b * p.K;
            int64_t pick = ((int64_t)b * p.E + e) * p.K + k;
            if constexpr (GATHER) {
                int32_t t = load_token(p.Ind, p.ind_dtype, pick, p.T);
                ao = t < 0 ? -1 : (int64_t)b * p.lda_b + (int64_t)t * p.lda_t;
                co = pick * N;
            } else {
                ao = pick * R;
                if constexpr (EPI == EPI_ATOMIC_F32) {
                    int32_t t = load_token(p.Ind, p.ind_dtype, pick, p.T);
                    co = t < 0 ? -1 : ((int64_t)b * p.T + t) * N;
                    if (t >= 0) {
                        const uint32_t key = (uint32_t)((int64_t)b * p.T + t) & (kDupBits - 1);
                        const uint32_t bit = 1u << (key & 31);
                        dup_row = (atomicOr(reinterpret_cast<uint32_t *>(smem_m) + (key >> 5), bit) & bit) != 0;
                    }
                } else {
                    co = pick * N;
                }
            }
        }
        a_off[tid] = ao;
        c_off[tid] = co;
    }
    bool tile_has_dups = false;
    if constexpr (EPI == EPI_ATOMIC_F32) tile_has_dups = __syncthreads_or(dup_row) != 0;
    else __syncthreads();

    // ---------------- row-side loader (K-major source rows)
    constexpr int NVM = BM * CH / NT;
    const int mc = tid % CH;
    const char *mrow[NVM];
    u32x4 mreg[NVM];
#pragma unroll
    for (int i = 0; i < NVM; ++i) {
        int64_t ao = a_off[tid / CH + i * (NT / CH)];
        mrow[i] = ao < 0 ? nullptr : p.A + ao * ES;
    }
    auto issue_m = [&](int kt) {
#pragma unroll
        for (int i = 0; i < NVM; ++i) mreg[i] = load_chunk<ES>(mrow[i], kt * BK + mc * VEC, R, a_vec);
    };
    auto commit_m = [&]() {
        u32x4 *tile_m = reinterpret_cast<u32x4 *>(smem_m);
#pragma unroll
        for (int i = 0; i < NVM; ++i) tile_m[tile_chunk_index<CH>(tid / CH + i * (NT / CH), mc)] = mreg[i];
    };
    issue_m(0);

    // ---------------- MFMA main loop
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int a = lane & 15, g = lane >> 4;
    const int wave_m0 = (wave / WN) * (BM / WM), wave_n0 = (wave % WN) * (BN / WN);
    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // fragment rows.  Without SWAP the weight side supplies the accumulator's row axis: lane (a, g) ends up
    // with columns 16 j + 4 g .. + 3 of row 16 i + a.
    int mrow_l[TM], nrow_l[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) mrow_l[i] = wave_m0 + i * 16 + a;
#pragma unroll
    for (int j = 0; j < TN; ++j)
        nrow_l[j] = wave_n0 + j * 16 + a;

    const int nk = (R + BK - 1) / BK;
    for (int kt = 0; kt < nk; ++kt) {
        commit_m();
        commit_n();
        __syncthreads();
        if (kt + 1 < nk) { issue_n(kt + 1); issue_m(kt + 1); }
        const u32x4 *tile_m = reinterpret_cast<const u32x4 *>(smem_m);
        const u32x4 *tile_n = reinterpret_cast<const u32x4 *>(smem_n);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            u32x4 mf[TM], nf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) mf[i] = tile_m[tile_chunk_index<CH>(mrow_l[i], ks * 4 + g)];
#pragma unroll
            for (int j = 0; j < TN; ++j) nf[j] = tile_n[tile_chunk_index<CH>(nrow_l[j], ks * 4 + g)];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if constexpr (SWAP) mma_chunk<TT>(acc[i][j], mf[i], nf[j]);
                    else mma_chunk<TT>(acc[i][j], nf[j], mf[i]);
                }
        }
        __syncthreads();
    }

    // ---------------- epilogue
    if constexpr (!SWAP) {
        // results are regrouped across lanes first (lane 4 r + c takes piece c of row r), so that the four
        // pieces of a row leave from adjacent lanes as one contiguous access
        constexpr int OES = (EPI == EPI_STORE_F32) ? 4 : ES;
        const bool c_vec = p.c_vec != 0;
        const int srow = lane >> 2, sg = lane & 3;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int64_t co = c_off[wave_m0 + i * 16 + srow];
            char *crow = p.C + (co < 0 ? 0 : co) * OES;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                f32x4 v = acc[i][j];
                if (p.w_scale != nullptr) {
                    const int nn = n0 + wave_n0 + j * 16 + g * 4;
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (nn + r < N) v[r] *= p.w_scale[(size_t)e * N + nn + r];
                }
                v = __builtin_bit_cast(f32x4, lanes_16g_a_to_4a_g(__builtin_bit_cast(u32x4, v), lane));
                const int n = n0 + wave_n0 + j * 16 + sg * 4;
                if (co < 0 || n >= N) continue;
                if (c_vec && n + 4 <= N) {
                    if constexpr (OES == 4) {
                        *reinterpret_cast<f32x4 *>(crow + (size_t)n * 4) = v;
                    } else {
                        u32x2 w;
                        w[0] = pack2<TT>(v[0], v[1]);
                        w[1] = pack2<TT>(v[2], v[3]);
                        *reinterpret_cast<u32x2 *>(crow + (size_t)n * 2) = w;
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (n + r >= N) continue;
                        if constexpr (OES == 4) reinterpret_cast<float *>(crow)[n + r] = v[r];
                        else reinterpret_cast<uint16_t *>(crow)[n + r] = (uint16_t)f32_to_elem_bits<TT>(v[r]);
                    }
                }
            }
        }
    } else {
        // fp32 atomics on the output.  Rows of the tile that land on the same token (a hot token under a skewed router:
        // tens of the 128 picks of a tile) are first added up inside the workgroup - LDS atomics into one of kSlots
        // rows of partial sums - so that the token receives one atomic per column from this tile, not one per pick.
        // A tile without such rows (the common case, known since the row bookkeeping) goes straight to memory.
        float *cbase = reinterpret_cast<float *>(p.C);
        constexpr int kSlots = (BM * BK * ES) / (BN * 4) < 32 ? (BM * BK * ES) / (BN * 4) : 32;
        static_assert(kSlots >= 8 && BN * BK * ES >= 4 * BM + 16, "bookkeeping of the tile's duplicate rows fits the slab buffers");
        int16_t *lead = reinterpret_cast<int16_t *>(smem_n);                 // [BM] first row of the tile with the same target
        int16_t *slot_of = lead + BM;                                        // [BM] slot of a leading row, -1: none
        int *nslots = reinterpret_cast<int *>(smem_n + 4 * BM);
        float *dupbuf = reinterpret_cast<float *>(smem_m);                   // [kSlots][BN]
        if (tile_has_dups) {                                                 // uniform per workgroup
            __syncthreads();                                                 // the slabs are no longer being read
            if (tid < BM) { lead[tid] = (int16_t)tid; slot_of[tid] = -1; }
            if (tid == 0) *nslots = 0;
            const int64_t my_co = tid < BM ? c_off[tid] : -1;
            for (int i = tid; i < kSlots * BN; i += NT) dupbuf[i] = 0.f;
            bool follows = false;
            if (tid < BM && my_co >= 0) {
                int l = tid;
                for (int r = 0; r < BM; ++r)                                 // no early exit: the reads stay independent
                    if (r < tid && c_off[r] == my_co) l = min(l, r);
                lead[tid] = (int16_t)l;
                follows = l != tid;
            }
            __syncthreads();
            if (follows) slot_of[lead[tid]] = -2;                            // every writer stores the same value
            __syncthreads();
            if (tid < BM && slot_of[tid] == -2) {
                const int sl = atomicAdd(nslots, 1);
                slot_of[tid] = (int16_t)(sl < kSlots ? sl : -1);
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = wave_m0 + i * 16 + g * 4 + r;
                    const int l = lead[row], sl = slot_of[l];
                    if (c_off[row] < 0 || l == row || sl < 0) continue;
#pragma unroll
                    for (int j = 0; j < TN; ++j) atomicAdd(&dupbuf[sl * BN + wave_n0 + j * 16 + a], acc[i][j][r]);
                }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = wave_m0 + i * 16 + g * 4 + r;
                    const int64_t co = c_off[row];
                    const int l = lead[row], sl = slot_of[l];
                    if (co < 0 || (l != row && sl >= 0)) continue;           // rejected pick, or folded into its leading row
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        const int nl = wave_n0 + j * 16 + a, n = n0 + nl;
                        const float extra = (l == row && sl >= 0) ? dupbuf[sl * BN + nl] : 0.f;
                        if (n < N) unsafeAtomicAdd(cbase + co + n, acc[i][j][r] + extra);
                    }
                }
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    int64_t co = c_off[wave_m0 + i * 16 + g * 4 + r];
                    if (co < 0) continue;
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        int n = n0 + wave_n0 + j * 16 + a;
                        if (n < N) unsafeAtomicAdd(cbase + co + n, acc[i][j][r]);
                    }
                }
        }
    }
}

}  // namespace egs
