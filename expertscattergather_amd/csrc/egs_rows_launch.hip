// Launch side of the tiled rows x weight products: picks the tile shape and kernel family
// (rows_gemm_kernel, or rows_gemm_dl_kernel for large well-formed 16-bit shapes) and instantiates them.
#include "egs_host.h"
#include "egs_rows_gemm_dl.h"

namespace egs {
namespace host {
namespace {

// ------------------------------------------------------------------------------ rows-GEMM dispatch
template <class TT, int WES, bool GATHER, bool W_TRANS, int EPI>
int launch_rows_gemm_cfg(RowsGemmParams &p, hipStream_t s)
{
    constexpr int BK = TT::ES == 4 ? 32 : 64;
    const int Me = p.B * p.K;
    if (Me == 0 || p.E == 0 || p.N == 0) return EGS_OK;
    const int e_groups = ceil_div(p.E, 8);
    // tile shape: 128 x 64 for narrow outputs, 256 x 256 (8 wavefronts) when the product is large
    // enough to be bound by operand traffic (16-bit types), else 128 x 128
    const bool big = TT::ES == 2 && EPI != EPI_ATOMIC_F32 && p.N >= 192 && Me >= 256 && p.R >= 128;
    if (p.N <= 64) {
        constexpr int BM = 128, BN = 64;
        p.m_tiles = ceil_div(Me, BM); p.n_tiles = ceil_div(p.N, BN);
        int64_t grid = (int64_t)8 * e_groups * p.m_tiles * p.n_tiles;
        if (grid > INT32_MAX) return EGS_ERR_BAD_SHAPE;
        hipLaunchKernelGGL((rows_gemm_kernel<TT, WES, BM, BN, BK, 4, 1, GATHER, W_TRANS, EPI>), dim3((unsigned)grid),
                           dim3(256), 0, s, p);
    } else if (big) {
        if constexpr (TT::ES == 2 && EPI != EPI_ATOMIC_F32) {
            constexpr int BM = 256, BN = 256;
            p.m_tiles = ceil_div(Me, BM); p.n_tiles = ceil_div(p.N, BN);
            int64_t grid = (int64_t)8 * e_groups * p.m_tiles * p.n_tiles;
            if (grid > INT32_MAX) return EGS_ERR_BAD_SHAPE;
            // well-formed shapes take the direct-to-LDS pipeline (256 x 256 x 64 slabs, two stages).  256 x 128 tiles of
            // four wavefronts on 32-deep slabs, two workgroups to a CU, measured for these shapes: gather at C3 156 -> 170 us
            // (gathered rows fetched once per column tile), fp32 product rows at C3 38.7 -> 40.2 us per group and at C5
            // 1.80 -> 2.09 ms; at C4 31.9 -> 28.7 us, which the table workgroups riding along take back
            const bool dl = !g_force_generic && p.R % 64 == 0 && p.N % (WES == 1 ? 16 : 8) == 0 && p.a_vec && p.w_vec &&
                            p.a_bytes != 0 && (uint64_t)p.R * p.N * 2 < (1ull << 31) && (WES == 1 || p.w_scale == nullptr) &&
                            (WES == 2 || aligned_to(p.W, 16)) &&
                            aligned_to(p.C, 16);
            if constexpr (WES == 2 || W_TRANS) {
                if (dl) {
                    const size_t smem = GATHER ? 0 : (size_t)dl_smem_bytes_scatter(256, 256, 64, 2);
                    p.csr_threads = 512;            // as many wavefronts as the histograms leave room for
                    while (p.csr_threads > kWave && csr_count_lds(p.T, p.csr_threads / kWave) > smem) p.csr_threads >>= 1;
                    if (GATHER || csr_count_lds(p.T, p.csr_threads / kWave) > smem) p.csr_blocks = 0;
                    // many picks per batch element: several workgroups per table, each ranking a share whose wavefront
                    // slices (512 picks) stay in registers; one workgroup ranking 32768 picks outlasts the product tiles
                    // of its launch (C3: 100 against 38 us; with eight parts the launch takes 54 us, one more round of workgroups)
                    p.csr_parts = 1;
                    if (p.csr_blocks > 0) {
                        const int64_t per = (int64_t)(p.csr_threads / kWave) * 512;
                        const int64_t parts = ((int64_t)p.E * p.K + per - 1) / per;
                        p.csr_parts = (int)(parts < 1 ? 1 : parts > 8 ? 8 : parts);
                        p.csr_blocks *= p.csr_parts;
                    }
                    grid += p.csr_blocks;
                    if (grid > INT32_MAX) return EGS_ERR_BAD_SHAPE;
                    p.csr_done = p.csr_blocks > 0;
                    if constexpr (WES == 1 && GATHER) {
                        // fp8 weights: a stage is 32 KB of rows + 16 KB of weight bytes, so three fit (C5 gather 1058 -> 1024 us)
                        hipLaunchKernelGGL((rows_gemm_dl_kernel<TT, WES, 256, 256, 64, 3, GATHER, W_TRANS, EPI>), dim3((unsigned)grid), dim3(512), 0, s, p);
                        EGS_CHECK_LAUNCH("rows_gemm_dl_kernel");
                        return EGS_OK;
                    }
                    hipLaunchKernelGGL((rows_gemm_dl_kernel<TT, WES, 256, 256, 64, 2, GATHER, W_TRANS, EPI>), dim3((unsigned)grid), dim3(512), 0, s, p);
                    EGS_CHECK_LAUNCH("rows_gemm_dl_kernel");
                    return EGS_OK;
                }
            }
            hipLaunchKernelGGL((rows_gemm_kernel<TT, WES, BM, BN, BK, 2, 4, GATHER, W_TRANS, EPI>), dim3((unsigned)grid),
                               dim3(512), 0, s, p);
        }
    } else {
        // 65..191 output columns.  The gathers of large, well-formed 16-bit shapes take the direct-to-LDS
        // pipeline with 256 x 128 tiles of four wavefronts in three stages of 32-deep slabs (75 KB), compiled for two
        // wavefronts per SIMD so that TWO workgroups share a CU and one's loads and stores run under the other's
        // matrix instructions: C4 gather 29.5 -> 21.5 us against 64-deep slabs in two stages with one workgroup per
        // CU.  (Left to itself the compiler gives a four-wavefront workgroup 144 + 128 accumulator registers, which
        // keeps a second workgroup off the CU whatever the LDS size.)
        if constexpr (TT::ES == 2 && WES == 2 && GATHER && EPI == EPI_STORE) {
            const bool dl = !g_force_generic && Me >= 256 && p.R >= 128 && p.R % 64 == 0 && p.N % 8 == 0 && p.a_vec && p.w_vec &&
                            p.a_bytes != 0 && (uint64_t)p.R * p.N * 2 < (1ull << 31) && p.w_scale == nullptr && aligned_to(p.C, 16);
            if (dl) {
                p.m_tiles = ceil_div(Me, 256); p.n_tiles = ceil_div(p.N, 128);
                int64_t grid = (int64_t)8 * e_groups * p.m_tiles * p.n_tiles;
                if (grid > INT32_MAX) return EGS_ERR_BAD_SHAPE;
                p.csr_blocks = 0;
                hipLaunchKernelGGL((rows_gemm_dl_kernel<TT, 2, 256, 128, 32, 3, true, W_TRANS, EPI_STORE>), dim3((unsigned)grid),
                                   dim3(dl_threads(256, 128)), 0, s, p);
                EGS_CHECK_LAUNCH("rows_gemm_dl_kernel");
                return EGS_OK;
            }
        }
        constexpr int BM = 128, BN = 128;
        p.m_tiles = ceil_div(Me, BM); p.n_tiles = ceil_div(p.N, BN);
        int64_t grid = (int64_t)8 * e_groups * p.m_tiles * p.n_tiles;
        if (grid > INT32_MAX) return EGS_ERR_BAD_SHAPE;
        hipLaunchKernelGGL((rows_gemm_kernel<TT, WES, BM, BN, BK, 2, 2, GATHER, W_TRANS, EPI>), dim3((unsigned)grid),
                           dim3(256), 0, s, p);
    }
    EGS_CHECK_LAUNCH("rows_gemm_kernel");
    return EGS_OK;
}

template <class TT, bool GATHER, int EPI>
int launch_rows_gemm_w(RowsGemmParams &p, bool w_trans, hipStream_t s)
{
    return w_trans ? launch_rows_gemm_cfg<TT, TT::ES, GATHER, true, EPI>(p, s)
                   : launch_rows_gemm_cfg<TT, TT::ES, GATHER, false, EPI>(p, s);
}

template <bool GATHER, int EPI>
int launch_rows_gemm(RowsGemmParams &p, int act_dtype, bool w_trans, hipStream_t s)
{
    switch (act_dtype) {
    case EGS_F32: return launch_rows_gemm_w<ElemF32, GATHER, EPI>(p, w_trans, s);
    case EGS_F16: return launch_rows_gemm_w<ElemF16, GATHER, EPI>(p, w_trans, s);
    case EGS_BF16: return launch_rows_gemm_w<ElemBF16, GATHER, EPI>(p, w_trans, s);
    default: return EGS_ERR_BAD_DTYPE;
    }
}


}  // namespace

int rows_gemm_gather(RowsGemmParams &p, int act_dtype, bool fp8_w, bool w_trans, hipStream_t s)
{
    if (fp8_w) {
        return w_trans ? launch_rows_gemm_cfg<ElemBF16, 1, true, true, EPI_STORE>(p, s)
                       : launch_rows_gemm_cfg<ElemBF16, 1, true, false, EPI_STORE>(p, s);
    }
    return launch_rows_gemm<true, EPI_STORE>(p, act_dtype, w_trans, s);
}

int rows_gemm_scatter(RowsGemmParams &p, int act_dtype, bool w_trans, int epi, hipStream_t s)
{
    switch (epi) {
    case EPI_STORE: return launch_rows_gemm<false, EPI_STORE>(p, act_dtype, w_trans, s);
    case EPI_STORE_F32: return launch_rows_gemm<false, EPI_STORE_F32>(p, act_dtype, w_trans, s);
    default: return launch_rows_gemm<false, EPI_ATOMIC_F32>(p, act_dtype, w_trans, s);
    }
}

}  // namespace host
}  // namespace egs
