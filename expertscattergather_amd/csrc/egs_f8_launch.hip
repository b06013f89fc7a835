// C ABI and launch side of the gather-GEMM with fp8 weights and fp8 activations (egs_rows_gemm_f8.h):
// the row quantiser followed by the fp8 x fp8 product, both on the caller's stream, intermediate rows and
// row scales in the caller's workspace.
#include "egs_host.h"
#include "egs_rows_gemm_f8.h"

namespace egs {
namespace host {
namespace {

struct F8Plan {
    size_t xq_bytes, xs_bytes, bytes;
};

bool f8_dims_ok(const egs_dims *d)
{
    return d != nullptr && d->B >= 0 && d->T >= 0 && d->E >= 0 && d->K >= 0 && d->I >= 0 && d->J >= 0;
}

F8Plan plan_f8(const egs_dims *d)
{
    F8Plan pl;
    pl.xq_bytes = align_up((size_t)d->B * d->T * d->I, 256);
    pl.xs_bytes = align_up((size_t)d->B * d->T * sizeof(float), 256);
    pl.bytes = pl.xq_bytes + pl.xs_bytes;
    return pl;
}

bool ind_dtype_known(int ind_dtype) { return ind_dtype >= EGS_IND_I16 && ind_dtype <= EGS_IND_U8; }

}  // namespace
}  // namespace host
}  // namespace egs

using namespace egs;
using namespace egs::host;

extern "C" {

size_t egs_gather_gemm_fp8act_workspace_bytes(const egs_dims *d)
{
    if (!f8_dims_ok(d)) return 0;
    return plan_f8(d).bytes;
}

int egs_gather_gemm_fp8act(const void *X, const void *Wq, const float *w_scale, const void *Ind, void *Y,
                           void *workspace, size_t workspace_bytes, const egs_dims *d,
                           int64_t ldx_b, int64_t ldx_t, int ind_dtype, void *stream)
{
    if (!f8_dims_ok(d)) return d == nullptr ? EGS_ERR_NULL_POINTER : EGS_ERR_BAD_SHAPE;
    if (!ind_dtype_known(ind_dtype)) return EGS_ERR_BAD_DTYPE;
    const size_t y_elems = (size_t)d->B * d->E * d->K * d->J;
    if (y_elems == 0) return EGS_OK;
    // the fp8 tile layout: whole 128-element slabs of the reduction, 16-byte weight chunks
    if (d->I == 0 || d->I % kF8BK != 0 || d->J % 16 != 0 || d->T == 0) return EGS_ERR_UNSUPPORTED;
    if (X == nullptr || Wq == nullptr || w_scale == nullptr || Ind == nullptr || Y == nullptr) return EGS_ERR_NULL_POINTER;
    if (ldx_t < d->I || (d->B > 1 && ldx_b < 0)) return EGS_ERR_BAD_STRIDE;
    if (ldx_t % 8 != 0 || (d->B > 1 && ldx_b % 8 != 0)) return EGS_ERR_ALIGNMENT;
    if (!aligned_to(X, 16) || !aligned_to(Wq, 16) || !aligned_to(Y, 16) || !aligned_to(w_scale, 4)) return EGS_ERR_ALIGNMENT;
    if ((uint64_t)d->B * d->T * d->I >= (1ull << 31) || (uint64_t)d->I * d->J >= (1ull << 31) ||
        (int64_t)d->B * d->K > INT32_MAX || (int64_t)d->B * d->T > INT32_MAX)
        return EGS_ERR_BAD_SHAPE;
    const F8Plan pl = plan_f8(d);
    if (workspace == nullptr || workspace_bytes < pl.bytes) return EGS_ERR_WORKSPACE;
    if (!aligned_to(workspace, 256)) return EGS_ERR_ALIGNMENT;
    hipStream_t s = (hipStream_t)stream;

    QuantRowsParams q;
    memset(&q, 0, sizeof(q));
    q.X = (const char *)X;
    q.Xq = (char *)workspace;
    q.xs = (float *)((char *)workspace + pl.xq_bytes);
    q.B = d->B; q.T = d->T; q.I = d->I;
    q.ldx_b = ldx_b; q.ldx_t = ldx_t;
    const int64_t rows = (int64_t)d->B * d->T;
    const int64_t qgrid = (rows + kThreads / 64 - 1) / (kThreads / 64);
    if (qgrid > INT32_MAX) return EGS_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(quantize_rows_e4m3_kernel, dim3((unsigned)qgrid), dim3(kThreads), 0, s, q);
    EGS_CHECK_LAUNCH("quantize_rows_e4m3_kernel");

    RowsGemmF8Params p;
    memset(&p, 0, sizeof(p));
    p.Aq = q.Xq; p.a_scale = q.xs; p.W = (const char *)Wq; p.w_scale = w_scale; p.Ind = Ind; p.C = (char *)Y;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K; p.R = d->I; p.N = d->J;
    p.ind_dtype = ind_dtype;
    p.m_tiles = ceil_div(d->B * d->K, kF8BM);
    p.n_tiles = ceil_div(d->J, kF8BN);
    p.a_bytes = (uint32_t)((uint64_t)d->B * d->T * d->I);
    const int64_t grid = (int64_t)8 * ceil_div(d->E, 8) * p.m_tiles * p.n_tiles;
    if (grid > INT32_MAX) return EGS_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(rows_gemm_f8_kernel, dim3((unsigned)grid), dim3(kF8Threads), 0, s, p);
    EGS_CHECK_LAUNCH("rows_gemm_f8_kernel");
    return EGS_OK;
}

}  // extern "C"
