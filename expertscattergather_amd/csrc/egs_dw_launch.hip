// Launch side of the tiled weight gradient: dw_kernel, or dw_dl_kernel for large well-formed 16-bit
// shapes, followed by the fixed-order sum over splits.
#include "egs_host.h"
#include "egs_dw_dl.h"

namespace egs {
namespace host {

int dw_general(const void *Xs, const void *Ys, const void *Ind, void *dW, void *workspace, const egs_dims *d,
               int64_t ldx_b, int64_t ldx_t, int act_dtype, int out_dtype, int ind_dtype, int dw_layout,
               const DwPlan &pl, hipStream_t s)
{
    const size_t w_elems = (size_t)d->E * d->I * d->J;
    const int ES = elem_size(act_dtype);
    DwParams p;
    memset(&p, 0, sizeof(p));
    p.Xs = (const char *)Xs; p.Ys = (const char *)Ys; p.Ind = Ind;
    p.part = (float *)workspace; p.dW = (char *)dW;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K; p.I = d->I; p.J = d->J;
    p.ldx_b = ldx_b; p.ldx_t = ldx_t;
    p.ind_dtype = ind_dtype;
    p.x_vec = aligned_to(Xs, 16) && (ldx_b * ES) % 16 == 0 && (ldx_t * ES) % 16 == 0;
    p.y_vec = aligned_to(Ys, 16) && ((int64_t)d->J * ES) % 16 == 0;
    p.o_vec = aligned_to(dW, 16) && d->J % 4 == 0;
    p.i_tiles = pl.i_tiles; p.j_tiles = pl.j_tiles; p.S = pl.S; p.rows_per_split = pl.rows_per_split;
    p.out_dtype = out_dtype; p.dw_layout = dw_layout;
    const uint64_t x_span = d->B > 0 && d->T > 0
        ? ((uint64_t)(d->B - 1) * (uint64_t)ldx_b + (uint64_t)(d->T - 1) * (uint64_t)ldx_t + (uint64_t)d->I) * ES : 0;
    const uint64_t y_span = (uint64_t)d->B * d->E * d->K * d->J * ES;
    if (dw_big_takes(pl, Xs, Ys, dW, d, ldx_b, ldx_t, act_dtype)) {
        DwDlParams q;
        q.d = p;
        q.d.i_tiles = pl.b_i_tiles; q.d.j_tiles = pl.b_j_tiles; q.d.S = pl.b_S; q.d.rows_per_split = pl.b_rows_per_split;
        q.x_bytes = (uint32_t)x_span; q.y_bytes = (uint32_t)y_span;
        const int64_t grid = (int64_t)8 * ceil_div(d->E, 8) * pl.b_i_tiles * pl.b_j_tiles * pl.b_S;
        if (grid > INT32_MAX) return EGS_ERR_BAD_SHAPE;
        // 128-column tiles: three 48 KB stages of 64 rows (C4: 42.2 -> 37.9 us per weight gradient with its sum over
        // splits); 256-column tiles: four 32 KB stages of 32 rows (C3: 178 -> 174 us)
        if (act_dtype == EGS_F16) {
            if (pl.b_bq == 256) hipLaunchKernelGGL((dw_dl_kernel<ElemF16, 256, 4, 32>), dim3((unsigned)grid), dim3(kDlThreads), 0, s, q);
            else hipLaunchKernelGGL((dw_dl_kernel<ElemF16, 128, 3>), dim3((unsigned)grid), dim3(kDlThreads), 0, s, q);
        } else {
            if (pl.b_bq == 256) hipLaunchKernelGGL((dw_dl_kernel<ElemBF16, 256, 4, 32>), dim3((unsigned)grid), dim3(kDlThreads), 0, s, q);
            else hipLaunchKernelGGL((dw_dl_kernel<ElemBF16, 128, 3>), dim3((unsigned)grid), dim3(kDlThreads), 0, s, q);
        }
        EGS_CHECK_LAUNCH("dw_dl_kernel");
        if (pl.b_S > 1) {       // partials are in the output's layout, I % 8 == 0 and J % 8 == 0: vectorised plain sum
            hipLaunchKernelGGL(dw_reduce4_kernel, dim3(grid_1d(w_elems / 4, 4096)), dim3(kThreads), 0, s,
                               (const float *)workspace, (char *)dW, pl.b_S, w_elems / 4, out_dtype);
            EGS_CHECK_LAUNCH("dw_reduce4_kernel");
        }
        return EGS_OK;
    }
    const int64_t grid = (int64_t)8 * ceil_div(d->E, 8) * pl.i_tiles * pl.j_tiles * pl.S;
    if (grid > INT32_MAX) return EGS_ERR_BAD_SHAPE;
    switch (act_dtype) {
    case EGS_F32: hipLaunchKernelGGL((dw_kernel<ElemF32, 128, 64, 32>), dim3((unsigned)grid), dim3(kThreads), 0, s, p); break;
    case EGS_F16: hipLaunchKernelGGL((dw_kernel<ElemF16, 128, 64, 64>), dim3((unsigned)grid), dim3(kThreads), 0, s, p); break;
    default: hipLaunchKernelGGL((dw_kernel<ElemBF16, 128, 64, 64>), dim3((unsigned)grid), dim3(kThreads), 0, s, p); break;
    }
    EGS_CHECK_LAUNCH("dw_kernel");
    if (pl.S > 1) {
        hipLaunchKernelGGL(dw_reduce_kernel, dim3(grid_1d(w_elems, 4096)), dim3(kThreads), 0, s, (const float *)workspace,
                           (char *)dW, pl.S, d->E, d->I, d->J, out_dtype, dw_layout);
        EGS_CHECK_LAUNCH("dw_reduce_kernel");
    }
    return EGS_OK;
}


}  // namespace host
}  // namespace egs
