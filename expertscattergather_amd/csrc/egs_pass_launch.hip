// Launch side of the one-kernel GEMM-scatter in passes (egs_scatter_pass.h): whether it takes a problem, its LDS
// layout, and its template instantiations (a translation unit of its own so that they compile beside the others).
#include "egs_host.h"
#include "egs_scatter_pass.h"

namespace egs {
namespace host {

namespace {
constexpr uint64_t kSpan32 = 0xFFFFFFFFull;      // the kernel addresses with 32-bit byte offsets
}

// Does the one-kernel scatter in passes (egs_scatter_pass.h: thousands of picks per batch element, one pass's product
// rows and its picks sorted by token block in LDS, token sums in accumulator tiles) take this problem?  Asked for the
// compact scatter mode, after the one-kernel scatters of small experts.
PassPlan scatter_pass_plan(const void *Y, const void *W, const void *Out, const egs_dims *d, int act_dtype)
{
    PassPlan no;
    memset(&no, 0, sizeof(no));
    const int R = d->J, N = d->I;
    const int64_t NP = (int64_t)d->E * d->K;
    if (g_force_generic || !(act_dtype == EGS_F16 || act_dtype == EGS_BF16) || !(R == 32 || R == 64 || R == 128)) return no;
    if (N < kPassCols || N % kPassCols != 0 || NP <= 1024 || NP > INT32_MAX / 2 || d->T < 1 || d->T > kPassMaxT || d->B < 1) return no;
    if (!aligned_to(Y, 16) || !aligned_to(W, 16) || !aligned_to(Out, 16)) return no;
    if ((uint64_t)d->B * NP * R * 2 > kSpan32 || (uint64_t)d->E * R * N * 2 > kSpan32) return no;
    const int slices = N / kPassCols;
    if ((int64_t)d->B * slices < 8 || (int64_t)8 * ceil_div(d->B, 8) * slices > INT32_MAX / 2) return no;
    // 32 units per pass (1024 picks, 128 KB of product rows); 16 when the batch element has no more than that
    const int64_t units_all = (int64_t)d->E * ceil_div(d->K, 32);
    PassPlan pl;
    pl.ok = true;
    pl.units_per_pass = units_all <= 16 ? 16 : kPassMaxUnits;
    pl.lds = scatter_pass_lds(pl.units_per_pass);
    if (pl.lds > 160 * 1024) return no;
    return pl;
}

namespace {

template <class TT>
int launch_scatter_pass_tt(const ScatterPassParams &p, int R, bool nmajor, size_t lds, int blocks, hipStream_t s)
{
#define EGS_PASS(NM, KS)                                                                                                    \
    do {                                                                                                                    \
        static LdsGrant told;                                                                                               \
        const int rc = allow_large_lds((const void *)scatter_pass_kernel<TT, NM, KS>, told, lds,                            \
                                       "hipFuncSetAttribute(scatter_pass_kernel)");                                        \
        if (rc != EGS_OK) return rc;                                                                                        \
        hipLaunchKernelGGL((scatter_pass_kernel<TT, NM, KS>), dim3(blocks), dim3(kPassThreads), lds, s, p);                \
    } while (0)
    if (nmajor) {
        if (R == 32) EGS_PASS(true, 1); else if (R == 64) EGS_PASS(true, 2); else EGS_PASS(true, 4);
    } else {
        if (R == 32) EGS_PASS(false, 1); else if (R == 64) EGS_PASS(false, 2); else EGS_PASS(false, 4);
    }
#undef EGS_PASS
    EGS_CHECK_LAUNCH("scatter_pass_kernel");
    return EGS_OK;
}

}  // namespace

// the caller has checked scatter_pass_plan()
int scatter_pass(const void *Y, const void *W, const void *Ind, void *Out, const egs_dims *d, int act_dtype, int ind_dtype,
                 int w_layout, hipStream_t s)
{
    const PassPlan pl = scatter_pass_plan(Y, W, Out, d, act_dtype);
    if (!pl.ok) return EGS_ERR_UNSUPPORTED;
    ScatterPassParams p;
    memset(&p, 0, sizeof(p));
    p.A = (const char *)Y; p.W = (const char *)W; p.Ind = Ind; p.out = (char *)Out;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K; p.N = d->I;
    p.ind_dtype = ind_dtype;
    p.slices = d->I / kPassCols;
    p.units_per_pass = pl.units_per_pass;
    const int blocks = 8 * ceil_div(d->B, 8) * p.slices;
    const bool nmajor = (w_layout == EGS_W_EJI);        // [E,J,I] = [E,R,N]
    return act_dtype == EGS_F16 ? launch_scatter_pass_tt<ElemF16>(p, d->J, nmajor, pl.lds, blocks, s)
                                : launch_scatter_pass_tt<ElemBF16>(p, d->J, nmajor, pl.lds, blocks, s);
}

}  // namespace host
}  // namespace egs
