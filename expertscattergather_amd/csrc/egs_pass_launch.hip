// Launch side of the one-kernel GEMM-scatter in passes (egs_scatter_pass.h): whether it takes a problem, its LDS
// layout, and its template instantiations (a translation unit of its own so that they compile beside the others).
#include "egs_host.h"
#include "egs_scatter_pass.h"

namespace egs {
namespace host {

namespace {
constexpr uint64_t kSpan32 = 0xFFFFFFFFull;      // the kernel addresses with 32-bit byte offsets
}

// Does the one-kernel scatter in passes (egs_scatter_pass.h: thousands of picks per batch element, 16-bit routing table
// and one pass's product rows in LDS, token sums in registers) take this problem?  Asked for the compact scatter mode,
// after the one-kernel scatters of small experts.
PassPlan scatter_pass_plan(const void *Y, const void *W, const void *Out, const egs_dims *d, int act_dtype)
{
    PassPlan no;
    memset(&no, 0, sizeof(no));
    const int R = d->J, N = d->I;
    const int64_t NP = (int64_t)d->E * d->K;
    if (g_force_generic || !(act_dtype == EGS_F16 || act_dtype == EGS_BF16) || !(R == 32 || R == 64 || R == 128)) return no;
    if (N < kPassCols || N % kPassCols != 0 || NP <= 1024 || NP > kPassMaxPicks || d->T < 1 || d->T > kPassMaxT || d->B < 1) return no;
    if (!aligned_to(Y, 16) || !aligned_to(W, 16) || !aligned_to(Out, 16)) return no;
    if ((uint64_t)d->B * NP * R * 2 > kSpan32 || (uint64_t)d->E * R * N * 2 > kSpan32) return no;
    const int slices = N / kPassCols;
    if ((int64_t)d->B * slices < 8 || (int64_t)8 * ceil_div(d->B, 8) * slices > INT32_MAX / 2) return no;
    const size_t budget = 156 * 1024, fixed = scatter_pass_fixed_lds(d->T, (int)NP);
    if (fixed + 16 * 32 * kPassCols * 4 > budget) return no;
    const int64_t units_all = (int64_t)d->E * ceil_div(d->K, 32);
    int64_t up = (int64_t)((budget - fixed) / (32 * kPassCols * 4));
    if (up > (units_all + 15) / 16 * 16) up = (units_all + 15) / 16 * 16;
    up = up / 16 * 16;
    if (up < 16) return no;
    PassPlan pl;
    pl.ok = true;
    pl.units_per_pass = (int)up;
    pl.perm_at = (int32_t)(up * 32 * kPassCols * 4);
    pl.seg_at = pl.perm_at + (int32_t)align_up((size_t)NP * 2, 16);
    pl.long_at = pl.seg_at + (int32_t)align_up((size_t)(d->T + 1) * 2, 16);
    pl.lds = (size_t)pl.long_at + kPassRecordBytes;
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

// the caller has checked scatter_pass_plan(); `seg` / `perm`: the routing table of all batch elements, in memory
int scatter_pass(const void *Y, const void *W, void *Out, const egs_dims *d, int act_dtype, int w_layout, const int32_t *seg,
                 const int32_t *perm, hipStream_t s)
{
    const PassPlan pl = scatter_pass_plan(Y, W, Out, d, act_dtype);
    if (!pl.ok) return EGS_ERR_UNSUPPORTED;
    ScatterPassParams p;
    memset(&p, 0, sizeof(p));
    p.A = (const char *)Y; p.W = (const char *)W; p.out = (char *)Out;
    p.tab_seg = seg; p.tab_perm = perm;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K; p.N = d->I;
    p.slices = d->I / kPassCols;
    p.units_per_pass = pl.units_per_pass;
    p.perm_at = pl.perm_at; p.seg_at = pl.seg_at; p.long_at = pl.long_at;
    const int blocks = 8 * ceil_div(d->B, 8) * p.slices;
    const bool nmajor = (w_layout == EGS_W_EJI);        // [E,J,I] = [E,R,N]
    return act_dtype == EGS_F16 ? launch_scatter_pass_tt<ElemF16>(p, d->J, nmajor, pl.lds, blocks, s)
                                : launch_scatter_pass_tt<ElemBF16>(p, d->J, nmajor, pl.lds, blocks, s);
}

}  // namespace host
}  // namespace egs
