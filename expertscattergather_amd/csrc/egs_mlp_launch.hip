// C ABI and launch side of the one-kernel inference block gather -> activation -> scatter of small experts
// (egs_mlp_fused.h).
#include "egs_host.h"
#include "egs_mlp_fused.h"

namespace egs {
namespace host {
namespace {

struct MlpPlan { bool ok; size_t lds; int slices; int64_t blocks; };

// shape and operand conditions of the kernel; operands may be null when only the shape is asked about
MlpPlan mlp_plan(const void *X, const void *Wg, const void *Ws, const void *Out, const egs_dims *d, int64_t ldx_b,
                 int64_t ldx_t, int dtype)
{
    const MlpPlan no = {false, 0, 0, 0};
    if (g_force_generic || !(dtype == EGS_F16 || dtype == EGS_BF16)) return no;
    if (!(d->I == 32 || d->I == 64 || d->I == 128) || !(d->J == 32 || d->J == 64)) return no;
    const int64_t NP = (int64_t)d->E * d->K;
    if (NP < 1 || NP > 1024 || d->T < 1 || d->B < 1) return no;
    const size_t lds = scatter_fused_lds(d->T, (int)NP);
    if (lds > 156 * 1024) return no;
    if (!aligned_to(X, 16) || !aligned_to(Wg, 16) || !aligned_to(Ws, 16) || !aligned_to(Out, 16)) return no;
    if ((ldx_b * 2) % 16 || (ldx_t * 2) % 16) return no;
    const uint64_t x_span = ((uint64_t)(d->B - 1) * (uint64_t)ldx_b + (uint64_t)(d->T - 1) * (uint64_t)ldx_t + d->I) * 2;
    if (x_span > 0xFFFFFFFFull) return no;
    const int slices = d->I / kFusedCols;
    const int64_t blocks = (int64_t)8 * ceil_div(d->B, 8) * slices;
    if (blocks > INT32_MAX / 2 || (int64_t)d->B * slices < 8) return no;
    return {true, lds, slices, blocks};
}

template <class TT, int KS1, int JT>
int launch_mlp_one(const MlpFusedParams &p, size_t lds, int blocks, hipStream_t s)
{
    static LdsGrant told;
    const int rc = allow_large_lds((const void *)mlp_fused_kernel<TT, KS1, JT>, told, lds, "hipFuncSetAttribute(mlp_fused_kernel)");
    if (rc != EGS_OK) return rc;
    hipLaunchKernelGGL((mlp_fused_kernel<TT, KS1, JT>), dim3(blocks), dim3(kFusedThreads), lds, s, p);
    EGS_CHECK_LAUNCH("mlp_fused_kernel");
    return EGS_OK;
}

template <class TT, int KS1>
int launch_mlp_jt(const MlpFusedParams &p, int J, size_t lds, int blocks, hipStream_t s)
{
    return J == 32 ? launch_mlp_one<TT, KS1, 2>(p, lds, blocks, s) : launch_mlp_one<TT, KS1, 4>(p, lds, blocks, s);
}

template <class TT>
int launch_mlp_tt(const MlpFusedParams &p, int I, int J, size_t lds, int blocks, hipStream_t s)
{
    switch (I) {
    case 32: return launch_mlp_jt<TT, 1>(p, J, lds, blocks, s);
    case 64: return launch_mlp_jt<TT, 2>(p, J, lds, blocks, s);
    default: return launch_mlp_jt<TT, 4>(p, J, lds, blocks, s);
    }
}

bool mlp_dims_ok(const egs_dims *d)
{
    return d != nullptr && d->B >= 0 && d->T >= 0 && d->E >= 0 && d->K >= 0 && d->I >= 0 && d->J >= 0;
}

void *const kAlignedStandIn = (void *)(uintptr_t)4096;

}  // namespace
}  // namespace host
}  // namespace egs

using namespace egs;
using namespace egs::host;

extern "C" {

int egs_expert_mlp_supported(const egs_dims *d, int dtype)
{
    if (!mlp_dims_ok(d)) return 0;
    return mlp_plan(kAlignedStandIn, kAlignedStandIn, kAlignedStandIn, kAlignedStandIn, d, (int64_t)d->T * d->I, d->I, dtype).ok ? 1 : 0;
}

int egs_expert_mlp_forward(const void *X, const void *Wg, const void *Ws, const void *Ind, void *Out, const egs_dims *d,
                           int64_t ldx_b, int64_t ldx_t, int dtype, int ind_dtype, int activation, void *stream)
{
    if (!mlp_dims_ok(d)) return d == nullptr ? EGS_ERR_NULL_POINTER : EGS_ERR_BAD_SHAPE;
    if (!(dtype == EGS_F32 || dtype == EGS_F16 || dtype == EGS_BF16)) return EGS_ERR_BAD_DTYPE;
    if (ind_dtype < EGS_IND_I16 || ind_dtype > EGS_IND_U8) return EGS_ERR_BAD_DTYPE;
    if (activation < EGS_ACT_NONE || activation > EGS_ACT_GELU_TANH) return EGS_ERR_BAD_MODE;
    // the same stride rule as the gather forward: rows must not overlap themselves, batch elements may sit in any
    // order (a transposed or batch-expanded view passes); the span is checked against the 32-bit offsets in mlp_plan
    if (ldx_t < d->I || (d->B > 1 && ldx_b < 0)) return EGS_ERR_BAD_STRIDE;
    if ((size_t)d->B * d->T * d->I == 0) return EGS_OK;            // nothing to write
    if (X == nullptr || Out == nullptr) return EGS_ERR_NULL_POINTER;
    if ((size_t)d->E * d->K > 0 && (Wg == nullptr || Ws == nullptr || Ind == nullptr)) return EGS_ERR_NULL_POINTER;
    const MlpPlan pl = mlp_plan(X, Wg, Ws, Out, d, ldx_b, ldx_t, dtype);
    if (!pl.ok) return EGS_ERR_UNSUPPORTED;
    const int64_t NP = (int64_t)d->E * d->K;
    MlpFusedParams p;
    memset(&p, 0, sizeof(p));
    p.X = (const char *)X; p.Wg = (const char *)Wg; p.Ws = (const char *)Ws; p.Ind = Ind; p.out = (char *)Out;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K;
    p.ldx_b = ldx_b; p.ldx_t = ldx_t; p.ind_dtype = ind_dtype;
    p.slices = pl.slices;
    p.perm_at = (int32_t)(NP * kFusedCols * 4);
    p.cnt_at = p.perm_at + (int32_t)(NP * 4);
    p.zero_at = (int32_t)scatter_fused_zero_at(d->T, (int)NP, (int)NP);
    p.act = activation;
    hipStream_t s = (hipStream_t)stream;
    return dtype == EGS_BF16 ? launch_mlp_tt<ElemBF16>(p, d->I, d->J, pl.lds, (int)pl.blocks, s)
                             : launch_mlp_tt<ElemF16>(p, d->I, d->J, pl.lds, (int)pl.blocks, s);
}

}  // extern "C"
