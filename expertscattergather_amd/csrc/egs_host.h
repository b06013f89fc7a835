// Host-side pieces shared by the translation units of the library: error plumbing, small helpers,
// plans, and the launch entry points that live in files of their own so that their kernel template
// instantiations compile in parallel with the rest.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/egs_hip.h"
#include "egs_device.h"
#include "egs_rows_gemm.h"
#include "egs_dw.h"

namespace egs {
namespace host {

extern std::atomic<bool> g_force_generic;       // testing aid (egs_testing_force_generic): skip the fast paths

int hip_fail(hipError_t err, const char *what);     // records the HIP error text for egs_last_hip_error, returns EGS_ERR_HIP
const char *last_hip_error();

// A kernel that takes more than 64 KB of dynamic LDS has to be granted it, per device.  One LdsGrant per kernel
// (a function-local static at the launch site) remembers the largest size granted on each device; growth is
// serialised so that a smaller request racing with a larger one cannot shrink the grant.
constexpr int kMaxDevices = 64;
struct LdsGrant { std::atomic<uint32_t> bytes[kMaxDevices]; };
int allow_large_lds(const void *fn, LdsGrant &grant, size_t lds, const char *what);

// testing aid (egs_testing_launch_log_begin / _end): while the calling thread keeps a log, the name of every kernel it
// launches is appended to it
void note_launch(const char *what);

#define EGS_CHECK_LAUNCH(what)                                         \
    do {                                                               \
        hipError_t err__ = hipGetLastError();                          \
        if (err__ != hipSuccess) return ::egs::host::hip_fail(err__, what); \
        ::egs::host::note_launch(what);                                \
    } while (0)

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

inline int elem_size(int dtype)
{
    switch (dtype) {
    case EGS_F32: return 4;
    case EGS_F16: case EGS_BF16: return 2;
    case EGS_FP8_E4M3: return 1;
    default: return 0;
    }
}

inline int ind_size(int ind_dtype)
{
    switch (ind_dtype) {
    case EGS_IND_U8: return 1;
    case EGS_IND_I16: return 2;
    case EGS_IND_I32: return 4;
    default: return 8;
    }
}

inline int grid_1d(size_t items, int cap = 8192)
{
    size_t g = (items + kThreads - 1) / kThreads;
    if (g < 1) g = 1;
    return (int)(g > (size_t)cap ? (size_t)cap : g);
}

// LDS the counting-sort routing table needs with `nw` wavefronts per batch element
inline size_t csr_count_lds(int T, int nw) { return ((size_t)(nw + 1) * T + 1) * 4; }

struct DwPlan {
    int BI, BJ, BK, i_tiles, j_tiles, S, rows_per_split;   // general tiled kernel
    bool small_ok;                                          // shape admits the small-expert kernel
    int s_i_tiles, s_j_tiles, s_S, s_rows_per_split;        // its plan
    bool big_ok;                                            // shape admits the direct-to-LDS kernel (256 x BQ tiles)
    int b_bq, b_i_tiles, b_j_tiles, b_S, b_rows_per_split;  // its plan
    size_t bytes_general, bytes_small, bytes_big;           // workspace of each of the three split kernels (0: no splits)
};

// does the direct-to-LDS weight gradient (dw_dl_kernel) take these operands?
inline bool dw_big_takes(const DwPlan &pl, const void *Xs, const void *Ys, const void *dW, const egs_dims *d, int64_t ldx_b,
                         int64_t ldx_t, int act_dtype)
{
    if (!pl.big_ok || g_force_generic || d->B < 1 || d->T < 1) return false;
    const int ES = elem_size(act_dtype);
    const bool x_vec = aligned_to(Xs, 16) && (ldx_b * ES) % 16 == 0 && (ldx_t * ES) % 16 == 0;
    const bool y_vec = aligned_to(Ys, 16) && ((int64_t)d->J * ES) % 16 == 0;
    const uint64_t x_span = ((uint64_t)(d->B - 1) * (uint64_t)ldx_b + (uint64_t)(d->T - 1) * (uint64_t)ldx_t + (uint64_t)d->I) * ES;
    const uint64_t y_span = (uint64_t)d->B * d->E * d->K * d->J * ES;
    return x_vec && y_vec && x_span < (1ull << 31) && y_span < (1ull << 31) && aligned_to(dW, 16);
}


// ---- egs_rows_launch.hip: tiled rows x weight products (general and direct-to-LDS kernels)
// gather: C = rows of A fetched through Ind times W, stored in the element type (fp8_w: e4m3 weights, bf16 activations)
int rows_gemm_gather(RowsGemmParams &p, int act_dtype, bool fp8_w, bool w_trans, hipStream_t s);
// scatter products: epi = EPI_STORE / EPI_STORE_F32 (rows in pick order) or EPI_ATOMIC_F32 (fp32 atomics on the output)
int rows_gemm_scatter(RowsGemmParams &p, int act_dtype, bool w_trans, int epi, hipStream_t s);

// ---- egs_pass_launch.hip: the one-kernel GEMM-scatter in passes (thousands of picks per batch element, 16-bit types)
struct PassPlan { bool ok; int units_per_pass; size_t lds; };
PassPlan scatter_pass_plan(const void *Y, const void *W, const void *Out, const egs_dims *d, int act_dtype);
int scatter_pass(const void *Y, const void *W, const void *Ind, void *Out, const egs_dims *d, int act_dtype, int ind_dtype,
                 int w_layout, hipStream_t s);

// ---- egs_dw_launch.hip: tiled weight gradient (general and direct-to-LDS kernels) with its second pass
int dw_general(const void *Xs, const void *Ys, const void *Ind, void *dW, void *workspace, const egs_dims *d,
               int64_t ldx_b, int64_t ldx_t, int act_dtype, int out_dtype, int ind_dtype, int dw_layout,
               const DwPlan &pl, hipStream_t s);

}  // namespace host
}  // namespace egs
