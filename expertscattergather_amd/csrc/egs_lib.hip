// Host side of the library: argument validation, workspace plans, kernel selection and the C ABI
// declared in include/egs_hip.h.  The two template-heavy launch families (tiled rows products,
// tiled weight gradients) live in egs_rows_launch.hip and egs_dw_launch.hip.
#include "egs_host.h"
#include "../../include/egs_hip_testing.h"
#include "egs_device.h"
#include "egs_scatter_aux.h"
#include "egs_small.h"
#include "egs_dw_tile.h"
#include "egs_small_f32.h"
#include "egs_scatter_fused.h"

#include <atomic>
#include <mutex>

using namespace egs;
using namespace egs::host;

namespace egs {
namespace host {

std::atomic<bool> g_force_generic{false};
static thread_local char g_hip_error_buf[256] = "";

int hip_fail(hipError_t err, const char *what)
{
    snprintf(g_hip_error_buf, sizeof(g_hip_error_buf), "%s: %s", what, hipGetErrorString(err));
    return EGS_ERR_HIP;
}
const char *last_hip_error() { return g_hip_error_buf; }

struct LaunchLog { bool on; size_t len; char text[1024]; };
static thread_local LaunchLog g_launch_log = {false, 0, ""};
void note_launch(const char *what)
{
    LaunchLog &l = g_launch_log;
    if (!l.on) return;
    const size_t n = strlen(what);
    if (l.len + n + 2 > sizeof(l.text)) return;
    if (l.len > 0) l.text[l.len++] = ',';
    memcpy(l.text + l.len, what, n + 1);
    l.len += n;
}

static std::mutex g_lds_mutex;
int allow_large_lds(const void *fn, LdsGrant &grant, size_t lds, const char *what)
{
    if (lds <= 64 * 1024) return EGS_OK;
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return hip_fail(err, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return EGS_ERR_UNSUPPORTED;
    if (grant.bytes[dev].load(std::memory_order_acquire) >= lds) return EGS_OK;
    std::lock_guard<std::mutex> lock(g_lds_mutex);
    if (grant.bytes[dev].load(std::memory_order_relaxed) >= lds) return EGS_OK;
    err = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) return hip_fail(err, what);
    grant.bytes[dev].store((uint32_t)lds, std::memory_order_release);
    return EGS_OK;
}

}  // namespace host
}  // namespace egs

namespace {

// ------------------------------------------------------------------------------ built-in scratch
// Device memory that exists from the moment the library's code object is loaded, for the one entry
// point that serves callers which cannot allocate (egs_dw_builtin_scratch).  Every GPU the library
// runs on holds its own copy of the array, at its own address, until the process ends.
// The array's name is only a host-side handle: host code never passes it to a kernel or a copy.  The
// device address is looked up once per device (with that device current) and kept.
static __device__ __align__(256) unsigned char scratch[EGS_BUILTIN_SCRATCH_BYTES];

std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];              // per device: address of that device's copy of `scratch`

int builtin_scratch_ptr(void **out)
{
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return hip_fail(err, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return EGS_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        err = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return hip_fail(err, "hipGetSymbolAddress(scratch)");
        if (ptr == nullptr) return EGS_ERR_HIP;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return EGS_OK;
}

bool act_dtype_ok(int d) { return d == EGS_F32 || d == EGS_F16 || d == EGS_BF16; }
bool ind_dtype_ok(int d) { return d >= EGS_IND_I16 && d <= EGS_IND_U8; }
bool layout_ok(int l) { return l == EGS_W_EIJ || l == EGS_W_EJI; }
bool mode_ok(int m) { return m == EGS_SCATTER_DETERMINISTIC || m == EGS_SCATTER_ATOMIC || m == EGS_SCATTER_COMPACT; }

int check_dims(const egs_dims *d)
{
    if (d == nullptr) return EGS_ERR_NULL_POINTER;
    if (d->B < 0 || d->T < 0 || d->E < 0 || d->K < 0 || d->I < 0 || d->J < 0) return EGS_ERR_BAD_SHAPE;
    // row counts and per-batch pick counts are held in 32-bit ints inside the kernels
    if ((int64_t)d->B * d->K > INT32_MAX || (int64_t)d->E * d->K > INT32_MAX) return EGS_ERR_BAD_SHAPE;
    if ((int64_t)d->B * d->T > INT32_MAX) return EGS_ERR_BAD_SHAPE;
    return EGS_OK;
}

// ------------------------------------------------------------------------------ plans
struct ScatterPlan {
    size_t seg_off_at, perm_at, rank_at, cnt_at, long_tab_at, long_part_at, rows_at;   // byte offsets inside the workspace
    size_t bytes;
};

// Workspace of the GEMM-scatter, for the kernels that will run:
//   fp32 atomic mode and the one-kernel scatter of small experts (`fused`) need none;
//   otherwise: routing table (segment offsets, picks in token order, scratch ranks, optional global counters),
//   long-segment records and partial rows, and the product rows in pick order - fp32 in deterministic mode
//   (fp32 accumulation with one final rounding), the element type in atomic ("fast") mode with 16-bit types
//   (half the traffic, one extra rounding per pick; the summation order is still fixed).
//   the one-kernel scatter in passes (SCATTER_PASS) needs nothing either (it sorts each pass's picks in LDS);
enum ScatterPath { SCATTER_FUSED, SCATTER_PASS, SCATTER_ROWS };

ScatterPlan plan_scatter(const egs_dims *d, int mode, int act_dtype, ScatterPath path)
{
    ScatterPlan pl;
    memset(&pl, 0, sizeof(pl));
    const size_t N = (size_t)d->E * d->K;
    if (mode == EGS_SCATTER_ATOMIC && act_dtype == EGS_F32) return pl;
    if (path == SCATTER_FUSED || path == SCATTER_PASS) return pl;
    const size_t row_es = (mode != EGS_SCATTER_ATOMIC || act_dtype == EGS_F32) ? 4 : (size_t)elem_size(act_dtype);
    size_t at = 0;
    pl.seg_off_at = at; at += align_up((size_t)d->B * ((size_t)d->T + 1) * 4, 256);
    pl.perm_at = at;    at += align_up((size_t)d->B * N * 4, 256);
    pl.rank_at = at;    at += align_up((size_t)d->B * N * 4, 256);
    pl.cnt_at = at;     at += d->T > kCsrLdsTokens ? align_up((size_t)d->B * d->T * 4, 256) : 0;
    // long segments (tokens picked more than kLongSegment times): records and fp32 partial rows
    pl.long_tab_at = at;  at += align_up((size_t)d->B * long_tab_stride((int)N) * 4, 256);
    pl.long_part_at = at; at += align_up((size_t)d->B * long_max_slots((int)N) * d->I * 4, 256);
    pl.rows_at = at;    at += align_up((size_t)d->B * N * d->I * row_es, 256);
    pl.bytes = at;
    return pl;
}

DwPlan plan_dw(const egs_dims *d, int act_dtype)
{
    DwPlan pl;
    memset(&pl, 0, sizeof(pl));
    pl.BI = 128; pl.BJ = 64;
    pl.BK = act_dtype == EGS_F32 ? 32 : 64;
    pl.i_tiles = ceil_div(d->I, pl.BI);
    pl.j_tiles = ceil_div(d->J, pl.BJ);
    const int64_t Me = (int64_t)d->B * d->K;
    const int64_t base = (int64_t)d->E * pl.i_tiles * pl.j_tiles;
    int64_t S = base > 0 ? (512 + base - 1) / base : 1;
    const int64_t max_s = Me > 0 ? (Me + pl.BK - 1) / pl.BK : 1;
    if (S > max_s) S = max_s;
    if (S > 64) S = 64;
    if (S < 1) S = 1;
    int64_t rows = Me > 0 ? (Me + S - 1) / S : pl.BK;
    rows = (rows + pl.BK - 1) / pl.BK * pl.BK;
    S = Me > 0 ? (Me + rows - 1) / rows : 1;
    pl.S = (int)S;
    pl.rows_per_split = (int)rows;
    pl.bytes_general = S > 1 ? align_up((size_t)S * d->E * d->I * d->J * 4, 256) : 0;

    // large 16-bit shapes: 256 x 256 (or 256 x 128) tiles, 64-row slabs, splits only to give every CU a workgroup
    // (C4: 2 splits 42 us, 4 splits 49 us, none 50 us)
    pl.big_ok = act_dtype != EGS_F32 && d->I % 8 == 0 && d->J % 8 == 0 && d->I > 128 && d->J > 64 && Me >= 256 && d->E > 0;
    if (pl.big_ok) {
        pl.b_bq = d->J > 128 ? 256 : 128;
        pl.b_i_tiles = ceil_div(d->I, 256);
        pl.b_j_tiles = ceil_div(d->J, pl.b_bq);
        const int64_t tiles = (int64_t)d->E * pl.b_i_tiles * pl.b_j_tiles;
        int64_t s3 = (256 + tiles - 1) / tiles;
        const int64_t most = (Me + 255) / 256;              // at least four slabs per split
        if (s3 > most) s3 = most;
        if (s3 > 32) s3 = 32;
        if (s3 < 1) s3 = 1;
        int64_t r3 = ((Me + s3 - 1) / s3 + 63) / 64 * 64;
        s3 = (Me + r3 - 1) / r3;
        pl.b_S = (int)s3;
        pl.b_rows_per_split = (int)r3;
        pl.bytes_big = s3 > 1 ? align_up((size_t)s3 * d->E * d->I * d->J * 4, 256) : 0;
    }

    // small experts: 64 x 64 tiles, up to 1024 picks per workgroup, enough workgroups to cover the device
    pl.small_ok = act_dtype != EGS_F32 && d->I % 8 == 0 && d->J % 8 == 0 && d->I >= 8 && d->J >= 8 && d->I <= 128 &&
                  d->J <= 128 && Me > 0 && d->E > 0;
    if (pl.small_ok) {
        pl.s_i_tiles = ceil_div(d->I, 64);
        pl.s_j_tiles = ceil_div(d->J, 64);
        const int64_t tiles = (int64_t)d->E * pl.s_i_tiles * pl.s_j_tiles;
        int64_t s2 = (256 + tiles - 1) / tiles;
        const int64_t need = (Me + kDwSmallMaxRows - 1) / kDwSmallMaxRows, most = (Me + 127) / 128;
        if (s2 < need) s2 = need;
        if (s2 > most) s2 = most;
        int64_t r2 = ((Me + s2 - 1) / s2 + 127) / 128 * 128;
        s2 = (Me + r2 - 1) / r2;
        pl.s_S = (int)s2;
        pl.s_rows_per_split = (int)r2;
        pl.bytes_small = s2 > 1 ? align_up((size_t)s2 * d->E * d->I * d->J * 4, 256) : 0;
    }
    return pl;
}

// ------------------------------------------------------------------------------ small-expert fast paths
constexpr uint64_t kSpan32 = 0xFFFFFFFFull;      // the small kernels address with 32-bit byte offsets

bool small_shape_ok(int act_dtype, int R, int N)
{
    return act_dtype != EGS_F32 && (R == 32 || R == 64 || R == 128) && N % 8 == 0 && N >= 8 && N <= 128;
}

// one launch of rows_small_kernel, or its share of a heterogeneous launch
struct SmallRowsJob {
    SmallRowsParams p;
    int R, act_dtype, blocks;
    bool nmajor, gather, out_f32;
    size_t lds;
};
// one launch of dw_small_kernel (or its share of a heterogeneous launch) plus the second pass
struct SmallDwJob {
    SmallDwParams q;
    int blocks, act_dtype;
    size_t w_elems;
    bool done;          // set once the first pass has been enqueued
};

// one launch of dw_tile_kernel (or its share of a heterogeneous launch): the whole weight gradient, no second pass
struct DwTileJob {
    DwTileParams q;
    int blocks, act_dtype;
    bool wide;          // 32 x 64 tiles and 8 wavefronts (dw_tile_wide_kernel) instead of 32 x 32 and 4
    bool done;          // set once it has been enqueued
};

// A routing table in caller-owned memory (egs_routing_table_bytes): seg [B][T+1], perm [B][E*K], the picks of each batch
// element in a stable order by token.  Built once per Ind by a gather forward, read by the one-kernel scatters that follow.
struct RoutingTable { int32_t *seg, *perm; };


// Workgroup -> (expert, row tile) map of the small-expert row kernels (decode_rows_block): which operand is worth keeping
// XCD-local - the source rows, each read by ~E*K/T experts and fetched from beyond the L2 once per XCD that uses them,
// or W(e), fetched once per XCD that runs one of the expert's row tiles.  Row tiles take the XCDs only where that leaves none
// idle: in groups of eight, or 2 / 4 of them on 4 / 2 XCDs each.
// whether the routing table that rides in a gather launch is built by two workgroups per batch element
// (csr_count_half_body) instead of one: its shares must fit the registers and its counters a modest piece of LDS, there must
// be picks enough to split, and the launch must not grow beyond what the device holds at once (two of these kernels'
// workgroups fit a CU)
bool table_split_pays(const egs_dims *d, int nwaves, int gather_blocks, int round_blocks)
{
    const int64_t N = (int64_t)d->E * d->K;
    return N >= 256 && N <= (int64_t)nwaves * 1024 && csr_half_lds(d->T, nwaves) <= 64 * 1024 &&
           (int64_t)gather_blocks + 2 * (int64_t)d->B <= round_blocks;
}
int rows_xcd_map(const egs_dims *d, int R, int N, int es, int tiles_per_e)
{
    const double picks_per_token = (double)d->E * d->K / (d->T > 0 ? d->T : 1);
    const double x_bytes = (double)d->B * d->T * R * es, w_bytes = (double)d->E * R * N * es;
    const double by_expert = x_bytes * (picks_per_token < 8 ? (picks_per_token < 1 ? 1 : picks_per_token) : 8) + w_bytes;
    const double by_rows = x_bytes + w_bytes * (tiles_per_e < 8 ? tiles_per_e : 8);
    if (by_rows >= by_expert) return 0;
    if (tiles_per_e == 2 || tiles_per_e == 4) return 8 / tiles_per_e;
    return (tiles_per_e % 8 == 0 || tiles_per_e > 16) ? 1 : 0;
}
int rows_xcd_blocks(int map, int tiles_per_e, int E)
{
    return map == 0 ? 8 * ceil_div(E, 8) * tiles_per_e : map == 1 ? 8 * ceil_div(tiles_per_e, 8) * E : 8 * ceil_div(E, map);
}

bool make_gather_small(const void *X, const void *W, const void *Ind, void *Y, const egs_dims *d, int64_t ldx_b,
                       int64_t ldx_t, int act_dtype, int w_dtype, int ind_dtype, int w_layout, SmallRowsJob &j,
                       const RoutingTable *build = nullptr)
{
    const int R = d->I, N = d->J;
    if (g_force_generic || w_dtype != act_dtype || !small_shape_ok(act_dtype, R, N)) return false;
    if (!aligned_to(X, 16) || !aligned_to(W, 16) || !aligned_to(Y, 16)) return false;
    if ((ldx_b * 2) % 16 || (ldx_t * 2) % 16 || d->T == 0) return false;
    const int64_t Me = (int64_t)d->B * d->K;
    if (Me == 0 || d->E == 0) return false;
    const uint64_t x_span = ((uint64_t)(d->B - 1) * (uint64_t)ldx_b + (uint64_t)(d->T - 1) * (uint64_t)ldx_t + R) * 2;
    if (x_span > kSpan32 || (uint64_t)d->E * R * N * 2 > kSpan32 || (uint64_t)Me * d->E * N * 2 > kSpan32) return false;
    memset(&j, 0, sizeof(j));
    SmallRowsParams &p = j.p;
    p.A = (const char *)X; p.W = (const char *)W; p.Ind = Ind; p.C = (char *)Y;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K; p.N = N;
    p.lda_b = ldx_b; p.lda_t = ldx_t; p.ind_dtype = ind_dtype;
    p.tiles_per_e = (int)((Me + 255) / 256);
    if ((int64_t)8 * (ceil_div(d->E, 8) + 1) * (p.tiles_per_e + 8) > INT32_MAX / 2) return false;
    p.rows_share_xcd = rows_xcd_map(d, R, N, 2, p.tiles_per_e);
    j.R = R; j.act_dtype = act_dtype; j.gather = true; j.out_f32 = false; j.lds = 0;
    j.nmajor = (w_layout == EGS_W_EIJ);                 // [E,I,J] = [E,R,N]
    if (build != nullptr) {             // the routing table of a later scatter rides along: B more workgroups, first in line
        p.csr_blocks = d->B;
        p.seg_off = build->seg; p.perm = build->perm;
        j.lds = csr_count_lds(d->T, 4);
        // ... or 2 B, each ranking half of the picks (the ranking is what the build consists of, and the gather's workgroups
        // alone take less time than one workgroup's whole table: B64 T256 E32 K32, 6.8 -> 6.3 us for the launch)
        const int gather_blocks = rows_xcd_blocks(p.rows_share_xcd, p.tiles_per_e, p.E);
        if (table_split_pays(d, 4, gather_blocks, 512)) { p.csr_blocks = 2 * d->B; p.csr_split = 1; j.lds = csr_half_lds(d->T, 4); }
    }
    j.blocks = rows_xcd_blocks(p.rows_share_xcd, p.tiles_per_e, p.E) + p.csr_blocks;
    return true;
}

// product rows of the scatter in pick order; with `ride` the routing table is built by extra
// workgroups of the same launch
bool make_scatter_rows_small(const void *Y, const void *W, void *rows, bool rows_f32, const egs_dims *d, int act_dtype,
                             int w_layout, bool ride, const void *Ind, int ind_dtype, int32_t *seg_off, int32_t *perm,
                             int32_t *rank_tmp, int32_t *long_tab, SmallRowsJob &j)
{
    const int R = d->J, N = d->I;
    if (g_force_generic || !small_shape_ok(act_dtype, R, N)) return false;
    if (!aligned_to(Y, 16) || !aligned_to(W, 16)) return false;
    const int64_t Me = (int64_t)d->B * d->K;
    if (Me == 0 || d->E == 0) return false;
    if ((uint64_t)Me * d->E * R * 2 > kSpan32 || (uint64_t)d->E * R * N * 2 > kSpan32 ||
        (uint64_t)Me * d->E * N * 4 > kSpan32) return false;
    memset(&j, 0, sizeof(j));
    SmallRowsParams &p = j.p;
    p.A = (const char *)Y; p.W = (const char *)W; p.C = (char *)rows;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K; p.N = N;
    p.tiles_per_e = (int)((Me + 255) / 256);
    if (ride) {
        p.csr_blocks = d->B; p.Ind = Ind; p.ind_dtype = ind_dtype;
        p.seg_off = seg_off; p.perm = perm; p.rank_tmp = rank_tmp; p.long_tab = long_tab;
        j.lds = csr_count_lds(d->T, 4);
    }
    if ((int64_t)8 * ceil_div(d->E, 8) * p.tiles_per_e + p.csr_blocks > INT32_MAX / 2) return false;
    j.R = R; j.act_dtype = act_dtype; j.gather = false; j.out_f32 = rows_f32;
    j.nmajor = (w_layout == EGS_W_EJI);                 // [E,J,I] = [E,R,N]
    j.blocks = 8 * ceil_div(p.E, 8) * p.tiles_per_e + p.csr_blocks;
    return true;
}

bool make_dw_small(const void *Xs, const void *Ys, const void *Ind, void *dW, void *workspace, const egs_dims *d,
                   int64_t ldx_b, int64_t ldx_t, int act_dtype, int out_dtype, int ind_dtype, int dw_layout,
                   const DwPlan &pl, SmallDwJob &j)
{
    if (!pl.small_ok || g_force_generic || d->T == 0) return false;
    const uint64_t x_span = ((uint64_t)(d->B - 1) * (uint64_t)ldx_b + (uint64_t)(d->T - 1) * (uint64_t)ldx_t + d->I) * 2;
    if (!aligned_to(Xs, 16) || !aligned_to(Ys, 16) || !aligned_to(dW, 16) || (ldx_b * 2) % 16 || (ldx_t * 2) % 16) return false;
    if (x_span > kSpan32 || (uint64_t)d->B * d->E * d->K * d->J * 2 > kSpan32) return false;
    if ((int64_t)8 * ceil_div(d->E, 8) * pl.s_i_tiles * pl.s_j_tiles * pl.s_S > INT32_MAX / 2) return false;
    memset(&j, 0, sizeof(j));
    SmallDwParams &q = j.q;
    q.Xs = (const char *)Xs; q.Ys = (const char *)Ys; q.Ind = Ind; q.part = (float *)workspace; q.dW = (char *)dW;
    q.B = d->B; q.T = d->T; q.E = d->E; q.K = d->K; q.I = d->I; q.J = d->J;
    q.ldx_b = ldx_b; q.ldx_t = ldx_t; q.ind_dtype = ind_dtype;
    q.i_tiles = pl.s_i_tiles; q.j_tiles = pl.s_j_tiles; q.S = pl.s_S; q.rows_per_split = pl.s_rows_per_split;
    q.out_dtype = out_dtype; q.dw_layout = dw_layout;
    j.blocks = 8 * ceil_div(d->E, 8) * pl.s_i_tiles * pl.s_j_tiles * pl.s_S;
    j.act_dtype = act_dtype;
    j.w_elems = (size_t)d->E * d->I * d->J;
    return true;
}

// The one-pass weight gradient (32 x 32 tiles of dW(e), every workgroup reduces all picks of its expert) is taken
// when its tiles alone fill the device; with fewer tiles the picks are split instead (dw_small_kernel + second pass).
bool make_dw_tile(const void *Xs, const void *Ys, const void *Ind, void *dW, const egs_dims *d, int64_t ldx_b, int64_t ldx_t,
                  int act_dtype, int out_dtype, int ind_dtype, int dw_layout, DwTileJob &j, bool wide = false)
{
    if (g_force_generic) return false;
    const int ES = elem_size(act_dtype);
    if (d->I % 8 || d->J % 8 || d->I < 8 || d->J < 8 || d->I > 2048 || d->J > 128) return false;
    const int64_t Me = (int64_t)d->B * d->K;
    if (Me == 0 || d->E == 0 || d->T == 0) return false;
    if (ES == 2 && d->I > 128 && d->J > 64 && Me >= 256) return false;      // the 256-row tiles of the direct-to-LDS kernel do better there
    const int it = ceil_div(d->I, 32), jt = ceil_div(d->J, wide ? 64 : 32);
    if ((int64_t)d->E * it * jt < (wide ? 64 : 128)) return false;
    if (!aligned_to(Xs, 16) || !aligned_to(Ys, 16) || !aligned_to(dW, 16) || (ldx_b * ES) % 16 || (ldx_t * ES) % 16) return false;
    const uint64_t x_span = ((uint64_t)(d->B - 1) * (uint64_t)ldx_b + (uint64_t)(d->T - 1) * (uint64_t)ldx_t + d->I) * ES;
    const uint64_t y_span = (uint64_t)Me * d->E * d->J * ES;
    if (x_span >= (1ull << 31) || y_span >= (1ull << 31)) return false;
    if ((int64_t)8 * ceil_div(d->E, 8) * it * jt > INT32_MAX / 2) return false;
    memset(&j, 0, sizeof(j));
    DwTileParams &q = j.q;
    q.Xs = (const char *)Xs; q.Ys = (const char *)Ys; q.Ind = Ind; q.dW = (char *)dW;
    q.B = d->B; q.T = d->T; q.E = d->E; q.K = d->K; q.I = d->I; q.J = d->J;
    q.ldx_b = ldx_b; q.ldx_t = ldx_t; q.ind_dtype = ind_dtype;
    q.i_tiles = it; q.j_tiles = jt;
    q.out_dtype = out_dtype; q.dw_layout = dw_layout;
    q.x_bytes = (uint32_t)x_span; q.y_bytes = (uint32_t)y_span;
    j.blocks = 8 * ceil_div(d->E, 8) * it * jt;
    j.act_dtype = act_dtype;
    j.wide = wide;
    return true;
}

// Which tile a one-pass weight gradient launched on its own should use.  32 x 64 tiles fetch whole 128-byte lines on
// the Ys side and send half the requests per pick; 32 x 32 tiles only win when they fill the device exactly once and the
// reduction is short (16-bit, the reference's default shape: 10.1 against 10.6 us; E48: 15.0 / 11.5, B160: 24.5 / 21.2,
// I256: 16.3 / 12.5 us).
// In fp32 a wide tile is twice the matrix instructions for the same four wavefronts, so only the tile count decides
// (default shape 19.5 / 30.1 us, B160: 41.7 / 67.3, E48: 36.2 / 30.5, I256: 36.6 / 31.0 us).
bool dw_tile_wide_alone(const egs_dims *d, int act_dtype)
{
    constexpr int64_t kCUs = 256;
    const int64_t narrow_tiles = (int64_t)d->E * ceil_div(d->I, 32) * ceil_div(d->J, 32);
    if (d->J <= 32) return false;
    return narrow_tiles > kCUs || (act_dtype != EGS_F32 && (int64_t)d->B * d->K >= 4096);
}

int launch_dw_tile_alone(DwTileJob &j, hipStream_t s)
{
    if (j.act_dtype == EGS_F32) {
        // four wavefronts either way; both sizes of staging tiles need more than the default LDS limit
        static LdsGrant told_narrow, told_wide;
        const size_t lds = dw_tile_lds(kThreads / 64, j.wide ? 64 : 32, 4);
        const int rc = j.wide
            ? allow_large_lds((const void *)dw_tile_wide_f32_kernel, told_wide, lds, "hipFuncSetAttribute(dw_tile_wide_f32_kernel)")
            : allow_large_lds((const void *)dw_tile_kernel<ElemF32>, told_narrow, lds, "hipFuncSetAttribute(dw_tile_kernel)");
        if (rc != EGS_OK) return rc;
        if (j.wide) hipLaunchKernelGGL(dw_tile_wide_f32_kernel, dim3(j.blocks), dim3(kThreads), lds, s, j.q);
        else hipLaunchKernelGGL(dw_tile_kernel<ElemF32>, dim3(j.blocks), dim3(kThreads), lds, s, j.q);
    } else if (j.wide) {
        static LdsGrant told_bf16, told_f16;
        const size_t lds = dw_tile_lds(kDwWideThreads / 64, 64);
        const int rc = j.act_dtype == EGS_BF16
            ? allow_large_lds((const void *)dw_tile_wide_kernel<ElemBF16>, told_bf16, lds, "hipFuncSetAttribute(dw_tile_wide_kernel)")
            : allow_large_lds((const void *)dw_tile_wide_kernel<ElemF16>, told_f16, lds, "hipFuncSetAttribute(dw_tile_wide_kernel)");
        if (rc != EGS_OK) return rc;
        if (j.act_dtype == EGS_BF16) hipLaunchKernelGGL(dw_tile_wide_kernel<ElemBF16>, dim3(j.blocks), dim3(kDwWideThreads), lds, s, j.q);
        else hipLaunchKernelGGL(dw_tile_wide_kernel<ElemF16>, dim3(j.blocks), dim3(kDwWideThreads), lds, s, j.q);
    } else {
        const size_t lds = dw_tile_lds(kThreads / 64);
        if (j.act_dtype == EGS_BF16) hipLaunchKernelGGL(dw_tile_kernel<ElemBF16>, dim3(j.blocks), dim3(kThreads), lds, s, j.q);
        else hipLaunchKernelGGL(dw_tile_kernel<ElemF16>, dim3(j.blocks), dim3(kThreads), lds, s, j.q);
    }
    EGS_CHECK_LAUNCH(j.act_dtype == EGS_F32 ? (j.wide ? "dw_tile_wide_f32_kernel" : "dw_tile_kernel") : (j.wide ? "dw_tile_wide_kernel" : "dw_tile_kernel"));
    j.done = true;
    return EGS_OK;
}

// ---- fp32 gather of small experts (W(e) in LDS, fp32 matrix instruction)
// Two 16-pick row tiles per wavefront and eight wavefronts per workgroup: two wavefronts per SIMD, so that one's waits
// (row transposition, LDS fragment reads) sit under the other's matrix instructions (default shape 18.4 -> 16.8 us against
// four row tiles and four wavefronts)
constexpr int kSmallF32Waves = 8;       // 16 / TQ with TQ = 2 below

template <bool W_NMAJOR, int KS>
int launch_gather_small_f32_ks(const SmallRowsParams &p, int blocks, hipStream_t s)
{
    constexpr int TQ = 2, threads = 64 * (16 / TQ);
    static_assert(threads == 64 * kSmallF32Waves, "wavefronts per workgroup");
    size_t lds = rows_small_f32_lds(16 * KS, p.N);
    const size_t csr_lds = p.csr_split ? csr_half_lds(p.T, kSmallF32Waves) : csr_count_lds(p.T, kSmallF32Waves);
    if (p.csr_blocks > 0 && csr_lds > lds) lds = csr_lds;
    switch (p.N / 16) {
    case 1: hipLaunchKernelGGL((rows_small_f32_kernel<W_NMAJOR, KS, 1, TQ>), dim3(blocks), dim3(threads), lds, s, p); break;
    case 2: hipLaunchKernelGGL((rows_small_f32_kernel<W_NMAJOR, KS, 2, TQ>), dim3(blocks), dim3(threads), lds, s, p); break;
    case 3: hipLaunchKernelGGL((rows_small_f32_kernel<W_NMAJOR, KS, 3, TQ>), dim3(blocks), dim3(threads), lds, s, p); break;
    default: hipLaunchKernelGGL((rows_small_f32_kernel<W_NMAJOR, KS, 4, TQ>), dim3(blocks), dim3(threads), lds, s, p); break;
    }
    EGS_CHECK_LAUNCH("rows_small_f32_kernel");
    return EGS_OK;
}

// `used` reports whether the shape and operands qualified
// whether the fp32 small-expert gather takes these sizes and operands
bool gather_small_f32_takes(const void *X, const void *W, const void *Y, const egs_dims *d, int64_t ldx_b, int64_t ldx_t)
{
    const int R = d->I, N = d->J;
    if (g_force_generic || !(R == 32 || R == 64 || R == 128) || N % 16 != 0 || N < 16 || N > 64 || d->T == 0) return false;
    if (!aligned_to(X, 16) || !aligned_to(W, 16) || !aligned_to(Y, 16) || (ldx_b * 4) % 16 || (ldx_t * 4) % 16) return false;
    const int64_t Me = (int64_t)d->B * d->K;
    if (Me == 0 || d->E == 0) return false;
    const uint64_t x_span = ((uint64_t)(d->B - 1) * (uint64_t)ldx_b + (uint64_t)(d->T - 1) * (uint64_t)ldx_t + R) * 4;
    if (x_span > kSpan32 || (uint64_t)d->E * R * N * 4 > kSpan32 || (uint64_t)Me * d->E * N * 4 > kSpan32) return false;
    const int tiles_per_e = (int)((Me + 255) / 256);
    return (int64_t)8 * (ceil_div(d->E, 8) + 1) * (tiles_per_e + 8) <= INT32_MAX / 2;
}

// `build` (optional): the routing table of a later scatter over the same Ind is built by B more workgroups of the launch
int gather_small_f32(const void *X, const void *W, const void *Ind, void *Y, const egs_dims *d, int64_t ldx_b, int64_t ldx_t,
                     int ind_dtype, int w_layout, hipStream_t s, bool &used, const RoutingTable *build = nullptr)
{
    used = false;
    if (!gather_small_f32_takes(X, W, Y, d, ldx_b, ldx_t)) return EGS_OK;
    const int R = d->I, N = d->J;
    const int64_t Me = (int64_t)d->B * d->K;
    SmallRowsParams p;
    memset(&p, 0, sizeof(p));
    p.A = (const char *)X; p.W = (const char *)W; p.Ind = Ind; p.C = (char *)Y;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K; p.N = N;
    p.lda_b = ldx_b; p.lda_t = ldx_t; p.ind_dtype = ind_dtype;
    p.tiles_per_e = (int)((Me + 255) / 256);
    if ((int64_t)8 * (ceil_div(d->E, 8) + 1) * (p.tiles_per_e + 8) > INT32_MAX / 2) return EGS_OK;
    p.rows_share_xcd = rows_xcd_map(d, R, N, 4, p.tiles_per_e);
    if (build != nullptr) {
        p.csr_blocks = d->B; p.seg_off = build->seg; p.perm = build->perm;
        if (table_split_pays(d, kSmallF32Waves, rows_xcd_blocks(p.rows_share_xcd, p.tiles_per_e, p.E), 512)) { p.csr_blocks = 2 * d->B; p.csr_split = 1; }
    }
    const int blocks = rows_xcd_blocks(p.rows_share_xcd, p.tiles_per_e, p.E) + p.csr_blocks;
    used = true;
    const bool nmajor = (w_layout == EGS_W_EIJ);        // [E,I,J] = [E,R,N]
    switch (R) {
    case 32: return nmajor ? launch_gather_small_f32_ks<true, 2>(p, blocks, s) : launch_gather_small_f32_ks<false, 2>(p, blocks, s);
    case 64: return nmajor ? launch_gather_small_f32_ks<true, 4>(p, blocks, s) : launch_gather_small_f32_ks<false, 4>(p, blocks, s);
    default: return nmajor ? launch_gather_small_f32_ks<true, 8>(p, blocks, s) : launch_gather_small_f32_ks<false, 8>(p, blocks, s);
    }
}

// ---- launch of a rows job, alone or sharing the launch with a weight gradient of the same call (its one-pass form,
// or the first pass of its split form)
template <class TT, bool W_NMAJOR, int KS, int TN, bool GATHER, bool OUT_F32>
int launch_rows_small_one(SmallRowsJob &j, SmallDwJob *dw, DwTileJob *dwt, hipStream_t s)
{
    if constexpr (GATHER) {
        if (dwt != nullptr) {       // dwt->wide, and j regridded for 8 wavefronts per workgroup (see pair_gather_with_dw_tile)
            static LdsGrant told;
            const size_t tile_lds = dw_tile_lds(kDwWideThreads / 64, 64);
            const int rc = allow_large_lds((const void *)rows_dw_tile_kernel<TT, W_NMAJOR, KS, TN>, told, tile_lds,
                                           "hipFuncSetAttribute(rows_dw_tile_kernel)");
            if (rc != EGS_OK) return rc;
            hipLaunchKernelGGL((rows_dw_tile_kernel<TT, W_NMAJOR, KS, TN>), dim3(j.blocks + dwt->blocks), dim3(kDwWideThreads),
                               tile_lds, s, j.p, dwt->q, j.blocks);
            EGS_CHECK_LAUNCH("rows_dw_tile_kernel");
            dwt->done = true;
            return EGS_OK;
        }
    }
    if (dw != nullptr) {
        hipLaunchKernelGGL((rows_dw_small_kernel<TT, W_NMAJOR, KS, TN, GATHER, OUT_F32>), dim3(j.blocks + dw->blocks),
                           dim3(kThreads), j.lds, s, j.p, dw->q, j.blocks);
        dw->done = true;
    } else {
        hipLaunchKernelGGL((rows_small_kernel<TT, W_NMAJOR, KS, TN, GATHER, OUT_F32>), dim3(j.blocks), dim3(kThreads),
                           j.lds, s, j.p);
    }
    EGS_CHECK_LAUNCH(dw != nullptr ? "rows_dw_small_kernel" : "rows_small_kernel");
    return EGS_OK;
}

template <class TT, bool W_NMAJOR, int TN, bool GATHER, bool OUT_F32>
int launch_rows_small_ks(SmallRowsJob &j, SmallDwJob *dw, DwTileJob *dwt, hipStream_t s)
{
    switch (j.R) {
    case 32: return launch_rows_small_one<TT, W_NMAJOR, 1, TN, GATHER, OUT_F32>(j, dw, dwt, s);
    case 64: return launch_rows_small_one<TT, W_NMAJOR, 2, TN, GATHER, OUT_F32>(j, dw, dwt, s);
    default: return launch_rows_small_one<TT, W_NMAJOR, 4, TN, GATHER, OUT_F32>(j, dw, dwt, s);
    }
}

template <class TT, bool GATHER, bool OUT_F32>
int launch_rows_small_tn(SmallRowsJob &j, SmallDwJob *dw, DwTileJob *dwt, hipStream_t s)
{
    if (j.p.N <= 64)
        return j.nmajor ? launch_rows_small_ks<TT, true, 4, GATHER, OUT_F32>(j, dw, dwt, s)
                        : launch_rows_small_ks<TT, false, 4, GATHER, OUT_F32>(j, dw, dwt, s);
    return j.nmajor ? launch_rows_small_ks<TT, true, 8, GATHER, OUT_F32>(j, dw, dwt, s)
                    : launch_rows_small_ks<TT, false, 8, GATHER, OUT_F32>(j, dw, dwt, s);
}

template <class TT>
int launch_rows_small_tt(SmallRowsJob &j, SmallDwJob *dw, DwTileJob *dwt, hipStream_t s)
{
    if (j.gather) return launch_rows_small_tn<TT, true, false>(j, dw, dwt, s);
    return j.out_f32 ? launch_rows_small_tn<TT, false, true>(j, dw, dwt, s) : launch_rows_small_tn<TT, false, false>(j, dw, dwt, s);
}

// `dwt` (one-pass weight gradient) shares the launch of a gather only; `dw` (first pass of the split form) any rows job
int launch_rows_small_job(SmallRowsJob &j, SmallDwJob *dw, DwTileJob *dwt, hipStream_t s)
{
    return j.act_dtype == EGS_BF16 ? launch_rows_small_tt<ElemBF16>(j, dw, dwt, s) : launch_rows_small_tt<ElemF16>(j, dw, dwt, s);
}

int launch_dw_small_alone(SmallDwJob &j, hipStream_t s)
{
    if (j.act_dtype == EGS_BF16) hipLaunchKernelGGL(dw_small_kernel<ElemBF16>, dim3(j.blocks), dim3(kThreads), 0, s, j.q);
    else hipLaunchKernelGGL(dw_small_kernel<ElemF16>, dim3(j.blocks), dim3(kThreads), 0, s, j.q);
    EGS_CHECK_LAUNCH("dw_small_kernel");
    j.done = true;
    return EGS_OK;
}

int launch_dw_reduce4(const SmallDwJob &j, hipStream_t s)
{
    if (j.q.S <= 1) return EGS_OK;
    hipLaunchKernelGGL(dw_reduce4_kernel, dim3(grid_1d(j.w_elems / 4, 2048)), dim3(kThreads), 0, s,
                       (const float *)j.q.part, j.q.dW, j.q.S, j.w_elems / 4, j.q.out_dtype);
    EGS_CHECK_LAUNCH("dw_reduce4_kernel");
    return EGS_OK;
}

// routing table of the deterministic scatter as a launch of its own: counting sort with
// per-wavefront histograms when they fit in LDS, bitonic sort in LDS for long sequences, else
// the one-wavefront counting sort
int launch_routing_table(const void *Ind, int ind_dtype, const egs_dims *d, int32_t *seg_off, int32_t *perm,
                         int32_t *rank_tmp, int32_t *cnt, int32_t *long_tab, hipStream_t s)
{
    const int64_t N = (int64_t)d->E * d->K;
    if (N >= 1) {
        // as many wavefronts as the per-wavefront histograms leave room for (up to 148 KB of LDS)
        const size_t budget = 148 * 1024;
        int nw = (int)((N + 63) / 64);
        if (nw > 16) nw = 16;
        while (nw > 1 && csr_count_lds(d->T, nw) > budget) nw >>= 1;
        const size_t lds = csr_count_lds(d->T, nw);
        if (lds <= budget) {
            static LdsGrant told;
            const int rc_lds = allow_large_lds((const void *)csr_count_kernel, told, lds, "hipFuncSetAttribute(csr_count_kernel)");
            if (rc_lds != EGS_OK) return rc_lds;
            hipLaunchKernelGGL(csr_count_kernel, dim3(d->B), dim3(64 * nw), lds, s, Ind, ind_dtype, d->T, (int32_t)N, seg_off, perm, rank_tmp, long_tab);
            EGS_CHECK_LAUNCH("csr_count_kernel");
            return EGS_OK;
        }
    }
    int NP = 1, QB = 0;
    while (NP < N) { NP <<= 1; ++QB; }
    const bool sortable = N >= 1 && NP <= 32768 && (((uint64_t)d->T << QB) <= 0xFFFFFFFFull);
    if (sortable) {
        const size_t lds = (size_t)NP * 4;
        static LdsGrant told;
        const int rc_lds = allow_large_lds((const void *)csr_sort_kernel, told, lds, "hipFuncSetAttribute(csr_sort_kernel)");
        if (rc_lds != EGS_OK) return rc_lds;
        int threads = NP / 2;
        if (threads < 64) threads = 64;
        if (threads > 1024) threads = 1024;
        hipLaunchKernelGGL(csr_sort_kernel, dim3(d->B), dim3(threads), lds, s, Ind, ind_dtype, d->T, (int32_t)N, NP, QB, seg_off, perm, long_tab);
        EGS_CHECK_LAUNCH("csr_sort_kernel");
        return EGS_OK;
    }
    const size_t lds = d->T > kCsrLdsTokens ? 0 : (size_t)d->T * 4;
    hipLaunchKernelGGL(csr_build_kernel, dim3(d->B), dim3(kWave), lds, s, Ind, ind_dtype, d->T, (int32_t)N, seg_off, perm, cnt, long_tab);
    EGS_CHECK_LAUNCH("csr_build_kernel");
    return EGS_OK;
}

template <class TT, class PT>
void launch_segment_sum8(const SegSumParams &sp, int seg_blocks, hipStream_t s)
{
    hipLaunchKernelGGL((segment_sum_kernel<TT, PT, 8>), dim3(seg_blocks), dim3(kThreads), 0, s, sp);
}

// fixed-order reduction of the product rows per token; when `reduce` is given (and qualifies) the
// second pass of that weight gradient shares the launch
int launch_segment_sum(const void *rows, bool rows_f32, const int32_t *seg_off, const int32_t *perm, int32_t *long_tab,
                       float *long_part, void *Out, const egs_dims *d, int act_dtype, SmallDwJob *reduce, hipStream_t s)
{
    const int N = d->E * d->K;
    const bool vw4 = d->I % 4 == 0 && aligned_to(Out, 16);
    // eight elements of a row per thread (16 bytes of a 16-bit row, two 16-byte loads of an fp32 row): half the threads,
    // table look-ups and address arithmetic per row
    const bool vw8 = vw4 && d->I % 8 == 0 && aligned_to(rows, 16) &&
                     !(reduce != nullptr && reduce->done && reduce->q.S > 1);
    const int iv = vw8 ? d->I / 8 : vw4 ? d->I / 4 : d->I;
    SegSumParams sp;
    memset(&sp, 0, sizeof(sp));
    sp.P = rows; sp.seg_off = seg_off; sp.perm = perm; sp.out = (char *)Out;
    sp.B = d->B; sp.T = d->T; sp.N = N; sp.I = d->I;
    while ((1 << sp.tpr_log2) < iv && sp.tpr_log2 < 8) ++sp.tpr_log2;      // threads sharing an output row (<= 256)
    sp.gx = ceil_div(d->T, kThreads >> sp.tpr_log2);
    sp.gy = d->B;
    while ((int64_t)sp.gx * sp.gy > (1 << 22)) sp.gy = (sp.gy + 1) / 2;     // stride loop over batch elements beyond that
    sp.long_tab = long_tab; sp.long_part = long_part;
    const int64_t all_seg_blocks = (int64_t)sp.gx * sp.gy + (int64_t)d->B * long_max_slots(N);
    if (all_seg_blocks > INT32_MAX / 2) return EGS_ERR_BAD_SHAPE;
    const int seg_blocks = (int)all_seg_blocks;
    const bool fuse = reduce != nullptr && reduce->done && reduce->q.S > 1 && vw4;
    const int red_blocks = fuse ? grid_1d(reduce->w_elems / 4, 1024) : 0;
#define EGS_SEGSUM(TT, PT)                                                                                                  \
    do {                                                                                                                    \
        if (fuse) hipLaunchKernelGGL((segsum_dwreduce_kernel<TT, PT, 4>), dim3(seg_blocks + red_blocks), dim3(kThreads), 0, \
                                     s, sp, seg_blocks, (const float *)reduce->q.part, reduce->q.dW, reduce->q.S,           \
                                     reduce->w_elems / 4, reduce->q.out_dtype);                                             \
        else if (vw8) launch_segment_sum8<TT, PT>(sp, seg_blocks, s);                                                       \
        else if (vw4) hipLaunchKernelGGL((segment_sum_kernel<TT, PT, 4>), dim3(seg_blocks), dim3(kThreads), 0, s, sp);      \
        else hipLaunchKernelGGL((segment_sum_kernel<TT, PT, 1>), dim3(seg_blocks), dim3(kThreads), 0, s, sp);               \
    } while (0)
    if (act_dtype == EGS_F32) EGS_SEGSUM(ElemF32, float);
    else if (act_dtype == EGS_F16) { if (rows_f32) EGS_SEGSUM(ElemF16, float); else EGS_SEGSUM(ElemF16, uint16_t); }
    else { if (rows_f32) EGS_SEGSUM(ElemBF16, float); else EGS_SEGSUM(ElemBF16, uint16_t); }
#undef EGS_SEGSUM
    EGS_CHECK_LAUNCH(fuse ? "segsum_dwreduce_kernel" : "segment_sum_kernel");
    if (fuse) reduce->q.S = 1;              // second pass done
    return EGS_OK;
}

// ------------------------------------------------------------------------------ fused small-expert scatter
template <class TT, bool W_NMAJOR, int KS>
int launch_scatter_fused_one(const ScatterFusedParams &p, size_t lds, int blocks, SmallDwJob *dw, DwTileJob *dwt, hipStream_t s)
{
    static LdsGrant told_plain, told_dw, told_dwt, told_multi;      // one set per template instantiation
    if constexpr (TT::ES != 2) { dw = nullptr; dwt = nullptr; }     // the small weight gradients exist for 16-bit types only
    const char *name = "scatter_fused_kernel";
    if (p.experts_per_pass < p.E && p.tab_seg != nullptr) {
        name = "scatter_fused_multi_table_kernel";
        static LdsGrant told_multi_tab;
        const int rc_lds = allow_large_lds((const void *)scatter_fused_multi_table_kernel<TT, W_NMAJOR, KS>, told_multi_tab, lds,
                                           "hipFuncSetAttribute(scatter_fused_multi_table_kernel)");
        if (rc_lds != EGS_OK) return rc_lds;
        hipLaunchKernelGGL((scatter_fused_multi_table_kernel<TT, W_NMAJOR, KS>), dim3(blocks), dim3(kFusedThreads), lds, s, p);
    } else if (p.experts_per_pass < p.E) {
        // several passes over groups of experts: a launch of its own (a weight gradient of the same call follows alone)
        name = "scatter_fused_multi_kernel";
        const int rc_lds = allow_large_lds((const void *)scatter_fused_multi_kernel<TT, W_NMAJOR, KS>, told_multi, lds,
                                           "hipFuncSetAttribute(scatter_fused_multi_kernel)");
        if (rc_lds != EGS_OK) return rc_lds;
        hipLaunchKernelGGL((scatter_fused_multi_kernel<TT, W_NMAJOR, KS>), dim3(blocks), dim3(kFusedThreads), lds, s, p);
    } else if (p.tab_seg != nullptr && dwt != nullptr && !dwt->wide && TT::ES == 2) {
      if constexpr (TT::ES == 2) {
        name = "scatter_fused_dwtile_table_kernel";
        static LdsGrant told_dwt_tab;
        const size_t tile_lds = dw_tile_lds(kFusedThreads / 64);
        const size_t need = lds > tile_lds ? lds : tile_lds;
        const int rc_lds = allow_large_lds((const void *)scatter_fused_dwtile_table_kernel<TT, W_NMAJOR, KS>, told_dwt_tab, need,
                                           "hipFuncSetAttribute(scatter_fused_dwtile_table_kernel)");
        if (rc_lds != EGS_OK) return rc_lds;
        hipLaunchKernelGGL((scatter_fused_dwtile_table_kernel<TT, W_NMAJOR, KS>), dim3(blocks + dwt->blocks), dim3(kFusedThreads), need,
                           s, p, dwt->q, blocks);
        dwt->done = true;
      }
    } else if (p.tab_seg != nullptr && dw == nullptr && (dwt == nullptr || dwt->wide || TT::ES != 2)) {
        name = "scatter_fused_table_kernel";
        static LdsGrant told_tab;
        const int rc_lds = allow_large_lds((const void *)scatter_fused_table_kernel<TT, W_NMAJOR, KS>, told_tab, lds,
                                           "hipFuncSetAttribute(scatter_fused_table_kernel)");
        if (rc_lds != EGS_OK) return rc_lds;
        hipLaunchKernelGGL((scatter_fused_table_kernel<TT, W_NMAJOR, KS>), dim3(blocks), dim3(kFusedThreads), lds, s, p);
    } else if (dwt != nullptr && !dwt->wide) {
      if constexpr (TT::ES == 2) {
        name = "scatter_fused_dwtile_kernel";
        const size_t tile_lds = dw_tile_lds(kFusedThreads / 64);
        const size_t need = lds > tile_lds ? lds : tile_lds;
        const int rc_lds = allow_large_lds((const void *)scatter_fused_dwtile_kernel<TT, W_NMAJOR, KS>, told_dwt, need,
                                           "hipFuncSetAttribute(scatter_fused_dwtile_kernel)");
        if (rc_lds != EGS_OK) return rc_lds;
        hipLaunchKernelGGL((scatter_fused_dwtile_kernel<TT, W_NMAJOR, KS>), dim3(blocks + dwt->blocks), dim3(kFusedThreads), need,
                           s, p, dwt->q, blocks);
        dwt->done = true;
      }
    } else if (dw != nullptr) {
      if constexpr (TT::ES == 2) {
        name = "scatter_fused_dw_kernel";
        const size_t dw_lds = (size_t)kDwSmallLdsBytes * (kFusedThreads / kThreads);       // one 16 KB tile per wavefront
        const size_t need = lds > dw_lds ? lds : dw_lds;
        const int rc_lds = allow_large_lds((const void *)scatter_fused_dw_kernel<TT, W_NMAJOR, KS>, told_dw, need,
                                           "hipFuncSetAttribute(scatter_fused_dw_kernel)");
        if (rc_lds != EGS_OK) return rc_lds;
        hipLaunchKernelGGL((scatter_fused_dw_kernel<TT, W_NMAJOR, KS>), dim3(blocks + dw->blocks), dim3(kFusedThreads), need, s, p,
                           dw->q, blocks);
        dw->done = true;
      }
    } else {
        const int rc_lds = allow_large_lds((const void *)scatter_fused_kernel<TT, W_NMAJOR, KS>, told_plain, lds,
                                           "hipFuncSetAttribute(scatter_fused_kernel)");
        if (rc_lds != EGS_OK) return rc_lds;
        hipLaunchKernelGGL((scatter_fused_kernel<TT, W_NMAJOR, KS>), dim3(blocks), dim3(kFusedThreads), lds, s, p);
    }
    EGS_CHECK_LAUNCH(name);
    return EGS_OK;
}

template <class TT, bool W_NMAJOR>
int launch_scatter_fused_ks(const ScatterFusedParams &p, int R, size_t lds, int blocks, SmallDwJob *dw, DwTileJob *dwt, hipStream_t s)
{
    switch (R / (4 * TT::VEC)) {        // MFMA steps of four 16-byte chunks
    case 1: return launch_scatter_fused_one<TT, W_NMAJOR, 1>(p, lds, blocks, dw, dwt, s);
    case 2: return launch_scatter_fused_one<TT, W_NMAJOR, 2>(p, lds, blocks, dw, dwt, s);
    default: return launch_scatter_fused_one<TT, W_NMAJOR, 4>(p, lds, blocks, dw, dwt, s);
    }
}

// Does the one-kernel scatter of small experts (product rows stay in LDS, no workspace) take this problem, and in how
// many passes over groups of experts?  experts_per_pass == E: one pass.
struct FusedPlan { bool ok; int experts_per_pass; size_t lds; };

FusedPlan scatter_fused_plan(const void *Y, const void *W, const void *Out, const egs_dims *d, int act_dtype)
{
    const FusedPlan no = {false, 0, 0};
    const int R = d->J, N = d->I;
    const int64_t NP = (int64_t)d->E * d->K;
    if (g_force_generic || !(R == 32 || R == 64 || (R == 128 && act_dtype != EGS_F32))) return no;
    const int ES = elem_size(act_dtype);
    if (N < kFusedCols || N % kFusedCols != 0 || NP < 1 || NP > 4096 || d->T < 1 || d->B < 1) return no;
    if (!aligned_to(Y, 16) || !aligned_to(W, 16) || !aligned_to(Out, 16)) return no;
    if ((uint64_t)d->B * NP * R * ES > kSpan32 || (uint64_t)d->E * R * N * ES > kSpan32) return no;
    const int slices = N / kFusedCols;
    const int64_t blocks = (int64_t)8 * ceil_div(d->B, 8) * slices;
    if (blocks > INT32_MAX / 2 || (int64_t)d->B * slices < 8) return no;        // fewer workgroups are not worth it
    const size_t budget = 156 * 1024;
    if (NP <= 1024 && scatter_fused_lds(d->T, (int)NP) <= budget) return {true, d->E, scatter_fused_lds(d->T, (int)NP)};
    // groups of experts: as few passes as the rows' share of LDS allows, of equal size
    if (d->T > (kFusedThreads >> 3) * kFusedMultiTokens) return no;
    const size_t fixed = scatter_fused_lds(d->T, (int)NP, 0);
    if (fixed >= budget) return no;
    const int64_t fit = (int64_t)((budget - fixed) / ((size_t)d->K * kFusedCols * 4));     // experts whose rows fit
    if (fit < 1) return no;
    const int passes = ceil_div(d->E, (int)(fit < d->E ? fit : d->E));
    if (passes < 2 || passes > kFusedMaxPasses) return no;
    const int per_pass = ceil_div(d->E, passes);
    return {true, per_pass, scatter_fused_lds(d->T, (int)NP, per_pass * d->K)};
}

// whether the one-kernel scatter planned as `fp` can take its routing table from memory: what the kernel's registers stage
// (one pass: 1024 picks, T + 1 <= 2048 offsets; in passes: 2048 picks, T <= 512, 16-bit types - in fp32 the pass kernel
// measured slower with the table than sorting for itself: 131 against 128 us for gather + scatter + gather backward at
// B64 T256 E60 K32 I128 J64)
bool fused_reads_table(const FusedPlan &fp, const egs_dims *d, int act_dtype)
{
    if (!fp.ok) return false;
    const int64_t NP = (int64_t)d->E * d->K;
    if (fp.experts_per_pass == d->E) return NP <= 1024 && d->T + 1 <= 2048;
    return act_dtype != EGS_F32 && NP <= 2048 && d->T <= 512;
}

bool scatter_fused_takes(const void *Y, const void *W, const void *Out, const egs_dims *d, int act_dtype)
{
    return scatter_fused_plan(Y, W, Out, d, act_dtype).ok;
}

// The one-kernel scatters come first where they apply (they are the fastest there and need no workspace).  Beyond them
// the product rows go through the workspace, unless the caller asks for the compact mode: the one-kernel scatter in
// passes keeps them in LDS and sorts each pass's picks there too, for any number of picks per batch element and with no
// workspace at all - at B16 T1024 E64 K128 I512 J128 in 136 us under Zipf routing and 133 us under even routing, where
// the product rows through 270 MB of workspace take 120 and 105 us.
ScatterPath scatter_choose(const void *Y, const void *W, const void *Out, const egs_dims *d, int act_dtype, int mode)
{
    if (scatter_fused_takes(Y, W, Out, d, act_dtype)) return SCATTER_FUSED;
    if (mode == EGS_SCATTER_COMPACT && scatter_pass_plan(Y, W, Out, d, act_dtype).ok) return SCATTER_PASS;
    return SCATTER_ROWS;
}

// GEMM-scatter of small experts in one kernel; the caller has checked scatter_fused_takes().  Both scatter modes
// take it: it is bitwise reproducible and needs no workspace.
int scatter_fused(const void *Y, const void *W, const void *Ind, void *Out, const egs_dims *d, int act_dtype, int ind_dtype,
                  int w_layout, SmallDwJob *dw, DwTileJob *dwt, hipStream_t s, const RoutingTable *use = nullptr)
{
    const int R = d->J, N = d->I;
    const int64_t NP = (int64_t)d->E * d->K;
    const FusedPlan fp = scatter_fused_plan(Y, W, Out, d, act_dtype);
    if (!fp.ok) return EGS_ERR_UNSUPPORTED;
    const size_t lds = fp.lds;
    const int slices = N / kFusedCols;
    const int64_t blocks = (int64_t)8 * ceil_div(d->B, 8) * slices;
    ScatterFusedParams p;
    memset(&p, 0, sizeof(p));
    p.A = (const char *)Y; p.W = (const char *)W; p.Ind = Ind; p.out = (char *)Out;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K; p.N = N;
    p.ind_dtype = ind_dtype;
    p.slices = slices;
    p.experts_per_pass = fp.experts_per_pass;
    if (use != nullptr && fused_reads_table(fp, d, act_dtype)) { p.tab_seg = use->seg; p.tab_perm = use->perm; }
    p.perm_at = (int32_t)((int64_t)fp.experts_per_pass * d->K * kFusedCols * 4);
    p.cnt_at = p.perm_at + (int32_t)(NP * 4);
    p.zero_at = (int32_t)scatter_fused_zero_at(d->T, (int)NP, fp.experts_per_pass * d->K);
    // where the rows come from a small-expert gather (256 picks of one expert per workgroup, row tiles mapped to XCDs), the
    // batch elements of one of its row tiles - 256 / K of them - were written on one XCD
    p.xcd_batch = (d->K == 32 || d->K == 64 || d->K == 128 || d->K == 256) ? 256 / d->K : 2;
    const bool nmajor = (w_layout == EGS_W_EJI);        // [E,J,I] = [E,R,N]
    if (act_dtype == EGS_F32)
        return nmajor ? launch_scatter_fused_ks<ElemF32, true>(p, R, lds, (int)blocks, nullptr, nullptr, s)
                      : launch_scatter_fused_ks<ElemF32, false>(p, R, lds, (int)blocks, nullptr, nullptr, s);
    if (act_dtype == EGS_F16)
        return nmajor ? launch_scatter_fused_ks<ElemF16, true>(p, R, lds, (int)blocks, dw, dwt, s)
                      : launch_scatter_fused_ks<ElemF16, false>(p, R, lds, (int)blocks, dw, dwt, s);
    return nmajor ? launch_scatter_fused_ks<ElemBF16, true>(p, R, lds, (int)blocks, dw, dwt, s)
                  : launch_scatter_fused_ks<ElemBF16, false>(p, R, lds, (int)blocks, dw, dwt, s);
}

// Which weight-gradient kernel takes these operands, and the workspace it needs.  egs_workspace_bytes asks with
// stand-in operands (dense, 16-byte aligned); the entry points ask with the real ones, so what is planned and what
// runs agree by construction.
enum DwPath { DW_TILE, DW_SMALL, DW_BIG, DW_GENERAL };
struct DwChoice { DwPath path; size_t bytes; };

DwChoice dw_choose(const void *Xs, const void *Ys, void *dW, const egs_dims *d, int64_t ldx_b, int64_t ldx_t, int act_dtype,
                   const DwPlan &pl)
{
    DwTileJob tj;
    if (make_dw_tile(Xs, Ys, nullptr, dW, d, ldx_b, ldx_t, act_dtype, act_dtype, 0, 0, tj)) return {DW_TILE, 0};
    SmallDwJob sj;
    if (make_dw_small(Xs, Ys, nullptr, dW, nullptr, d, ldx_b, ldx_t, act_dtype, act_dtype, 0, 0, pl, sj)) return {DW_SMALL, pl.bytes_small};
    if (dw_big_takes(pl, Xs, Ys, dW, d, ldx_b, ldx_t, act_dtype)) return {DW_BIG, pl.bytes_big};
    return {DW_GENERAL, pl.bytes_general};
}

void *const kStandInPtr = (void *)(uintptr_t)4096;      // aligned, never dereferenced

size_t dw_bytes_planned(const egs_dims *d, int act_dtype)
{
    return dw_choose(kStandInPtr, kStandInPtr, kStandInPtr, d, (int64_t)d->T * d->I, d->I, act_dtype, plan_dw(d, act_dtype)).bytes;
}
size_t scatter_bytes_planned(const egs_dims *d, int mode, int act_dtype)
{
    return plan_scatter(d, mode, act_dtype, scatter_choose(kStandInPtr, kStandInPtr, kStandInPtr, d, act_dtype, mode)).bytes;
}

// Layout of a caller-owned routing table, for the sizes whose one-kernel scatter can read one (16-bit types, one pass,
// T + 1 <= 2048 table offsets per batch element); `ok` false: a table would not be used.
struct TableLayout { bool ok; size_t perm_at, bytes; };
TableLayout routing_table_layout(const egs_dims *d, int act_dtype)
{
    TableLayout l = {false, 0, 0};
    if (!(act_dtype == EGS_F16 || act_dtype == EGS_BF16 || act_dtype == EGS_F32)) return l;
    const FusedPlan fp = scatter_fused_plan(kStandInPtr, kStandInPtr, kStandInPtr, d, act_dtype);
    if (!fused_reads_table(fp, d, act_dtype)) return l;
    // the table pays only when its build rides in the gather forward's launch (as a launch of its own it costs more than
    // the two scatters save): the small-expert gather of the type must take these sizes too
    if (act_dtype == EGS_F32) {
        if (!gather_small_f32_takes(kStandInPtr, kStandInPtr, kStandInPtr, d, (int64_t)d->T * d->I, d->I) ||
            csr_count_lds(d->T, kSmallF32Waves) > 64 * 1024)
            return l;
    } else {
        SmallRowsJob gj;
        if (!make_gather_small(kStandInPtr, kStandInPtr, kStandInPtr, kStandInPtr, d, (int64_t)d->T * d->I, d->I, act_dtype,
                               act_dtype, EGS_IND_I32, EGS_W_EIJ, gj))
            return l;
    }
    l.ok = true;
    l.perm_at = align_up((size_t)d->B * (d->T + 1) * 4, 256);
    l.bytes = l.perm_at + align_up((size_t)d->B * d->E * d->K * 4, 256);
    return l;
}

// checks a table argument of an entry point; fills `t` when the table is to be used
int check_table_arg(void *table, size_t table_bytes, const egs_dims *d, int act_dtype, RoutingTable &t, bool &have)
{
    have = false;
    if (table == nullptr) return EGS_OK;
    const TableLayout l = routing_table_layout(d, act_dtype);
    if (!l.ok) return EGS_ERR_UNSUPPORTED;
    if (!aligned_to(table, 256)) return EGS_ERR_ALIGNMENT;
    if (table_bytes < l.bytes) return EGS_ERR_WORKSPACE;
    t.seg = (int32_t *)table;
    t.perm = (int32_t *)((char *)table + l.perm_at);
    have = true;
    return EGS_OK;
}

// ------------------------------------------------------------------------------ implementations
int gather_gemm_impl(const void *X, const void *W, const void *Ind, void *Y, const float *w_scale,
                     const egs_dims *d, int64_t ldx_b, int64_t ldx_t, int act_dtype, int w_dtype, int ind_dtype,
                     int w_layout, hipStream_t s, const RoutingTable *build = nullptr)
{
    const int ES = elem_size(act_dtype), WES = elem_size(w_dtype);
    if (w_scale == nullptr) {
        SmallRowsJob j;
        if (make_gather_small(X, W, Ind, Y, d, ldx_b, ldx_t, act_dtype, w_dtype, ind_dtype, w_layout, j, build))
            return launch_rows_small_job(j, nullptr, nullptr, s);
    }
    if (w_scale == nullptr && act_dtype == EGS_F32 && w_dtype == EGS_F32) {
        bool used = false;
        const int rc = gather_small_f32(X, W, Ind, Y, d, ldx_b, ldx_t, ind_dtype, w_layout, s, used, build);
        if (used) return rc;
    }
    if (build != nullptr) {             // no launch for the table to ride in: a launch of its own
        const int rc = launch_routing_table(Ind, ind_dtype, d, build->seg, build->perm, nullptr, nullptr, nullptr, s);
        if (rc != EGS_OK) return rc;
    }
    RowsGemmParams p;
    memset(&p, 0, sizeof(p));
    p.A = (const char *)X; p.W = (const char *)W; p.Ind = Ind; p.C = (char *)Y; p.w_scale = w_scale;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K;
    p.R = d->I; p.N = d->J;
    p.lda_b = ldx_b; p.lda_t = ldx_t;
    p.ind_dtype = ind_dtype;
    const bool w_trans = (w_layout == EGS_W_EIJ);       // [E,I,J]: the reduction index selects the row
    p.a_vec = aligned_to(X, 16) && (ldx_b * ES) % 16 == 0 && (ldx_t * ES) % 16 == 0;
    const int64_t w_row = w_trans ? d->J : d->I;
    p.w_vec = WES == 1 ? (aligned_to(W, 8) && w_row % 8 == 0) : (aligned_to(W, 16) && (w_row * WES) % 16 == 0);   // stricter than the 8-byte blocks of the transposed loader need
    p.c_vec = aligned_to(Y, 16) && d->J % 4 == 0;
    {
        const uint64_t span = d->B > 0 && d->T > 0
            ? ((uint64_t)(d->B - 1) * (uint64_t)ldx_b + (uint64_t)(d->T - 1) * (uint64_t)ldx_t + (uint64_t)d->I) * ES : 0;
        p.a_bytes = span < (1ull << 31) ? (uint32_t)span : 0;
    }
    return rows_gemm_gather(p, act_dtype, w_dtype == EGS_FP8_E4M3, w_trans, s);
}

// `dw` (optional): a weight gradient of the same call whose first pass may share the product
// launch and whose second pass may share the reduction launch
int gemm_scatter_impl(const void *Y, const void *W, const void *Ind, void *Out, void *workspace,
                      const egs_dims *d, int act_dtype, int ind_dtype, int w_layout, int mode, SmallDwJob *dw,
                      DwTileJob *dwt, hipStream_t s, const RoutingTable *use = nullptr)
{
    const int ES = elem_size(act_dtype);
    const size_t out_elems = (size_t)d->B * d->T * d->I;
    if (out_elems == 0) return EGS_OK;
    const ScatterPath path = scatter_choose(Y, W, Out, d, act_dtype, mode);
    const bool fused = path == SCATTER_FUSED;
    const ScatterPlan pl = plan_scatter(d, mode, act_dtype, path);
    char *ws = (char *)workspace;
    const int N = d->E * d->K;

    RowsGemmParams p;
    memset(&p, 0, sizeof(p));
    p.A = (const char *)Y; p.W = (const char *)W; p.Ind = Ind;
    p.B = d->B; p.T = d->T; p.E = d->E; p.K = d->K;
    p.R = d->J; p.N = d->I;
    p.ind_dtype = ind_dtype;
    const bool w_trans = (w_layout == EGS_W_EJI);       // [E,J,I]: the reduction index j selects the row
    p.a_vec = aligned_to(Y, 16) && ((int64_t)d->J * ES) % 16 == 0;
    const int64_t w_row = w_trans ? d->I : d->J;
    p.w_vec = aligned_to(W, 16) && (w_row * ES) % 16 == 0;
    {
        const uint64_t span = (uint64_t)d->B * d->E * d->K * d->J * ES;
        p.a_bytes = span < (1ull << 31) ? (uint32_t)span : 0;
    }

    if (mode == EGS_SCATTER_ATOMIC && act_dtype == EGS_F32) {
        float *acc32 = (float *)Out;
        hipLaunchKernelGGL(fill_zero_f32_kernel, dim3(grid_1d(out_elems / 4 + 1)), dim3(kThreads), 0, s, acc32, out_elems,
                           (int)aligned_to(acc32, 16));
        EGS_CHECK_LAUNCH("fill_zero_f32_kernel");
        p.C = (char *)acc32;
        p.c_vec = 0;
        return rows_gemm_scatter(p, act_dtype, w_trans, EPI_ATOMIC_F32, s);
    }

    if (fused) return scatter_fused(Y, W, Ind, Out, d, act_dtype, ind_dtype, w_layout, dw, dwt, s, use);   // small experts: one kernel
    // compact mode, thousands of picks per batch element: one kernel in passes, nothing in the workspace
    if (path == SCATTER_PASS) return scatter_pass(Y, W, Ind, Out, d, act_dtype, ind_dtype, w_layout, s);

    // routing table (picks in token order) + product rows in pick order, then one fixed-order
    // gather-and-sum per token that writes every output row exactly once
    int32_t *seg_off = (int32_t *)(ws + pl.seg_off_at);
    int32_t *perm = (int32_t *)(ws + pl.perm_at);
    int32_t *rank_tmp = (int32_t *)(ws + pl.rank_at);
    int32_t *cnt = d->T > kCsrLdsTokens ? (int32_t *)(ws + pl.cnt_at) : nullptr;
    int32_t *long_tab = (int32_t *)(ws + pl.long_tab_at);
    float *long_part = (float *)(ws + pl.long_part_at);
    void *rows = ws + pl.rows_at;
    bool rows_f32 = (mode != EGS_SCATTER_ATOMIC);
    // small experts: the sort rides along with the product when its histograms are small
    const bool ride = csr_count_lds(d->T, 4) <= 16 * 1024 && N <= 4096 && N > 0;
    SmallRowsJob j;
    int rc;
    if (N > 0 && make_scatter_rows_small(Y, W, rows, rows_f32, d, act_dtype, w_layout, ride, Ind, ind_dtype, seg_off, perm,
                                         rank_tmp, long_tab, j)) {
        if (!ride) {
            rc = launch_routing_table(Ind, ind_dtype, d, seg_off, perm, rank_tmp, cnt, long_tab, s);
            if (rc != EGS_OK) return rc;
        }
        rc = launch_rows_small_job(j, dw, nullptr, s);
    } else {
        rows_f32 = mode != EGS_SCATTER_ATOMIC || act_dtype == EGS_F32;   // fast mode: rows in the element type
        // Product rows that one launch writes and the next reads back are still in the 256 MB memory-side
        // cache when there are few enough of them.  A call with more is processed as groups of batch
        // elements (independent of each other; the routing tables of all of them are built with the first
        // group): the largest groups whose rows take at most 144 MB, provided the weights, which every
        // group reads again, fit beside them and the groups still fill the 256-row tiles of the product
        // kernel.  C4: 2 groups of 8, 142 -> 123 us; C3: 8 groups of 1, 600 -> 565 us.  Smaller groups than
        // necessary lose more in the product kernel than the cache returns (C4, groups of 4: 168 us).
        int G = d->B;
        {
            const uint64_t per_b = (uint64_t)N * d->I * (rows_f32 ? 4 : ES);
            const uint64_t keep = 144ull << 20;
            if (per_b > 0 && per_b * d->B > (192ull << 20) && per_b <= keep) {
                const int fit = (int)(keep / per_b);
                const int groups = ceil_div(d->B, fit);
                const int g = ceil_div(d->B, groups);
                const uint64_t w_bytes = (uint64_t)d->E * d->I * d->J * ES;
                const int64_t rows_e = (int64_t)g * d->K;                     // rows per expert and group
                const int64_t padded = (rows_e + 255) / 256 * 256;
                if (groups > 1 && rows_e >= 256 && padded * 100 <= rows_e * 115 && w_bytes <= keep / 2) G = g;
            }
        }
        p.C = (char *)rows;
        p.c_vec = d->I % 4 == 0;
        p.seg_off = seg_off; p.perm = perm; p.rank_tmp = rank_tmp; p.long_tab = long_tab;
        for (int b0 = 0; b0 < d->B; b0 += G) {
            egs_dims sub = *d;
            sub.B = d->B - b0 < G ? d->B - b0 : G;
            p.A = (const char *)Y + (size_t)b0 * N * d->J * ES;
            p.B = sub.B;
            const uint64_t span = (uint64_t)sub.B * N * d->J * ES;
            p.a_bytes = span < (1ull << 31) ? (uint32_t)span : 0;
            // the routing table may ride along with the (first) product launch (large shapes); otherwise it is a
            // launch of its own
            p.csr_blocks = (b0 == 0 && N > 0) ? d->B : 0; p.csr_done = 0;
            rc = rows_gemm_scatter(p, act_dtype, w_trans, rows_f32 ? EPI_STORE_F32 : EPI_STORE, s);
            if (rc == EGS_OK && b0 == 0 && !p.csr_done)
                rc = launch_routing_table(Ind, ind_dtype, d, seg_off, perm, rank_tmp, cnt, long_tab, s);
            if (rc != EGS_OK) return rc;
            rc = launch_segment_sum(rows, rows_f32, seg_off + (size_t)b0 * (d->T + 1), perm + (size_t)b0 * N,
                                    long_tab + (size_t)b0 * long_tab_stride(N), long_part + (size_t)b0 * long_max_slots(N) * d->I,
                                    (char *)Out + (size_t)b0 * d->T * d->I * ES, &sub, act_dtype,
                                    b0 + G >= d->B ? dw : nullptr, s);
            if (rc != EGS_OK) return rc;
        }
        return EGS_OK;
    }
    if (rc != EGS_OK) return rc;
    return launch_segment_sum(rows, rows_f32, seg_off, perm, long_tab, long_part, Out, d, act_dtype, dw, s);
}

int dw_impl(const void *Xs, const void *Ys, const void *Ind, void *dW, void *workspace, const egs_dims *d,
            int64_t ldx_b, int64_t ldx_t, int act_dtype, int out_dtype, int ind_dtype, int dw_layout, hipStream_t s)
{
    if ((size_t)d->E * d->I * d->J == 0) return EGS_OK;
    DwPlan pl = plan_dw(d, act_dtype);
    switch (dw_choose(Xs, Ys, dW, d, ldx_b, ldx_t, act_dtype, pl).path) {
    case DW_TILE: {
        DwTileJob jt;
        make_dw_tile(Xs, Ys, Ind, dW, d, ldx_b, ldx_t, act_dtype, out_dtype, ind_dtype, dw_layout, jt, dw_tile_wide_alone(d, act_dtype));
        return launch_dw_tile_alone(jt, s);
    }
    case DW_SMALL: {
        SmallDwJob j;
        make_dw_small(Xs, Ys, Ind, dW, workspace, d, ldx_b, ldx_t, act_dtype, out_dtype, ind_dtype, dw_layout, pl, j);
        const int rc = launch_dw_small_alone(j, s);
        return rc != EGS_OK ? rc : launch_dw_reduce4(j, s);
    }
    default:
        return dw_general(Xs, Ys, Ind, dW, workspace, d, ldx_b, ldx_t, act_dtype, out_dtype, ind_dtype, dw_layout, pl, s);
    }
}

// ------------------------------------------------------------------------------ validation
int validate_gather(const void *X, const void *W, const void *Ind, const void *Y, const float *w_scale,
                    const egs_dims *d, int64_t ldx_b, int64_t ldx_t, int act_dtype, int w_dtype, int ind_dtype,
                    int w_layout)
{
    int rc = check_dims(d);
    if (rc != EGS_OK) return rc;
    if (!act_dtype_ok(act_dtype) || !ind_dtype_ok(ind_dtype)) return EGS_ERR_BAD_DTYPE;
    if (w_dtype == EGS_FP8_E4M3) {
        if (act_dtype != EGS_BF16) return EGS_ERR_UNSUPPORTED;    // fp8 weights pair with bf16 activations
        if (w_scale == nullptr) return EGS_ERR_NULL_POINTER;
    } else if (w_dtype != act_dtype) {
        return act_dtype_ok(w_dtype) ? EGS_ERR_UNSUPPORTED : EGS_ERR_BAD_DTYPE;
    }
    if (!layout_ok(w_layout)) return EGS_ERR_BAD_LAYOUT;
    const size_t y_elems = (size_t)d->B * d->E * d->K * d->J;
    if (y_elems == 0) return EGS_OK;
    if (Y == nullptr || Ind == nullptr) return EGS_ERR_NULL_POINTER;
    if (d->I > 0 && (X == nullptr || W == nullptr)) return EGS_ERR_NULL_POINTER;
    if (d->I > 0 && d->T == 0) return EGS_OK;                      // every pick is out of range
    if (ldx_t < d->I || (d->B > 1 && ldx_b < 0)) return EGS_ERR_BAD_STRIDE;
    const int ES = elem_size(act_dtype);
    if (!aligned_to(X, ES) || !aligned_to(Y, ES) || !aligned_to(W, elem_size(w_dtype))) return EGS_ERR_ALIGNMENT;
    return EGS_OK;
}

int validate_scatter(const void *Y, const void *W, const void *Ind, const void *Out, const void *workspace,
                     size_t workspace_bytes, const egs_dims *d, int act_dtype, int ind_dtype, int w_layout, int mode)
{
    int rc = check_dims(d);
    if (rc != EGS_OK) return rc;
    if (!act_dtype_ok(act_dtype) || !ind_dtype_ok(ind_dtype)) return EGS_ERR_BAD_DTYPE;
    if (!layout_ok(w_layout)) return EGS_ERR_BAD_LAYOUT;
    if (!mode_ok(mode)) return EGS_ERR_BAD_MODE;
    const size_t out_elems = (size_t)d->B * d->T * d->I;
    if (out_elems == 0) return EGS_OK;
    if (Out == nullptr) return EGS_ERR_NULL_POINTER;
    const size_t picks = (size_t)d->B * d->E * d->K;
    if (picks > 0 && Ind == nullptr) return EGS_ERR_NULL_POINTER;
    if (picks > 0 && d->J > 0 && (Y == nullptr || W == nullptr)) return EGS_ERR_NULL_POINTER;
    const size_t need = plan_scatter(d, mode, act_dtype, scatter_choose(Y, W, Out, d, act_dtype, mode)).bytes;
    if (need > 0 && (workspace == nullptr || workspace_bytes < need)) return EGS_ERR_WORKSPACE;
    if (need > 0 && !aligned_to(workspace, 256)) return EGS_ERR_ALIGNMENT;
    const int ES = elem_size(act_dtype);
    if (!aligned_to(Y, ES) || !aligned_to(Out, ES) || !aligned_to(W, ES)) return EGS_ERR_ALIGNMENT;
    return EGS_OK;
}

int validate_dw(const void *Xs, const void *Ys, const void *Ind, const void *dW, const void *workspace,
                size_t workspace_bytes, const egs_dims *d, int64_t ldx_b, int64_t ldx_t, int act_dtype,
                int out_dtype, int ind_dtype, int dw_layout)
{
    int rc = check_dims(d);
    if (rc != EGS_OK) return rc;
    if (!act_dtype_ok(act_dtype) || !act_dtype_ok(out_dtype) || !ind_dtype_ok(ind_dtype)) return EGS_ERR_BAD_DTYPE;
    if (!layout_ok(dw_layout)) return EGS_ERR_BAD_LAYOUT;
    const size_t w_elems = (size_t)d->E * d->I * d->J;
    if (w_elems == 0) return EGS_OK;
    if (dW == nullptr) return EGS_ERR_NULL_POINTER;
    const size_t picks = (size_t)d->B * d->K;
    if (picks > 0 && (Xs == nullptr || Ys == nullptr || Ind == nullptr)) return EGS_ERR_NULL_POINTER;
    if (picks > 0 && d->T > 0 && (ldx_t < d->I || (d->B > 1 && ldx_b < 0))) return EGS_ERR_BAD_STRIDE;
    const size_t need = picks > 0 ? dw_choose(Xs, Ys, const_cast<void *>(dW), d, ldx_b, ldx_t, act_dtype, plan_dw(d, act_dtype)).bytes : 0;
    if (need > 0 && (workspace == nullptr || workspace_bytes < need)) return EGS_ERR_WORKSPACE;
    if (need > 0 && !aligned_to(workspace, 256)) return EGS_ERR_ALIGNMENT;
    const int ES = elem_size(act_dtype);
    if (!aligned_to(Xs, ES) || !aligned_to(Ys, ES) || !aligned_to(dW, elem_size(out_dtype))) return EGS_ERR_ALIGNMENT;
    return EGS_OK;
}

}  // namespace

// ================================================================================ C ABI
extern "C" {

int egs_abi_version(void) { return EGS_ABI_VERSION; }

const char *egs_status_string(int status)
{
    switch (status) {
    case EGS_OK: return "ok";
    case EGS_ERR_NULL_POINTER: return "null pointer argument";
    case EGS_ERR_BAD_SHAPE: return "negative or too large dimension";
    case EGS_ERR_BAD_DTYPE: return "Unknown dtype";
    case EGS_ERR_BAD_LAYOUT: return "unknown weight layout";
    case EGS_ERR_BAD_MODE: return "unknown scatter mode";
    case EGS_ERR_WORKSPACE: return "workspace missing or too small";
    case EGS_ERR_ALIGNMENT: return "pointer not aligned to its element size (workspace: 256 bytes)";
    case EGS_ERR_HIP: return "HIP runtime error";
    case EGS_ERR_UNSUPPORTED: return "unsupported dtype combination";
    case EGS_ERR_BAD_STRIDE: return "source stride smaller than its row";
    case EGS_ERR_SCRATCH_LIMIT: return "sizes need more scratch than the built-in buffer holds (EGS_BUILTIN_SCRATCH_BYTES)";
    default: return "unknown status";
    }
}

const char *egs_last_hip_error(void) { return last_hip_error(); }

void egs_testing_force_generic(int on) { g_force_generic.store(on != 0); }

void egs_testing_launch_log_begin(void)
{
    g_launch_log.on = true; g_launch_log.len = 0; g_launch_log.text[0] = 0;
}

size_t egs_testing_launch_log_end(char *buf, size_t n)
{
    const size_t len = g_launch_log.len;
    if (buf != nullptr && n > 0) {
        const size_t c = len < n - 1 ? len : n - 1;
        memcpy(buf, g_launch_log.text, c);
        buf[c] = 0;
    }
    g_launch_log.on = false; g_launch_log.len = 0; g_launch_log.text[0] = 0;
    return len;
}

size_t egs_workspace_bytes(int op, int mode, const egs_dims *d, int act_dtype)
{
    if (check_dims(d) != EGS_OK || !act_dtype_ok(act_dtype)) return 0;
    if (!mode_ok(mode)) mode = EGS_SCATTER_DETERMINISTIC;
    switch (op) {
    case EGS_OP_GATHER_GEMM: return 0;
    case EGS_OP_GEMM_SCATTER: return scatter_bytes_planned(d, mode, act_dtype);
    case EGS_OP_DW: return dw_bytes_planned(d, act_dtype);
    case EGS_OP_GATHER_BACKWARD: return scatter_bytes_planned(d, mode, act_dtype) + dw_bytes_planned(d, act_dtype);
    case EGS_OP_SCATTER_BACKWARD: return dw_bytes_planned(d, act_dtype);
    default: return 0;
    }
}

int egs_gather_gemm(const void *X, const void *W, const void *Ind, void *Y, const float *w_scale,
                    const egs_dims *d, int64_t ldx_b, int64_t ldx_t,
                    int act_dtype, int w_dtype, int ind_dtype, int w_layout, void *stream)
{
    int rc = validate_gather(X, W, Ind, Y, w_scale, d, ldx_b, ldx_t, act_dtype, w_dtype, ind_dtype, w_layout);
    if (rc != EGS_OK) return rc;
    if ((size_t)d->B * d->E * d->K * d->J == 0) return EGS_OK;
    return gather_gemm_impl(X, W, Ind, Y, w_scale, d, ldx_b, ldx_t, act_dtype, w_dtype, ind_dtype, w_layout,
                            (hipStream_t)stream);
}

int egs_gemm_scatter(const void *Y, const void *W, const void *Ind, void *Out,
                     void *workspace, size_t workspace_bytes, const egs_dims *d,
                     int act_dtype, int ind_dtype, int w_layout, int mode, void *stream)
{
    int rc = validate_scatter(Y, W, Ind, Out, workspace, workspace_bytes, d, act_dtype, ind_dtype, w_layout, mode);
    if (rc != EGS_OK) return rc;
    return gemm_scatter_impl(Y, W, Ind, Out, workspace, d, act_dtype, ind_dtype, w_layout, mode, nullptr, nullptr,
                             (hipStream_t)stream);
}

int egs_dw(const void *Xsrc, const void *Ysrc, const void *Ind, void *dW,
           void *workspace, size_t workspace_bytes, const egs_dims *d,
           int64_t ldx_b, int64_t ldx_t,
           int act_dtype, int out_dtype, int ind_dtype, int dw_layout, void *stream)
{
    int rc = validate_dw(Xsrc, Ysrc, Ind, dW, workspace, workspace_bytes, d, ldx_b, ldx_t, act_dtype, out_dtype,
                         ind_dtype, dw_layout);
    if (rc != EGS_OK) return rc;
    return dw_impl(Xsrc, Ysrc, Ind, dW, workspace, d, ldx_b, ldx_t, act_dtype, out_dtype, ind_dtype, dw_layout,
                   (hipStream_t)stream);
}

int egs_dw_builtin_scratch(const void *Xsrc, const void *Ysrc, const void *Ind, void *dW, const egs_dims *d,
                           int64_t ldx_b, int64_t ldx_t,
                           int act_dtype, int out_dtype, int ind_dtype, int dw_layout, void *stream)
{
    int rc = check_dims(d);
    if (rc != EGS_OK) return rc;
    if (!act_dtype_ok(act_dtype)) return EGS_ERR_BAD_DTYPE;
    if (!layout_ok(dw_layout)) return EGS_ERR_BAD_LAYOUT;
    const size_t need = dw_choose(Xsrc, Ysrc, dW, d, ldx_b, ldx_t, act_dtype, plan_dw(d, act_dtype)).bytes;
    if (need > (size_t)EGS_BUILTIN_SCRATCH_BYTES) return EGS_ERR_SCRATCH_LIMIT;
    // the remaining checks are those of egs_dw; the stand-in address only has to look like a valid workspace
    rc = validate_dw(Xsrc, Ysrc, Ind, dW, need > 0 ? (const void *)(uintptr_t)256 : nullptr, need, d, ldx_b, ldx_t, act_dtype,
                     out_dtype, ind_dtype, dw_layout);
    if (rc != EGS_OK) return rc;
    if ((size_t)d->E * d->I * d->J == 0) return EGS_OK;
    void *ws = nullptr;
    if (need > 0) {
        rc = builtin_scratch_ptr(&ws);
        if (rc != EGS_OK) return rc;
    }
    // the partial sums of every split are written before the second pass reads them: nothing in the
    // buffer has to start at zero
    return dw_impl(Xsrc, Ysrc, Ind, dW, ws, d, ldx_b, ldx_t, act_dtype, out_dtype, ind_dtype, dw_layout,
                   (hipStream_t)stream);
}

int egs_expert_gather_forward(const void *X, const void *W, const void *Ind, void *Y,
                              const egs_dims *d, int64_t ldx_b, int64_t ldx_t,
                              int dtype, int ind_dtype, void *stream)
{
    return egs_gather_gemm(X, W, Ind, Y, nullptr, d, ldx_b, ldx_t, dtype, dtype, ind_dtype, EGS_W_EIJ, stream);
}

static int gather_backward_impl(const void *X, const void *W, const void *Ind, const void *grad_Y,
                                void *grad_X, void *grad_W,
                                void *workspace, size_t workspace_bytes, const egs_dims *d,
                                int64_t ldx_b, int64_t ldx_t,
                                int dtype, int ind_dtype, int mode, void *stream, void *table, size_t table_bytes)
{
    int rc = check_dims(d);
    if (rc != EGS_OK) return rc;
    if (!act_dtype_ok(dtype)) return EGS_ERR_BAD_DTYPE;
    if (!mode_ok(mode)) return EGS_ERR_BAD_MODE;
    if (grad_X == nullptr && (size_t)d->B * d->T * d->I > 0) return EGS_ERR_NULL_POINTER;
    RoutingTable tab;
    bool have_tab = false;
    rc = check_table_arg(table, table_bytes, d, dtype, tab, have_tab);
    if (rc != EGS_OK) return rc;
    const size_t ws_scatter = plan_scatter(d, mode, dtype, scatter_choose(grad_Y, W, grad_X, d, dtype, mode)).bytes;
    const size_t ws_dw = (size_t)d->B * d->K > 0 && (size_t)d->E * d->I * d->J > 0 && grad_W != nullptr
        ? dw_choose(X, grad_Y, grad_W, d, ldx_b, ldx_t, dtype, plan_dw(d, dtype)).bytes : 0;
    if (ws_scatter + ws_dw > 0 && (workspace == nullptr || workspace_bytes < ws_scatter + ws_dw)) return EGS_ERR_WORKSPACE;
    // validate both halves before enqueuing anything
    rc = validate_scatter(grad_Y, W, Ind, grad_X, workspace, ws_scatter, d, dtype, ind_dtype, EGS_W_EIJ, mode);
    if (rc != EGS_OK) return rc;
    void *ws2 = workspace ? (char *)workspace + ws_scatter : nullptr;
    rc = validate_dw(X, grad_Y, Ind, grad_W, ws2, ws_dw, d, ldx_b, ldx_t, dtype, dtype, ind_dtype, EGS_W_EIJ);
    if (rc != EGS_OK) return rc;
    // grad_X[b,t,i] = sum_picks sum_j grad_Y[b,e,k,j] * W[e,i,j];  grad_W[e,i,j] = sum X[b,Ind,i] * grad_Y[b,e,k,j].
    // The two are independent: for small experts the weight gradient shares the scatter's launches.
    hipStream_t s = (hipStream_t)stream;
    const size_t w_elems = (size_t)d->E * d->I * d->J;
    const DwPlan dpl = plan_dw(d, dtype);
    SmallDwJob dwj;
    DwTileJob dwt;
    // 32 x 32 tiles when they can share the launch of the one-kernel scatter (one pass) and come after it in one round of
    // workgroups, else what suits a launch of its own (I = 256: 42.9 us sharing, 37 us as two launches with 32 x 64 tiles)
    const FusedPlan fpl = scatter_fused_plan(grad_Y, W, grad_X, d, dtype);
    const bool shares_launch = dtype != EGS_F32 && fpl.ok && fpl.experts_per_pass == d->E &&
                               (int64_t)d->E * ceil_div(d->I, 32) * ceil_div(d->J, 32) <= 256;
    const bool dw_tile = w_elems > 0 && make_dw_tile(X, grad_Y, Ind, grad_W, d, ldx_b, ldx_t, dtype, dtype, ind_dtype, EGS_W_EIJ, dwt,
                                                     !shares_launch && dw_tile_wide_alone(d, dtype));
    const bool dw_small = !dw_tile && w_elems > 0 && make_dw_small(X, grad_Y, Ind, grad_W, ws2, d, ldx_b, ldx_t, dtype, dtype,
                                                                   ind_dtype, EGS_W_EIJ, dpl, dwj);
    rc = gemm_scatter_impl(grad_Y, W, Ind, grad_X, workspace, d, dtype, ind_dtype, EGS_W_EIJ, mode, dw_small ? &dwj : nullptr,
                           dw_tile ? &dwt : nullptr, s, have_tab ? &tab : nullptr);
    if (rc != EGS_OK) return rc;
    if (w_elems == 0) return EGS_OK;
    if (dw_tile) return dwt.done ? EGS_OK : launch_dw_tile_alone(dwt, s);
    if (dw_small) {
        if (!dwj.done) { rc = launch_dw_small_alone(dwj, s); if (rc != EGS_OK) return rc; }
        return launch_dw_reduce4(dwj, s);       // no-op when the reduction launch already did it
    }
    return dw_general(X, grad_Y, Ind, grad_W, ws2, d, ldx_b, ldx_t, dtype, dtype, ind_dtype, EGS_W_EIJ, dpl, s);
}

int egs_expert_gather_backward(const void *X, const void *W, const void *Ind, const void *grad_Y,
                               void *grad_X, void *grad_W,
                               void *workspace, size_t workspace_bytes, const egs_dims *d,
                               int64_t ldx_b, int64_t ldx_t,
                               int dtype, int ind_dtype, int mode, void *stream)
{
    return gather_backward_impl(X, W, Ind, grad_Y, grad_X, grad_W, workspace, workspace_bytes, d, ldx_b, ldx_t, dtype, ind_dtype,
                                mode, stream, nullptr, 0);
}

int egs_expert_gather_backward_table(const void *X, const void *W, const void *Ind, const void *table, size_t table_bytes,
                                     const void *grad_Y, void *grad_X, void *grad_W,
                                     void *workspace, size_t workspace_bytes, const egs_dims *d,
                                     int64_t ldx_b, int64_t ldx_t,
                                     int dtype, int ind_dtype, int mode, void *stream)
{
    return gather_backward_impl(X, W, Ind, grad_Y, grad_X, grad_W, workspace, workspace_bytes, d, ldx_b, ldx_t, dtype, ind_dtype,
                                mode, stream, const_cast<void *>(table), table_bytes);
}

int egs_expert_scatter_forward(const void *Y, const void *W, const void *Ind, void *Out,
                               void *workspace, size_t workspace_bytes, const egs_dims *d,
                               int dtype, int ind_dtype, int mode, void *stream)
{
    return egs_gemm_scatter(Y, W, Ind, Out, workspace, workspace_bytes, d, dtype, ind_dtype, EGS_W_EJI, mode, stream);
}

int egs_expert_scatter_forward_table(const void *Y, const void *W, const void *Ind, const void *table, size_t table_bytes,
                                     void *Out, void *workspace, size_t workspace_bytes, const egs_dims *d,
                                     int dtype, int ind_dtype, int mode, void *stream)
{
    int rc = validate_scatter(Y, W, Ind, Out, workspace, workspace_bytes, d, dtype, ind_dtype, EGS_W_EJI, mode);
    if (rc != EGS_OK) return rc;
    RoutingTable tab;
    bool have_tab = false;
    rc = check_table_arg(const_cast<void *>(table), table_bytes, d, dtype, tab, have_tab);
    if (rc != EGS_OK) return rc;
    return gemm_scatter_impl(Y, W, Ind, Out, workspace, d, dtype, ind_dtype, EGS_W_EJI, mode, nullptr, nullptr,
                             (hipStream_t)stream, have_tab ? &tab : nullptr);
}

size_t egs_routing_table_bytes(const egs_dims *d, int dtype)
{
    if (check_dims(d) != EGS_OK) return 0;
    const TableLayout l = routing_table_layout(d, dtype);
    return l.ok ? l.bytes : 0;
}

int egs_expert_gather_forward_table(const void *X, const void *W, const void *Ind, void *Y, void *table, size_t table_bytes,
                                    const egs_dims *d, int64_t ldx_b, int64_t ldx_t,
                                    int dtype, int ind_dtype, void *stream)
{
    int rc = validate_gather(X, W, Ind, Y, nullptr, d, ldx_b, ldx_t, dtype, dtype, ind_dtype, EGS_W_EIJ);
    if (rc != EGS_OK) return rc;
    RoutingTable tab;
    bool have_tab = false;
    rc = check_table_arg(table, table_bytes, d, dtype, tab, have_tab);
    if (rc != EGS_OK) return rc;
    if ((size_t)d->B * d->E * d->K * d->J == 0) return EGS_OK;
    return gather_gemm_impl(X, W, Ind, Y, nullptr, d, ldx_b, ldx_t, dtype, dtype, ind_dtype, EGS_W_EIJ, (hipStream_t)stream,
                            have_tab ? &tab : nullptr);
}

int egs_expert_scatter_backward(const void *Y, const void *W, const void *Ind, const void *grad_Out,
                                void *grad_Y, void *grad_W,
                                void *workspace, size_t workspace_bytes, const egs_dims *d,
                                int64_t ldg_b, int64_t ldg_t,
                                int dtype, int ind_dtype, void *stream)
{
    int rc = validate_gather(grad_Out, W, Ind, grad_Y, nullptr, d, ldg_b, ldg_t, dtype, dtype, ind_dtype, EGS_W_EJI);
    if (rc != EGS_OK) return rc;
    rc = validate_dw(grad_Out, Y, Ind, grad_W, workspace, workspace_bytes, d, ldg_b, ldg_t, dtype, dtype, ind_dtype,
                     EGS_W_EJI);
    if (rc != EGS_OK) return rc;
    // grad_Y[b,e,k,j] = sum_i grad_Out[b,Ind,i] * W[e,j,i];  grad_W[e,j,i] = sum grad_Out[b,Ind,i] * Y[b,e,k,j].
    // Independent of each other: for small experts they share one launch.
    hipStream_t s = (hipStream_t)stream;
    const size_t y_elems = (size_t)d->B * d->E * d->K * d->J, w_elems = (size_t)d->E * d->I * d->J;
    const DwPlan dpl = plan_dw(d, dtype);
    SmallRowsJob gj;
    SmallDwJob dwj;
    const bool g_small = y_elems > 0 && make_gather_small(grad_Out, W, Ind, grad_Y, d, ldg_b, ldg_t, dtype, dtype, ind_dtype,
                                                          EGS_W_EJI, gj);
    DwTileJob dwt;
    if (g_small && w_elems > 0 &&
        make_dw_tile(grad_Out, Y, Ind, grad_W, d, ldg_b, ldg_t, dtype, dtype, ind_dtype, EGS_W_EJI, dwt, /*wide=*/true)) {
        // One launch: the gather regridded to 8 wavefronts per workgroup, the weight-gradient workgroups first in launch
        // order (they run longest).  The launch's LDS size admits one workgroup per CU, so the two bodies never share a
        // CU (sharing one costs the sum of their times); with more workgroups than CUs the gather's fill the CUs the
        // weight gradient leaves and then follow on each CU as it frees (B64 T256 E48 K32 I128 J64: 26.5 -> 21.1 us
        // against two launches, B128 E32: 30.9 -> 21.3 us).
        SmallRowsJob g8 = gj;
        const int64_t Me = (int64_t)d->B * d->K;
        g8.p.tiles_per_e = (int)((Me + 511) / 512);
        // (row tiles on the XCDs in groups of eight only: with four row tiles on two XCDs each this launch measured
        // 11.4 against 11.05 us at B64 T256 E32 K32 I128 J64 - its other half reads the same rows expert by expert)
        g8.p.rows_share_xcd = g8.p.tiles_per_e % 8 == 0 ? rows_xcd_map(d, d->I, d->J, 2, g8.p.tiles_per_e) : 0;
        g8.blocks = rows_xcd_blocks(g8.p.rows_share_xcd, g8.p.tiles_per_e, g8.p.E);
        if ((int64_t)g8.blocks + dwt.blocks <= INT32_MAX / 2) return launch_rows_small_job(g8, nullptr, &dwt, s);
    }
    const bool dw_tile = w_elems > 0 && make_dw_tile(grad_Out, Y, Ind, grad_W, d, ldg_b, ldg_t, dtype, dtype, ind_dtype, EGS_W_EJI, dwt,
                                                     dw_tile_wide_alone(d, dtype));
    if (dw_tile) {
        if (y_elems > 0) {
            rc = gather_gemm_impl(grad_Out, W, Ind, grad_Y, nullptr, d, ldg_b, ldg_t, dtype, dtype, ind_dtype, EGS_W_EJI, s);
            if (rc != EGS_OK) return rc;
        }
        return launch_dw_tile_alone(dwt, s);
    }
    const bool dw_small = !dw_tile && w_elems > 0 && make_dw_small(grad_Out, Y, Ind, grad_W, workspace, d, ldg_b, ldg_t, dtype,
                                                                   dtype, ind_dtype, EGS_W_EJI, dpl, dwj);
    if (g_small && dw_small) {
        rc = launch_rows_small_job(gj, &dwj, nullptr, s);
        if (rc != EGS_OK) return rc;
        return launch_dw_reduce4(dwj, s);
    }
    if (y_elems > 0) {
        rc = gather_gemm_impl(grad_Out, W, Ind, grad_Y, nullptr, d, ldg_b, ldg_t, dtype, dtype, ind_dtype, EGS_W_EJI, s);
        if (rc != EGS_OK) return rc;
    }
    return dw_impl(grad_Out, Y, Ind, grad_W, workspace, d, ldg_b, ldg_t, dtype, dtype, ind_dtype, EGS_W_EJI, s);
}

int egs_stream_capture_id(void *stream, unsigned long long *id)
{
    if (id == nullptr) return EGS_ERR_NULL_POINTER;
    *id = 0;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long cid = 0;
    const hipError_t err = hipStreamGetCaptureInfo((hipStream_t)stream, &status, &cid);
    if (err != hipSuccess) return hip_fail(err, "hipStreamGetCaptureInfo");
    if (status == hipStreamCaptureStatusActive) *id = cid;
    return EGS_OK;
}

int egs_validate_indices(const void *Ind, int ind_dtype, int64_t n, int32_t T, int32_t *d_bad_count, void *stream)
{
    if (n < 0) return EGS_ERR_BAD_SHAPE;
    if (!ind_dtype_ok(ind_dtype)) return EGS_ERR_BAD_DTYPE;
    if (n == 0) return EGS_OK;
    if (Ind == nullptr || d_bad_count == nullptr) return EGS_ERR_NULL_POINTER;
    hipLaunchKernelGGL(validate_indices_kernel, dim3(grid_1d((size_t)n, 1024)), dim3(kThreads), 0, (hipStream_t)stream,
                       Ind, ind_dtype, n, T, d_bad_count);
    EGS_CHECK_LAUNCH("validate_indices_kernel");
    return EGS_OK;
}

}  // extern "C"
