// Weight gradient of small experts in ONE pass, no split of the picks and therefore no partial sums
// and no second launch:
//
//   dW(e, i, j) = sum over all picks m = (b, k) of expert e of  Xs[b, Ind[b,e,k], i] * Ys[b, e, k, j]
//
// A workgroup owns a 32 x TJ tile of dW(e) (TJ = 32 or 64) and reduces ALL of the expert's picks; with
// E * (I/32) * (J/TJ) workgroups (256 or 128 at the reference's default shape E32 I128 J64) the device is busy
// without splitting the reduction.  Its wavefronts take contiguous parts of the picks, each accumulating the
// whole tile, and are summed through LDS in wavefront order (fixed order -> bitwise reproducible, no atomics).
// What bounds the kernel is the rate at which a CU can send requests to its L2 (about one per 2.4 cycles,
// whatever their size up to a 128-byte line): 64 columns on the Ys side make that side's requests full lines.
//
// Both operands are "reduction-strided" in memory (a pick selects a row, the output index runs along it),
// the opposite of what the matrix instruction wants (per lane: 8 consecutive picks of one column).  Per
// 32-pick step a wavefront fetches the 64-byte pieces of 32 gathered Xs rows and the 64- or 128-byte pieces of
// 32 Ys rows with 16-byte buffer loads (adjacent lanes take adjacent chunks of a pick's piece: one access per
// row), one step ahead of the step it multiplies, drops each step into a wavefront-private LDS tile
// as [pick][column] and reads the fragments back with the LDS transpose read.  No barrier in the main loop.  Row byte
// offsets come from a table in LDS that the wavefront decodes from Ind one chunk (128 or 256 picks) ahead; picks that do not exist (bad index, ragged end) get an offset outside the buffer
// descriptor and arrive as zeros on both sides.
//
// Replaces the reference's expert_gather_scatter_dW_kernel (egs/triton_kernels.py:261-356), which reduces
// over the batch only and adds the K partial tiles with atomics in the output type.
#pragma once
#include <type_traits>
#include "egs_device.h"

namespace egs {

struct DwTileParams {
    const char *Xs;         // [B,T,I] rows, strides (ldx_b, ldx_t, 1) in elements; x_bytes < 2 GiB
    const char *Ys;         // [B,E,K,J] dense; y_bytes < 2 GiB
    const void *Ind;
    char *dW;               // [E,I,J] or [E,J,I] in out_dtype
    int32_t B, T, E, K, I, J;       // I % 8 == 0, J % 8 == 0
    int64_t ldx_b, ldx_t;
    int32_t ind_dtype;
    int32_t i_tiles, j_tiles;       // 32-column tiles of I and of J
    int32_t out_dtype, dw_layout;
    uint32_t x_bytes, y_bytes;
};

// `ES` = bytes per element (2, or 4 for fp32, whose pieces are twice as long and whose fragments are read untransposed)
// picks whose row offsets a wavefront decodes at a time (a chunk; its steps have registers of their own: 16 or 24 per 32-pick step; 32 or 48 in fp32)
__host__ __device__ constexpr int dw_tile_chunk(int TJ, int ES = 2) { return (TJ == 32 ? 256 : 128) / (ES / 2); }
// byte strides of a pick's piece inside a staging tile.  16-bit: dense (the transpose reads are XOR-swizzled instead).
// fp32: 48 or 80 floats, so that the four picks a 4-byte fragment read touches (16 lanes each) fall on different banks
__host__ __device__ constexpr int dw_tile_xstride(int ES) { return ES == 2 ? 64 : 192; }
__host__ __device__ constexpr int dw_tile_ystride(int TJ, int ES) { return ES == 2 ? TJ * 2 : (TJ == 32 ? 192 : 320); }
// per wavefront: row-offset tables of two chunks (Xs and Ys side) + two staging tiles (32 picks of each side)
__host__ __device__ constexpr int dw_tile_lds_per_wave(int TJ, int ES = 2)
{
    return 2 * 2 * dw_tile_chunk(TJ, ES) * 4 + 2 * 32 * (dw_tile_xstride(ES) + dw_tile_ystride(TJ, ES));
}
__host__ __device__ constexpr size_t dw_tile_lds(int waves, int TJ = 32, int ES = 2) { return (size_t)waves * dw_tile_lds_per_wave(TJ, ES); }

__device__ __forceinline__ u32x4 buffer_load16(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff)
{
    return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff, 0, 0));
}

// Requirements (checked by the launcher): 2-byte elements, I % 8 == 0, J % 8 == 0, rows of Xs and Ys 16-byte
// aligned, both tensors below 2 GiB, dW 16-byte aligned, T >= 1; j_tiles counts TJ-column tiles.
// `smem`: dw_tile_lds(NW, TJ) bytes, 16-byte aligned.
template <class TT, int NW, int TJ = 32>
__device__ __forceinline__ void dw_tile_body(const DwTileParams &p, const int block, char *smem)
{
    static_assert(TJ == 32 || TJ == 64, "Ys-side tile width");
    constexpr int ES = TT::ES;
    constexpr int CH = dw_tile_chunk(TJ, ES), NS = CH / 32;
    constexpr int kLdsPerWave = dw_tile_lds_per_wave(TJ, ES);
    constexpr int XB = 32 * ES;                 // bytes of an Xs piece (32 columns)
    constexpr int XL = XB / 16;                 // lanes per Xs piece (4; fp32: 8)
    constexpr int XN = 32 * XL / 64;            // Xs loads per step (2; fp32: 4), 64 / XL picks each
    constexpr int YB = TJ * ES;                 // bytes of a Ys piece
    constexpr int YL = YB / 16;                 // lanes per Ys piece (4 or 8; fp32: 8 or 16)
    constexpr int YN = 32 * YL / 64;            // Ys loads per step (2 or 4; fp32: 4 or 8), 64 / YL picks each
    constexpr int XS = dw_tile_xstride(ES), YS = dw_tile_ystride(TJ, ES);
    constexpr int XT = 32 * XS;                 // bytes of the Xs half of a staging tile
    constexpr int STG = XT + 32 * YS;           // bytes of a staging tile
    constexpr int NY = TJ / 16;                 // 16-column groups on the Ys side
    int e, tile;
    const int tiles_per_e = p.i_tiles * p.j_tiles;
    if (!decode_expert_tile(block, tiles_per_e, p.E, e, tile)) return;
    const int it = tile / p.j_tiles, jt = tile - it * p.j_tiles;
    const int i0 = it * 32, j0 = jt * TJ;
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int a = lane & 15, g = lane >> 4;
    const int Me = p.B * p.K;
    const int per_wave = ((Me + NW - 1) / NW + 31) & ~31;
    const int w_begin = min(Me, wave * per_wave), w_end = min(Me, w_begin + per_wave);
    const int nchunks = (w_end - w_begin + CH - 1) / CH;

    char *mine = smem + wave * kLdsPerWave;
    uint32_t *tab = reinterpret_cast<uint32_t *>(mine);         // [2][x: CH | y: CH]
    char *stage = mine + 2 * 2 * CH * 4;                        // [2][Xs piece 2 KB | Ys piece 32 * YB]

    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(p.Xs), 0, (int)p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_y = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(p.Ys), 0, (int)p.y_bytes, 0x00020000);

    // this lane's share of a step: Xs picks (lane / XL) + (64 / XL) * h, 16-byte chunk lane % XL of the tile's
    // columns; Ys picks (lane / YL) + (64 / YL) * h, chunk lane % YL
    const int xc = i0 + (lane % XL) * (16 / ES), yc = j0 + (lane % YL) * (16 / ES);
    const uint32_t xcol = xc < p.I ? (uint32_t)xc * (uint32_t)ES : kVoffInvalid;
    const uint32_t ycol = yc < p.J ? (uint32_t)yc * (uint32_t)ES : kVoffInvalid;

    uint64_t iw[CH / 64];
    auto pick_of = [&](int c, int u, int &m, int &b) -> int64_t {
        m = w_begin + c * CH + u * 64 + lane;
        const int mm = min(m, Me - 1);
        b = mm / p.K;
        return ((int64_t)b * p.E + e) * p.K + (mm - b * p.K);
    };
    auto load_idx = [&](int c) {
#pragma unroll
        for (int u = 0; u < CH / 64; ++u) {
            int m, b;
            const int64_t pick = pick_of(c, u, m, b);
            iw[u] = load_index_word(p.Ind, p.ind_dtype, pick);
        }
    };
    auto store_tab = [&](int c) {
        uint32_t *t = tab + (c & 1) * 2 * CH;
#pragma unroll
        for (int u = 0; u < CH / 64; ++u) {
            int m, b;
            const int64_t pick = pick_of(c, u, m, b);
            const int64_t raw = decode_index_word(iw[u], p.Ind, p.ind_dtype, pick);
            const bool live = m < w_end && raw >= 0 && raw < (int64_t)p.T;
            t[u * 64 + lane] = live ? (uint32_t)(((int64_t)b * p.ldx_b + raw * p.ldx_t) * ES) : kVoffInvalid;
            t[CH + u * 64 + lane] = live ? (uint32_t)(pick * p.J * ES) : kVoffInvalid;
        }
    };

    u32x4 rx[NS][XN], ry[NS][YN];
    auto issue = [&](int c, int s) {
        const uint32_t *t = tab + (c & 1) * 2 * CH;
#pragma unroll
        for (int h = 0; h < XN; ++h) {
            const uint32_t xo = t[s * 32 + h * (64 / XL) + lane / XL];
            rx[s][h] = buffer_load16(rs_x, (xo == kVoffInvalid || xcol == kVoffInvalid) ? kVoffInvalid : xo + xcol);
        }
#pragma unroll
        for (int h = 0; h < YN; ++h) {
            const uint32_t yo = t[CH + s * 32 + h * (64 / YL) + lane / YL];
            ry[s][h] = buffer_load16(rs_y, (yo == kVoffInvalid || ycol == kVoffInvalid) ? kVoffInvalid : yo + ycol);
        }
    };

    f32x4 acc[2][NY];
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int y = 0; y < NY; ++y) acc[x][y] = f32x4{0.f, 0.f, 0.f, 0.f};

    // 16-bit fragment addresses inside a piece ([32 picks][64 or YB bytes]): the lane points at pick 8 g + 4 h + a / 4 and
    // the four columns 4 (a % 4) of a 16-column group, and receives column a of picks 8 g + 4 h .. + 3
    // The 32-byte units of a row (one 16-column group each) are XOR-swizzled by the pick number so that the 16 rows a
    // transpose read touches (four picks per 16 lanes, lane groups eight picks apart) spread over the banks: eight picks
    // are 512 or 1024 bytes, a multiple of the banks' 256-byte period, so without a term in pick / 8 the four lane groups
    // would read the same banks (measured: 52 % of the LDS-active cycles were bank conflicts).  Key of pick p:
    // (p / 2 % 2) ^ (p / 8 % 2) in the 64-byte rows, (p % 4) ^ (p / 8 % 4) in the 128-byte rows: the 512 bytes of a
    // read then fall two deep on every bank, the least possible.  p = 8 g + 4 h + a / 4 below.
    // fp32 fragments are single elements: matrix-instruction step k of a 32-pick step takes pick 4 k + g from lane group g,
    // column a of a 16-column group; rows are padded instead of swizzled (dw_tile_xstride).
    const int fr = a >> 2;                              // pick of the lane inside its group of four
    const int xkey = ((fr >> 1) & 1) ^ (g & 1), ykey = YB == 64 ? ((fr >> 1) & 1) ^ (g & 1) : (fr & 3) ^ g;
    const int at0 = ES == 2 ? (g * 8 + fr) * 64 + (a & 3) * 8 : g * XS + a * 4, at1 = at0 + 4 * 64;
    const int yat0 = ES == 2 ? (g * 8 + fr) * YB + (a & 3) * 8 : g * YS + a * 4, yat1 = yat0 + 4 * YB;
    // writers: lane holds chunk c (16 bytes; 16-bit: half a unit) of pick p
    const int xp = lane / XL, xcn = lane % XL;
    const int wr = ES == 2 ? xp * 64 + (((xcn >> 1) ^ ((xp >> 1) & 1) ^ ((xp >> 3) & 1)) << 5) + (xcn & 1) * 16 : xp * XS + xcn * 16;
    const int yp = lane / YL, ycn = lane % YL;
    // (a load of the 128-byte rows covers eight picks: pick / 8 is the load's number h, added in stage_write)
    const int ywr = ES == 2 ? yp * YB + (((ycn >> 1) ^ (YB == 64 ? ((yp >> 1) & 1) ^ ((yp >> 3) & 1) : yp & 3)) << 5) + (ycn & 1) * 16
                            : yp * YS + ycn * 16;
    // A step goes registers -> LDS tile (stage_write), LDS tile -> fragments (stage_read), fragments -> MFMAs.  The
    // loop is software-pipelined: the fragments of step s are requested first, then the registers of step s+1 are
    // dropped into the other tile (and refilled from the next chunk), then the MFMAs of step s run - so the LDS
    // round trip of one step hides behind the work of its neighbours.
    auto stage_write = [&](int s) {
        char *st = stage + (s & 1) * STG;
#pragma unroll
        for (int h = 0; h < XN; ++h) *reinterpret_cast<u32x4 *>(st + h * (64 / XL) * XS + wr) = rx[s][h];
#pragma unroll
        for (int h = 0; h < YN; ++h)
            *reinterpret_cast<u32x4 *>(st + XT + h * (64 / YL) * YS + (ES == 2 && YB == 128 ? ywr ^ ((h & 3) << 5) : ywr)) = ry[s][h];
    };
    // fragments of a step: 16-bit, one 16-byte operand per 16-column group (8 picks per lane group);
    // fp32, eight single elements per group (one per matrix-instruction step)
    struct Frag16 { u32x4 v; };
    struct Frag32 { float v[8]; };
    typedef typename std::conditional<ES == 2, Frag16, Frag32>::type Frag;
    auto stage_read = [&](int s, Frag (&pf)[2], Frag (&qf)[NY]) {
        const char *st = stage + (s & 1) * STG;
        if constexpr (ES == 2) {
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const u32x2 lo = lds_read_tr16(st + at0 + ((x ^ xkey) << 5)), hi = lds_read_tr16(st + at1 + ((x ^ xkey) << 5));
                pf[x].v = u32x4{lo[0], lo[1], hi[0], hi[1]};
            }
#pragma unroll
            for (int y = 0; y < NY; ++y) {
                const u32x2 lo = lds_read_tr16(st + XT + yat0 + ((y ^ ykey) << 5)), hi = lds_read_tr16(st + XT + yat1 + ((y ^ ykey) << 5));
                qf[y].v = u32x4{lo[0], lo[1], hi[0], hi[1]};
            }
        } else {
#pragma unroll
            for (int x = 0; x < 2; ++x)
#pragma unroll
                for (int k = 0; k < 8; ++k) pf[x].v[k] = *reinterpret_cast<const float *>(st + at0 + k * 4 * XS + x * 64);
#pragma unroll
            for (int y = 0; y < NY; ++y)
#pragma unroll
                for (int k = 0; k < 8; ++k) qf[y].v[k] = *reinterpret_cast<const float *>(st + XT + yat0 + k * 4 * YS + y * 64);
        }
    };
    auto chunk_len = [&](int c) { return c < nchunks ? min(CH, w_end - w_begin - c * CH) : 0; };

    // Steps whose rows are requested ahead of the step being multiplied: one.  Not the whole chunk: a CU's wavefronts
    // share one address path, a wavefront cannot drop its first step into LDS before its own requests are accepted, and
    // with a chunk (8 or 4 steps) requested up front all of them queued there first (B64 T256 E32 K32 I128 J64, the launches
    // that carry this body: 11.1 -> 10.5 us and 17.1 -> 16.1 us; two steps ahead the same, three and four slower).
    constexpr int P = 1;
    static_assert(P <= NS, "a chunk has at least one step");
    auto issue_step = [&](int c, int sp) {              // step sp >= 0 counted from the start of chunk c; may lie in the next chunks
        const int cc = c + sp / NS, ss = sp % NS;
        if (ss * 32 < chunk_len(cc)) issue(cc, ss);
    };
    if (nchunks > 0) {
        load_idx(0);
        store_tab(0);
        if (nchunks > 1) { load_idx(1); }
#pragma unroll
        for (int s = 0; s < P; ++s) issue_step(0, s);
        if (nchunks > 1) { store_tab(1); }
        if (nchunks > 2) load_idx(2);
        stage_write(0);
        issue_step(0, P);
    }
    for (int c = 0; c < nchunks; ++c) {
        const int len = chunk_len(c), len1 = chunk_len(c + 1);
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            // the table of chunk c+2 replaces that of chunk c once the last step of chunk c has been requested (at the
            // step before this one); its index words were requested a chunk ago
            if (s == NS - P) {
                if (chunk_len(c + 2) > 0) store_tab(c + 2);
                if (c + 3 < nchunks) load_idx(c + 3);
            }
            if (s * 32 < len) {
                Frag pf[2], qf[NY];
                stage_read(s, pf, qf);
                __builtin_amdgcn_sched_barrier(0);
                if (s + 1 < NS && (s + 1) * 32 < len) {
                    stage_write(s + 1);
                    issue_step(c, s + 1 + P);
                } else if (len1 > 0) {                  // last step of the chunk: the next chunk's first step
                    stage_write(0);
                    issue_step(c + 1, P);
                }
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (ES == 2) {
#pragma unroll
                    for (int x = 0; x < 2; ++x)
#pragma unroll
                        for (int y = 0; y < NY; ++y) mma_chunk<TT>(acc[x][y], qf[y].v, pf[x].v);
                } else {
                    // accumulators interleaved: consecutive matrix instructions never wait for each other's result
#pragma unroll
                    for (int k = 0; k < 8; ++k)
#pragma unroll
                        for (int x = 0; x < 2; ++x)
#pragma unroll
                            for (int y = 0; y < NY; ++y)
                                acc[x][y] = __builtin_amdgcn_mfma_f32_16x16x4f32(qf[y].v[k], pf[x].v[k], acc[x][y], 0, 0, 0);
                }
            }
        }
    }
    __syncthreads();                                    // every wavefront is done with its tables and staging tiles

    // lane (a, g) holds dW rows i0 + 16 x + a, columns j0 + 16 y + 4 g .. + 3
    // A row of the exchange buffer is TJ + 4 floats: with rows of 128 or 256 bytes the 16 lanes of a 16-byte write
    // (16 rows, same columns) would all fall on the same 4 banks, and the column-wise reads of the [E,J,I] layout on one.
    constexpr int RS = TJ + 4;
    float *red = reinterpret_cast<float *>(smem);       // [NW][32 i][RS]
    static_assert(32 * RS * 4 <= kLdsPerWave, "reduction buffer fits");
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int y = 0; y < NY; ++y)
            *reinterpret_cast<f32x4 *>(red + wave * (32 * RS) + (x * 16 + a) * RS + y * 16 + g * 4) = acc[x][y];
    __syncthreads();
    // wavefront tiles are added in wavefront order; 4 consecutive elements of the requested layout per thread
    const bool eji = p.dw_layout != 0;
    for (int item = tid; item < 8 * TJ; item += NW * 64) {
        // a thread sums four consecutive j of one row i over the wavefronts.  [E,I,J]: consecutive threads take consecutive
        // groups of j (one 16-byte piece of the output each); [E,J,I]: consecutive threads take consecutive i, whose four
        // elements go out one by one, each next to its neighbour thread's (rows of the exchange buffer are 4 banks apart:
        // 16 lanes x 16 bytes cover the banks once)
        const int gi_l = eji ? item & 31 : item / (TJ / 4);
        const int gj_l = (eji ? item >> 5 : item % (TJ / 4)) * 4;
        f32x4 v = *reinterpret_cast<const f32x4 *>(red + gi_l * RS + gj_l);
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            const f32x4 u = *reinterpret_cast<const f32x4 *>(red + w * (32 * RS) + gi_l * RS + gj_l);
            v[0] += u[0]; v[1] += u[1]; v[2] += u[2]; v[3] += u[3];
        }
        const int gi = i0 + gi_l, gj = j0 + gj_l;
        if (gi >= p.I || gj >= p.J) continue;           // J % 4 == 0: a group of four j is inside or outside
        if (!eji) {
            const size_t at = ((size_t)e * p.I + gi) * p.J + gj;
            if (p.out_dtype == 0) {
                *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(p.dW) + at) = v;
            } else {
                u32x2 w2;
                w2[0] = p.out_dtype == 1 ? pack2<ElemF16>(v[0], v[1]) : pack2<ElemBF16>(v[0], v[1]);
                w2[1] = p.out_dtype == 1 ? pack2<ElemF16>(v[2], v[3]) : pack2<ElemBF16>(v[2], v[3]);
                *reinterpret_cast<u32x2 *>(reinterpret_cast<uint16_t *>(p.dW) + at) = w2;
            }
        } else {
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const size_t at = ((size_t)e * p.J + gj + x) * p.I + gi;
                if (p.out_dtype == 0) reinterpret_cast<float *>(p.dW)[at] = v[x];
                else reinterpret_cast<uint16_t *>(p.dW)[at] =
                         (uint16_t)((p.out_dtype == 1 ? pack2<ElemF16>(v[x], 0.f) : pack2<ElemBF16>(v[x], 0.f)) & 0xffffu);
            }
        }
    }
}

template <class TT>
__global__ __launch_bounds__(kThreads) void dw_tile_kernel(DwTileParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_dw_tile[];
    dw_tile_body<TT, kThreads / 64>(p, (int)blockIdx.x, smem_dw_tile);
}

// fp32: 32 x 64 tiles, 4 wavefronts (the staging tiles of 8 would not fit)
static __global__ __launch_bounds__(kThreads) void dw_tile_wide_f32_kernel(DwTileParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_dw_tile_wide_f32[];
    dw_tile_body<ElemF32, kThreads / 64, 64>(p, (int)blockIdx.x, smem_dw_tile_wide_f32);
}

// 32 x 64 tiles, 8 wavefronts
constexpr int kDwWideThreads = 512;
template <class TT>
__global__ __launch_bounds__(kDwWideThreads) void dw_tile_wide_kernel(DwTileParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_dw_tile_wide[];
    dw_tile_body<TT, kDwWideThreads / 64, 64>(p, (int)blockIdx.x, smem_dw_tile_wide);
}

}  // namespace egs
