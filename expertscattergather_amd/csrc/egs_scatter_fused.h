// GEMM-scatter for small experts in ONE kernel, product rows never leaving the CU:
//
//   out[b, t, c0:c0+32] = sum over the picks (e, k) of token t, in routing-table order, of
//                         A[b, e, k, :] . W(e)[:, c0:c0+32]
//
// A workgroup owns one batch element b and one 32-column slice of the output.  It
//   (0) sorts the picks of b by token in LDS (the counting sort of csr_count_body; the slices of
//       one batch element repeat it, which is cheaper than a launch of its own),
//   (1) multiplies every pick's row by its expert's weight slice on the MFMAs (operands straight
//       from global memory into registers, several (expert, 32-pick) units in flight per wavefront)
//       and parks the fp32 products in LDS, one 128-byte row per pick,
//   (2) walks each token's segment of the table, adds its product rows in table order in fp32,
//       rounds once and writes the output row slice (tokens nobody picked become zero).
// Nothing but the inputs and the output touches memory: compared with product rows in a
// workspace plus a segment-sum launch this removes 2 x 32 MB of traffic and a launch at the
// reference's default shape.  Bitwise reproducible (fixed order), no atomics.
//
// Fits when a batch element's picks (E*K <= 1024) times 128 bytes, the table and the sort's
// histograms fit in LDS; 16-bit elements with reduction 32/64/128 or fp32 with reduction 32/64, output
// columns a multiple of 32.
//
// More picks than fit (MULTI, up to four passes): the table is in expert order inside a token's segment, so the
// experts are taken in consecutive groups; each pass parks the products of one group in LDS and every thread
// continues its tokens' sums where the previous pass stopped (a cursor per token, partial sums in
// registers).  The order of the additions is the order of the table, as in one pass: same bits.
//
// Replaces the reference's expert_scatter_kernel (egs/triton_kernels.py:156-247), which adds every
// output element with a global atomic.
#pragma once
#include "egs_device.h"
#include "egs_scatter_aux.h"
#include "egs_small.h"

namespace egs {

constexpr int kFusedCols = 32;          // output columns per workgroup
constexpr int kFusedThreads = 512;      // 8 wavefronts: enough units in flight to cover the memory latency in two rounds

struct ScatterFusedParams {
    const char *A;          // [B,E,K,R] dense rows
    const char *W;          // [E,R,N] (W_NMAJOR) or [E,N,R]
    const void *Ind;        // [B,E,K]
    char *out;              // [B,T,N] element type
    int32_t B, T, E, K, N;
    int32_t ind_dtype;
    int32_t slices;         // N / kFusedCols
    int32_t perm_at, cnt_at;    // byte offsets of the table and of the sort's counters in dynamic LDS (rows start at 0)
    int32_t zero_at;            // ... and of 128 bytes of zeros (128-byte aligned), scatter_fused_zero_at()
    int32_t xcd_batch;          // consecutive batch elements per XCD: 1, 2, 4 or 8
    int32_t experts_per_pass;   // MULTI: experts whose product rows are in LDS at a time (E otherwise)
    // TABLE: routing table built beforehand (seg [B][T+1], perm [B][E*K]); the workgroup copies its batch element's part
    // into LDS instead of sorting the picks itself
    const int32_t *tab_seg, *tab_perm;
};

constexpr int kFusedMaxPasses = 4;
constexpr int kFusedMultiTokens = 8;    // MULTI: tokens per thread (64 threads groups of 8 walk the tokens) -> T <= 512

// LDS bytes: product rows (of `rows` picks at a time), table of all NP picks, counters of the sort (one histogram
// per wavefront + offsets), a row of zeros
__host__ __device__ inline size_t scatter_fused_zero_at(int T, int NP, int rows)
{
    const size_t at = (size_t)rows * kFusedCols * 4 + (size_t)NP * 4 + ((size_t)(kFusedThreads / 64 + 1) * T + 1) * 4 + 64;
    return (at + 127) & ~(size_t)127;
}
__host__ __device__ inline size_t scatter_fused_lds(int T, int NP, int rows)
{
    return scatter_fused_zero_at(T, NP, rows) + kFusedCols * 4;
}
__host__ __device__ inline size_t scatter_fused_lds(int T, int NP) { return scatter_fused_lds(T, NP, NP); }

template <class TT, bool W_NMAJOR, int KS, bool MULTI = false, bool TABLE = false>
__device__ __forceinline__ void scatter_fused_body(const ScatterFusedParams &p, const int block, char *smem)
{
    // KS = reduction length in MFMA steps of four 16-byte chunks: 32 elements of a 16-bit type, 16 of fp32
    constexpr int ES = TT::ES, VEC = TT::VEC;
    constexpr int R = 4 * VEC * KS;
    constexpr int kFusedDepth = KS == 4 ? 2 : 4;         // (expert, 32-pick) units a wavefront has registers for
    // Units requested ahead of the one being multiplied.  One pass: a single one - the wavefronts of a CU then take turns
    // at its one address path, which is what bounds this phase (about 200 cycles of it per unit with the 4-byte pieces of an
    // [E,R,N] weight; with all four units requested up front a wavefront spent 5000 cycles issuing before it multiplied
    // anything, 8.3 against 9.8 us at B64 T256 E32 K32 I128 J64 together with the summing loop below).  In passes: all.
    constexpr int kAhead = MULTI ? kFusedDepth : 1;
    // a table that this workgroup parks itself (TABLE, one pass) is parked as row addresses, see (2)
    constexpr bool kEncoded = TABLE && !MULTI;
    // the wavefront index is made known as uniform: units, experts and base addresses derived from it are then
    // scalar work, and the loads take a scalar base with a per-lane 32-bit offset
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int a = lane & 15, g = lane >> 4;
    // slices of one batch element sit on one XCD (ids congruent modulo 8 share an XCD), so that its
    // rows are fetched from memory once
    const int grp = block & 7, idx = block >> 3;
    const int qb = idx / p.slices, slice = idx % p.slices;
    // XCD grp takes runs of xcd_batch consecutive batch elements (a power of two up to 8: the batch elements of one 256-pick
    // row tile of the gather that wrote this scatter's rows, which ran on the XCD of the same number), i.e. the elements
    // xcd_batch * grp .. + xcd_batch - 1 of every 8 * xcd_batch; a last incomplete block: grp of every 8
    const int nb = p.xcd_batch;
    const int b = (qb | (nb - 1)) < ((p.B + 7) >> 3) ? ((qb / nb) * 8 + grp) * nb + (qb & (nb - 1)) : qb * 8 + grp;
    if (b >= p.B) return;
    const int c0 = slice * kFusedCols;
    const int T = p.T, E = p.E, K = p.K, N = p.N, NP = E * K;

    float *rows = reinterpret_cast<float *>(smem);
    int32_t *perm = reinterpret_cast<int32_t *>(smem + p.perm_at);
    int32_t *cnt = reinterpret_cast<int32_t *>(smem + p.cnt_at);
    constexpr int NWV = kFusedThreads / 64;
    const int32_t *seg = cnt + NWV * T;                 // token offsets left there by the sort
    if (!MULTI && tid < kFusedCols) reinterpret_cast<float *>(smem + p.zero_at)[tid] = 0.f;     // read after the barrier before (2)

    // ---------------- (1) units of work of this wavefront: (expert, pair of 16-pick row tiles); the weight
    // fragments of a unit serve both row tiles
    // A pass covers the experts [e0, e0 + ne): all of them, unless MULTI
    const int KT2 = (K + 31) >> 5;
    struct Unit { u32x4 y[2][KS]; u32x4 w[2 * KS]; };
    Unit buf[kFusedDepth];
    const uint32_t a_base_b = (uint32_t)b * (uint32_t)NP * R * ES;
    auto load_unit = [&](Unit &u, int unit, int e0, int ne) {
        if (unit >= ne * KT2) return;                   // uniform per wavefront; a unit's own loads are unconditional
        const int el = unit / KT2, rp = unit - el * KT2, e = e0 + el;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            // coalesced: lanes 4r .. 4r+3 fetch four consecutive chunks of row r; transposed to operand order at use
            const int k = min(rp * 32 + h * 16 + (lane >> 2), K - 1);
            const char *yrow = p.A + a_base_b + (uint32_t)((e * K + k) * R * ES);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) u.y[h][ks] = *reinterpret_cast<const u32x4 *>(yrow + (ks * 4 + (lane & 3)) * 16);
        }
        if constexpr (!W_NMAJOR) {
            // [E,N,R]: the lane's output column is a row of W
#pragma unroll
            for (int ct = 0; ct < 2; ++ct) {
                const char *wrow = p.W + ((size_t)e * N + c0 + ct * 16 + (lane >> 2)) * (R * ES);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) u.w[ct * KS + ks] = *reinterpret_cast<const u32x4 *>(wrow + (ks * 4 + (lane & 3)) * 16);
            }
        } else {
            // [E,R,N]: VEC (reduction) x 2 (columns 2a, 2a+1) blocks, transposed in registers below; raw rows kept here
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const char *wblk = p.W + (((size_t)e * R + ks * 4 * VEC + g * VEC) * N + c0 + 2 * a) * ES;
                if constexpr (ES == 2) {
#pragma unroll
                    for (int x = 0; x < 8; ++x)
                        u.w[ks * 2 + (x >> 2)][x & 3] = *reinterpret_cast<const uint32_t *>(wblk + (size_t)x * N * 2);
                } else {
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        const u32x2 two = *reinterpret_cast<const u32x2 *>(wblk + (size_t)x * N * 4);
                        u.w[ks * 2 + (x >> 1)][(x & 1) * 2] = two[0];
                        u.w[ks * 2 + (x >> 1)][(x & 1) * 2 + 1] = two[1];
                    }
                }
            }
        }
    };
    auto compute_unit = [&](const Unit &u, int unit, int ne) {
        if (unit >= ne * KT2) return;
        const int e = unit / KT2, rp = unit - e * KT2;  // expert counted from the first of the pass: rows are local to the pass
        f32x4 acc[2][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) { acc[h][0] = f32x4{0.f, 0.f, 0.f, 0.f}; acc[h][1] = f32x4{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 wf[2];
            if constexpr (!W_NMAJOR) {
                wf[0] = lanes_4a_g_to_16g_a(u.w[ks], lane); wf[1] = lanes_4a_g_to_16g_a(u.w[KS + ks], lane);
            } else if constexpr (ES == 2) {
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const uint32_t lo = u.w[ks * 2 + (pp >> 1)][(pp & 1) * 2], hi = u.w[ks * 2 + (pp >> 1)][(pp & 1) * 2 + 1];
                    wf[0][pp] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);     // column 2a   of rows 2pp, 2pp+1
                    wf[1][pp] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);     // column 2a+1
                }
            } else {
#pragma unroll
                for (int x = 0; x < 4; ++x) {                                   // row x of the block: columns 2a, 2a+1
                    wf[0][x] = u.w[ks * 2 + (x >> 1)][(x & 1) * 2];
                    wf[1][x] = u.w[ks * 2 + (x >> 1)][(x & 1) * 2 + 1];
                }
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const u32x4 yf = lanes_4a_g_to_16g_a(u.y[h][ks], lane);
                mma_chunk<TT>(acc[h][0], wf[0], yf);
                mma_chunk<TT>(acc[h][1], wf[1], yf);
            }
        }
        // lane (a, g) holds, for pick k = 32 rp + 16 h + a, slice columns
        //   [E,N,R]: 16 ct + 4 g + r            -> chunk 4 ct + g of the row
        //   [E,R,N]: 2 (4 g + r) + ct = 8 g + 2 r + ct -> chunks 2 g, 2 g + 1 after interleaving the two tiles
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = rp * 32 + h * 16 + a;
            if (k < K) {
                const int q = e * K + k;
                f32x4 *row = reinterpret_cast<f32x4 *>(rows + (size_t)q * kFusedCols);
                if constexpr (!W_NMAJOR) {
                    row[(g) ^ (q & 7)] = acc[h][0];
                    row[(4 + g) ^ (q & 7)] = acc[h][1];
                } else {
                    row[(2 * g) ^ (q & 7)] = f32x4{acc[h][0][0], acc[h][1][0], acc[h][0][1], acc[h][1][1]};
                    row[(2 * g + 1) ^ (q & 7)] = f32x4{acc[h][0][2], acc[h][1][2], acc[h][0][3], acc[h][1][3]};
                }
            }
        }
    };

    // ---------------- (0) routing table of batch element b in LDS; the first units' operands go in flight
    // right behind the sort's token loads and travel while it runs
    const int EP = MULTI ? p.experts_per_pass : E;
    if constexpr (TABLE) {
        // the table comes from memory: its loads go first, the operands behind them; it is parked in LDS in the places
        // the sort would have left it while the operands travel (one pass: NP <= 1024, T < 2048; in passes: NP <= 2048,
        // T <= 512 - checked by the host)
        constexpr int PV = (MULTI ? 2048 : 1024) / kFusedThreads, SV = (MULTI ? 1024 : 2048) / kFusedThreads;
        const int32_t *gseg = p.tab_seg + (size_t)b * (T + 1), *gperm = p.tab_perm + (size_t)b * NP;
        int32_t pv[PV], sv[SV];
#pragma unroll
        for (int x = 0; x < PV; ++x) pv[x] = gperm[min(tid + x * kFusedThreads, NP - 1)];
#pragma unroll
        for (int x = 0; x < SV; ++x) sv[x] = gseg[min(tid + x * kFusedThreads, T)];
#pragma unroll
        for (int d = 0; d < kAhead; ++d) load_unit(buf[d], wave + NWV * d, 0, min(EP, E));
        int32_t *seg_w = cnt + NWV * T;
        // entries are clamped to what a table of these sizes can hold: whatever a caller hands over (a table of other
        // indices, memory that was never filled), every loop below ends and every access stays inside the workgroup's rows
#pragma unroll
        for (int x = 0; x < PV; ++x)
            if (tid + x * kFusedThreads < NP) {
                const int q = min(max(pv[x], 0), NP - 1);
                perm[tid + x * kFusedThreads] = kEncoded ? (q << 7) | ((q & 7) << 4) : q;
            }
#pragma unroll
        for (int x = 0; x < SV; ++x)
            if (tid + x * kFusedThreads <= T) seg_w[tid + x * kFusedThreads] = min(max(sv[x], 0), NP);
    } else {
    csr_count_body(cnt, b, 0, tid, kFusedThreads, p.Ind, p.ind_dtype, T, NP, nullptr, perm, nullptr, nullptr, [&]() {
#pragma unroll
        for (int d = 0; d < kAhead; ++d) load_unit(buf[d], wave + NWV * d, 0, min(EP, E));
    });
    }

    const int cc = tid & 7;
    auto store_row = [&](int t, const f32x4 &sum) {
        char *dst = p.out + (((size_t)b * T + t) * N + c0 + cc * 4) * ES;
        if constexpr (ES == 4) {
            *reinterpret_cast<f32x4 *>(dst) = sum;
        } else {
            u32x2 w;
            w[0] = pack2<TT>(sum[0], sum[1]);
            w[1] = pack2<TT>(sum[2], sum[3]);
            *reinterpret_cast<u32x2 *>(dst) = w;
        }
    };

    if constexpr (!MULTI) {
        for (int u0 = wave; u0 < E * KT2; u0 += NWV * kFusedDepth) {
#pragma unroll
            for (int d = 0; d < kFusedDepth; ++d) {
                // the request for the unit kAhead further on goes out before this one is multiplied: a CU's wavefronts
                // then take turns at its one address path instead of all queueing there first and multiplying afterwards
                if constexpr (kAhead < kFusedDepth) load_unit(buf[(d + kAhead) % kFusedDepth], u0 + NWV * (d + kAhead), 0, E);
                compute_unit(buf[d], u0 + NWV * d, E);
                if constexpr (kAhead == kFusedDepth) load_unit(buf[d], u0 + NWV * d + NWV * kFusedDepth, 0, E);
            }
        }
        __syncthreads();

        // ---------------- (2) per token: add its product rows in table order; 4 threads x 8 columns per token.
        // The table entries of a segment are read four at a time without looking at its end (what follows in LDS is the next
        // segment or the sort's counters: inside the allocation either way); an entry past the end selects a row of zeros
        // instead of its own, so that the additions need no condition.  Entry q stands for byte (q << 7) | ((q & 7) << 4),
        // chunk 0 of row q in the rows' XOR order: a thread's two chunks are one XOR away each.  (The phase is bound by
        // vector-ALU issue - two wavefronts per SIMD, all in it at once - so it is written for few instructions per pick.)
        const uint32_t c2 = (uint32_t)(tid & 3) << 5, zero_sel = (uint32_t)p.zero_at;
        for (int t = tid >> 2; t < T; t += kFusedThreads >> 2) {
            const int s0 = seg[t], s1 = seg[t + 1];
            f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
            for (int s = s0; s < s1; s += 4) {
                const int n = s1 - s;
                uint32_t en[4];
                f32x4 v[4][2];
#pragma unroll
                for (int x = 0; x < 4; ++x) en[x] = (uint32_t)perm[s + x];
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const uint32_t at = kEncoded ? en[x] : (en[x] << 7) | ((en[x] & 7u) << 4);
                    const uint32_t sel = (x < n) ? at : zero_sel;
                    v[x][0] = *reinterpret_cast<const f32x4 *>(smem + (sel ^ c2));
                    v[x][1] = *reinterpret_cast<const f32x4 *>(smem + (sel ^ (c2 | 16u)));
                }
#pragma unroll
                for (int x = 0; x < 4; ++x) { lo += v[x][0]; hi += v[x][1]; }
            }
            char *dst = p.out + (((size_t)b * T + t) * N + c0 + (tid & 3) * 8) * ES;
            if constexpr (ES == 4) {
                reinterpret_cast<f32x4 *>(dst)[0] = lo;
                reinterpret_cast<f32x4 *>(dst)[1] = hi;
            } else {
                u32x4 w;
                w[0] = pack2<TT>(lo[0], lo[1]); w[1] = pack2<TT>(lo[2], lo[3]);
                w[2] = pack2<TT>(hi[0], hi[1]); w[3] = pack2<TT>(hi[2], hi[3]);
                *reinterpret_cast<u32x4 *>(dst) = w;
            }
        }
    } else {
        // ---------------- (1) + (2) in passes over groups of EP experts.  A thread keeps, for each of its tokens, the
        // place in the segment where the previous pass stopped and the sum so far.
        constexpr int TOK = kFusedMultiTokens, TSTRIDE = kFusedThreads >> 3;
        int cur[TOK], end[TOK];
        f32x4 sum[TOK];
        for (int e0 = 0; e0 < E; e0 += EP) {
            const int ne = min(EP, E - e0), ne_next = min(EP, E - e0 - ne);
            for (int u0 = wave; u0 < ne * KT2; u0 += NWV * kFusedDepth) {
#pragma unroll
                for (int d = 0; d < kFusedDepth; ++d) {
                    compute_unit(buf[d], u0 + NWV * d, ne);
                    load_unit(buf[d], u0 + NWV * d + NWV * kFusedDepth, e0, ne);
                }
            }
            // the next group's first operands travel while this group's rows are added
            if (ne_next > 0) {
#pragma unroll
                for (int d = 0; d < kFusedDepth; ++d) load_unit(buf[d], wave + NWV * d, e0 + ne, ne_next);
            }
            __syncthreads();                            // products (and, in the first pass, the table) are in LDS
            if (e0 == 0) {
#pragma unroll
                for (int i = 0; i < TOK; ++i) {
                    const int t = (tid >> 3) + i * TSTRIDE;
                    cur[i] = t < T ? seg[t] : 0;
                    end[i] = t < T ? seg[t + 1] : 0;
                    sum[i] = f32x4{0.f, 0.f, 0.f, 0.f};
                }
            }
            const int lo = e0 * K, hi = (e0 + ne) * K;  // picks whose rows are in LDS now; a segment lists its picks in increasing order
#pragma unroll
            for (int i = 0; i < TOK; ++i) {
                while (cur[i] < end[i]) {
                    int q[4];
                    f32x4 v[4];
#pragma unroll
                    for (int x = 0; x < 4; ++x) q[x] = perm[min(cur[i] + x, end[i] - 1)];
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        const int ql = (q[x] < hi && q[x] >= lo) ? q[x] - lo : 0;   // picks of later groups (or, in a table that is not this Ind's, of earlier ones): any valid row
                        v[x] = reinterpret_cast<const f32x4 *>(rows + (size_t)ql * kFusedCols)[cc ^ (ql & 7)];
                    }
                    int n = 0;
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        if (cur[i] + x < end[i] && q[x] < hi) { sum[i] += v[x]; ++n; }
                    cur[i] += n;
                    if (n < 4) break;
                }
            }
            if (ne_next > 0) __syncthreads();           // everybody is done with this group's rows
        }
#pragma unroll
        for (int i = 0; i < TOK; ++i) {
            const int t = (tid >> 3) + i * TSTRIDE;
            if (t < T) store_row(t, sum[i]);
        }
    }
}

template <class TT, bool W_NMAJOR, int KS>
__global__ __launch_bounds__(kFusedThreads) void scatter_fused_kernel(ScatterFusedParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_fused[];
    scatter_fused_body<TT, W_NMAJOR, KS>(p, (int)blockIdx.x, smem_fused);
}

// more picks per batch element than LDS holds product rows for: groups of experts, one after the other
template <class TT, bool W_NMAJOR, int KS>
__global__ __launch_bounds__(kFusedThreads) void scatter_fused_multi_kernel(ScatterFusedParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_fused_multi[];
    scatter_fused_body<TT, W_NMAJOR, KS, true>(p, (int)blockIdx.x, smem_fused_multi);
}

// the same with the first pass of a small weight gradient of the same backward call in the launch:
// workgroups [0, fused_blocks) run the scatter, the rest the weight gradient
template <class TT, bool W_NMAJOR, int KS>
__global__ __launch_bounds__(kFusedThreads) void scatter_fused_dw_kernel(ScatterFusedParams p, SmallDwParams q, int fused_blocks)
{
    extern __shared__ __attribute__((aligned(16))) char smem_fused_dw[];
    if ((int)blockIdx.x < fused_blocks) {
        scatter_fused_body<TT, W_NMAJOR, KS>(p, (int)blockIdx.x, smem_fused_dw);
    } else {
        dw_small_body<TT, kFusedThreads / 64>(q, (int)blockIdx.x - fused_blocks, reinterpret_cast<float *>(smem_fused_dw));
    }
}

// with the routing table read from memory instead of sorted in the kernel
template <class TT, bool W_NMAJOR, int KS>
__global__ __launch_bounds__(kFusedThreads) void scatter_fused_multi_table_kernel(ScatterFusedParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_fused_multi_table[];
    scatter_fused_body<TT, W_NMAJOR, KS, true, true>(p, (int)blockIdx.x, smem_fused_multi_table);
}

template <class TT, bool W_NMAJOR, int KS>
__global__ __launch_bounds__(kFusedThreads) void scatter_fused_table_kernel(ScatterFusedParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_fused_table[];
    scatter_fused_body<TT, W_NMAJOR, KS, false, true>(p, (int)blockIdx.x, smem_fused_table);
}

template <class TT, bool W_NMAJOR, int KS>
__global__ __launch_bounds__(kFusedThreads) void scatter_fused_dwtile_table_kernel(ScatterFusedParams p, DwTileParams q, int fused_blocks)
{
    extern __shared__ __attribute__((aligned(16))) char smem_fused_dwtile_table[];
    if ((int)blockIdx.x < fused_blocks) {
        scatter_fused_body<TT, W_NMAJOR, KS, false, true>(p, (int)blockIdx.x, smem_fused_dwtile_table);
    } else {
        if constexpr (TT::ES == 2) dw_tile_body<TT, kFusedThreads / 64>(q, (int)blockIdx.x - fused_blocks, smem_fused_dwtile_table);
    }
}

// ... or with the one-pass weight gradient (egs_dw_tile.h) of the same backward call
template <class TT, bool W_NMAJOR, int KS>
__global__ __launch_bounds__(kFusedThreads) void scatter_fused_dwtile_kernel(ScatterFusedParams p, DwTileParams q, int fused_blocks)
{
    extern __shared__ __attribute__((aligned(16))) char smem_fused_dwtile[];
    if ((int)blockIdx.x < fused_blocks) {
        scatter_fused_body<TT, W_NMAJOR, KS>(p, (int)blockIdx.x, smem_fused_dwtile);
    } else {
        if constexpr (TT::ES == 2) dw_tile_body<TT, kFusedThreads / 64>(q, (int)blockIdx.x - fused_blocks, smem_fused_dwtile);
    }
}

}  // namespace egs
