// GEMM-scatter in ONE kernel for batch elements with thousands of picks: product rows never reach memory.
//
//   out[b, t, c0:c0+32] = sum over the picks (e, k) of token t, in a fixed order, of A[b, e, k, :] . W(e)[:, c0:c0+32]
//
// A workgroup (8 wavefronts) owns one batch element b and one 32-column slice of the output, like the one-kernel
// scatter of small experts (egs_scatter_fused.h), but where that kernel parks the product rows of ALL picks of the
// batch element in LDS, this one works through the picks in passes:
//   - the routing table of b (picks in a stable order by token, built beforehand) is copied into LDS as 16-bit entries;
//   - a pass takes the next `units_per_pass` (expert, 32-pick) units in pick order; a wavefront takes a contiguous
//     share of them (so that its units share an expert and the expert's weight slice is fetched once), multiplies on the
//     matrix cores with the operands coming straight from global memory into registers, two units in flight, and parks
//     the fp32 products in LDS, one 128-byte row per pick;
//   - after a barrier every group of 8 threads continues the sums of its 16 tokens (kept in registers for the whole
//     kernel): a token's segment of the table lists its picks in increasing pick number, so the picks of a pass are
//     the next entries of every segment, and the additions happen in table order;
//   - the first operands of the next pass are in flight while the sums are continued.
// A token with more than kPassLong picks (skewed routing) is not walked by its 8 threads: in every pass a whole
// wavefront adds that token's rows of the pass, eight rows per step, lane group r taking entries r, r + 8, ... of
// each 64-entry chunk, then the eight lane groups are added in order r = 0..7 and the result joins the token's
// running total in LDS.  Which wavefront does it and the order of every addition depend on the table alone:
// bitwise reproducible, no atomics on data.
//
// Takes 16-bit elements, reduction length 32 / 64 / 128, output columns a multiple of 32, T <= 1024, and as many
// picks per batch element as the 16-bit table leaves room for beside at least 16 units of rows.
// Replaces, at these sizes, the reference's expert_scatter_kernel (egs/triton_kernels.py:156-247), which adds every
// output element with a global atomic.
#pragma once
#include "egs_device.h"
#include "egs_scatter_fused.h"

namespace egs {

constexpr int kPassTokens = 16;                                     // tokens per group of 8 threads
constexpr int kPassMaxT = (kFusedThreads >> 3) * kPassTokens;       // 1024
constexpr int kPassLong = 128;                                      // longer segments are summed by a whole wavefront
constexpr int kPassMaxPicks = 32768;                                // 16-bit table entries, with room to spare

struct ScatterPassParams {
    const char *A;              // [B,E,K,R] dense rows
    const char *W;              // [E,R,N] (W_NMAJOR) or [E,N,R]
    char *out;                  // [B,T,N] element type
    const int32_t *tab_seg;     // [B][T+1] routing table: segment offsets ...
    const int32_t *tab_perm;    // [B][E*K]  ... and picks in token order
    int32_t B, T, E, K, N;
    int32_t slices;             // N / kFusedCols
    int32_t units_per_pass;     // (expert, 32-pick) units whose product rows are in LDS at a time; a multiple of 16
    int32_t long_slots;         // long tokens a batch element can have: E*K / (kPassLong + 1) + 1
    int32_t perm_at, seg_at, long_at, tot_at;   // byte offsets in dynamic LDS (product rows start at 0)
};

__host__ __device__ inline int pass_long_slots(int NP) { return NP / (kPassLong + 1) + 1; }
// LDS bytes beside the product rows: 16-bit table, long-token records (counter, token, cursor, end) and totals
__host__ __device__ inline size_t scatter_pass_fixed_lds(int T, int NP)
{
    const size_t slots = (size_t)pass_long_slots(NP);
    return (((size_t)NP * 2 + 15) & ~(size_t)15) + (((size_t)(T + 1) * 2 + 15) & ~(size_t)15) + 16 + 3 * 4 * slots + slots * kFusedCols * 4;
}

template <class TT, bool W_NMAJOR, int KS>
__global__ __launch_bounds__(kFusedThreads) void scatter_pass_kernel(ScatterPassParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_pass[];
    static_assert(TT::ES == 2, "16-bit element types");
    constexpr int ES = 2, VEC = 8, R = 4 * VEC * KS, NWV = kFusedThreads / 64, TOK = kPassTokens;
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int a = lane & 15, g = lane >> 4;
    // slices of one batch element sit on one XCD (ids congruent modulo 8 share an XCD): its rows come from memory once
    const int block = (int)blockIdx.x, grp = block & 7, idx = block >> 3;
    const int b = (idx / p.slices) * 8 + grp, slice = idx % p.slices;
    if (b >= p.B) return;
    const int c0 = slice * kFusedCols;
    const int T = p.T, E = p.E, K = p.K, N = p.N, NP = E * K;
    const int KT2 = (K + 31) >> 5, NU = E * KT2;        // units per expert, units in all
    const int UP = p.units_per_pass, UPW = UP / NWV;    // units per pass, and per pass and wavefront (even)
    const int npass = (NU + UP - 1) / UP;

    float *rows = reinterpret_cast<float *>(smem_pass);
    uint16_t *perm = reinterpret_cast<uint16_t *>(smem_pass + p.perm_at);
    uint16_t *seg = reinterpret_cast<uint16_t *>(smem_pass + p.seg_at);
    int32_t *lctr = reinterpret_cast<int32_t *>(smem_pass + p.long_at);
    int32_t *ltok = lctr + 4, *lcur = ltok + p.long_slots, *lend = lcur + p.long_slots;
    float *ltot = reinterpret_cast<float *>(smem_pass + p.tot_at);

    // first pick of unit u (units are numbered in pick order); NP past the last unit
    auto first_pick = [&](int u) { const int e = u / KT2; return u >= NU ? NP : e * K + (u - e * KT2) * 32; };

    // ---------------- operands of a unit: 32 rows of A (two 16-row tiles), and the weight slice of its expert
    const uint32_t a_base_b = (uint32_t)b * (uint32_t)NP * R * ES;
    struct RowsOp { u32x4 y[2][KS]; };
    RowsOp buf[2];
    u32x4 wreg[2 * KS];
    int w_e = -1;                                       // expert whose slice wreg holds (uniform)
    auto load_rows = [&](RowsOp &u, int unit) {
        if (unit >= NU) return;                         // uniform per wavefront; a unit's own loads are unconditional
        const int e = unit / KT2, rp = unit - e * KT2;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            // coalesced: lanes 4r .. 4r+3 fetch four consecutive chunks of row r; moved to operand order at use
            const int k = min(rp * 32 + h * 16 + (lane >> 2), K - 1);
            const char *yrow = p.A + a_base_b + (uint32_t)((e * K + k) * R * ES);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) u.y[h][ks] = *reinterpret_cast<const u32x4 *>(yrow + (ks * 4 + (lane & 3)) * 16);
        }
    };
    auto load_w = [&](int e) {
        if constexpr (!W_NMAJOR) {
            // [E,N,R]: the lane's output column is a row of W
#pragma unroll
            for (int ct = 0; ct < 2; ++ct) {
                const char *wrow = p.W + ((size_t)e * N + c0 + ct * 16 + (lane >> 2)) * (R * ES);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) wreg[ct * KS + ks] = *reinterpret_cast<const u32x4 *>(wrow + (ks * 4 + (lane & 3)) * 16);
            }
        } else {
            // [E,R,N]: 8 (reduction) x 2 (columns 2a, 2a+1) blocks, transposed in registers at use; raw rows kept here
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const char *wblk = p.W + (((size_t)e * R + ks * 4 * VEC + g * VEC) * N + c0 + 2 * a) * ES;
#pragma unroll
                for (int x = 0; x < 8; ++x)
                    wreg[ks * 2 + (x >> 2)][x & 3] = *reinterpret_cast<const uint32_t *>(wblk + (size_t)x * N * 2);
            }
        }
        w_e = e;
    };
    // products of a unit into LDS rows [first pick of the unit - lo ...)
    auto compute_unit = [&](const RowsOp &u, int unit, int lo) {
        const int e = unit / KT2, rp = unit - e * KT2;
        f32x4 acc[2][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) { acc[h][0] = f32x4{0.f, 0.f, 0.f, 0.f}; acc[h][1] = f32x4{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 wf[2];
            if constexpr (!W_NMAJOR) {
                wf[0] = lanes_4a_g_to_16g_a(wreg[ks], lane); wf[1] = lanes_4a_g_to_16g_a(wreg[KS + ks], lane);
            } else {
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const uint32_t lo2 = wreg[ks * 2 + (pp >> 1)][(pp & 1) * 2], hi2 = wreg[ks * 2 + (pp >> 1)][(pp & 1) * 2 + 1];
                    wf[0][pp] = __builtin_amdgcn_perm(hi2, lo2, 0x05040100u);     // column 2a   of rows 2pp, 2pp+1
                    wf[1][pp] = __builtin_amdgcn_perm(hi2, lo2, 0x07060302u);     // column 2a+1
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
        //   [E,N,R]: 16 ct + 4 g + r                   -> chunk 4 ct + g of the row
        //   [E,R,N]: 2 (4 g + r) + ct = 8 g + 2 r + ct -> chunks 2 g, 2 g + 1 after interleaving the two tiles
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = rp * 32 + h * 16 + a;
            if (k < K) {
                const int q = e * K + k - lo;
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
    auto unit_of = [&](int pass, int i) { return pass * UP + wave * UPW + i; };

    // ---------------- (0) the table of batch element b goes to LDS as 16-bit entries; the first operands travel behind it
    {
        const int32_t *gseg = p.tab_seg + (size_t)b * (T + 1), *gperm = p.tab_perm + (size_t)b * NP;
        // entries are clamped to what a table of these sizes can hold: whatever memory a caller hands over, every loop
        // below ends and every access stays inside the workgroup's LDS
        for (int s0 = 0; s0 < NP; s0 += 8 * kFusedThreads) {
            int32_t v[8];
#pragma unroll
            for (int x = 0; x < 8; ++x) v[x] = gperm[min(s0 + x * kFusedThreads + tid, NP - 1)];
            if (s0 == 0) {
                const int u0 = unit_of(0, 0);
                if (u0 < NU) load_w(u0 / KT2);
                load_rows(buf[0], u0);
                load_rows(buf[1], u0 + 1);
            }
#pragma unroll
            for (int x = 0; x < 8; ++x)
                if (s0 + x * kFusedThreads + tid < NP) perm[s0 + x * kFusedThreads + tid] = (uint16_t)min(max(v[x], 0), NP - 1);
        }
        for (int t = tid; t <= T; t += kFusedThreads) seg[t] = (uint16_t)min(max(gseg[t], 0), NP);
        if (tid == 0) lctr[0] = 0;
        for (int x = tid; x < p.long_slots * kFusedCols; x += kFusedThreads) ltot[x] = 0.f;
    }
    __syncthreads();

    // ---------------- per-thread state of the sums: 8 threads x 4 columns per token, 16 tokens per thread
    const int cc = tid & 7;
    uint32_t ce[TOK];               // cursor | end << 16 into the token's segment
    f32x4 sum[TOK];
    uint32_t long_mask = 0;         // tokens of this thread that a wavefront sums instead
#pragma unroll
    for (int i = 0; i < TOK; ++i) {
        const int t = (tid >> 3) + i * (kFusedThreads >> 3);
        int s0 = t < T ? (int)seg[t] : 0, s1 = t < T ? (int)seg[t + 1] : 0;
        if (s1 - s0 > kPassLong) {
            if (cc == 0) {
                const int slot = atomicAdd(lctr, 1);        // which slot a token gets does not enter any sum
                if (slot < p.long_slots) { ltok[slot] = t; lcur[slot] = s0; lend[slot] = s1; }
            }
            long_mask |= 1u << i;
            s0 = s1 = 0;
        }
        ce[i] = (uint32_t)s0 | ((uint32_t)s1 << 16);
        sum[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    for (int pass = 0; pass < npass; ++pass) {
        const int lo = first_pick(pass * UP), hi = first_pick(pass * UP + UP);
        // ---------------- (1) products of this wavefront's units of the pass; as a unit's operands are consumed, those
        // of the unit two further on (of this pass, or the first two of the next) are requested
        for (int i = 0; i < UPW; i += 2) {
#pragma unroll
            for (int d = 0; d < 2; ++d) {
                const int unit = unit_of(pass, i + d);
                if (unit < NU) {
                    if (unit / KT2 != w_e) load_w(unit / KT2);          // a wavefront's units of a pass are consecutive
                    compute_unit(buf[d], unit, lo);
                }
                const int nxt = i + d + 2 < UPW ? unit_of(pass, i + d + 2) : unit_of(pass + 1, i + d + 2 - UPW);
                load_rows(buf[d], nxt);
            }
        }
        {   // the weight slice of the next pass's first unit travels while the sums are continued
            const int u0 = unit_of(pass + 1, 0);
            if (u0 < NU && u0 / KT2 != w_e) load_w(u0 / KT2);
        }
        __syncthreads();                                    // the products of the pass are in LDS

        // ---------------- (2) every token's sum continues with its picks in [lo, hi): rounds of up to two entries per
        // token, four tokens at a time (their table entries first, then their rows), until no token has entries left
        bool more = true;
        while (more) {
            more = false;
#pragma unroll
            for (int t4 = 0; t4 < TOK; t4 += 4) {
                int qa[4], qb[4];
                f32x4 va[4], vb[4];
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const int cur = (int)(ce[t4 + x] & 0xffffu);
                    qa[x] = perm[min(cur, NP - 1)];
                    qb[x] = perm[min(cur + 1, NP - 1)];
                }
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const int la = (qa[x] >= lo && qa[x] < hi) ? qa[x] - lo : 0, lb = (qb[x] >= lo && qb[x] < hi) ? qb[x] - lo : 0;
                    va[x] = reinterpret_cast<const f32x4 *>(rows + (size_t)la * kFusedCols)[cc ^ (la & 7)];
                    vb[x] = reinterpret_cast<const f32x4 *>(rows + (size_t)lb * kFusedCols)[cc ^ (lb & 7)];
                }
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const int cur = (int)(ce[t4 + x] & 0xffffu), end = (int)(ce[t4 + x] >> 16);
                    const bool ina = cur < end && qa[x] >= lo && qa[x] < hi;
                    const bool inb = ina && cur + 1 < end && qb[x] >= lo && qb[x] < hi;
                    if (ina) sum[t4 + x] += va[x];
                    if (inb) sum[t4 + x] += vb[x];
                    ce[t4 + x] += (ina ? 1u : 0u) + (inb ? 1u : 0u);
                    more |= inb && cur + 2 < end;
                }
            }
        }

        // ---------------- (2b) long tokens: wavefront (slot mod 8) adds the token's rows of this pass
        {
            const int nlong = min(lctr[0], p.long_slots);
            const int r = lane >> 3, c8 = lane & 7;
            for (int slot = wave; slot < nlong; slot += NWV) {
                int cur = lcur[slot];
                const int end = lend[slot];
                f32x4 part = {0.f, 0.f, 0.f, 0.f};
                bool any = false;
                while (cur < end) {
                    const int at = cur + lane;
                    const int q = perm[min(at, NP - 1)];
                    const bool valid = at < end && q >= lo && q < hi;
                    const int n = __popcll(__ballot(valid));        // a segment is increasing: the valid entries are the first n
                    if (n == 0) break;
                    any = true;
                    f32x4 v[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int qj = __shfl(q, j * 8 + r, kWave);
                        const int lj = (j * 8 + r < n && qj >= lo && qj < hi) ? qj - lo : 0;
                        v[j] = reinterpret_cast<const f32x4 *>(rows + (size_t)lj * kFusedCols)[c8 ^ (lj & 7)];
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (j * 8 + r < n) part += v[j];
                    cur += n;
                    if (n < kWave) break;
                }
                if (any) {
                    // the eight lane groups, added in order r = 0 .. 7; lanes 0..7 then hold the pass's share of the token
                    f32x4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int rr = 0; rr < 8; ++rr) {
#pragma unroll
                        for (int x = 0; x < 4; ++x) tot[x] += __shfl(part[x], rr * 8 + c8, kWave);
                    }
                    if (r == 0) {
                        f32x4 *dst = reinterpret_cast<f32x4 *>(ltot + (size_t)slot * kFusedCols) + c8;
                        f32x4 run = *dst;
                        run += tot;
                        *dst = run;
                    }
                    if (lane == 0) lcur[slot] = cur;
                }
            }
        }
        if (pass + 1 < npass) __syncthreads();              // everybody is done with this pass's rows
    }

    // ---------------- (3) one rounding, every output row written exactly once (tokens nobody picked become zero)
    auto store_row = [&](int t, int col4, const f32x4 &s) {
        char *dst = p.out + (((size_t)b * T + t) * N + c0 + col4 * 4) * ES;
        u32x2 w2;
        w2[0] = pack2<TT>(s[0], s[1]);
        w2[1] = pack2<TT>(s[2], s[3]);
        *reinterpret_cast<u32x2 *>(dst) = w2;
    };
#pragma unroll
    for (int i = 0; i < TOK; ++i) {
        const int t = (tid >> 3) + i * (kFusedThreads >> 3);
        if (t < T && !((long_mask >> i) & 1u)) store_row(t, cc, sum[i]);
    }
    {
        const int nlong = min(lctr[0], p.long_slots);
        for (int slot = wave; slot < nlong; slot += NWV)
            if (lane < 8) store_row(ltok[slot], lane, reinterpret_cast<const f32x4 *>(ltot + (size_t)slot * kFusedCols)[lane]);
    }
}

}  // namespace egs
