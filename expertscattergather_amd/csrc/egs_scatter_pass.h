// GEMM-scatter in ONE kernel for batch elements with thousands of picks: product rows never reach memory.
//
//   out[b, t, c0:c0+32] = sum over the picks (e, k) of token t, in a fixed order, of A[b, e, k, :] . W(e)[:, c0:c0+32]
//
// A workgroup (8 wavefronts) owns one batch element b and one 32-column slice of the output, like the one-kernel
// scatter of small experts (egs_scatter_fused.h), but where that kernel parks the product rows of ALL picks of the
// batch element in LDS, this one works through the picks in passes:
//   - the routing table of b (picks in a stable order by token, built beforehand) is copied into LDS as 16-bit entries;
//   - a pass takes the next `units_per_pass` (expert, 32-pick) units in pick order; a wavefront takes a contiguous
//     share of them (so that its units share an expert and the expert's weight slice is fetched and put into operand
//     order once), multiplies on the matrix cores with the operands coming straight from global memory into
//     registers, two units in flight, and parks the fp32 products in LDS, one 128-byte row per pick;
//   - after a barrier every PAIR of threads continues the sums of its 4 tokens (16 columns per thread, kept in
//     registers for the whole kernel): a token's segment of the table lists its picks in increasing pick number, so
//     the picks of a pass are the next entries of every segment, and the additions happen in table order.  Two
//     threads per token, not eight: what a thread spends per table entry on the entry itself (is it of this pass,
//     where is its row) is then spent 256 times per pass and entry slot, not 1024 times;
//   - the first operands of the next pass are in flight while the sums are continued.
// A token with more than kPassLong picks (skewed routing) is not walked by its two threads: in every pass a whole
// wavefront adds that token's rows of the pass, lane group r (of 8 lanes, 16 bytes of the row each) taking entries r,
// r + 8, ... of each 64-entry chunk of the segment, into per-lane partial sums that live in registers until the end;
// there the eight lane groups are added in order r = 0..7.  The first kPassLongSlots such tokens of a batch element,
// in token order, are treated so; any further ones stay with their threads.  A token with more than kPassHuge picks
// (a quarter of all picks on one token) would still keep one wavefront busy while seven wait: the 64-entry chunks of
// its segment are dealt to the wavefronts round robin (chunk c to wavefront c mod 8), and at the end the wavefronts'
// sums are added in wavefront order.  Which wavefront adds what and the order of every addition depend on the table
// alone: bitwise reproducible, no atomics.
//
// Takes 16-bit elements, reduction length 32 / 64 / 128, output columns a multiple of 32, T <= 1024, and as many
// picks per batch element as the 16-bit table leaves room for beside at least 16 units of rows.
// Replaces, at these sizes, the reference's expert_scatter_kernel (egs/triton_kernels.py:156-247), which adds every
// output element with a global atomic.
#pragma once
#include "egs_device.h"

namespace egs {

constexpr int kPassCols = 32;                                       // output columns per workgroup
constexpr int kPassThreads = 512;                                   // 8 wavefronts
constexpr int kPassTokens = 4;                                      // tokens per pair of threads
constexpr int kPassMaxT = (kPassThreads >> 1) * kPassTokens;        // 1024
constexpr int kPassDepth = 2;                                       // units whose rows a wavefront has in flight
constexpr int kPassLong = 64;                                       // longer segments are summed by a whole wavefront ...
constexpr int kPassLongPerWave = 2;                                 // ... each wavefront keeps the partial sums of so many
constexpr int kPassLongSlots = (kPassThreads / 64) * kPassLongPerWave;     // ... the first 16 of a batch element, in token order
constexpr int kPassHuge = 512;                                      // a segment longer than this is shared by all wavefronts ...
constexpr int kPassHugeSlots = 4;                                   // ... the first so many of a batch element
constexpr int kPassMaxPicks = 32768;                                // 16-bit table entries, with room to spare

struct ScatterPassParams {
    const char *A;              // [B,E,K,R] dense rows
    const char *W;              // [E,R,N] (W_NMAJOR) or [E,N,R]
    char *out;                  // [B,T,N] element type
    const int32_t *tab_seg;     // [B][T+1] routing table: segment offsets ...
    const int32_t *tab_perm;    // [B][E*K]  ... and picks in token order
    int32_t B, T, E, K, N;
    int32_t slices;             // N / kPassCols
    int32_t units_per_pass;     // (expert, 32-pick) units whose product rows are in LDS at a time; a multiple of 16 (2 per wavefront and step)
    int32_t perm_at, seg_at, long_at;   // byte offsets in dynamic LDS (product rows start at 0)
};

// LDS bytes beside the product rows: 16-bit table and the long-token records (counts; token, cursor, end per long slot;
// token, start, end per huge slot)
constexpr int kPassRecordBytes = 16 + 3 * 4 * (kPassLongSlots + kPassHugeSlots);
__host__ __device__ inline size_t scatter_pass_fixed_lds(int T, int NP)
{
    return (((size_t)NP * 2 + 15) & ~(size_t)15) + (((size_t)(T + 1) * 2 + 15) & ~(size_t)15) + kPassRecordBytes;
}

template <class TT, bool W_NMAJOR, int KS>
__global__ __launch_bounds__(kPassThreads) void scatter_pass_kernel(ScatterPassParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_pass[];
    static_assert(TT::ES == 2, "16-bit element types");
    constexpr int ES = 2, VEC = 8, R = 4 * VEC * KS, NWV = kPassThreads / 64, TOK = kPassTokens, LPW = kPassLongPerWave;
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int a = lane & 15, g = lane >> 4;
    // slices of one batch element sit on one XCD (ids congruent modulo 8 share an XCD): its rows come from memory once
    const int block = (int)blockIdx.x, grp = block & 7, idx = block >> 3;
    const int b = (idx / p.slices) * 8 + grp, slice = idx % p.slices;
    if (b >= p.B) return;
    const int c0 = slice * kPassCols;
    const int T = p.T, E = p.E, K = p.K, N = p.N, NP = E * K;
    const int KT2 = (K + 31) >> 5, NU = E * KT2;        // units per expert, units in all
    const int UP = p.units_per_pass, UPW = UP / NWV;    // units per pass, and per pass and wavefront (even)
    const int npass = (NU + UP - 1) / UP;

    float *rows = reinterpret_cast<float *>(smem_pass);
    uint16_t *perm = reinterpret_cast<uint16_t *>(smem_pass + p.perm_at);
    uint16_t *seg = reinterpret_cast<uint16_t *>(smem_pass + p.seg_at);
    int32_t *lctr = reinterpret_cast<int32_t *>(smem_pass + p.long_at);
    int32_t *ltok = lctr + 4, *lcur = ltok + kPassLongSlots, *lend = lcur + kPassLongSlots;
    int32_t *htok = lend + kPassLongSlots, *hbeg = htok + kPassHugeSlots, *hend = hbeg + kPassHugeSlots;

    // first pick of unit u (units are numbered in pick order); NP past the last unit
    auto first_pick = [&](int u) { const int e = u / KT2; return u >= NU ? NP : e * K + (u - e * KT2) * 32; };

    // ---------------- operands of a unit: 32 rows of A (two 16-row tiles), and the weight slice of its expert
    const uint32_t a_base_b = (uint32_t)b * (uint32_t)NP * R * ES;
    struct RowsOp { u32x4 y[2][KS]; };
    RowsOp buf[kPassDepth];
    u32x4 wreg[2 * KS];                                 // weight slice: as it is loaded, then (w_ready) in operand order, in place
    int w_e = -1;                                       // expert whose slice wreg holds (uniform)
    bool w_ready = false;
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
            // [E,R,N]: 8 (reduction) x 2 (columns 2a, 2a+1) blocks, transposed in registers below; raw rows kept here
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const char *wblk = p.W + (((size_t)e * R + ks * 4 * VEC + g * VEC) * N + c0 + 2 * a) * ES;
#pragma unroll
                for (int x = 0; x < 8; ++x)
                    wreg[ks * 2 + (x >> 2)][x & 3] = *reinterpret_cast<const uint32_t *>(wblk + (size_t)x * N * 2);
            }
        }
        w_e = e;
        w_ready = false;
    };
    // the slice in operand order, once per expert (not per unit), in the registers it was loaded into: afterwards the two
    // 16-column tiles of reduction step ks are wreg[ks], wreg[KS + ks] ([E,N,R]) or wreg[2 ks], wreg[2 ks + 1] ([E,R,N])
    auto ready_w = [&]() {
        if (w_ready) return;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if constexpr (!W_NMAJOR) {
                wreg[ks] = lanes_4a_g_to_16g_a(wreg[ks], lane); wreg[KS + ks] = lanes_4a_g_to_16g_a(wreg[KS + ks], lane);
            } else {
                u32x4 t0, t1;
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const uint32_t lo2 = wreg[ks * 2 + (pp >> 1)][(pp & 1) * 2], hi2 = wreg[ks * 2 + (pp >> 1)][(pp & 1) * 2 + 1];
                    t0[pp] = __builtin_amdgcn_perm(hi2, lo2, 0x05040100u);     // column 2a   of rows 2pp, 2pp+1
                    t1[pp] = __builtin_amdgcn_perm(hi2, lo2, 0x07060302u);     // column 2a+1
                }
                wreg[ks * 2] = t0; wreg[ks * 2 + 1] = t1;
            }
        }
        w_ready = true;
    };
    // products of a unit into LDS rows [first pick of the unit - lo ...)
    auto compute_unit = [&](const RowsOp &u, int unit, int lo) {
        const int e = unit / KT2, rp = unit - e * KT2;
        f32x4 acc[2][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) { acc[h][0] = f32x4{0.f, 0.f, 0.f, 0.f}; acc[h][1] = f32x4{0.f, 0.f, 0.f, 0.f}; }
        // the rows' chunks go to operand order two reduction steps at a time: enough cross-lane moves in flight to hide
        // their latency, few enough registers
        constexpr int KB = KS >= 2 ? 2 : 1;
#pragma unroll
        for (int k0 = 0; k0 < KS; k0 += KB) {
            u32x4 yf[2][KB];
#pragma unroll
            for (int kk = 0; kk < KB; ++kk)
#pragma unroll
                for (int h = 0; h < 2; ++h) yf[h][kk] = lanes_4a_g_to_16g_a(u.y[h][k0 + kk], lane);
#pragma unroll
            for (int kk = 0; kk < KB; ++kk)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    mma_chunk<TT>(acc[h][0], wreg[W_NMAJOR ? 2 * (k0 + kk) : k0 + kk], yf[h][kk]);
                    mma_chunk<TT>(acc[h][1], wreg[W_NMAJOR ? 2 * (k0 + kk) + 1 : KS + k0 + kk], yf[h][kk]);
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
                f32x4 *row = reinterpret_cast<f32x4 *>(rows + (size_t)q * kPassCols);
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
        for (int s0 = 0; s0 < NP; s0 += 8 * kPassThreads) {
            int32_t v[8];
#pragma unroll
            for (int x = 0; x < 8; ++x) v[x] = gperm[min(s0 + x * kPassThreads + tid, NP - 1)];
            if (s0 == 0) {
                const int u0 = unit_of(0, 0);
                if (u0 < NU) load_w(u0 / KT2);
#pragma unroll
                for (int dd = 0; dd < kPassDepth; ++dd) load_rows(buf[dd], u0 + dd);
            }
#pragma unroll
            for (int x = 0; x < 8; ++x)
                if (s0 + x * kPassThreads + tid < NP) perm[s0 + x * kPassThreads + tid] = (uint16_t)min(max(v[x], 0), NP - 1);
        }
        for (int t = tid; t <= T; t += kPassThreads) seg[t] = (uint16_t)min(max(gseg[t], 0), NP);
    }
    __syncthreads();

    // ---------------- long tokens get slots in token order: flags (in the rows area, free until the first products),
    // then one wavefront numbers them
    {
        int32_t *flag = reinterpret_cast<int32_t *>(rows);
        __syncthreads();
        if (wave == 0) {
            int base = 0, hbase = 0;
            for (int t0 = 0; t0 < T; t0 += kWave) {
                const int t = t0 + lane;
                const int len = t < T ? (int)seg[t + 1] - (int)seg[t] : 0;
                // huge tokens first come first served (in token order) up to kPassHugeSlots, the others that are long likewise
                const bool hf0 = len > kPassHuge;
                const uint64_t hbal = __ballot(hf0);
                const int hslot = hbase + __popcll(hbal & (lane == 0 ? 0ull : (~0ull >> (64 - lane))));
                const bool hf = hf0 && hslot < kPassHugeSlots;
                const bool f = len > kPassLong && !hf;
                const uint64_t bal = __ballot(f);
                const int slot = base + __popcll(bal & (lane == 0 ? 0ull : (~0ull >> (64 - lane))));
                if (t < T) flag[t] = hf ? kPassLongSlots + hslot : ((f && slot < kPassLongSlots) ? slot : -1);
                if (hf) { htok[hslot] = t; hbeg[hslot] = (int)seg[t]; hend[hslot] = (int)seg[t + 1]; }
                if (f && slot < kPassLongSlots) { ltok[slot] = t; lcur[slot] = (int)seg[t]; lend[slot] = (int)seg[t + 1]; }
                base += __popcll(bal);
                hbase += __popcll(hbal);
            }
            if (lane == 0) { lctr[0] = min(base, kPassLongSlots); lctr[1] = min(hbase, kPassHugeSlots); }
        }
        __syncthreads();
    }

    // ---------------- per-thread state of the sums: 2 threads x 16 columns per token, 4 tokens per thread
    const int half = tid & 1;                           // which 16 columns (64 bytes) of a row
    uint32_t ce[TOK];               // cursor | end << 16 into the token's segment
    f32x4 sum[TOK][4];
    uint32_t long_mask = 0;         // tokens of this thread that a wavefront sums instead
#pragma unroll
    for (int i = 0; i < TOK; ++i) {
        const int t = (tid >> 1) + i * (kPassThreads >> 1);
        int s0 = t < T ? (int)seg[t] : 0, s1 = t < T ? (int)seg[t + 1] : 0;
        if (t < T && reinterpret_cast<const int32_t *>(rows)[t] >= 0) { long_mask |= 1u << i; s0 = s1 = 0; }
        ce[i] = (uint32_t)s0 | ((uint32_t)s1 << 16);
#pragma unroll
        for (int c = 0; c < 4; ++c) sum[i][c] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const int nlong = min(lctr[0], kPassLongSlots), nhuge = min(lctr[1], kPassHugeSlots);
    // long tokens of this wavefront: slots wave, wave + 8, ...; lane (r, c8) keeps a partial sum of chunk c8 of the row
    const int lr = lane >> 3, c8 = lane & 7;
    f32x4 lpart[LPW];
#pragma unroll
    for (int s = 0; s < LPW; ++s) lpart[s] = f32x4{0.f, 0.f, 0.f, 0.f};
    // huge tokens: this wavefront's share of every one of them, and the next 64-entry chunk of the segment it looks at
    f32x4 hpart[kPassHugeSlots];
    int hck[kPassHugeSlots];
#pragma unroll
    for (int s = 0; s < kPassHugeSlots; ++s) { hpart[s] = f32x4{0.f, 0.f, 0.f, 0.f}; hck[s] = wave; }
    __syncthreads();                    // the flags are read: the rows area may take products

    for (int pass = 0; pass < npass; ++pass) {
        const int lo = first_pick(pass * UP), hi = first_pick(pass * UP + UP);
        // ---------------- (1) products of this wavefront's units of the pass; as a unit's operands are consumed, those
        // of the unit two further on (of this pass, or one of the first two of the next) are requested
        for (int i = 0; i < UPW; i += kPassDepth) {
#pragma unroll
            for (int d = 0; d < kPassDepth; ++d) {
                const int unit = unit_of(pass, i + d);
                if (unit < NU) {
                    if (unit / KT2 != w_e) load_w(unit / KT2);          // a wavefront's units of a pass are consecutive
                    ready_w();
                    compute_unit(buf[d], unit, lo);
                }
                const int nxt = i + d + kPassDepth < UPW ? unit_of(pass, i + d + kPassDepth) : unit_of(pass + 1, i + d + kPassDepth - UPW);
                load_rows(buf[d], nxt);
            }
        }
        {   // the weight slice of the next pass's first unit travels while the sums are continued
            const int u0 = unit_of(pass + 1, 0);
            if (u0 < NU && u0 / KT2 != w_e) load_w(u0 / KT2);
        }
        __syncthreads();                                    // the products of the pass are in LDS

        // ---------------- (2) every token's sum continues with its picks in [lo, hi): up to four entries per token in
        // straight-line code (the table entries first, then the rows); a token with more entries in this pass
        // finishes in a loop of its own
        constexpr int EN = 4;
        auto in_pass = [&](int q) { return q >= lo && q < hi; };
        auto add_row = [&](f32x4 (&s)[4], int q) {
            const int l = q - lo;
            const f32x4 *row = reinterpret_cast<const f32x4 *>(rows + (size_t)l * kPassCols);
#pragma unroll
            for (int c = 0; c < 4; ++c) s[c] += row[(half * 4 + c) ^ (l & 7)];
        };
        uint32_t left = 0;              // tokens with all EN entries taken and more to look at
#pragma unroll
        for (int i = 0; i < TOK; ++i) {
            const int cur = (int)(ce[i] & 0xffffu), end = (int)(ce[i] >> 16);
            int q[EN];
#pragma unroll
            for (int n = 0; n < EN; ++n) q[n] = perm[min(cur + n, NP - 1)];
            bool in = true;
            uint32_t took = 0;
#pragma unroll
            for (int n = 0; n < EN; ++n) {
                in = in && cur + n < end && in_pass(q[n]);
                if (in) { add_row(sum[i], q[n]); ++took; }
            }
            ce[i] += took;
            if (in && cur + EN < end) left |= 1u << i;
        }
        if (__ballot(left != 0) != 0) {
#pragma unroll
            for (int i = 0; i < TOK; ++i) {
                if ((left >> i) & 1u) {
                    int cur = (int)(ce[i] & 0xffffu);
                    const int end = (int)(ce[i] >> 16);
                    while (cur < end) {
                        const int q0 = perm[cur];
                        if (!in_pass(q0)) break;
                        add_row(sum[i], q0);
                        ++cur;
                    }
                    ce[i] = (uint32_t)cur | ((uint32_t)end << 16);
                }
            }
        }

        // ---------------- (2b) long tokens: this wavefront adds the rows of the pass of its slots; lane group r takes the
        // entries r, r + 8, ... of every 64-entry chunk of the segment (entries first, then their rows)
#pragma unroll
        for (int s = 0; s < LPW; ++s) {
            const int slot = wave + s * NWV;
            if (slot < nlong) {
                int cur = lcur[slot];
                const int end = lend[slot];
                const int cur0 = cur;
                while (cur < end) {
                    int q[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) q[j] = perm[min(cur + j * 8 + lr, NP - 1)];
                    int n = 0;
#pragma unroll
                    for (int j0 = 0; j0 < 8; j0 += 4) {         // four rows in flight at a time
                        f32x4 v[4];
                        bool ok[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            ok[j] = cur + (j0 + j) * 8 + lr < end && in_pass(q[j0 + j]);
                            const int l = ok[j] ? q[j0 + j] - lo : 0;
                            v[j] = reinterpret_cast<const f32x4 *>(rows + (size_t)l * kPassCols)[c8 ^ (l & 7)];
                            n += __popcll(__ballot(ok[j] && c8 == 0));  // a segment is increasing: the entries of the pass come first
                        }
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (ok[j]) lpart[s] += v[j];
                    }
                    cur += n;
                    if (n < kWave) break;
                }
                if (lane == 0 && cur != cur0) lcur[slot] = cur;
            }
        }
        // ---------------- (2c) huge tokens: chunk c of the segment belongs to wavefront c mod 8; a chunk is left when none of
        // its entries is of a later pass
#pragma unroll
        for (int s = 0; s < kPassHugeSlots; ++s) {
            if (s < nhuge) {
                const int beg = hbeg[s], end = hend[s];
                while (beg + hck[s] * kWave < end) {
                    const int pos0 = beg + hck[s] * kWave;
                    int q[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) q[j] = perm[min(pos0 + j * 8 + lr, NP - 1)];
                    bool later = false;
#pragma unroll
                    for (int j0 = 0; j0 < 8; j0 += 4) {         // four rows in flight at a time
                        f32x4 v[4];
                        bool ok[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const bool there = pos0 + (j0 + j) * 8 + lr < end;
                            ok[j] = there && in_pass(q[j0 + j]);
                            later = later || (there && q[j0 + j] >= hi);
                            const int l = ok[j] ? q[j0 + j] - lo : 0;
                            v[j] = reinterpret_cast<const f32x4 *>(rows + (size_t)l * kPassCols)[c8 ^ (l & 7)];
                        }
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (ok[j]) hpart[s] += v[j];
                    }
                    if (__ballot(later) != 0) break;
                    hck[s] += NWV;
                }
            }
        }
        if (pass + 1 < npass) __syncthreads();              // everybody is done with this pass's rows
    }

    // ---------------- (3) one rounding, every output row written exactly once (tokens nobody picked become zero)
    int tid_late = tid;                 // opaque: keeps the output addresses from being formed (and held) before the passes
    asm volatile("" : "+v"(tid_late));
#pragma unroll
    for (int i = 0; i < TOK; ++i) {
        const int t = (tid_late >> 1) + i * (kPassThreads >> 1);
        if (t < T && !((long_mask >> i) & 1u)) {
            char *dst = p.out + (((size_t)b * T + t) * N + c0 + (tid_late & 1) * 16) * ES;
            u32x4 w0, w1;
            w0[0] = pack2<TT>(sum[i][0][0], sum[i][0][1]); w0[1] = pack2<TT>(sum[i][0][2], sum[i][0][3]);
            w0[2] = pack2<TT>(sum[i][1][0], sum[i][1][1]); w0[3] = pack2<TT>(sum[i][1][2], sum[i][1][3]);
            w1[0] = pack2<TT>(sum[i][2][0], sum[i][2][1]); w1[1] = pack2<TT>(sum[i][2][2], sum[i][2][3]);
            w1[2] = pack2<TT>(sum[i][3][0], sum[i][3][1]); w1[3] = pack2<TT>(sum[i][3][2], sum[i][3][3]);
            reinterpret_cast<u32x4 *>(dst)[0] = w0;
            reinterpret_cast<u32x4 *>(dst)[1] = w1;
        }
    }
    // huge tokens: every wavefront adds its eight lane groups in order r = 0 .. 7 and leaves the result in LDS (the rows
    // area is free now); wavefront s then adds the eight wavefronts' results in wavefront order and stores the row
    if (nhuge > 0) {
        __syncthreads();
        f32x4 *hsum = reinterpret_cast<f32x4 *>(rows);      // [huge slot][wavefront][8 chunks]
#pragma unroll
        for (int s = 0; s < kPassHugeSlots; ++s) {
            if (s < nhuge) {
                f32x4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int rr = 0; rr < 8; ++rr)
#pragma unroll
                    for (int x = 0; x < 4; ++x) tot[x] += __shfl(hpart[s][x], rr * 8 + c8, kWave);
                if (lr == 0) hsum[(s * NWV + wave) * 8 + c8] = tot;
            }
        }
        __syncthreads();
        if (wave < nhuge && lane < 8) {
            f32x4 tot = hsum[(wave * NWV) * 8 + lane];
#pragma unroll
            for (int w = 1; w < NWV; ++w) tot += hsum[(wave * NWV + w) * 8 + lane];
            char *dst = p.out + (((size_t)b * T + htok[wave]) * N + c0 + lane * 4) * ES;
            u32x2 w2;
            w2[0] = pack2<TT>(tot[0], tot[1]);
            w2[1] = pack2<TT>(tot[2], tot[3]);
            *reinterpret_cast<u32x2 *>(dst) = w2;
        }
    }
    // long tokens: the eight lane groups of a slot's partial sums, added in order r = 0 .. 7; lanes 0 .. 7 store the row
#pragma unroll
    for (int s = 0; s < LPW; ++s) {
        const int slot = wave + s * NWV;
        if (slot < nlong) {
            f32x4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int rr = 0; rr < 8; ++rr)
#pragma unroll
                for (int x = 0; x < 4; ++x) tot[x] += __shfl(lpart[s][x], rr * 8 + c8, kWave);
            if (lr == 0) {
                char *dst = p.out + (((size_t)b * T + ltok[slot]) * N + c0 + c8 * 4) * ES;
                u32x2 w2;
                w2[0] = pack2<TT>(tot[0], tot[1]);
                w2[1] = pack2<TT>(tot[2], tot[3]);
                *reinterpret_cast<u32x2 *>(dst) = w2;
            }
        }
    }
}

}  // namespace egs
