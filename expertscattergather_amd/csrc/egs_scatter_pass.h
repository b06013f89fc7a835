// GEMM-scatter in ONE kernel for batch elements with thousands of picks: product rows never reach memory, and there
// is no routing table in memory either.
//
//   out[b, t, c0:c0+32] = sum over the picks (e, k) of token t, in a fixed order, of A[b, e, k, :] . W(e)[:, c0:c0+32]
//
// A workgroup (8 wavefronts) owns one batch element b and one 32-column slice of the output, like the one-kernel
// scatter of small experts (egs_scatter_fused.h), but where that kernel parks the product rows of ALL picks of the
// batch element in LDS, this one works through the picks in passes of `units_per_pass` (expert, 32-pick) units:
//   (a) the picks of the pass are sorted, stably, by the 16-token BLOCK their token lies in (a counting sort over at
//       most 64 blocks: the tokens come straight from Ind; ranks inside a wavefront by ballots, one small histogram
//       per wavefront in LDS, every wavefront adds the histograms up for itself); an entry is 32 bits: where the pick's
//       product row lies in LDS, and its token's place in the block; a block's list is filled up to a multiple of 8
//       with entries that point at a row of zeros, so that the sums need no bounds inside a list;
//   (b) every wavefront multiplies its contiguous share of the units on the matrix cores (its units share an expert,
//       whose weight slice is fetched and put into operand order once; rows straight from global memory, two units in
//       flight; the first operands of the next pass travel during (c)) and parks the fp32 products in LDS, one
//       128-byte row per pick;
//   (c) the per-token sums are a matrix product as well: out(block)[token, column] += S^T . P, where P are the
//       block's product rows of this pass and S[entry, token] is 1 where the entry's token is that token.  Wavefront
//       w owns the token blocks 8 w .. 8 w + 7: for each it walks the block's entries four at a time (lane group g
//       takes the g-th quarter of them) and issues v_mfma_f32_16x16x4_f32 with the product values as one operand and
//       the selector (1.0 or 0.0, exact) as the other; the 16 x 32 sums of a block are two accumulator tiles that stay
//       in the wavefront's registers for the whole kernel.  Skewed routing: a hot token only makes its block's list
//       longer, but one wavefront would then sum while seven wait.  A census of the batch element's picks at the start
//       names up to two blocks that hold an eighth or more of all picks; their lists are put behind all others, every
//       wavefront sums an eighth of each into two tiles of its own, and at the end the eight wavefronts' tiles are added
//       in wavefront order.
// Which entry is added where, and in which matrix instruction, depends on Ind alone: bitwise reproducible, no atomics.
// A selector of 0.0 would turn a product that is not finite (an overflow, a NaN in the input) into NaNs for the other
// tokens of its block; a pass in which any product is not finite therefore takes its sums with plain selects and
// additions instead (same lists, same owners, slower), so such a value reaches its own token only, as in the reference.
//
// Takes 16-bit elements, reduction length 32 / 64 / 128, output columns a multiple of 32, T <= 1024.
// Replaces, at these sizes, the reference's expert_scatter_kernel (egs/triton_kernels.py:156-247), which adds every
// output element with a global atomic.
#pragma once
#include "egs_device.h"

namespace egs {

constexpr int kPassCols = 32;                                       // output columns per workgroup
constexpr int kPassThreads = 512;                                   // 8 wavefronts
constexpr int kPassWaves = kPassThreads / 64;
constexpr int kPassMaxT = 1024;                                     // 64 token blocks of 16, 8 per wavefront
constexpr int kPassBlocks = kPassMaxT / 16;
constexpr int kPassOwn = kPassBlocks / kPassWaves;                  // token blocks whose sums a wavefront keeps
constexpr int kPassDepth = 2;                                       // units whose rows a wavefront has in flight
constexpr int kPassMaxUnits = 32;                                   // units per pass at most: 1024 picks, 128 KB of rows
constexpr int kPassRounds = kPassMaxUnits * 32 / kPassThreads;      // picks per thread and pass in the sort
constexpr int kPassListPad = 8;                                     // a block's list is a multiple of so many entries
constexpr int kPassShared = 1;                                      // blocks whose lists all wavefronts sum together

struct ScatterPassParams {
    const char *A;              // [B,E,K,R] dense rows
    const char *W;              // [E,R,N] (W_NMAJOR) or [E,N,R]
    const void *Ind;            // [B,E,K]
    char *out;                  // [B,T,N] element type
    int32_t B, T, E, K, N;
    int32_t ind_dtype;
    int32_t slices;             // N / kPassCols
    int32_t units_per_pass;     // 16 or 32: (expert, 32-pick) units whose product rows are in LDS at a time
};

// entries of the lists of a pass at most: its picks, the lists' padding, and what a read one step ahead may touch
__host__ __device__ constexpr int scatter_pass_list_entries(int units_per_pass)
{
    return units_per_pass * 32 + kPassBlocks * (kPassListPad - 1) + 64;
}
// LDS: product rows of a pass, one row of zeros (what a list's padding points at), the lists, one histogram
// per wavefront, the blocks' offsets into the lists, a flag
__host__ __device__ inline size_t scatter_pass_lds(int units_per_pass)
{
    return (size_t)units_per_pass * 32 * kPassCols * 4 + kPassCols * 4 +
           (((size_t)scatter_pass_list_entries(units_per_pass) * 4 + 15) & ~(size_t)15) +
           (size_t)kPassWaves * kPassBlocks * 4 + (kPassBlocks + 8) * 4 + 16 +
           (size_t)kPassShared * kPassWaves * 2 * 64 * 16;
}

// inclusive prefix sum over the 64 lanes of a wavefront: shifts inside the rows of 16 lanes, then the last lane of a row
// added to the rows after it
__device__ __forceinline__ int wave_prefix_sum(int x)
{
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, true);      // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, true);      // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, true);      // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, true);      // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);     // row_bcast:15 into rows 1 and 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);     // row_bcast:31 into rows 2 and 3
    return x;
}

template <class TT, bool W_NMAJOR, int KS>
__global__ __launch_bounds__(kPassThreads) void scatter_pass_kernel(ScatterPassParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_pass[];
    static_assert(TT::ES == 2, "16-bit element types");
    constexpr int ES = 2, VEC = 8, R = 4 * VEC * KS, NWV = kPassWaves;
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
    const int PW = UP * 32 / NWV;                       // picks of a pass whose entries a wavefront ranks: 64 or 128

    float *rows = reinterpret_cast<float *>(smem_pass);
    float *zrow = rows + (size_t)UP * 32 * kPassCols;
    uint32_t *sorted = reinterpret_cast<uint32_t *>(zrow + kPassCols);
    const int list_cap = scatter_pass_list_entries(UP);
    int32_t *hist = reinterpret_cast<int32_t *>(reinterpret_cast<char *>(sorted) + (((size_t)list_cap * 4 + 15) & ~(size_t)15));  // [wavefront][block]
    int32_t *boff = hist + NWV * kPassBlocks;                                    // [blocks + 1]
    int32_t *flag = boff + kPassBlocks + 8;           // (behind the blocks' starts: start and length of each shared list)
    f32x4 *shared_part = reinterpret_cast<f32x4 *>(flag + 4);           // [shared block][wavefront][half][lane]
    const uint32_t null_entry = (uint32_t)UP * 32u * (kPassCols * 4);   // the row of zeros, token 0 of the block

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
        // a product that is not finite sends the pass's sums down the path without multiplications
        bool odd = false;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int ct = 0; ct < 2; ++ct)
#pragma unroll
                for (int r = 0; r < 4; ++r) odd = odd || !__builtin_isfinite(acc[h][ct][r]);
        if (odd) flag[0] = 1;
        // lane (a, g) holds, for pick k = 32 rp + 16 h + a, slice columns
        //   [E,N,R]: 16 ct + 4 g + r                   -> chunk 4 ct + g of the row
        //   [E,R,N]: 2 (4 g + r) + ct = 8 g + 2 r + ct -> chunks 2 g, 2 g + 1 after interleaving the two tiles
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = rp * 32 + h * 16 + a;
            if (k < K) {
                const int q = e * K + k - lo;
                f32x4 *row = reinterpret_cast<f32x4 *>(rows + (size_t)q * kPassCols);
                // the four 16-byte chunks of each 64-byte half of a row are XORed with the row number's low two bits
                if constexpr (!W_NMAJOR) {
                    row[g ^ (q & 3)] = acc[h][0];
                    row[4 + (g ^ (q & 3))] = acc[h][1];
                } else {
                    row[(g & 2) * 2 + (((2 * g) & 3) ^ (q & 3))] = f32x4{acc[h][0][0], acc[h][1][0], acc[h][0][1], acc[h][1][1]};
                    row[(g & 2) * 2 + (((2 * g + 1) & 3) ^ (q & 3))] = f32x4{acc[h][0][2], acc[h][1][2], acc[h][0][3], acc[h][1][3]};
                }
            }
        }
    };
    auto unit_of = [&](int pass, int i) { return pass * UP + wave * UPW + i; };

    // tokens of the picks this thread ranks in a pass: local rows wave * PW + 64 r + lane (-1: no such pick, or a token
    // outside [0, T), which contributes nothing)
    int tok[kPassRounds];
    auto load_tokens = [&](int pass) {
        const int lo = first_pick(pass * UP), hi = first_pick(pass * UP + UP);
#pragma unroll
        for (int r = 0; r < kPassRounds; ++r) {
            const int l = wave * PW + r * 64 + lane;
            tok[r] = (r * 64 < PW && lo + l < hi) ? load_token(p.Ind, p.ind_dtype, (int64_t)b * NP + lo + l, T) : -1;
        }
    };

    // ---------------- the sums: two accumulator tiles (16 tokens x 16 columns each) per owned token block
    f32x4 sum[kPassOwn][2];
#pragma unroll
    for (int i = 0; i < kPassOwn; ++i) { sum[i][0] = f32x4{0.f, 0.f, 0.f, 0.f}; sum[i][1] = f32x4{0.f, 0.f, 0.f, 0.f}; }

    if (tid < kPassCols) zrow[tid] = 0.f;
    // ---------------- census: picks per token block over the whole batch element (counts, so the order of the additions
    // does not matter), and from it the blocks that all wavefronts will sum together: those with an eighth of the picks
    // or more, the first kPassShared of them in block order
    int hb[kPassShared];                                // uniform; -1: no such block
    {
        if (tid < kPassBlocks) hist[tid] = 0;
        __syncthreads();
        for (int i = tid; i < NP; i += kPassThreads) {
            const int t = load_token(p.Ind, p.ind_dtype, (int64_t)b * NP + i, T);
            if (t >= 0) atomicAdd(&hist[t >> 4], 1);
        }
        __syncthreads();
        const int c = hist[lane];
        uint64_t many = __ballot(c >= 64 && (int64_t)c * 8 >= NP);
#pragma unroll
        for (int x = 0; x < kPassShared; ++x) {
            hb[x] = many != 0 ? (int)__builtin_ctzll(many) : -1;
            many &= many - 1;
        }
        __syncthreads();                                // the histogram rows are cleared again below
    }
    // this wavefront's share of the shared blocks' sums lives in LDS between the passes
#pragma unroll
    for (int x = 0; x < kPassShared; ++x) {
        shared_part[((x * NWV + wave) * 2 + 0) * 64 + lane] = f32x4{0.f, 0.f, 0.f, 0.f};
        shared_part[((x * NWV + wave) * 2 + 1) * 64 + lane] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    load_tokens(0);
    {
        const int u0 = unit_of(0, 0);
        if (u0 < NU) load_w(u0 / KT2);
#pragma unroll
        for (int dd = 0; dd < kPassDepth; ++dd) load_rows(buf[dd], u0 + dd);
    }

    for (int pass = 0; pass < npass; ++pass) {
        const int lo = first_pick(pass * UP);
        // ---------------- (a) entries of the pass in block order.  Ranks inside the wavefront: lanes with the same block
        // find each other with one ballot per bit of the block number; the wavefront's count so far comes from its
        // histogram row, which the first lane of each group of equals moves on.
        hist[tid] = 0;                                  // thread tid clears an entry of its own wavefront's row
        if (tid == 0) flag[0] = 0;
        for (int x = tid; x < list_cap; x += kPassThreads) sorted[x] = null_entry;     // what is not a pick selects the row of zeros
        int rank[kPassRounds];
#pragma unroll
        for (int r = 0; r < kPassRounds; ++r) {
            const bool live = tok[r] >= 0;
            const int key = live ? (tok[r] >> 4) : 0;
            uint64_t peers = __ballot(live);
#pragma unroll
            for (int bit = 0; bit < 6; ++bit) {
                const bool one = (key >> bit) & 1;
                const uint64_t set = __ballot(live && one);
                peers &= one ? set : ~set;
            }
            const int below = __popcll(peers & ((1ull << lane) - 1ull));
            int32_t *mine = hist + wave * kPassBlocks + key;
            const int before = live ? *mine : 0;
            if (live && below == 0) *mine = before + __popcll(peers);
            rank[r] = before + below;
        }
        __syncthreads();
        {
            // block `lane`: its entries start where the blocks before it end; inside, wavefront by wavefront.  Every
            // wavefront adds the histograms up for itself (no second barrier) and keeps, in lane `block`, where its own
            // entries of that block start; the first wavefront leaves the blocks' starts for the sums
            int tot = 0, before_me = 0;
#pragma unroll
            for (int w = 0; w < NWV; ++w) {
                const int c = hist[w * kPassBlocks + lane];
                before_me += w < wave ? c : 0;
                tot += c;
            }
            const int len = (tot + kPassListPad - 1) & ~(kPassListPad - 1);
            bool is_shared = false;
#pragma unroll
            for (int x = 0; x < kPassShared; ++x) is_shared = is_shared || lane == hb[x];
            const int padded = is_shared ? 0 : len;         // a shared block's list is not among the others
            const int incl = wave_prefix_sum(padded);
            int start = incl - padded + before_me;
            int behind = __builtin_amdgcn_readlane(incl, 63);      // where the shared lists begin
#pragma unroll
            for (int x = 0; x < kPassShared; ++x) {
                if (hb[x] >= 0) {                           // uniform
                    const int ln = __builtin_amdgcn_readlane(len, hb[x]);
                    if (lane == hb[x]) start = behind + before_me;
                    if (wave == 0 && lane == 0) { boff[kPassBlocks + 1 + 2 * x] = behind; boff[kPassBlocks + 2 + 2 * x] = ln; }
                    behind += ln;
                }
            }
            if (wave == 0) {
                boff[lane] = incl - padded;
                if (lane == 63) boff[kPassBlocks] = incl;
            }
#pragma unroll
            for (int r = 0; r < kPassRounds; ++r) {
                const int at = __shfl(start, tok[r] >= 0 ? (tok[r] >> 4) : 0, kWave) + rank[r];
                if (tok[r] >= 0) {
                    const uint32_t l = (uint32_t)(wave * PW + r * 64 + lane);
                    sorted[at] = (l << 7) | ((l & 3u) << 4) | (uint32_t)(tok[r] & 15);
                }
            }
        }
        if (pass + 1 < npass) load_tokens(pass + 1);     // they travel during the products

        // ---------------- (b) products of this wavefront's units of the pass; as a unit's operands are consumed, those
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
                if (i + d + kPassDepth < UPW) load_rows(buf[d], unit_of(pass, i + d + kPassDepth));
            }
        }
        w_e = -1;                                           // the slice's registers are free for the sums
        __syncthreads();                                    // products and entries of the pass are in LDS

        // ---------------- (c) sums.  One copy of the code serves the eight lists of the wavefront's own blocks and its eighth of
        // each shared list: a list's sums of the pass are formed in two tiles of their own and then added to the block's
        // running sums (registers, picked by name) or to the wavefront's tiles of the shared block (LDS).
        {
            const bool plain = flag[0] != 0;                // uniform: some product of the pass is not finite
            const int bl = boff[wave * kPassOwn + min(lane, kPassOwn)];
            const char *rows_b = reinterpret_cast<const char *>(rows);
            const uint32_t *mine = sorted + 2 * g;
            const uint32_t lane4 = (uint32_t)a * 4u;
            // An entry's upper bits are the byte offset of its row with the row's chunk key in place: XORed with 4 a they
            // give the address of column a of the row, and column 16 + a lies 64 bytes further.  After the matrix
            // instruction lane (a, g) holds, for token a of the block, columns 4 g .. 4 g + 3 of each half.
            struct Pair { float x[4], sel[2]; };
            auto request = [&](const u32x2 e, Pair &pr) {
                const float *r0 = reinterpret_cast<const float *>(rows_b + ((e[0] & ~15u) ^ lane4));
                const float *r1 = reinterpret_cast<const float *>(rows_b + ((e[1] & ~15u) ^ lane4));
                pr.sel[0] = (int)(e[0] & 15u) == a ? 1.f : 0.f;
                pr.sel[1] = (int)(e[1] & 15u) == a ? 1.f : 0.f;
                pr.x[0] = r0[0]; pr.x[1] = r0[16]; pr.x[2] = r1[0]; pr.x[3] = r1[16];
            };
            // The rows of the next step are requested, and the entries of the step after it read, before the matrix
            // instructions of a step are issued; the own blocks' lists lie one behind the other, so what was requested
            // past the end of one list is the beginning of the next (`primed`: the entry `cur` was requested for).
            Pair cur;
            u32x2 ahead = {0u, 0u};
            int primed = -1;
#pragma unroll 1
            for (int k = 0; k < kPassOwn + kPassShared; ++k) {
                int at, upto;                               // uniform: the entries [at, upto) in steps of eight
                if (k < kPassOwn) {
                    at = __builtin_amdgcn_readlane(bl, 0); upto = at;
#pragma unroll
                    for (int x = 0; x < kPassOwn; ++x)
                        if (k == x) { at = __builtin_amdgcn_readlane(bl, x); upto = __builtin_amdgcn_readlane(bl, x + 1); }
                } else {
                    const int x = k - kPassOwn;
                    bool have = false;
#pragma unroll
                    for (int y = 0; y < kPassShared; ++y) have = have || (x == y && hb[y] >= 0);
                    if (!have) break;
                    const int h0 = __builtin_amdgcn_readfirstlane(boff[kPassBlocks + 1 + 2 * x]);
                    const int steps = __builtin_amdgcn_readfirstlane(boff[kPassBlocks + 2 + 2 * x]) >> 3;
                    const int share = (steps + NWV - 1) / NWV;
                    at = h0 + 8 * min(wave * share, steps);
                    upto = h0 + 8 * min(wave * share + share, steps);
                }
                if (at >= upto) continue;
                f32x4 part0 = {0.f, 0.f, 0.f, 0.f}, part1 = {0.f, 0.f, 0.f, 0.f};
                if (!plain) {
                    if (at != primed) {                         // uniform
                        request(*reinterpret_cast<const u32x2 *>(mine + at), cur);
                        ahead = *reinterpret_cast<const u32x2 *>(mine + at + 8);
                    }
#pragma unroll 1
                    for (; at < upto; at += 8) {
                        Pair nxt;
                        request(ahead, nxt);
                        ahead = *reinterpret_cast<const u32x2 *>(mine + at + 16);
                        __builtin_amdgcn_sched_barrier(0);
                        part0 = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.x[0], cur.sel[0], part0, 0, 0, 0);
                        part1 = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.x[1], cur.sel[0], part1, 0, 0, 0);
                        part0 = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.x[2], cur.sel[1], part0, 0, 0, 0);
                        part1 = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.x[3], cur.sel[1], part1, 0, 0, 0);
                        __builtin_amdgcn_sched_barrier(0);
                        cur = nxt;
                    }
                    primed = at;
                } else {
                    // one entry at a time, in list order; a value is added where its token is, and nowhere else
#pragma unroll 1
                    for (int j = at; j < upto; ++j) {
                        const uint32_t ent = sorted[j];
                        const int l = (int)(ent >> 7);
                        const f32x4 *row = reinterpret_cast<const f32x4 *>(rows_b + ((size_t)l << 7));
                        const f32x4 u0 = row[g ^ (l & 3)], u1 = row[4 + (g ^ (l & 3))];
                        if ((int)(ent & 15u) == a) { part0 += u0; part1 += u1; }
                    }
                }
#pragma unroll
                for (int x = 0; x < kPassOwn; ++x)
                    if (k == x) { sum[x][0] += part0; sum[x][1] += part1; }
#pragma unroll
                for (int x = 0; x < kPassShared; ++x)
                    if (k == kPassOwn + x) {
                        shared_part[((x * NWV + wave) * 2 + 0) * 64 + lane] += part0;
                        shared_part[((x * NWV + wave) * 2 + 1) * 64 + lane] += part1;
                    }
            }
        }
        {   // the first operands of the next pass travel while its picks are sorted
            const int u0 = unit_of(pass + 1, 0);
            if (u0 < NU && u0 / KT2 != w_e) load_w(u0 / KT2);
#pragma unroll
            for (int dd = 0; dd < kPassDepth; ++dd) load_rows(buf[dd], u0 + dd);
        }
        if (pass + 1 < npass) __syncthreads();              // everybody is done with this pass's rows and lists
    }

    // ---------------- one rounding, every output row written exactly once (tokens nobody picked become zero):
    // lane (a, g) stores, for token 16 tb + a, columns 4 g .. 4 g + 3 of each half
    auto store_block = [&](int tb, const f32x4 &s0, const f32x4 &s1) {
        const int t = tb * 16 + a;
        if (t < T) {
            char *dst = p.out + (((size_t)b * T + t) * N + c0 + g * 4) * ES;
            u32x2 w2;
            w2[0] = pack2<TT>(s0[0], s0[1]); w2[1] = pack2<TT>(s0[2], s0[3]);
            *reinterpret_cast<u32x2 *>(dst) = w2;
            w2[0] = pack2<TT>(s1[0], s1[1]); w2[1] = pack2<TT>(s1[2], s1[3]);
            *reinterpret_cast<u32x2 *>(dst + 16 * ES) = w2;
        }
    };
#pragma unroll
    for (int i = 0; i < kPassOwn; ++i) {
        const int tb = wave * kPassOwn + i;
        bool is_shared = false;
#pragma unroll
        for (int x = 0; x < kPassShared; ++x) is_shared = is_shared || tb == hb[x];
        if (!is_shared) store_block(tb, sum[i][0], sum[i][1]);      // uniform
    }
    // shared blocks: wavefront x adds the eight wavefronts' tiles of block hb[x] in wavefront order
    if (hb[0] >= 0) {                                   // uniform
        __syncthreads();
#pragma unroll
        for (int x = 0; x < kPassShared; ++x) {
            if (hb[x] >= 0 && wave == x) {
                f32x4 s0 = shared_part[((x * NWV + 0) * 2 + 0) * 64 + lane], s1 = shared_part[((x * NWV + 0) * 2 + 1) * 64 + lane];
#pragma unroll
                for (int w = 1; w < NWV; ++w) {
                    s0 += shared_part[((x * NWV + w) * 2 + 0) * 64 + lane];
                    s1 += shared_part[((x * NWV + w) * 2 + 1) * 64 + lane];
                }
                store_block(hb[x], s0, s1);
            }
        }
    }
}

}  // namespace egs
