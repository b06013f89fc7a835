// Inference block of small experts in ONE kernel: gather-GEMM, activation and GEMM-scatter with the
// intermediate rows Y[b,e,k,:] never leaving the CU:
//
//   Y[b,e,k,:]  = act( X[b, Ind[b,e,k], :] . Wg(e) )                 Wg(e): [I,J]
//   out[b,t,:]  = sum over the picks (e,k) of token t, in routing-table order, of  Y[b,e,k,:] . Ws(e)      Ws(e): [J,I]
//
// The second half is the one-kernel scatter of egs_scatter_fused.h (a workgroup owns one batch element and one
// 32-column slice of the output, sorts the picks in LDS, parks fp32 product rows in LDS and adds them per token in
// table order: bitwise reproducible, no atomics, no workspace).  What is new is where its row operand comes from: each
// (expert, 32-pick) unit first multiplies its gathered rows of X by Wg(e) - computed as the TRANSPOSED tile
// Yt = Wg(e)t . Xt, so that after the matrix instructions lane (a, g) holds, for pick a, sixteen consecutive
// reduction elements j of the second product (16 g .. 16 g + 15 of each 64-column block of Y).  That is already the
// operand layout of the second matrix instruction (a lane supplies eight reduction-consecutive elements of its row):
// the activation is applied in registers in fp32, the values are rounded to the element type (as a stored Y would be)
// and fed straight back, with the rows of Ws(e) fetched in the matching order.  No LDS round trip, no cross-lane moves.
// The four slice workgroups of a batch element each redo the gather product (it is a quarter of the work of the
// kernel and all of it hits the L2); in exchange Y (8 MB at the reference's default shape, written once and read
// once), the activation's read and write of it and two launches disappear.
//
// 16-bit elements, I in {32, 64, 128}, J in {32, 64}, E*K <= 1024 picks per batch element.  (J = 128 compiles - JT = 8 -
// but the two 64-column blocks of Wg(e) no longer fit the register file next to the other operands: 159 us where the
// separate launches take 33 us, so the host does not instantiate it.)
// Measured at the reference's default shape (bf16, relu): 22.8 us against 27.3 us for gather, torch.relu and scatter as
// three launches; 14.6 against 23.3 us with 16 experts.  A workgroup's life is four units per wavefront one after the
// other, each waiting for its 24 KB of operands; with an activation that costs many instructions (erf) the fourfold
// repetition across the slice workgroups outweighs the saved launches.
//
// Replaces the reference's call pattern  scatter(act(gather(x, Ind)), Ind, T)  (test_speed.ipynb:73-75; kernels
// egs/triton_kernels.py:49-143 and :156-247) for inference.
#pragma once
#include "egs_scatter_fused.h"

namespace egs {

enum MlpAct { MLP_ACT_NONE = 0, MLP_ACT_RELU = 1, MLP_ACT_GELU = 2, MLP_ACT_SILU = 3, MLP_ACT_GELU_TANH = 4 };

struct MlpFusedParams {
    const char *X;          // [B,T,I] rows, strides (ldx_b, ldx_t, 1) in elements
    const char *Wg;         // [E,I,J]
    const char *Ws;         // [E,J,I]
    const void *Ind;        // [B,E,K]
    char *out;              // [B,T,I]
    int32_t B, T, E, K;
    int64_t ldx_b, ldx_t;
    int32_t ind_dtype;
    int32_t slices;         // I / kFusedCols
    int32_t perm_at, cnt_at, zero_at;   // as in ScatterFusedParams
    int32_t act;            // MlpAct
};

// KS1 = I / 32 (matrix-instruction steps of the gather product; I is also the output width), JT = J / 16
template <class TT, int KS1, int JT>
__device__ __forceinline__ void mlp_fused_body(const MlpFusedParams &p, const int block, char *smem)
{
    static_assert(TT::ES == 2, "16-bit element types");
    static_assert(JT == 2 || JT == 4 || JT == 8, "J = 32, 64 or 128");
    constexpr int I = 32 * KS1, J = 16 * JT, N = I;
    constexpr int JB = JT <= 4 ? 1 : 2;                 // 64-column blocks of Y (J = 32: half a block)
    constexpr int KS2 = 2 * JB;                         // matrix-instruction steps of the second product
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int a = lane & 15, g = lane >> 4;
    const int grp = block & 7, idx = block >> 3;
    const int b = (idx / p.slices) * 8 + grp, slice = idx % p.slices;
    if (b >= p.B) return;
    const int c0 = slice * kFusedCols;
    const int T = p.T, E = p.E, K = p.K, NP = E * K;

    float *rows = reinterpret_cast<float *>(smem);
    int32_t *perm = reinterpret_cast<int32_t *>(smem + p.perm_at);
    int32_t *cnt = reinterpret_cast<int32_t *>(smem + p.cnt_at);
    constexpr int NWV = kFusedThreads / 64;
    const int32_t *seg = cnt + NWV * T;
    if (tid < kFusedCols) reinterpret_cast<float *>(smem + p.zero_at)[tid] = 0.f;       // read after the barrier before the sums

    const int KT2 = (K + 31) >> 5;
    const int units = E * KT2;                          // (expert, 32 picks); a wavefront takes units wave, wave + 8, ...

    // ---- operands of a unit
    u32x2 wg[JB][KS1][8];       // Wg(e): 8 (reduction i) x 4 (columns j = 64 jb + 4 a ..) blocks, transposed at use
    u32x4 xr[2][KS1];           // gathered rows, coalesced order (lanes 4r .. 4r+3: four consecutive chunks of row r)
    struct WsFrag { u32x4 w[2 * KS2]; };
    WsFrag ws_cur, ws_next;     // Ws(e): rows j in the order the first product leaves them, columns c0 + 2a, c0 + 2a + 1

    auto unit_pick = [&](int unit, int &e, int &rp) -> int64_t {      // this lane's pick of the unit (lanes >= 32 repeat)
        e = unit / KT2; rp = unit - e * KT2;
        const int k = min(rp * 32 + (lane & 31), K - 1);
        return ((int64_t)b * E + e) * K + k;
    };
    auto load_index = [&](int unit) -> uint64_t {
        if (unit >= units) return 0;
        int e, rp;
        return load_index_word(p.Ind, p.ind_dtype, unit_pick(unit, e, rp));
    };
    auto load_wg = [&](int unit) {
        if (unit >= units) return;
        const int e = unit / KT2;
#pragma unroll
        for (int jb = 0; jb < JB; ++jb) {
            const int col = min(jb * 64 + 4 * a, J - 4);        // J = 32: lanes a >= 8 repeat a valid block; their rows of Yt meet zeros
#pragma unroll
            for (int ks = 0; ks < KS1; ++ks)
#pragma unroll
                for (int x = 0; x < 8; ++x)
                    wg[jb][ks][x] = *reinterpret_cast<const u32x2 *>(p.Wg + (((size_t)e * I + ks * 32 + g * 8 + x) * J + col) * 2);
        }
    };
    auto load_ws = [&](WsFrag &f, int unit) {
        if (unit >= units) return;
        const int e = unit / KT2;
#pragma unroll
        for (int ks2 = 0; ks2 < KS2; ++ks2) {
            // lane group g supplies, in step ks2 = 2 jb + half, the reduction elements j = 64 jb + 16 g + 8 half + x
            const int j0 = (ks2 >> 1) * 64 + 16 * g + (ks2 & 1) * 8;
#pragma unroll
            for (int x = 0; x < 8; ++x) {
                uint32_t v = 0;
                if (j0 + x < J) v = *reinterpret_cast<const uint32_t *>(p.Ws + (((size_t)e * J + j0 + x) * N + c0 + 2 * a) * 2);
                f.w[ks2 * 2 + (x >> 2)][x & 3] = v;
            }
        }
    };
    auto load_rows = [&](int unit, uint64_t iw) {
        if (unit >= units) return;
        int e, rp;
        const int64_t pick = unit_pick(unit, e, rp);
        const int64_t raw = decode_index_word(iw, p.Ind, p.ind_dtype, pick);
        // a rejected pick has no place in the table: whatever row it reads is never added
        const int64_t t = (raw < 0 || raw >= (int64_t)T) ? 0 : raw;
        const uint32_t aoff = (uint32_t)(((int64_t)b * p.ldx_b + t * p.ldx_t) * 2);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t xo = (uint32_t)__shfl((int)aoff, h * 16 + (lane >> 2), kWave) + (uint32_t)((lane & 3) * 16);
#pragma unroll
            for (int ks = 0; ks < KS1; ++ks) xr[h][ks] = *reinterpret_cast<const u32x4 *>(p.X + xo + ks * 64);
        }
    };

    // ---------------- (0) routing table of batch element b in LDS; the first unit's index and weights go in flight
    // right behind the sort's token loads
    uint64_t iw_cur = 0;
    csr_count_body(cnt, b, 0, tid, kFusedThreads, p.Ind, p.ind_dtype, T, NP, nullptr, perm, nullptr, nullptr, [&]() {
        iw_cur = load_index(wave);
        load_wg(wave);
        load_ws(ws_cur, wave);
    });
    load_rows(wave, iw_cur);
    uint64_t iw_next = load_index(wave + NWV);

    for (int unit = wave; unit < units; unit += NWV) {
        const int e = unit / KT2, rp = unit - e * KT2;
        // ---- first product, transposed: lane (a, g) ends with Y[pick 16 h + a][j = 64 jb + 16 g + 4 r + c] in acc1[h][4 jb + c][r]
        f32x4 acc1[2][4 * JB];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int t = 0; t < 4 * JB; ++t) acc1[h][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS1; ++ks) {
            u32x4 xf[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) xf[h] = lanes_4a_g_to_16g_a(xr[h][ks], lane);
#pragma unroll
            for (int jb = 0; jb < JB; ++jb) {
                u32x4 wf[4];
                transpose8x4_16b(wg[jb][ks], wf);
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int c = 0; c < 4; ++c) mma_chunk<TT>(acc1[h][4 * jb + c], wf[c], xf[h]);
            }
        }
        // ---- the next unit's operands go in flight now that this unit's are consumed
        load_rows(unit + NWV, iw_next);
        load_wg(unit + NWV);
        load_ws(ws_next, unit + NWV);
        iw_next = load_index(unit + 2 * NWV);

        // ---- activation (fp32; one uniform branch per unit), rounding to the element type, second product
        auto activate = [&](auto fn) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int t = 0; t < 4 * JB; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc1[h][t][r] = fn(acc1[h][t][r]);
        };
        // The transcendental ones are written with the hardware exponential and reciprocal (a few instructions per value
        // instead of the ~100 of the library erff / tanhf: every slice workgroup repeats them).  gelu_tanh(v) = v * sigmoid(2u);
        // erf by the rational approximation of Abramowitz & Stegun 7.1.26 (absolute error < 1.5e-7, far below the rounding
        // to a 16-bit type that follows).
        switch (p.act) {
        case MLP_ACT_RELU: activate([](float v) { return fmaxf(v, 0.f); }); break;
        case MLP_ACT_GELU:
            activate([](float v) {
                const float x = fabsf(v) * 0.70710678118654752f;
                const float t = __frcp_rn(1.f + 0.3275911f * x);
                const float poly = ((((1.061405429f * t - 1.453152027f) * t + 1.421413741f) * t - 0.284496736f) * t + 0.254829592f) * t;
                const float erf_abs = 1.f - poly * __expf(-x * x);
                return 0.5f * v * (1.f + copysignf(erf_abs, v));
            });
            break;
        case MLP_ACT_SILU: activate([](float v) { return v * __frcp_rn(1.f + __expf(-v)); }); break;
        case MLP_ACT_GELU_TANH:
            activate([](float v) {
                const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
                return v * __frcp_rn(1.f + __expf(-2.f * u));
            });
            break;
        default: break;
        }
        f32x4 acc2[2][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) { acc2[h][0] = f32x4{0.f, 0.f, 0.f, 0.f}; acc2[h][1] = f32x4{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
        for (int ks2 = 0; ks2 < KS2; ++ks2) {
            const int jb = ks2 >> 1, r0 = (ks2 & 1) * 2;
            u32x4 wf[2];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                const uint32_t lo = ws_cur.w[ks2 * 2 + (pp >> 1)][(pp & 1) * 2], hi = ws_cur.w[ks2 * 2 + (pp >> 1)][(pp & 1) * 2 + 1];
                wf[0][pp] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);     // column 2a   of rows 2pp, 2pp+1
                wf[1][pp] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);     // column 2a+1
            }
            const bool real = jb * 64 + 16 * g + (ks2 & 1) * 8 < J;        // J = 32: lane groups 2 and 3 hold nothing of Y
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                u32x4 q = {0u, 0u, 0u, 0u};
                if (real) {
#pragma unroll
                    for (int rr = 0; rr < 2; ++rr) {
                        const int r = r0 + rr;
                        q[rr * 2] = pack2<TT>(acc1[h][4 * jb + 0][r], acc1[h][4 * jb + 1][r]);
                        q[rr * 2 + 1] = pack2<TT>(acc1[h][4 * jb + 2][r], acc1[h][4 * jb + 3][r]);
                    }
                }
                mma_chunk<TT>(acc2[h][0], wf[0], q);
                mma_chunk<TT>(acc2[h][1], wf[1], q);
            }
        }
        // lane (a, g) holds, for pick k = 32 rp + 16 h + a, slice columns 2 (4 g + r) + ct = 8 g + 2 r + ct
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = rp * 32 + h * 16 + a;
            if (k < K) {
                const int q = e * K + k;
                f32x4 *row = reinterpret_cast<f32x4 *>(rows + (size_t)q * kFusedCols);
                row[(2 * g) ^ (q & 7)] = f32x4{acc2[h][0][0], acc2[h][1][0], acc2[h][0][1], acc2[h][1][1]};
                row[(2 * g + 1) ^ (q & 7)] = f32x4{acc2[h][0][2], acc2[h][1][2], acc2[h][0][3], acc2[h][1][3]};
            }
        }
        ws_cur = ws_next;
    }
    __syncthreads();

    // ---------------- per token: add its product rows in table order; 4 threads x 8 columns per token, four table entries
    // at a time read without looking at the segment's end, those past it replaced by a row of zeros (the loop of
    // scatter_fused_body, which is bound by vector-ALU issue)
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
                const uint32_t sel = (x < n) ? (en[x] << 7) | ((en[x] & 7u) << 4) : zero_sel;
                v[x][0] = *reinterpret_cast<const f32x4 *>(smem + (sel ^ c2));
                v[x][1] = *reinterpret_cast<const f32x4 *>(smem + (sel ^ (c2 | 16u)));
            }
#pragma unroll
            for (int x = 0; x < 4; ++x) { lo += v[x][0]; hi += v[x][1]; }
        }
        u32x4 w;
        w[0] = pack2<TT>(lo[0], lo[1]); w[1] = pack2<TT>(lo[2], lo[3]);
        w[2] = pack2<TT>(hi[0], hi[1]); w[3] = pack2<TT>(hi[2], hi[3]);
        *reinterpret_cast<u32x4 *>(p.out + (((size_t)b * T + t) * N + c0 + (tid & 3) * 8) * 2) = w;
    }
}

template <class TT, int KS1, int JT>
__global__ __launch_bounds__(kFusedThreads) void mlp_fused_kernel(MlpFusedParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem_mlp_fused[];
    mlp_fused_body<TT, KS1, JT>(p, (int)blockIdx.x, smem_mlp_fused);
}

}  // namespace egs
