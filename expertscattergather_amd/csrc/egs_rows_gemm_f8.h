// Gather-GEMM with fp8 (OCP e4m3fn) weights AND fp8 activations on the gfx950 fp8 matrix
// instruction (v_mfma_f32_16x16x128_f8f6f4, fp32 accumulation):
//
//   Y[b,e,k,n] = xs[b,t] * ws[e,n] * sum_r Xq[b,t,r] * Wq[e,r,n],   t = Ind[b,e,k]
//
// Two kernels.
//   quantize_rows_e4m3_kernel   every source row X[b,t,:] (bf16) is quantised ONCE to e4m3 with its own
//       scale xs[b,t] = max|X[b,t,:]| / 448; a row is picked by many experts, so quantising before the gather
//       instead of inside it divides the conversion work by the number of picks per token and halves the bytes
//       the gather moves.
//   rows_gemm_f8_kernel         the direct-to-LDS pipeline of egs_rows_gemm_dl.h at one byte per element:
//       256 x 256 tile of one expert's product per workgroup (8 wavefronts, 2 x 4, 128 x 64 each), 128-deep
//       slabs (32 KB of gathered rows + 32 KB of weights), two stages, one barrier per slab.  Rows are K-major
//       in LDS and read with 16-byte reads, weights stay [reduction][column] and are read with the 8-bit LDS
//       transpose read; both operands of one MFMA are 32 bytes per lane and use the same order of reduction
//       elements within a lane group, which is all the instruction needs.
//
// The reference has no quantised path (its kernels take fp32/fp16/bf16 only, egs/triton_kernels.py:15-23);
// this is the inference variant of expert_gather_kernel (egs/triton_kernels.py:49-143) for e4m3 weights.
#pragma once
#include "egs_device.h"

namespace egs {

typedef int i32x8 __attribute__((ext_vector_type(8)));

constexpr float kE4M3Max = 448.0f;

// ---------------------------------------------------------------------------- row quantiser
struct QuantRowsParams {
    const char *X;          // [B,T,I] bf16, strides (ldx_b, ldx_t, 1) in elements, rows 16-byte aligned
    char *Xq;               // [B*T, I] e4m3, dense
    float *xs;              // [B*T] row scales
    int32_t B, T, I;        // I % 8 == 0
    int64_t ldx_b, ldx_t;
};

// one wavefront per row: pass 1 finds max|x|, pass 2 (the row is in the cache by then) scales,
// clamps and converts with round-to-nearest-even; adjacent lanes write adjacent 8-byte pieces
static __global__ __launch_bounds__(kThreads) void quantize_rows_e4m3_kernel(QuantRowsParams p)
{
    const int lane = (int)threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kThreads / 64) + ((int)threadIdx.x >> 6);
    if (row >= (int64_t)p.B * p.T) return;
    const int64_t b = row / p.T, t = row - b * p.T;
    const char *src = p.X + (b * p.ldx_b + t * p.ldx_t) * 2;
    const int chunks = p.I >> 3;
    // max|x| over the row as an integer maximum of the magnitude bits: for non-negative floats the bit patterns
    // order like the values, infinities sort above every finite value and NaNs above the infinities, so a NaN
    // anywhere in the row survives the reduction (fmaxf would drop it)
    uint32_t amax_bits = 0u;
    for (int c = lane; c < chunks; c += 64) {
        const u32x4 v = *reinterpret_cast<const u32x4 *>(src + (size_t)c * 16);
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            amax_bits = max(amax_bits, (v[x] << 16) & 0x7fffffffu);
            amax_bits = max(amax_bits, v[x] & 0x7fff0000u);
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) amax_bits = max(amax_bits, (uint32_t)__shfl_xor((int)amax_bits, m));
    const float amax = bits_f32(amax_bits);
    // a row that holds a NaN or an infinity gets a NaN scale: every product that uses the row comes out NaN,
    // as it does in unquantised arithmetic (the quantised values themselves are then meaningless)
    const bool finite = amax_bits < 0x7f800000u;
    const float scale = !finite ? bits_f32(0x7fc00000u) : (amax > 0.f ? amax / kE4M3Max : 1.0f);
    const float inv = finite ? 1.0f / scale : 0.f;
    if (lane == 0) p.xs[row] = scale;
    char *dst = p.Xq + row * p.I;
    for (int c = lane; c < chunks; c += 64) {
        const u32x4 v = *reinterpret_cast<const u32x4 *>(src + (size_t)c * 16);
        u32x2 q;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float f[4];
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                f[2 * x] = fminf(fmaxf(bits_f32(v[2 * h + x] << 16) * inv, -kE4M3Max), kE4M3Max);
                f[2 * x + 1] = fminf(fmaxf(bits_f32(v[2 * h + x] & 0xffff0000u) * inv, -kE4M3Max), kE4M3Max);
            }
            int w = 0;
            w = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], w, false);
            w = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w, true);
            q[h] = (uint32_t)w;
        }
        *reinterpret_cast<u32x2 *>(dst + (size_t)c * 8) = q;
    }
}

// ---------------------------------------------------------------------------- fp8 x fp8 gather-GEMM
struct RowsGemmF8Params {
    const char *Aq;         // [B*T, R] e4m3 rows (the quantiser's output)
    const float *a_scale;   // [B*T]
    const char *W;          // [E, R, N] e4m3
    const float *w_scale;   // [E, N]
    const void *Ind;        // [B,E,K]
    char *C;                // [B,E,K,N] bf16
    int32_t B, T, E, K, R, N;   // R % 128 == 0, N % 16 == 0
    int32_t ind_dtype;
    int32_t m_tiles, n_tiles;
    uint32_t a_bytes;       // B*T*R, below 2 GiB
};

constexpr int kF8BM = 256, kF8BN = 256, kF8BK = 128, kF8Stages = 2, kF8Threads = 512;
constexpr int kF8StageBytes = kF8BM * kF8BK + kF8BK * kF8BN;

// swizzle key of the K-major byte rows (8 chunks of 16 bytes), XORed into the chunk index: the 16-byte
// fragment reads of consecutive rows spread over the banks
__device__ __forceinline__ int f8_key_rows(int row) { return row & 7; }

static __global__ __launch_bounds__(kF8Threads) void rows_gemm_f8_kernel(RowsGemmF8Params p)
{
    constexpr int BM = kF8BM, BN = kF8BN, BK = kF8BK, NSTAGE = kF8Stages;
    constexpr int NW = kF8Threads / 64, WN = 4;
    constexpr int TM = 8, TN = 4;                       // 16 x 16 tiles per wavefront: 128 x 64
    constexpr int P_BYTES = BM * BK, STAGE = kF8StageBytes;
    constexpr int PL = BM * (BK / 16) / 64 / NW;        // row-side loads per wavefront and slab (1 KB = 8 rows each)
    constexpr int QL = BK / 4 / NW;                     // weight-side loads (1 KB = 4 reduction rows of 256 bytes)
    static_assert(PL == 4 && QL == 4, "loads per slab");

    __shared__ __attribute__((aligned(1024))) char smem[NSTAGE * STAGE + BM * 16];
    uint32_t *a_voff = reinterpret_cast<uint32_t *>(smem + NSTAGE * STAGE);
    float *a_scl = reinterpret_cast<float *>(smem + NSTAGE * STAGE + BM * 4);
    int64_t *c_off = reinterpret_cast<int64_t *>(smem + NSTAGE * STAGE + BM * 8);

    const int tid = (int)threadIdx.x;
    int e, tile;
    if (!decode_expert_tile((int)blockIdx.x, p.m_tiles * p.n_tiles, p.E, e, tile)) return;
    const int mt = tile / p.n_tiles, nt = tile - mt * p.n_tiles;
    const int m0 = mt * BM, n0 = nt * BN;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int R = p.R, N = p.N;
    const int Me = p.B * p.K;

    // ---------------- per-row bookkeeping: byte offset of the quantised source row, its scale, output offset
    if (tid < BM) {
        const int m = m0 + tid;
        uint32_t ao = kVoffInvalid;
        float sc = 0.f;
        int64_t co = -1;
        if (m < Me) {
            const int b = m / p.K, k = m - b * p.K;
            const int64_t pick = ((int64_t)b * p.E + e) * p.K + k;
            const int32_t t = load_token(p.Ind, p.ind_dtype, pick, p.T);
            if (t >= 0) {
                const int64_t src = (int64_t)b * p.T + t;
                ao = (uint32_t)(src * R);
                sc = p.a_scale[src];
            }
            co = pick * N;
        }
        a_voff[tid] = ao;
        a_scl[tid] = sc;
        c_off[tid] = co;
    }
    __syncthreads();

    const u32x4 rs_a = make_rsrc(p.Aq, p.a_bytes);
    const u32x4 rs_w = make_rsrc(p.W + (size_t)e * R * N, (uint32_t)((size_t)R * N));

    // ---------------- loaders: lane l of a row-side load lands on row 8 j + l/8, physical chunk l%8 and so
    // fetches logical chunk (l%8) ^ key(row); lane l of a weight-side load lands on reduction row 4 j + l/16,
    // physical chunk l%16 and fetches the 16 columns of logical chunk (l%16) ^ (row & 15)
    uint32_t pv[PL], qv[QL];
#pragma unroll
    for (int jj = 0; jj < PL; ++jj) {
        const int row = (wave * PL + jj) * 8 + (lane >> 3);
        const uint32_t ao = a_voff[row];
        pv[jj] = ao == kVoffInvalid ? kVoffInvalid : ao + (uint32_t)(((lane & 7) ^ f8_key_rows(row)) << 4);
    }
#pragma unroll
    for (int jj = 0; jj < QL; ++jj) {
        const int row = (wave * QL + jj) * 4 + (lane >> 4);
        const int n = n0 + ((lane & 15) ^ (row & 15)) * 16;
        qv[jj] = n < N ? (uint32_t)row * (uint32_t)N + (uint32_t)n : kVoffInvalid;
    }
    auto issue = [&](int kt, int stage) {
        char *pbase = smem + stage * STAGE + wave * (PL * 1024);
        char *qbase = smem + stage * STAGE + P_BYTES + wave * (QL * 1024);
        const uint32_t so_a = (uint32_t)kt * BK;
        const uint32_t so_w = (uint32_t)kt * BK * (uint32_t)N;
#pragma unroll
        for (int jj = 0; jj < PL; ++jj) direct_load16(rs_a, pv[jj], so_a, pbase + jj * 1024);
#pragma unroll
        for (int jj = 0; jj < QL; ++jj) direct_load16(rs_w, qv[jj], so_w, qbase + jj * 1024);
    };

    // ---------------- fragment addresses.  The 32 operand bytes of lane group g are, in this order, the
    // reduction elements 64 u + 16 g + 8 h .. + 7 for (u, h) = (0,0), (0,1), (1,0), (1,1): one 16-byte read per
    // u on the row side (chunk 4 u + g of the row), one transpose read per (u, h) on the weight side
    const int a = lane & 15, g = lane >> 4;
    const int wave_m0 = (wave / WN) * 128, wave_n0 = (wave % WN) * 64;
    int m_at[2], n_at[4];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int row = wave_m0 + a;                                // + 16 i: the key does not depend on i
        m_at[u] = row * BK + (((4 * u + g) ^ f8_key_rows(row)) << 4);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int kr = u * 64 + g * 16 + h * 8 + (a >> 1);      // the transpose read's row of this lane
            n_at[2 * u + h] = kr * BN + (((wave_n0 >> 4) ^ (kr & 15)) << 4) + (a & 1) * 8;
        }
    }

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nk = R / BK;
    if (nk > 0) issue(0, 0);
    for (int kt = 0; kt < nk; ++kt) {
        wait_vmem<0>();
        __syncthreads();            // slab kt visible to all; everyone is done reading the stage refilled next
        if (kt + 1 < nk) issue(kt + 1, (kt + 1) & 1);
        const char *tile_m = smem + (kt & 1) * STAGE;
        const char *tile_n = tile_m + P_BYTES;
        i32x8 nf[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const u32x2 v = lds_read_tr8(tile_n + (n_at[q] ^ (j << 4)));     // chunk wave_n0/16 + j, j < 4
                nf[j][2 * q] = (int)v[0];
                nf[j][2 * q + 1] = (int)v[1];
            }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            i32x8 mf;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(tile_m + m_at[u] + i * (16 * BK));
#pragma unroll
                for (int x = 0; x < 4; ++x) mf[4 * u + x] = (int)v[x];
            }
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(nf[j], mf, acc[i][j], 0, 0, 0, 0, 0, 0);
        }
    }

    // ---------------- epilogue.  Lane (a, g) holds, for row 16 i + a, the four columns 16 j + 4 g .. + 3.  Both
    // scales are applied, the bf16 tile goes through LDS (the slab stages are free now: 256 rows x 512 bytes)
    // and leaves as whole row segments, 512 contiguous bytes of each of two rows per store instruction.
    constexpr int ROW_BYTES = BN * 2;
    static_assert(BM * ROW_BYTES <= NSTAGE * STAGE, "staging tile fits the slab stages");
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int row = wave_m0 + i * 16 + a;
        const float rs = a_scl[row];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            f32x4 v = acc[i][j];
            const int col = wave_n0 + j * 16 + g * 4;
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] *= n0 + col + r < N ? p.w_scale[(size_t)e * N + n0 + col + r] * rs : 0.f;
            const int chunk = (col >> 3) ^ (row & 15);
            const u32x2 w = {pack2<ElemBF16>(v[0], v[1]), pack2<ElemBF16>(v[2], v[3])};
            *reinterpret_cast<u32x2 *>(smem + row * ROW_BYTES + chunk * 16 + (col & 4) * 2) = w;
        }
    }
    __syncthreads();
    const int lrow = lane >> 5, lchunk = lane & 31;
    const int n_here = n0 + lchunk * 8;
    for (int r0 = wave * 2; r0 < BM; r0 += NW * 2) {
        const int row = r0 + lrow;
        const int64_t co = c_off[row];
        const u32x4 v = *reinterpret_cast<const u32x4 *>(smem + row * ROW_BYTES + ((lchunk ^ (row & 15)) << 4));
        if (co >= 0 && n_here < N) *reinterpret_cast<u32x4 *>(p.C + co * 2 + (size_t)n_here * 2) = v;
    }
}

}  // namespace egs
