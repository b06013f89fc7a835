// Device-side building blocks shared by the gfx950 kernels: 16-byte chunk loads with
// tail/alignment guards, the swizzled K-major LDS tile, in-register block transposes,
// MFMA steps per element type and index decoding.
//
// Vocabulary used throughout:
//   pick    one (b, e, k) entry of Ind; picks of one expert form the rows m = b*K + k of a
//           dense per-expert matrix product
//   chunk   16 bytes = VEC consecutive elements along the reduction axis
//   slab    BK reduction elements staged in LDS at a time
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace egs {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;   // 4 wavefronts of 64 lanes per workgroup
constexpr int kWave = 64;

// ---------------------------------------------------------------------------- element types
struct ElemF32 {
    static constexpr int ES = 4;      // bytes per element
    static constexpr int VEC = 4;     // elements per 16-byte chunk
    static constexpr int ID = 0;
};
struct ElemF16 {
    static constexpr int ES = 2;
    static constexpr int VEC = 8;
    static constexpr int ID = 1;
};
struct ElemBF16 {
    static constexpr int ES = 2;
    static constexpr int VEC = 8;
    static constexpr int ID = 2;
};

__device__ __forceinline__ uint32_t f32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }

// round-to-nearest-even float -> bf16 bits
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f)
{
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;      // NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f)
{
    _Float16 h = (_Float16)f;
    return (uint32_t)__builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return bits_f32(h << 16); }
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// two floats -> two 16-bit elements in one dword (round to nearest even; one hardware
// instruction for bf16 on gfx950)
template <class TT> __device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2<ElemBF16>(float lo, float hi)
{
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2_t){lo, hi}, bf16x2_t));
}
template <> __device__ __forceinline__ uint32_t pack2<ElemF16>(float lo, float hi)
{
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2_t){lo, hi}, f16x2_t));
}
template <> __device__ __forceinline__ uint32_t pack2<ElemF32>(float lo, float) { return f32_bits(lo); }

template <class TT> __device__ __forceinline__ uint32_t f32_to_elem_bits(float f);
template <> __device__ __forceinline__ uint32_t f32_to_elem_bits<ElemF32>(float f) { return f32_bits(f); }
template <> __device__ __forceinline__ uint32_t f32_to_elem_bits<ElemF16>(float f) { return f32_to_f16_bits(f); }
template <> __device__ __forceinline__ uint32_t f32_to_elem_bits<ElemBF16>(float f) { return f32_to_bf16_bits(f); }

// one MFMA "chunk step": every lane supplies one 16-byte chunk per operand; lane group
// g = lane/16 supplies reduction elements [g*VEC, g*VEC+VEC) of a 4*VEC wide step, rows /
// columns are lane%16.  The accumulator holds rows 4*g..4*g+3 of column lane%16, where
// "rows" index the first operand's lanes and "columns" the second operand's.
template <class TT> __device__ __forceinline__ void mma_chunk(f32x4 &acc, const u32x4 &p, const u32x4 &q);
template <> __device__ __forceinline__ void mma_chunk<ElemBF16>(f32x4 &acc, const u32x4 &p, const u32x4 &q)
{
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, p), __builtin_bit_cast(bf16x8, q), acc, 0, 0, 0);
}
template <> __device__ __forceinline__ void mma_chunk<ElemF16>(f32x4 &acc, const u32x4 &p, const u32x4 &q)
{
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, p), __builtin_bit_cast(f16x8, q), acc, 0, 0, 0);
}
template <> __device__ __forceinline__ void mma_chunk<ElemF32>(f32x4 &acc, const u32x4 &p, const u32x4 &q)
{
#pragma unroll
    for (int c = 0; c < 4; ++c)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(bits_f32(p[c]), bits_f32(q[c]), acc, 0, 0, 0);
}

// ---------------------------------------------------------------------------- index decode
// Ind is read in its own integer width and never narrowed.  Branch-free for every width (so that
// several index loads can be in flight): one 8-byte load of the aligned window that contains the
// element, then shift and sign- or zero-extend.  The window never leaves the allocation because
// device allocations start and end on multiples of 8 bytes and elements are naturally aligned.
// The load and the decoding are separate functions so that a kernel can put other loads between them.
__device__ __forceinline__ uint64_t load_index_word(const void *ind, int ind_dtype, int64_t at)
{
    const int es_log2 = (0x0321 >> (4 * ind_dtype)) & 0xF;          // int16 -> 1, int32 -> 2, int64 -> 3, uint8 -> 0
    // pointer arithmetic on `ind` itself (not on its integer value): the compiler then knows the load is a
    // global one, which returns in order with the other global loads of the wavefront
    const int64_t mis = (int64_t)(reinterpret_cast<uint64_t>(ind) & 7ull);
    const int64_t off = (at << es_log2) + mis;
    return *reinterpret_cast<const uint64_t *>(static_cast<const char *>(ind) - mis + (off & ~(int64_t)7));
}
__device__ __forceinline__ int64_t decode_index_word(uint64_t w, const void *ind, int ind_dtype, int64_t at)
{
    const int es_log2 = (0x0321 >> (4 * ind_dtype)) & 0xF;
    const uint64_t addr = reinterpret_cast<uint64_t>(ind) + ((uint64_t)at << es_log2);
    const int bits = 8 << es_log2;
    w <<= 64 - bits - (int)(addr & 7ull) * 8;                       // element now in the top `bits` bits
    const int64_t sx = (int64_t)w >> (64 - bits);                   // sign-extended
    const int64_t zx = (int64_t)(w >> (64 - bits));                 // zero-extended (uint8)
    return ind_dtype == 3 ? zx : sx;
}
__device__ __forceinline__ int64_t load_index_raw(const void *ind, int ind_dtype, int64_t at)
{
    return decode_index_word(load_index_word(ind, ind_dtype, at), ind, ind_dtype, at);
}
__device__ __forceinline__ int32_t load_token(const void *ind, int ind_dtype, int64_t at, int32_t T)
{
    int64_t t = load_index_raw(ind, ind_dtype, at);
    return (t < 0 || t >= (int64_t)T) ? -1 : (int32_t)t;
}

// ---------------------------------------------------------------------------- guarded chunk loads
// `row` points at element 0 of a source row (nullptr => the row reads as zeros), `k0` is the
// first element wanted and `klim` the number of valid elements in the row.  `vec_ok` says the
// row start is 16-byte aligned and k0 is a multiple of VEC, so an in-range chunk is one load.
template <int ES>
__device__ __forceinline__ u32x4 load_chunk(const char *row, int k0, int klim, bool vec_ok)
{
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row == nullptr || k0 >= klim) return v;
    constexpr int VEC = 16 / ES;
    if (vec_ok && k0 + VEC <= klim) {
        return *reinterpret_cast<const u32x4 *>(row + (size_t)k0 * ES);
    }
    if constexpr (ES == 2) {
        const uint16_t *p = reinterpret_cast<const uint16_t *>(row) + k0;
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            uint32_t h = (k0 + x < klim) ? (uint32_t)p[x] : 0u;
            v[x >> 1] |= h << (16 * (x & 1));
        }
    } else {
        const uint32_t *p = reinterpret_cast<const uint32_t *>(row) + k0;
#pragma unroll
        for (int x = 0; x < 4; ++x) v[x] = (k0 + x < klim) ? p[x] : 0u;
    }
    return v;
}

// 8 consecutive fp8 (OCP e4m3fn) bytes -> 8 bf16 in one chunk.  Exact: e4m3 has 3 mantissa bits.
__device__ __forceinline__ u32x4 fp8x8_to_bf16_chunk(uint32_t lo, uint32_t hi)
{
    u32x4 v;
    auto a = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, false);
    auto b = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, true);
    auto c = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, false);
    auto d = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, true);
    v[0] = (f32_bits(a[0]) >> 16) | (f32_bits(a[1]) & 0xffff0000u);
    v[1] = (f32_bits(b[0]) >> 16) | (f32_bits(b[1]) & 0xffff0000u);
    v[2] = (f32_bits(c[0]) >> 16) | (f32_bits(c[1]) & 0xffff0000u);
    v[3] = (f32_bits(d[0]) >> 16) | (f32_bits(d[1]) & 0xffff0000u);
    return v;
}
// fp8 source row, result is a bf16 chunk (8 elements); same guards as load_chunk.
__device__ __forceinline__ u32x4 load_chunk_fp8_as_bf16(const char *row, int k0, int klim, bool vec_ok)
{
    u32x4 z = {0u, 0u, 0u, 0u};
    if (row == nullptr || k0 >= klim) return z;
    uint32_t lo = 0, hi = 0;
    if (vec_ok && k0 + 8 <= klim) {
        u32x2 w = *reinterpret_cast<const u32x2 *>(row + k0);
        lo = w[0]; hi = w[1];
    } else {
        const uint8_t *p = reinterpret_cast<const uint8_t *>(row) + k0;
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            uint32_t b = (k0 + x < klim) ? (uint32_t)p[x] : 0u;
            if (x < 4) lo |= b << (8 * x); else hi |= b << (8 * (x - 4));
        }
    }
    return fp8x8_to_bf16_chunk(lo, hi);
}

// 4 consecutive 16-bit elements (8 bytes) with the same guards as load_chunk; `vec_ok` = the row
// start is 8-byte aligned and k0 is a multiple of 4.
__device__ __forceinline__ u32x2 load_half_chunk16(const char *row, int k0, int klim, bool vec_ok)
{
    u32x2 v = {0u, 0u};
    if (row == nullptr || k0 >= klim) return v;
    if (vec_ok && k0 + 4 <= klim) return *reinterpret_cast<const u32x2 *>(row + (size_t)k0 * 2);
    const uint16_t *p = reinterpret_cast<const uint16_t *>(row) + k0;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        uint32_t h = (k0 + x < klim) ? (uint32_t)p[x] : 0u;
        v[x >> 1] |= h << (16 * (x & 1));
    }
    return v;
}
// 4 consecutive fp8 (e4m3fn) bytes -> 4 bf16; `vec_ok` = 4-byte aligned row start, k0 % 4 == 0.
__device__ __forceinline__ u32x2 load_half_chunk_fp8_as_bf16(const char *row, int k0, int klim, bool vec_ok)
{
    u32x2 z = {0u, 0u};
    if (row == nullptr || k0 >= klim) return z;
    uint32_t w = 0;
    if (vec_ok && k0 + 4 <= klim) {
        w = *reinterpret_cast<const uint32_t *>(row + k0);
    } else {
        const uint8_t *p = reinterpret_cast<const uint8_t *>(row) + k0;
#pragma unroll
        for (int x = 0; x < 4; ++x) w |= ((k0 + x < klim) ? (uint32_t)p[x] : 0u) << (8 * x);
    }
    auto a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    auto b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    u32x2 v;
    v[0] = (f32_bits(a[0]) >> 16) | (f32_bits(a[1]) & 0xffff0000u);
    v[1] = (f32_bits(b[0]) >> 16) | (f32_bits(b[1]) & 0xffff0000u);
    return v;
}

// ---------------------------------------------------------------------------- direct global -> LDS loads
// A raw buffer descriptor over `bytes` bytes starting at `base`: loads whose byte offset is not
// below `bytes` return zeros instead of touching memory, which is how tile rows that do not exist
// (ragged tile edges, rejected picks) are filled.
typedef __attribute__((address_space(3))) void lds_void_t;
constexpr uint32_t kVoffInvalid = 0x80000000u;      // never below a descriptor's size (sizes stay under 2 GiB)

__device__ __forceinline__ u32x4 make_rsrc(const void *base, uint32_t bytes)
{
    const uint64_t addr = reinterpret_cast<uint64_t>(base);
    u32x4 r;
    r[0] = __builtin_amdgcn_readfirstlane((uint32_t)addr);
    r[1] = __builtin_amdgcn_readfirstlane((uint32_t)(addr >> 32) & 0xffffu);     // stride 0: raw byte offsets
    r[2] = __builtin_amdgcn_readfirstlane(bytes);
    r[3] = 0x00020000u;                                                          // 32-bit raw data format
    return r;
}
// One wavefront-wide instruction: lane l fetches the 16 bytes at byte offset voff + soff of the
// descriptor and the hardware writes them to LDS at `lds_base + 16*l` (lds_base wavefront-uniform),
// without passing through registers.  Completion is tracked by the vector-memory counter.
// Written as assembly on purpose: for the builtin form the compiler orders every later LDS read
// behind all outstanding direct loads, which would serialise the prefetch of the next slab with the
// reads of the current one.  Callers order the LDS accesses themselves with wait_vmem + a barrier.
__device__ __forceinline__ void direct_load16(u32x4 rsrc, uint32_t voff, uint32_t soff, char *lds_base)
{
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_void_t *)lds_base;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory", "m0");
}
// Wait until at most N of this wavefront's vector-memory operations are outstanding (N < 64; loads and
// stores complete in issue order as far as this counter is concerned).
template <int N> __device__ __forceinline__ void wait_vmem()
{
    static_assert(N >= 0 && N < 64, "immediate range");
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}
// LDS transpose read: the 16 lanes of a group each point at 4 consecutive 16-bit elements of a
// row (lanes 4k..4k+3 cover 16 columns of row k, k = 0..3); lane n receives column n of those four
// rows, i.e. four reduction-consecutive elements of a row-major [reduction][column] tile.
__device__ __forceinline__ u32x2 lds_read_tr16(const char *at)
{
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(lds_void_t *)at);
    return __builtin_bit_cast(u32x2, v);
}

// 8-bit LDS transpose read: of 16 lanes, lanes 2k and 2k+1 point at bytes 0..7 and 8..15 of row k
// (k = 0..7); lane n receives byte n of those eight rows, i.e. eight reduction-consecutive fp8 values
// of column n of a row-major [reduction][column] byte tile.
__device__ __forceinline__ u32x2 lds_read_tr8(const char *at)
{
    typedef int i32x2 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(3))) i32x2 lds_i32x2;
    i32x2 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2 *)(lds_void_t *)at);
    return __builtin_bit_cast(u32x2, v);
}

// ---------------------------------------------------------------------------- LDS tile
// A tile holds ROWS rows of BK reduction elements, K-major (a row's chunks are adjacent), so
// an MFMA operand fragment is one 16-byte LDS read per lane.  Chunk positions inside each
// 128-byte group are XOR-swizzled by the row so that both the row-wise staging writes, the
// transposed staging writes (8 rows apart) and the fragment reads (consecutive rows) spread
// over the banks.
template <int CH>   // chunks per row, power of two
__device__ __forceinline__ int tile_chunk_index(int row, int c)
{
    constexpr int SW = (CH >= 8 ? 8 : CH) - 1;
    return row * CH + (c ^ ((row ^ (row >> 3)) & SW));
}

// VEC x VEC block transpose in registers: in[r] holds VEC consecutive n of source row r;
// out[c] holds the VEC consecutive r of column c.
__device__ __forceinline__ void transpose8x8_16b(const u32x4 (&in)[8], u32x4 (&out)[8])
{
#pragma unroll
    for (int c = 0; c < 8; ++c) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            uint32_t lo = in[2 * p][c >> 1], hi = in[2 * p + 1][c >> 1];
            out[c][p] = (c & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
        }
    }
}
// 8 rows x 4 columns of 16-bit values (in[x] = 4 columns of row x) -> out[c] = the 8 rows of column c
__device__ __forceinline__ void transpose8x4_16b(const u32x2 (&in)[8], u32x4 (&out)[4])
{
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            uint32_t lo = in[2 * p][c >> 1], hi = in[2 * p + 1][c >> 1];
            out[c][p] = (c & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u) : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        }
}

__device__ __forceinline__ void transpose4x4_32b(const u32x4 (&in)[4], u32x4 (&out)[4])
{
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) out[c][r] = in[r][c];
}

// Lane transposition 16 x 4 -> 4 x 16: lane 16 g + a receives what lane 4 a + g holds.  A global load in
// which lanes 4a .. 4a+3 fetch four consecutive 16-byte chunks of row a is what the memory pipeline
// coalesces (one 64-byte access per row instead of four 16-byte ones); an MFMA operand wants row a's
// chunk g in lane 16 g + a.  Four cross-lane moves (no LDS storage involved) convert one into the other.
__device__ __forceinline__ u32x4 lanes_4a_g_to_16g_a(const u32x4 &v, int lane)
{
    const int src = ((lane & 15) << 2 | (lane >> 4)) << 2;       // byte address of the source lane
    u32x4 r;
#pragma unroll
    for (int x = 0; x < 4; ++x) r[x] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)v[x]);
    return r;
}

// The inverse move: lane 4 a + g receives what lane 16 g + a holds.  Results of an MFMA tile have the four
// lanes g = 0..3 of row a holding four consecutive 16-byte pieces of that row; regrouped, adjacent lanes
// store adjacent addresses (one 64-byte access per row instead of four 16-byte ones).
__device__ __forceinline__ u32x4 lanes_16g_a_to_4a_g(const u32x4 &v, int lane)
{
    const int src = ((lane & 3) << 4 | (lane >> 2)) << 2;
    u32x4 r;
#pragma unroll
    for (int x = 0; x < 4; ++x) r[x] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)v[x]);
    return r;
}

// workgroup id -> (expert, tile): consecutive workgroup ids land on consecutive XCDs (8 per
// device), so expert = 8*group + (id % 8) keeps all tiles of one expert on one XCD and its
// weight tile in that XCD's L2.
__device__ __forceinline__ bool decode_expert_tile(int bid, int tiles_per_expert, int E, int &e, int &tile)
{
    int xcd = bid & 7, slot = bid >> 3;
    int eg = slot / tiles_per_expert;
    tile = slot - eg * tiles_per_expert;
    e = eg * 8 + xcd;
    return e < E;
}

// The other choice: consecutive row tiles of all experts share an XCD (row tile = 8*group +
// id % 8), so the source rows of a batch element, which several experts pick, are fetched into
// one L2 only, at the price of every XCD fetching every W[e].
__device__ __forceinline__ bool decode_tile_expert(int bid, int tiles_per_expert, int E, int &e, int &tile)
{
    int xcd = bid & 7, slot = bid >> 3;
    int tg = slot / E;
    e = slot - tg * E;
    tile = tg * 8 + xcd;
    return tile < tiles_per_expert;
}

// The three maps behind one switch.  `rows_share`: 0 = experts map to XCDs (decode_expert_tile); 1 = row tiles map to
// XCDs in groups of eight (decode_tile_expert); 2 or 4 = there are 8 / rows_share row tiles per expert in all, each
// owns rows_share XCDs, and the experts are dealt among those (few row tiles must not leave XCDs without work).
__device__ __forceinline__ bool decode_rows_block(int bid, int rows_share, int tiles_per_expert, int E, int &e, int &tile)
{
    if (rows_share == 0) return decode_expert_tile(bid, tiles_per_expert, E, e, tile);
    if (rows_share == 1) return decode_tile_expert(bid, tiles_per_expert, E, e, tile);
    const int xcd = bid & 7, slot = bid >> 3;
    tile = xcd / rows_share;
    e = slot * rows_share + xcd % rows_share;
    return e < E && tile < tiles_per_expert;
}

}  // namespace egs
