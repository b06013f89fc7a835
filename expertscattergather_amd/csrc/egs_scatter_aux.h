// Helpers around the GEMM-scatter: the inverse routing table (which picks land on which
// token, in a fixed order), the fixed-order row reduction of the deterministic mode, and
// the zero-fill / down-convert passes of the atomic mode.
#pragma once
#include "egs_device.h"
#include <type_traits>

namespace egs {

constexpr int kCsrLdsTokens = 16384;     // token counters kept in LDS up to this T (64 KB)

// token counters live in LDS or, for very long sequences, in global memory; agent-scope
// relaxed atomics keep one lane's update visible to the other lanes' later reads either way
__device__ __forceinline__ int32_t cnt_load(int32_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void cnt_store(int32_t *p, int32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// ---------------------------------------------------------------------------- long segments
// A token picked more than kLongSegment times (hot tokens under skewed routing) is not reduced by
// the thread group that owns its output row: its segment is cut into chunks of kLongSegment
// picks, every chunk is summed by a workgroup of its own into an fp32 partial row, and whichever
// of those workgroups finishes last adds the partial rows in chunk order and writes the output
// row.  Chunk boundaries and the order of the final additions depend only on the routing table,
// so the result is still bitwise reproducible.
//
// Partial rows cross workgroups (and L2s) inside one kernel.  They are written and read with
// device-scope atomic accesses, which go through to memory, and a workgroup counts its arrival
// only after its stores have completed; a device-scope fence would do as well, but it writes back
// and invalidates the whole L2 each time, which on skewed routing cost more than the reduction.
//
// The routing-table kernels leave, per batch element, a table of these tokens:
//   tab[0]            number of records
//   tab[4 + 4 r ...]  record r = { token, chunks, first partial-row slot, arrival counter }
// Records and slots are handed out in whatever order the threads get there; nothing downstream
// depends on that order.
constexpr int kLongSegment = 64;
__host__ __device__ inline int long_max_records(int N) { return N / kLongSegment + 1; }
__host__ __device__ inline int long_max_slots(int N) { return 2 * (N / kLongSegment) + 2; }
__host__ __device__ inline size_t long_tab_stride(int N) { return 4 + 4 * (size_t)long_max_records(N); }

// Called by every thread of the workgroup that built batch element b's segment offsets, after
// those are final in global memory (`seg_off_b` = that element's T+1 offsets).
__device__ __forceinline__ void emit_long_tokens(const int32_t *seg_off_b, int T, int N, int32_t *long_tab, int b, int tid,
                                                 int nthreads)
{
    __shared__ int32_t long_ctr[2];
    if (long_tab == nullptr) return;
    int32_t *tab = long_tab + (size_t)b * long_tab_stride(N);
    if (tid == 0) { long_ctr[0] = 0; long_ctr[1] = 0; }
    __syncthreads();            // also orders the seg_off stores of the other threads before the loads below
    for (int t = tid; t < T; t += nthreads) {
        const int len = seg_off_b[t + 1] - seg_off_b[t];
        if (len > kLongSegment) {
            const int nch = (len + kLongSegment - 1) / kLongSegment;
            const int r = atomicAdd(&long_ctr[0], 1);
            const int slot = atomicAdd(&long_ctr[1], nch);
            int32_t *rec = tab + 4 + 4 * r;
            rec[0] = t; rec[1] = nch; rec[2] = slot; rec[3] = 0;
        }
    }
    __syncthreads();
    if (tid == 0) tab[0] = long_ctr[0];
}

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane)
{
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        int o = __shfl_up(v, d, kWave);
        if (lane >= d) v += o;
    }
    return v;
}

// Routing table of one batch element: its [N = E*K] picks in a stable order by token,
//   seg_off[b][t] .. seg_off[b][t+1]  = sorted positions of the picks that selected token t
//   perm[b][s]                        = pick q = e*K + k at sorted position s, increasing inside
//                                       a token's segment (picks with a bad index are left out)
// Stability is what fixes the summation order of the deterministic scatter.
//
// General version: one wavefront per batch element does a counting sort.  Ranks inside a
// 64-pick chunk come from ballots over the bits of the token id, not from atomics, so the
// result does not depend on hardware ordering.  Works for any T and N; slow for large N.
static __global__ __launch_bounds__(kWave) void csr_build_kernel(const void *Ind, int32_t ind_dtype, int32_t T, int32_t N,
                                                          int32_t *seg_off, int32_t *perm, int32_t *cnt_global,
                                                          int32_t *long_tab)
{
    extern __shared__ int32_t cnt_lds[];
    const int lane = (int)threadIdx.x, b = (int)blockIdx.x;
    int32_t *cnt = (T <= kCsrLdsTokens) ? cnt_lds : cnt_global + (size_t)b * T;
    const int64_t base_pick = (int64_t)b * N;

    for (int t = lane; t < T; t += kWave) cnt_store(&cnt[t], 0);
    __syncthreads();
    for (int q0 = 0; q0 < N; q0 += kWave) {
        int q = q0 + lane;
        int32_t t = q < N ? load_token(Ind, ind_dtype, base_pick + q, T) : -1;
        if (t >= 0) atomicAdd(&cnt[t], 1);          // integer counts: order does not matter
    }
    __syncthreads();
    int running = 0;
    for (int t0 = 0; t0 < T; t0 += kWave) {
        int t = t0 + lane;
        int c = t < T ? cnt_load(&cnt[t]) : 0;
        int incl = wave_inclusive_scan(c, lane);
        int excl = running + incl - c;
        if (t < T) {
            seg_off[(size_t)b * (T + 1) + t] = excl;
            cnt_store(&cnt[t], excl);               // becomes the write cursor of token t
        }
        running += __shfl(incl, kWave - 1, kWave);
    }
    if (lane == 0) seg_off[(size_t)b * (T + 1) + T] = running;
    __syncthreads();

    const int nbits = T > 1 ? 32 - __clz(T - 1) : 0;
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    for (int q0 = 0; q0 < N; q0 += kWave) {
        int q = q0 + lane;
        int32_t t = q < N ? load_token(Ind, ind_dtype, base_pick + q, T) : -1;
        uint64_t same = __ballot(t >= 0);
        for (int bit = 0; bit < nbits; ++bit) {
            bool one = (t >> bit) & 1;
            uint64_t bal = __ballot(one);
            same &= one ? bal : ~bal;
        }
        if (t >= 0) {
            int rank = __popcll(same & lt_mask);
            int group = __popcll(same);
            int start = cnt_load(&cnt[t]);
            perm[base_pick + start + rank] = q;
            if (rank == group - 1) cnt_store(&cnt[t], start + group);
        }
        __syncthreads();                             // cursor update visible to the next chunk
    }
    emit_long_tokens(seg_off + (size_t)b * (T + 1), T, N, long_tab, b, lane, kWave);
}

// Fast version when T counters per wavefront fit in LDS: one workgroup of NW wavefronts per
// batch element.  Wavefront w ranks the picks of its contiguous slice against a private
// histogram (ballot matching inside each 64-pick chunk, no atomics), then the per-token counts
// are prefix-summed over wavefronts and over tokens, and every pick goes to
//   start of its token + picks of that token in earlier slices + rank inside its slice.
// LDS (sh_cnt): (NW + 1) * T + 1 int32.  `rank_tmp` is [B][N] scratch (only touched when a wavefront's
// slice exceeds 512 picks).  Picks are read at batch element `b`; results are written at batch element
// `out_b` of seg_off / perm (a caller that keeps them in LDS passes 0 and seg_off = nullptr: the
// offsets are left in sh_cnt[NW * T ..]).  `after_token_loads` runs once the tokens have been decoded, before the
// table is built: a caller's own prefetches belong there, they travel while the table is built and the wait
// for the tokens does not have to cover them.
// `parts` > 1: the batch element's table is built by `parts` workgroups, this one being number `part`.  It ranks only
// its own contiguous share of the picks (so that a wavefront's slice stays in registers where one workgroup's would
// not) and merely counts the others, with LDS atomics: the picks before its share into the first wavefront's
// counters, which therefore start at that count and carry it into every rank and prefix, the picks after its share
// into the token totals.  Every part computes the same offsets; part 0 stores them and lists the long tokens.
struct NoPrefetch { __device__ __forceinline__ void operator()() const {} };

template <class AfterTokenLoads = NoPrefetch>
__device__ __forceinline__ void csr_count_body(int32_t *sh_cnt, int b, int out_b, int tid, int nthreads, const void *Ind,
                                               int32_t ind_dtype, int32_t T, int32_t N, int32_t *seg_off,
                                               int32_t *perm, int32_t *rank_tmp, int32_t *long_tab,
                                               AfterTokenLoads after_token_loads = AfterTokenLoads(), int part = 0, int parts = 1)
{
    constexpr int MAXC = 8;                             // 64-pick chunks whose tokens (and ranks) are held in registers at a time
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), NW = nthreads >> 6;
    int32_t *hist = sh_cnt + (size_t)wave * T;          // this wavefront's counters
    int32_t *tok_start = sh_cnt + (size_t)NW * T;       // [T + 1]
    const int64_t base_pick = (int64_t)b * N;           // where this batch element's picks start in Ind
    const int64_t out_pick = (int64_t)out_b * N;        // ... and in perm / rank_tmp
    const int own = parts > 1 ? (((N + parts - 1) / parts + 63) & ~63) : N;
    const int own_begin = min(N, part * own), own_end = min(N, own_begin + own);
    const int slice = ((own_end - own_begin + NW - 1) / NW + 63) & ~63;
    const int q_begin = own_begin + wave * slice, q_end = min(own_end, q_begin + slice);
    const bool in_regs = slice <= MAXC * kWave;

    // tokens of the slice go in flight before anything else.  Only the loads: decoding a token here would make
    // each (uniformly guarded) load wait for its own result, one trip to memory after the other
    int32_t tk[MAXC], rk[MAXC];
    uint64_t tw[MAXC];
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        tw[c] = 0;
        if (in_regs && c * kWave < slice)        // uniform; within the slice the loads are unconditional so that they overlap
            tw[c] = load_index_word(Ind, ind_dtype, base_pick + min(q_begin + c * kWave + lane, N - 1));
    }

    // every wavefront clears its own counters: they are private until the prefix below, and a wavefront's LDS
    // accesses happen in order, so no barrier is needed before it ranks
    for (int i = lane; i < T; i += kWave) cnt_store(&hist[i], 0);
    __builtin_amdgcn_wave_barrier();
    if (parts > 1) {
        for (int i = tid; i <= T; i += nthreads) cnt_store(&tok_start[i], 0);
        __syncthreads();                                // every counter is clear
        constexpr int U = 16;                           // token loads in flight per thread
        for (int q0 = 0; q0 < N; q0 += U * nthreads) {
            int32_t ft[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int q = q0 + u * nthreads + tid;
                const bool foreign = q < N && (q < own_begin || q >= own_end);
                ft[u] = foreign ? load_token(Ind, ind_dtype, base_pick + q, T) : -1;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int q = q0 + u * nthreads + tid;
                if (ft[u] >= 0) atomicAdd(q < own_begin ? &sh_cnt[ft[u]] : &tok_start[ft[u]], 1);
            }
        }
        __syncthreads();                                // the first wavefront's counters start at the picks before this share
    }
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int q = q_begin + c * kWave + lane;
        int32_t t = -1;
        if (in_regs && c * kWave < slice) {
            const int64_t raw = decode_index_word(tw[c], Ind, ind_dtype, base_pick + min(q, N - 1));
            t = (raw < 0 || raw >= (int64_t)T) ? -1 : (int32_t)raw;
        }
        tk[c] = q < q_end ? t : -1;
        rk[c] = 0;
    }
    // whatever else the caller wants in flight while the table is built.  Only now: the wait for the tokens
    // would otherwise have to cover these loads too (the counter of outstanding loads holds 63 at most).
    // Issuing many loads is bound by the CU's one address path and ranking by VALU issue: the first four
    // wavefronts prefetch and then rank, the others rank first, so that the two overlap on every SIMD
    const bool prefetch_first = (wave & 4) == 0;
    if (prefetch_first) after_token_loads();

    const int nbits = T > 1 ? 32 - __clz(T - 1) : 0;
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    auto rank_chunk = [&](int32_t t) -> int {           // rank of this lane's pick among equal tokens seen so far by this wavefront
        uint64_t same = __ballot(t >= 0);
        for (int bit = 0; bit < nbits; ++bit) {
            const bool one = (t >> bit) & 1;
            const uint64_t bal = __ballot(one);
            same &= one ? bal : ~bal;
        }
        int r = 0;
        if (t >= 0) {
            const int rank = __popcll(same & lt_mask), group = __popcll(same);
            const int start = cnt_load(&hist[t]);
            r = start + rank;
            if (rank == group - 1) cnt_store(&hist[t], start + group);
        }
        __builtin_amdgcn_wave_barrier();
        return r;
    };
    if (in_regs) {
#pragma unroll
        for (int c = 0; c < MAXC; ++c)
            if (q_begin + c * kWave < q_end) rk[c] = rank_chunk(tk[c]);
    } else {
        // long slices: MAXC chunks of tokens in flight at a time, ranks parked in global scratch
        for (int q0 = q_begin; q0 < q_end; q0 += MAXC * kWave) {
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                const int q = q0 + c * kWave + lane;
                const int32_t t = load_token(Ind, ind_dtype, base_pick + min(q, N - 1), T);
                tk[c] = q < q_end ? t : -1;
            }
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                if (q0 + c * kWave >= q_end) break;
                const int r = rank_chunk(tk[c]);
                if (tk[c] >= 0) rank_tmp[out_pick + q0 + c * kWave + lane] = r;
            }
        }
    }
    if (!prefetch_first) after_token_loads();
    __syncthreads();

    // per token: counts -> exclusive prefix over wavefronts; total per token
    // (all counts of a token are read before any is overwritten, so that the reads are in flight together)
    constexpr int kMaxWaves = 16;                       // workgroups have at most 1024 threads
    for (int t = tid; t < T; t += nthreads) {
        int c[kMaxWaves];
#pragma unroll
        for (int w = 0; w < kMaxWaves; ++w) c[w] = w < NW ? sh_cnt[(size_t)w * T + t] : 0;
        int run = 0;
#pragma unroll
        for (int w = 0; w < kMaxWaves; ++w) {
            if (w < NW) sh_cnt[(size_t)w * T + t] = run;
            run += c[w];
        }
        tok_start[t] = parts > 1 ? run + tok_start[t] : run;     // + the picks after this share
    }
    __syncthreads();
    {   // exclusive scan of the totals over tokens: each wavefront scans a contiguous part,
        // then the parts are offset by the totals of the parts before them
        __shared__ int32_t part_total[16];
        const int tw = ((T + NW - 1) / NW + 63) & ~63;
        const int t_begin = wave * tw, t_end = min(T, t_begin + tw);
        int running = 0;
        for (int t0 = t_begin; t0 < t_end; t0 += kWave) {
            const int t = t0 + lane;
            const int c = t < t_end ? tok_start[t] : 0;
            const int incl = wave_inclusive_scan(c, lane);
            if (t < t_end) tok_start[t] = running + incl - c;
            running += __shfl(incl, kWave - 1, kWave);
        }
        if (lane == 0) part_total[wave] = running;
        __syncthreads();
        int before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kMaxWaves; ++w) {
            const int c = w < NW ? part_total[w] : 0;
            if (w < wave) before += c;
            total += c;
        }
        for (int t = t_begin + lane; t < t_end; t += kWave) tok_start[t] += before;
        if (tid == 0) tok_start[T] = total;
    }
    __syncthreads();
    if (seg_off != nullptr && part == 0)
        for (int t = tid; t <= T; t += nthreads) seg_off[(size_t)out_b * (T + 1) + t] = tok_start[t];
    if (in_regs) {
#pragma unroll
        for (int c = 0; c < MAXC; ++c)
            if (tk[c] >= 0) perm[out_pick + tok_start[tk[c]] + hist[tk[c]] + rk[c]] = q_begin + c * kWave + lane;
    } else {
        for (int q0 = q_begin; q0 < q_end; q0 += MAXC * kWave) {
            int32_t rr[MAXC];
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                const int q = q0 + c * kWave + lane;
                const int32_t t = load_token(Ind, ind_dtype, base_pick + min(q, N - 1), T);
                rr[c] = rank_tmp[out_pick + min(q, N - 1)];
                tk[c] = q < q_end ? t : -1;
            }
#pragma unroll
            for (int c = 0; c < MAXC; ++c)
                if (tk[c] >= 0) perm[out_pick + tok_start[tk[c]] + hist[tk[c]] + rr[c]] = q0 + c * kWave + lane;
        }
    }
    if (part == 0) emit_long_tokens(tok_start, T, N, long_tab, out_b, tid, nthreads);
}

// The same table built by TWO workgroups per batch element (`h` = 0 or 1), for the case where it rides in a launch that has
// compute units to spare: the ranking (eight ballot rounds per 64-pick chunk) is what the build consists of, and each
// workgroup ranks only one half of the picks - the lower pick numbers (h = 0) or the upper ones - and merely counts the other
// half with LDS atomics (counts do not depend on the order of arrival).  Both compute the same segment offsets; a token's
// segment lists the lower half's picks before the upper half's, i.e. in increasing pick number as csr_count_body does.
// Workgroup 0 writes seg_off, each writes its half of perm.  LDS: (2 NW + 1) T + 1 int32 (csr_half_lds).  Requires
// N <= NW * 1024 (a wavefront's share of a half in registers) - checked by the host.
__host__ __device__ constexpr size_t csr_half_lds(int T, int nwaves) { return ((size_t)(2 * nwaves + 1) * T + 1) * 4; }

__device__ __forceinline__ void csr_count_half_body(int32_t *sh, int b, int h, int tid, int nthreads, const void *Ind,
                                                    int32_t ind_dtype, int32_t T, int32_t N, int32_t *seg_off, int32_t *perm)
{
    constexpr int MAXC = 8, MAXO = 8;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), NW = nthreads >> 6;
    int32_t *hist = sh + (size_t)wave * T;              // own half: this wavefront's counters
    int32_t *oth = sh + (size_t)(NW + wave) * T;        // other half: this wavefront's counts
    int32_t *tok_start = sh + (size_t)2 * NW * T;       // [T + 1]
    int32_t *own_at = sh + (size_t)NW * T;              // after the prefix: where the own half starts inside a token's segment
    const int split = min(N, ((N + 1) / 2 + 63) & ~63);
    const int own_begin = h ? split : 0, own_end = h ? N : split;
    const int oth_begin = h ? 0 : split, oth_end = h ? split : N;
    const int64_t base_pick = (int64_t)b * N;
    const int slice = ((own_end - own_begin + NW - 1) / NW + 63) & ~63;
    const int q_begin = own_begin + wave * slice, q_end = min(own_end, q_begin + slice);

    int32_t tk[MAXC], rk[MAXC];
    uint64_t tw[MAXC], ow[MAXO];
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        tw[c] = 0;
        if (c * kWave < slice) tw[c] = load_index_word(Ind, ind_dtype, base_pick + min(q_begin + c * kWave + lane, N - 1));
    }
#pragma unroll
    for (int i = 0; i < MAXO; ++i) {
        ow[i] = 0;
        if (oth_begin + i * nthreads < oth_end)         // uniform
            ow[i] = load_index_word(Ind, ind_dtype, base_pick + min(oth_begin + i * nthreads + tid, N - 1));
    }
    for (int i = lane; i < T; i += kWave) { cnt_store(&hist[i], 0); cnt_store(&oth[i], 0); }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int q = q_begin + c * kWave + lane;
        int32_t t = -1;
        if (c * kWave < slice) {
            const int64_t raw = decode_index_word(tw[c], Ind, ind_dtype, base_pick + min(q, N - 1));
            t = (raw < 0 || raw >= (int64_t)T) ? -1 : (int32_t)raw;
        }
        tk[c] = q < q_end ? t : -1;
        rk[c] = 0;
    }
    const int nbits = T > 1 ? 32 - __clz(T - 1) : 0;
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        if (q_begin + c * kWave < q_end) {              // uniform
            const int32_t t = tk[c];
            uint64_t same = __ballot(t >= 0);
            for (int bit = 0; bit < nbits; ++bit) {
                const bool one = (t >> bit) & 1;
                const uint64_t bal = __ballot(one);
                same &= one ? bal : ~bal;
            }
            if (t >= 0) {
                const int rank = __popcll(same & lt_mask), group = __popcll(same);
                const int start = cnt_load(&hist[t]);
                rk[c] = start + rank;
                if (rank == group - 1) cnt_store(&hist[t], start + group);
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
#pragma unroll
    for (int i = 0; i < MAXO; ++i) {
        const int q = oth_begin + i * nthreads + tid;
        if (oth_begin + i * nthreads < oth_end) {
            const int64_t raw = decode_index_word(ow[i], Ind, ind_dtype, base_pick + min(q, N - 1));
            if (q < oth_end && raw >= 0 && raw < (int64_t)T)
                __hip_atomic_fetch_add(&oth[(int32_t)raw], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
    __syncthreads();

    constexpr int kMaxWaves = 16;
    for (int t = tid; t < T; t += nthreads) {
        int c[kMaxWaves], o = 0;
#pragma unroll
        for (int w = 0; w < kMaxWaves; ++w) {
            c[w] = w < NW ? sh[(size_t)w * T + t] : 0;
            o += w < NW ? sh[(size_t)(NW + w) * T + t] : 0;
        }
        int run = 0;
#pragma unroll
        for (int w = 0; w < kMaxWaves; ++w) {
            if (w < NW) sh[(size_t)w * T + t] = run;
            run += c[w];
        }
        tok_start[t] = run + o;
        own_at[t] = h ? o : 0;
    }
    __syncthreads();
    {   // exclusive scan of the totals over tokens, as in csr_count_body
        __shared__ int32_t part_total_half[16];
        const int tw_ = ((T + NW - 1) / NW + 63) & ~63;
        const int t_begin = wave * tw_, t_end = min(T, t_begin + tw_);
        int running = 0;
        for (int t0 = t_begin; t0 < t_end; t0 += kWave) {
            const int t = t0 + lane;
            const int c = t < t_end ? tok_start[t] : 0;
            const int incl = wave_inclusive_scan(c, lane);
            if (t < t_end) tok_start[t] = running + incl - c;
            running += __shfl(incl, kWave - 1, kWave);
        }
        if (lane == 0) part_total_half[wave] = running;
        __syncthreads();
        int before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kMaxWaves; ++w) {
            const int c = w < NW ? part_total_half[w] : 0;
            if (w < wave) before += c;
            total += c;
        }
        for (int t = t_begin + lane; t < t_end; t += kWave) tok_start[t] += before;
        if (tid == 0) tok_start[T] = total;
    }
    __syncthreads();
    if (h == 0)
        for (int t = tid; t <= T; t += nthreads) seg_off[(size_t)b * (T + 1) + t] = tok_start[t];
#pragma unroll
    for (int c = 0; c < MAXC; ++c)
        if (tk[c] >= 0) perm[base_pick + tok_start[tk[c]] + own_at[tk[c]] + hist[tk[c]] + rk[c]] = q_begin + c * kWave + lane;
}


static __global__ __launch_bounds__(1024) void csr_count_kernel(const void *Ind, int32_t ind_dtype, int32_t T, int32_t N,
                                                         int32_t *seg_off, int32_t *perm, int32_t *rank_tmp,
                                                         int32_t *long_tab)
{
    extern __shared__ int32_t sh_cnt_dyn[];
    csr_count_body(sh_cnt_dyn, (int)blockIdx.x, (int)blockIdx.x, (int)threadIdx.x, (int)blockDim.x, Ind, ind_dtype, T, N, seg_off, perm,
                   rank_tmp, long_tab);
}

// Fast version for N <= 32768 picks whose (token, pick) pair fits 32 bits: one workgroup per
// batch element sorts the keys (token << QB | q) with a bitonic network in LDS.  Keys are
// unique, so the sorted order is the stable order by token.  NP = N rounded up to a power of
// two; dynamic LDS = NP * 4 bytes.
static __global__ __launch_bounds__(1024) void csr_sort_kernel(const void *Ind, int32_t ind_dtype, int32_t T, int32_t N,
                                                        int32_t NP, int32_t QB, int32_t *seg_off, int32_t *perm,
                                                        int32_t *long_tab)
{
    extern __shared__ uint32_t keys[];
    const int tid = (int)threadIdx.x, nthreads = (int)blockDim.x, b = (int)blockIdx.x;
    const int64_t base_pick = (int64_t)b * N;
    for (int q = tid; q < NP; q += nthreads) {
        uint32_t key = 0xFFFFFFFFu;
        if (q < N) {
            int32_t t = load_token(Ind, ind_dtype, base_pick + q, T);
            if (t >= 0) key = ((uint32_t)t << QB) | (uint32_t)q;
        }
        keys[q] = key;
    }
    __syncthreads();
    for (int k = 2; k <= NP; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = tid; i < (NP >> 1); i += nthreads) {
                // pair (lo, lo + j) of the j-stride butterfly
                const int lo = ((i & ~(j - 1)) << 1) | (i & (j - 1));
                const int hi = lo + j;
                const bool ascending = (lo & k) == 0;
                const uint32_t x = keys[lo], y = keys[hi];
                if ((x > y) == ascending) { keys[lo] = y; keys[hi] = x; }
            }
            __syncthreads();
        }
    }
    const uint32_t qmask = (1u << QB) - 1u;
    for (int s = tid; s < N; s += nthreads) {
        const uint32_t key = keys[s];
        if (key != 0xFFFFFFFFu) perm[base_pick + s] = (int32_t)(key & qmask);
    }
    // seg_off[t] = number of keys below (t << QB); seg_off[T] = number of valid keys
    for (int t = tid; t <= T; t += nthreads) {
        const uint32_t want = t < T ? ((uint32_t)t << QB) : 0xFFFFFFFFu;
        int lo = 0, hi = NP;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (keys[mid] < want) lo = mid + 1; else hi = mid;
        }
        seg_off[(size_t)b * (T + 1) + t] = lo;
    }
    emit_long_tokens(seg_off + (size_t)b * (T + 1), T, N, long_tab, b, tid, nthreads);
}

// out[b,t,:] = sum, in routing-table order, of the product rows of the picks of token t
// (rows perm[b][s] of P[b], seg_off[t] <= s < seg_off[t+1]); every row of out is written
// exactly once (tokens nobody picked become zero).  P rows hold PT (float, or 16-bit values
// of the element type TT); VW elements per thread.
struct SegSumParams {
    const void *P;              // product rows [B, N, I], fp32 or 16-bit
    const int32_t *seg_off, *perm;
    char *out;                  // [B, T, I]
    int32_t B, T, N, I;
    int32_t tpr_log2;           // 2^tpr_log2 threads share an output row
    int32_t gx, gy;             // logical grid: gx row groups x gy batch slots
    int32_t *long_tab;          // long-segment records (see emit_long_tokens), or nullptr
    float *long_part;           // [B, long_max_slots(N), I] fp32 partial rows
};

template <class TT, class PT, int VW>
__device__ __forceinline__ void segment_sum_body(const SegSumParams &sp, const int bx, const int by)
{
    static_assert(VW == 1 || VW == 4 || VW == 8, "a thread takes 1, 4 or 8 elements of a row");
    // 2^tpr_log2 threads share an output row (VW columns each, looping if the row is wider);
    // bx selects a group of rows of batch element by (+ a stride loop over b)
    const PT *P = reinterpret_cast<const PT *>(sp.P);
    const int32_t *seg_off = sp.seg_off, *perm = sp.perm;
    char *out = sp.out;
    const int B = sp.B, T = sp.T, N = sp.N, I = sp.I, tpr_log2 = sp.tpr_log2;
    const int IV = (I + VW - 1) / VW;
    const int tpr = 1 << tpr_log2;
    const int t = bx * (kThreads >> tpr_log2) + ((int)threadIdx.x >> tpr_log2);
    if (t >= T) return;
    for (int b = by; b < B; b += sp.gy)
    for (int iv = (int)threadIdx.x & (tpr - 1); iv < IV; iv += tpr) {
        const size_t row = (size_t)b * T + t;
        int s0 = seg_off[(size_t)b * (T + 1) + t], s1 = seg_off[(size_t)b * (T + 1) + t + 1];
        if (sp.long_tab != nullptr && s1 - s0 > kLongSegment) continue;      // segment_sum_long_body writes this row
        float acc[VW];
#pragma unroll
        for (int x = 0; x < VW; ++x) acc[x] = 0.f;
        // rows are fetched 4 at a time (their table entries first, then the rows) so that a
        // short segment costs two memory round trips; they are still added in table order
        auto add_row = [&](const PT *src) {
            if constexpr (sizeof(PT) == 4) {
                if constexpr (VW == 4) {
                    f32x4 v = *reinterpret_cast<const f32x4 *>(src);
#pragma unroll
                    for (int x = 0; x < 4; ++x) acc[x] += v[x];
                } else {
                    acc[0] += src[0];
                }
            } else {
                if constexpr (VW == 4) {
                    u32x2 v = *reinterpret_cast<const u32x2 *>(src);
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        uint32_t hbits = (v[x >> 1] >> (16 * (x & 1))) & 0xffffu;
                        acc[x] += TT::ID == 2 ? bf16_bits_to_f32(hbits) : f16_bits_to_f32(hbits);
                    }
                } else {
                    uint32_t hbits = (uint32_t)src[0];
                    acc[0] += TT::ID == 2 ? bf16_bits_to_f32(hbits) : f16_bits_to_f32(hbits);
                }
            }
        };
        const int32_t *pb = perm + (size_t)b * N;
        const PT *Pb = P + (size_t)b * N * I + (size_t)iv * VW;
        int s = s0;
        if constexpr (VW >= 4) {
            struct alignas(16) F32x8 { f32x4 lo, hi; };
            typedef typename std::conditional<sizeof(PT) == 4, typename std::conditional<VW == 8, F32x8, f32x4>::type,
                                              typename std::conditional<VW == 8, u32x4, u32x2>::type>::type vec_t;
            auto add_vec = [&](const vec_t &v) {
                if constexpr (sizeof(PT) == 4 && VW == 8) {
#pragma unroll
                    for (int x = 0; x < 4; ++x) { acc[x] += v.lo[x]; acc[4 + x] += v.hi[x]; }
                } else if constexpr (sizeof(PT) == 4) {
#pragma unroll
                    for (int x = 0; x < 4; ++x) acc[x] += v[x];
                } else {
#pragma unroll
                    for (int x = 0; x < VW; ++x) {
                        uint32_t hbits = (v[x >> 1] >> (16 * (x & 1))) & 0xffffu;
                        acc[x] += TT::ID == 2 ? bf16_bits_to_f32(hbits) : f16_bits_to_f32(hbits);
                    }
                }
            };
            // long segments (hot tokens): 16 rows (256 bytes) in flight per thread; added in table order all the same
            constexpr int LB = sizeof(vec_t) == 32 ? 8 : 16;
            for (; s + LB <= s1; s += LB) {
                int q[LB];
                vec_t v[LB];
#pragma unroll
                for (int u = 0; u < LB; ++u) q[u] = pb[s + u];
#pragma unroll
                for (int u = 0; u < LB; ++u) v[u] = *reinterpret_cast<const vec_t *>(Pb + (size_t)q[u] * I);
#pragma unroll
                for (int u = 0; u < LB; ++u) add_vec(v[u]);
            }
            // 16-bit rows are half the bytes per load: twice the rows per round trip keep as many bytes in flight
            constexpr int RB = sizeof(PT) == 2 ? 8 : 4;
            for (; s < s1; s += RB) {
                const int nb = min(RB, s1 - s);
                int q[RB];
                vec_t v[RB];
#pragma unroll
                for (int u = 0; u < RB; ++u) q[u] = pb[min(s + u, s1 - 1)];
#pragma unroll
                for (int u = 0; u < RB; ++u) v[u] = *reinterpret_cast<const vec_t *>(Pb + (size_t)q[u] * I);
#pragma unroll
                for (int u = 0; u < RB; ++u)
                    if (u < nb) add_vec(v[u]);
            }
        } else {
            for (; s < s1; ++s) add_row(Pb + (size_t)pb[s] * I);
        }
        size_t at = row * I + (size_t)iv * VW;
        if constexpr (TT::ES == 4) {
            float *dst = reinterpret_cast<float *>(out) + at;
            if constexpr (VW >= 4) *reinterpret_cast<f32x4 *>(dst) = f32x4{acc[0], acc[1], acc[2], acc[3]};
            else dst[0] = acc[0];
            if constexpr (VW == 8) *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{acc[4], acc[5], acc[6], acc[7]};
        } else {
            uint16_t *dst = reinterpret_cast<uint16_t *>(out) + at;
            if constexpr (VW == 8) {
                u32x4 w;
#pragma unroll
                for (int x = 0; x < 4; ++x) w[x] = pack2<TT>(acc[2 * x], acc[2 * x + 1]);
                *reinterpret_cast<u32x4 *>(dst) = w;
            } else if constexpr (VW == 4) {
                u32x2 w;
                w[0] = pack2<TT>(acc[0], acc[1]);
                w[1] = pack2<TT>(acc[2], acc[3]);
                *reinterpret_cast<u32x2 *>(dst) = w;
            } else {
                dst[0] = (uint16_t)f32_to_elem_bits<TT>(acc[0]);
            }
        }
    }
}

// One chunk of a long segment: workgroup (b, slot) sums the up to kLongSegment product rows of its
// chunk into partial row `slot`; the workgroup that arrives last at the record's counter adds the
// token's partial rows in chunk order and writes the output row.  Slots no record covers exit.
template <class TT, class PT, int VW>
__device__ __forceinline__ void segment_sum_long_body(const SegSumParams &sp, const int b, const int slot)
{
    __shared__ int32_t sh_rec, sh_last;
    const int tid = (int)threadIdx.x;
    const int T = sp.T, N = sp.N, I = sp.I;
    int32_t *tab = sp.long_tab + (size_t)b * long_tab_stride(N);
    const int nrec = tab[0];
    if (nrec == 0) return;
    if (tid == 0) sh_rec = -1;
    __syncthreads();
    for (int r = tid; r < nrec; r += kThreads) {
        const int first = tab[4 + 4 * r + 2], nch = tab[4 + 4 * r + 1];
        if (slot >= first && slot < first + nch) sh_rec = r;
    }
    __syncthreads();
    const int r = sh_rec;
    if (r < 0) return;
    int32_t *rec = tab + 4 + 4 * r;
    const int t = rec[0], nch = rec[1], first = rec[2];
    const int c = slot - first;
    const int seg0 = sp.seg_off[(size_t)b * (T + 1) + t], seg1 = sp.seg_off[(size_t)b * (T + 1) + t + 1];
    const int s0 = seg0 + c * kLongSegment, s1 = min(seg1, s0 + kLongSegment);
    const int IV = (I + VW - 1) / VW;
    const PT *P = reinterpret_cast<const PT *>(sp.P);
    const int32_t *pb = sp.perm + (size_t)b * N;
    const size_t slots = (size_t)long_max_slots(N);
    float *part = sp.long_part + ((size_t)b * slots + slot) * I;

    for (int iv = tid; iv < IV; iv += kThreads) {
        const PT *Pb = P + (size_t)b * N * I + (size_t)iv * VW;
        float acc[VW];
#pragma unroll
        for (int x = 0; x < VW; ++x) acc[x] = 0.f;
        auto add_elems = [&](const PT *src) {
#pragma unroll
            for (int x = 0; x < VW; ++x) {
                if constexpr (sizeof(PT) == 4) acc[x] += src[x];
                else acc[x] += TT::ID == 2 ? bf16_bits_to_f32((uint32_t)src[x]) : f16_bits_to_f32((uint32_t)src[x]);
            }
        };
        int s = s0;
        for (; s + 8 <= s1; s += 8) {                    // 8 rows in flight, added in table order
            int q[8];
            PT v[8][VW];
#pragma unroll
            for (int u = 0; u < 8; ++u) q[u] = pb[s + u];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const PT *src = Pb + (size_t)q[u] * I;
                if constexpr (VW == 4) {
                    typedef typename std::conditional<sizeof(PT) == 4, f32x4, u32x2>::type vec_t;
                    *reinterpret_cast<vec_t *>(v[u]) = *reinterpret_cast<const vec_t *>(src);
                } else {
                    v[u][0] = src[0];
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) add_elems(v[u]);
        }
        for (; s < s1; ++s) {
            const PT *src = Pb + (size_t)pb[s] * I;
            PT v[VW];
#pragma unroll
            for (int x = 0; x < VW; ++x) v[x] = src[x];
            add_elems(v);
        }
        if constexpr (VW == 4) {
            uint64_t *dst = reinterpret_cast<uint64_t *>(part + (size_t)iv * 4);
            __hip_atomic_store(dst, (uint64_t)f32_bits(acc[0]) | ((uint64_t)f32_bits(acc[1]) << 32), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(dst + 1, (uint64_t)f32_bits(acc[2]) | ((uint64_t)f32_bits(acc[3]) << 32), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        } else {
            __hip_atomic_store(part + iv, acc[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // Hand-off to the workgroup that arrives last.  The partial-row stores above are agent-scope atomic stores:
    // they bypass this XCD's non-coherent cache state and are acknowledged by the memory side.  The wait below
    // (stores count on the vector-memory counter) returns once this thread's stores have been acknowledged, and
    // as a volatile statement with a memory clobber it also keeps the compiler from moving any of them past it.
    // The barrier then orders every thread's acknowledged stores before thread 0's arrival count, which is an
    // agent-scope read-modify-write at the same memory side; a workgroup that observes nch - 1 there therefore
    // reads, with agent-scope loads that also go to the memory side, rows that are complete.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0)
        sh_last = (__hip_atomic_fetch_add(&rec[3], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nch - 1) ? 1 : 0;
    __syncthreads();
    if (!sh_last) return;
    const float *pt = sp.long_part + ((size_t)b * slots + first) * I;
    for (int iv = tid; iv < IV; iv += kThreads) {
        float acc[VW];
#pragma unroll
        for (int x = 0; x < VW; ++x) acc[x] = 0.f;
        // eight partial rows in flight at a time; added in chunk order all the same
        for (int c0 = 0; c0 < nch; c0 += 8) {
            if constexpr (VW == 4) {
                uint64_t lo[8], hi[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const float *src = pt + (size_t)min(c0 + u, nch - 1) * I + (size_t)iv * VW;
                    lo[u] = __hip_atomic_load(reinterpret_cast<const uint64_t *>(src), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    hi[u] = __hip_atomic_load(reinterpret_cast<const uint64_t *>(src) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (c0 + u < nch) {
                        acc[0] += bits_f32((uint32_t)lo[u]); acc[1] += bits_f32((uint32_t)(lo[u] >> 32));
                        acc[2] += bits_f32((uint32_t)hi[u]); acc[3] += bits_f32((uint32_t)(hi[u] >> 32));
                    }
            } else {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    v[u] = __hip_atomic_load(pt + (size_t)min(c0 + u, nch - 1) * I + iv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (c0 + u < nch) acc[0] += v[u];
            }
        }
        const size_t at = ((size_t)b * T + t) * I + (size_t)iv * VW;
        if constexpr (TT::ES == 4) {
            float *dst = reinterpret_cast<float *>(sp.out) + at;
            if constexpr (VW == 4) *reinterpret_cast<f32x4 *>(dst) = f32x4{acc[0], acc[1], acc[2], acc[3]};
            else dst[0] = acc[0];
        } else {
            uint16_t *dst = reinterpret_cast<uint16_t *>(sp.out) + at;
            if constexpr (VW == 4) {
                u32x2 w;
                w[0] = pack2<TT>(acc[0], acc[1]);
                w[1] = pack2<TT>(acc[2], acc[3]);
                *reinterpret_cast<u32x2 *>(dst) = w;
            } else {
                dst[0] = (uint16_t)f32_to_elem_bits<TT>(acc[0]);
            }
        }
    }
}

// workgroups [0, B * long_max_slots(N)): chunks of long segments (first, because they are the longest
// dependent chains of the launch); then gx * gy workgroups for the ordinary rows
template <class TT, class PT, int VW>
__device__ __forceinline__ void segment_sum_dispatch(const SegSumParams &sp, const int block)
{
    const int slots = long_max_slots(sp.N);
    const int long_blocks = sp.B * slots;
    if (block < long_blocks) {
        segment_sum_long_body<TT, PT, (VW == 8 ? 4 : VW)>(sp, block / slots, block % slots);   // its partial rows are laid out for 4
    } else {
        const int sb = block - long_blocks;
        segment_sum_body<TT, PT, VW>(sp, sb % sp.gx, sb / sp.gx);
    }
}

template <class TT, class PT, int VW>
__global__ __launch_bounds__(kThreads) void segment_sum_kernel(SegSumParams sp)
{
    segment_sum_dispatch<TT, PT, VW>(sp, (int)blockIdx.x);
}

// zero n floats (the atomic mode's accumulator).  A kernel rather than a memset so that the
// call sequence can be captured into a graph.  `vec` = dst is 16-byte aligned.
static __global__ __launch_bounds__(kThreads) void fill_zero_f32_kernel(float *dst, size_t n, int vec)
{
    const size_t n4 = vec ? n / 4 : 0;
    const size_t gid = (size_t)blockIdx.x * kThreads + threadIdx.x, stride = (size_t)gridDim.x * kThreads;
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    for (size_t i = gid; i < n4; i += stride) reinterpret_cast<f32x4 *>(dst)[i] = z;
    for (size_t i = n4 * 4 + gid; i < n; i += stride) dst[i] = 0.f;
}

// fp32 accumulator -> 16-bit output element type, n elements.  `vec` = dst is 8-byte aligned
// (src is a 256-byte aligned workspace).
template <class TT>
__global__ __launch_bounds__(kThreads) void downconvert_kernel(const float *src, uint16_t *dst, size_t n, int vec)
{
    const size_t n4 = vec ? n / 4 : 0;
    const size_t gid = (size_t)blockIdx.x * kThreads + threadIdx.x, stride = (size_t)gridDim.x * kThreads;
    for (size_t i = gid; i < n4; i += stride) {
        f32x4 v = reinterpret_cast<const f32x4 *>(src)[i];
        u32x2 w;
        w[0] = pack2<TT>(v[0], v[1]);
        w[1] = pack2<TT>(v[2], v[3]);
        reinterpret_cast<u32x2 *>(dst)[i] = w;
    }
    for (size_t i = n4 * 4 + gid; i < n; i += stride) dst[i] = (uint16_t)f32_to_elem_bits<TT>(src[i]);
}

static __global__ __launch_bounds__(kThreads) void validate_indices_kernel(const void *Ind, int32_t ind_dtype, int64_t n,
                                                                    int32_t T, int32_t *bad)
{
    int local = 0;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
        int64_t t = load_index_raw(Ind, ind_dtype, i);
        local += (t < 0 || t >= (int64_t)T) ? 1 : 0;
    }
    if (local) atomicAdd(bad, local);
}

}  // namespace egs
