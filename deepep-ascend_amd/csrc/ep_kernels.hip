// Device code object for the EP dispatch/combine path on gfx950 (wave64).  Built ahead of time with
// `hipcc --genco` and launched by the host runtime through hipModuleLaunchKernel.
//
// Kernels (all HBM-bound, no MFMA):
//   ep_layout_count / ep_layout_assign (/ ep_layout_scan)  stable counting sort of the (token, slot)
//       entries by destination partition and by local expert -> every handle tensor; with several
//       partitions once on the send side (slots in the destinations' regions) and once on the receive
//       side (slots of the rows that arrived).  Two launches up to a few hundred workgroups (the
//       assignment sums the histograms of the workgroups before it itself), three beyond.
//   ep_scatter_copy / ep_scatter_quant                     token (or receive-stream row) -> its expanded slots
//   ep_scatter_copy_pack / ep_scatter_quant_pack           token -> one packed row per destination partition
//   ep_sf_transpose                                        scale rows -> scale columns
//   ep_quant_rows                                          the quantiser alone (rows in place)
//   ep_combine_k<K> / ep_combine_generic                   K-way gather + fp32 reduce back to token order
//   ep_combine_partial_* / ep_combine_final_*              the same reduce in its owner-side and token-side halves
//   ep_fp8_selftest                                        hardware vs integer e4m3fn conversion
// (The calibration code object of the benchmarks, ep_calib.hip, includes this file and instantiates some of
// its bodies once more; nothing of it is built into this code object.)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ep_args.h"
#include "ep_fp8.h"

#define WAVE 64

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// Streaming stores of the row kernels.  The policy bits of the store instruction (sc0, sc1 = scope,
// nt = non-temporal) decide how the L2 treats the lines; which combination moves rows fastest is a
// measured choice per kernel (EP_*_ST_POL below; bit 0 = nt, bit 1 = sc0, bit 2 = sc1).
template <int POL>
__device__ __forceinline__ void stream_store(u32x4* p, u32x4 v) {
    if (POL == 0) *p = v;
    else if (POL == 1) __builtin_nontemporal_store(v, p);
    else if (POL == 2) asm volatile("global_store_dwordx4 %0, %1, off sc0" ::"v"(p), "v"(v) : "memory");
    else if (POL == 3) asm volatile("global_store_dwordx4 %0, %1, off sc0 nt" ::"v"(p), "v"(v) : "memory");
    else if (POL == 4) asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
    else if (POL == 5) asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" ::"v"(p), "v"(v) : "memory");
    else if (POL == 6) asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
    else asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt" ::"v"(p), "v"(v) : "memory");
}
template <int POL>
__device__ __forceinline__ void stream_store(u32x2* p, u32x2 v) {
    if (POL == 0) *p = v;
    else if (POL == 1) __builtin_nontemporal_store(v, p);
    else if (POL == 2) asm volatile("global_store_dwordx2 %0, %1, off sc0" ::"v"(p), "v"(v) : "memory");
    else if (POL == 3) asm volatile("global_store_dwordx2 %0, %1, off sc0 nt" ::"v"(p), "v"(v) : "memory");
    else if (POL == 4) asm volatile("global_store_dwordx2 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
    else if (POL == 5) asm volatile("global_store_dwordx2 %0, %1, off sc1 nt" ::"v"(p), "v"(v) : "memory");
    else if (POL == 6) asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
    else asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1 nt" ::"v"(p), "v"(v) : "memory");
}
#ifndef EP_SCATTER_ST_POL
#define EP_SCATTER_ST_POL 1
#endif
#ifndef EP_PAD_ST_POL
#define EP_PAD_ST_POL 1
#endif
#ifndef EP_COMBINE_ST_POL
#define EP_COMBINE_ST_POL 1
#endif

__device__ __forceinline__ int lane_id() { return threadIdx.x & (WAVE - 1); }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }
__device__ __forceinline__ int align_up(int x, int a) { return (x + a - 1) / a * a; }

__device__ __forceinline__ int readlane(int v, int l) { return __builtin_amdgcn_readlane(v, l); }

// Lanes of the wave holding the same key.  Every lane must call it; `key` < 2^nbits.
__device__ __forceinline__ uint64_t match_any(int key, int nbits) {
    uint64_t peers = ~0ull;
    for (int b = 0; b < nbits; ++b) {
        const bool bit = (key >> b) & 1;
        const uint64_t ones = __ballot(bit);
        peers &= bit ? ones : ~ones;
    }
    return peers;
}

__device__ __forceinline__ int wave_inclusive_sum(int v) {
    const int lane = lane_id();
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) {
        const int o = __shfl_up(v, off, WAVE);
        if (lane >= off) v += o;
    }
    return v;
}

// ------------------------------------------------------------------------------------------------
// Entries of the layout passes: (token, j) of topk_idx on the send side, (row, j) of the receive
// stream on the receive side.
// ------------------------------------------------------------------------------------------------
// Receive side: inclusive row counts per source partition from the inbox, in LDS.  Every thread of
// the workgroup calls it (blockDim >= R); returns the length of the receive stream.  s_psum holds
// R + blockDim/64 ints.
__device__ __forceinline__ int recv_scan_sources(const EpLayoutArgs& a, int* s_psum) {
    const int R = a.num_ranks, tid = threadIdx.x, lane = lane_id(), w = wave_id();
    int* s_w = s_psum + R;
    int v = 0;
    if (tid < R) v = max(0, min(a.inbox[tid], a.max_tokens));
    const int incl = wave_inclusive_sum(v);
    if (lane == WAVE - 1) s_w[w] = incl;
    __syncthreads();
    int off = 0;
    for (int i = 0; i < w; ++i) off += s_w[i];
    if (tid < R) s_psum[tid] = off + incl;
    __syncthreads();
    return s_psum[R - 1];
}

// Row g of the receive stream (the regions of the source partitions one after the other, each up to
// its row count: the PSumIterator of dispatch_copy_epilogue.hpp:130-174) -> packed row index.
__device__ __forceinline__ int64_t recv_packed_row(const int* psum, int R, int max_tokens, int g) {
    int lo = 0, hi = R - 1;                       // first source whose inclusive count exceeds g
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (psum[mid] > g) hi = mid; else lo = mid + 1;
    }
    return (int64_t)lo * max_tokens + (g - (lo ? psum[lo - 1] : 0));
}

// Stages the expert ids of this workgroup's entries.  Send side: entry (t, j) of topk_idx.  Receive
// side: entry (row, j) of the receive stream, read from the packed row; partitions play no role there.
// num_rows: rows (tokens) the entries range over (layout_num_rows).
// (recv: a.recv_mode, or the constant an instance of the slot assignment was built for)
__device__ __forceinline__ int layout_num_rows(const EpLayoutArgs& a, int* s_psum, bool recv) {
    return recv ? recv_scan_sources(a, s_psum) : a.num_tokens;
}
__device__ __forceinline__ void layout_load_keys(const EpLayoutArgs& a, short* s_key, short* s_rk, const int* s_psum,
                                                 int num_rows, bool recv, int block) {
    const int K = a.num_topk;
    const int n = EP_TOKENS_PER_BLOCK * K;
    if (recv) {
        const int N = num_rows;
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const int row = i / K, j = i - row * K;
            const int g = block * EP_TOKENS_PER_BLOCK + row;
            int e = -1;
            if (g < N) {
                const int64_t pr = recv_packed_row(s_psum, a.num_ranks, a.max_tokens, g);
                const int64_t v = ((const int64_t*)(a.packed_base + pr * a.packed_row_bytes + a.idx_off))[j];
                e = (v >= 0 && v < a.num_experts) ? (int)v : -1;
            }
            s_key[i] = (short)e;
            s_rk[i] = -1;
        }
        return;
    }
    const int64_t base = (int64_t)block * n;
    const int64_t total = (int64_t)a.num_tokens * K;
    if (total <= 0) {
        for (int i = threadIdx.x; i < n; i += blockDim.x) s_key[i] = s_rk[i] = -1;
        return;
    }
    // four loads a thread in flight, none under a per-lane condition (an entry past the end re-reads the last one
    // and is masked): the ids come from memory, and one trip for a workgroup's entries is all this pass waits for
    for (int i0 = threadIdx.x; i0 < n; i0 += 4 * blockDim.x) {
        int64_t v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = a.topk_idx[min(base + i0 + u * (int)blockDim.x, total - 1)];
        __builtin_amdgcn_sched_barrier(0);      // (the scheduler otherwise uses the first value before it issues the other loads)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = i0 + u * (int)blockDim.x;
            if (i >= n) break;
            const int e = (base + i < total && v[u] >= 0 && v[u] < a.num_experts) ? (int)v[u] : -1;
            s_key[i] = (short)e;
            s_rk[i] = (short)(e < 0 ? -1 : e / a.experts_per_rank);
        }
    }
}

// Destination partition of entry idx if it is the last slot of its token going there, else -1
// (the "master" of common/simt.hpp:24-34).
__device__ __forceinline__ int master_rank(const short* s_rk, int idx, int j, int K) {      // j = idx % K
    const int r = s_rk[idx];
    if (r < 0) return -1;
    for (int jj = j + 1; jj < K; ++jj)
        if (s_rk[idx - j + jj] == r) return -1;
    return r;
}

// ------------------------------------------------------------------------------------------------
// Layout pass A: per-block histograms of expert ids and of destination-partition masters.
// Reference semantics: impls/ep/dispatch.hpp:166-194 (expert histogram, dedup by partition).
// ------------------------------------------------------------------------------------------------
extern "C" __global__ __launch_bounds__(EP_LAYOUT_THREADS) void ep_layout_count(EpLayoutArgs a) {
    extern __shared__ int smem[];
    const int E = a.num_experts, R = a.num_ranks, K = a.num_topk;
    int* s_ecnt = smem;                 // [E]
    int* s_rcnt = s_ecnt + E;           // [R]
    short* s_key = (short*)(s_rcnt + R);
    short* s_rk = s_key + EP_TOKENS_PER_BLOCK * K;
    int* s_psum = (int*)(s_rk + EP_TOKENS_PER_BLOCK * K);      // [R + waves]  (receive side)
    for (int i = threadIdx.x; i < E + R; i += blockDim.x) smem[i] = 0;
    const int num_rows = layout_num_rows(a, s_psum, a.recv_mode != 0);
    // the scan stops at the last workgroup that has rows: the ones behind it leave nothing
    if ((int)blockIdx.x > 0 && (int)blockIdx.x * EP_TOKENS_PER_BLOCK >= num_rows) return;
    layout_load_keys(a, s_key, s_rk, s_psum, num_rows, a.recv_mode != 0, blockIdx.x);
    __syncthreads();
    const int n = EP_TOKENS_PER_BLOCK * K;
    // (the position of an entry inside its token is carried along: a division by a run-time top-k is forty instructions)
    int j = (int)threadIdx.x % K;
    const int jstep = (int)blockDim.x % K;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int e = s_key[i];
        if (e >= 0) atomicAdd(&s_ecnt[e], 1);
        const int mr = master_rank(s_rk, i, j, K);
        if (mr >= 0) atomicAdd(&s_rcnt[mr], 1);
        j += jstep;
        if (j >= K) j -= K;
    }
    __syncthreads();
    // one row of the count matrix: this partition's experts, then the partitions, then zero fill.  For the scan kernel
    // the counts are ints; the slot assignment that sums the rows itself takes them as 16-bit halves (a count is at
    // most EP_TOKENS_PER_BLOCK * EP_MAX_TOPK = 4096), eight columns a 16-byte load and two columns an add.
    const int El = a.experts_per_rank, lo = a.rank_idx * El;
    if (a.scan_mode == EP_LAYOUT_FOLDED) {
        unsigned* row = (unsigned*)a.blk_cnt + (int64_t)blockIdx.x * (a.cnt_stride >> 1);
        auto count_of = [&](int i) -> unsigned { return i < El ? s_ecnt[lo + i] : (i < El + R ? s_rcnt[i - El] : 0); };
        for (int i = threadIdx.x; i < (a.cnt_stride >> 1); i += blockDim.x) row[i] = count_of(2 * i) | count_of(2 * i + 1) << 16;
        return;
    }
    int* row = a.blk_cnt + (int64_t)blockIdx.x * a.cnt_stride;
    for (int i = threadIdx.x; i < a.cnt_stride; i += blockDim.x)
        row[i] = i < El ? s_ecnt[lo + i] : (i < El + R ? s_rcnt[i - El] : 0);
}

// ------------------------------------------------------------------------------------------------
// Layout pass B: exclusive prefix over the workgroups of pass A for every histogram column, plus
// column totals.  One workgroup owns 16 columns; its 1024 threads are 64 row groups x 16 columns, a
// thread walks the rows of its group (consecutive threads read consecutive columns of one row).
// ------------------------------------------------------------------------------------------------
#define EP_SCAN_COLS 16
#define EP_SCAN_GROUPS (EP_SCAN_THREADS / EP_SCAN_COLS)

extern "C" __global__ __launch_bounds__(EP_SCAN_THREADS) void ep_layout_scan(EpLayoutArgs a) {
    __shared__ int s_part[EP_SCAN_GROUPS][EP_SCAN_COLS + 1];
    __shared__ int s_rows;
    const int R = a.num_ranks, W = a.cnt_stride;
    int B = a.num_blocks;
    if (a.recv_mode) {
        // rows exist only up to the length of the receive stream
        if (threadIdx.x == 0) s_rows = 0;
        __syncthreads();
        if ((int)threadIdx.x < R) atomicAdd(&s_rows, max(0, min(a.inbox[threadIdx.x], a.max_tokens)));
        __syncthreads();
        B = min(B, max(1, (s_rows + EP_TOKENS_PER_BLOCK - 1) / EP_TOKENS_PER_BLOCK));
    }
    const int c = threadIdx.x % EP_SCAN_COLS, g = threadIdx.x / EP_SCAN_COLS;
    const int col = blockIdx.x * EP_SCAN_COLS + c;
    const bool live = col < W;
    int* base = a.blk_cnt + col;
    const int rpg = (B + EP_SCAN_GROUPS - 1) / EP_SCAN_GROUPS;
    const int r0 = min(B, g * rpg), r1 = min(B, r0 + rpg);
    int sum = 0;
    if (live)
        for (int r = r0; r < r1; ++r) sum += base[(int64_t)r * W];
    s_part[g][c] = sum;
    __syncthreads();
    int off = 0, total = 0;
    for (int i = 0; i < EP_SCAN_GROUPS; ++i) {
        const int v = s_part[i][c];
        if (i < g) off += v;
        total += v;
    }
    if (live) {
        int run = off;
        for (int r = r0; r < r1; ++r) {
            const int v = base[(int64_t)r * W];
            base[(int64_t)r * W] = run;
            run += v;
        }
        if (g == 0) a.col_total[col] = total;
    }
}

// ------------------------------------------------------------------------------------------------
// Layout pass C: slot of every entry.
//   dst_buffer_slot_idx[t,j] = number of earlier tokens with a master for the same partition
//                               (masters only)                       -- impls/ep/dispatch.hpp:258-281
//   slot_map[t,j]            = expert_start[e] + number of earlier (t',j') entries with the same
//                               local expert (lexicographic order)    -- dispatch_copy_epilogue.hpp:471-488
//                               with the canonical order of deep_ep/buffers/ep.py:100-160
// One workgroup (the only one, or one launched beside the ranking ones) publishes the per-partition / per-expert
// counts and prefix sums (impls/ep/dispatch.hpp:469-545) and, when asked, the host count page.
//
// Where the counts of the other blocks come from (a.scan_mode):
//   EP_LAYOUT_SCANNED  ep_layout_scan left exclusive prefixes in blk_cnt and totals in col_total
//   EP_LAYOUT_FOLDED   ep_layout_count left plain counts in blk_cnt (16-bit halves): every block sums the rows
//                      before it itself (cheaper than a launch of its own up to a few hundred blocks)
//   EP_LAYOUT_SINGLE   one block owns every token: nothing ran before, its own LDS counts are the totals
//   EP_LAYOUT_RECOUNTED  a few blocks of one partition: nothing ran before, every workgroup counts the ids of all
//                      blocks itself (a launch less; the ids of 1024 tokens are 48 KB)
// Only the local experts and the partitions need prefixes: slots of other experts are never used.
// ------------------------------------------------------------------------------------------------
#define EP_FOLD_DEPTH 22
#define EP_KEY_MASTER 0x4000          // flag in a staged key: the entry is the master of its partition (ids < 2048)
#define EP_LAYOUT_MAX_COLS_PER_THREAD ((EP_MAX_EXPERTS + EP_MAX_RANKS + EP_LAYOUT_THREADS - 1) / EP_LAYOUT_THREADS)

// Four instances.  FOLD: for EP_LAYOUT_FOLDED (the other modes run one without the summing code).  RECV: for the
// receive side of a node (a.recv_mode).
template <bool FOLD, bool RECV>
__device__ __forceinline__ void layout_assign_body(const EpLayoutArgs& a) {
    extern __shared__ int smem[];
    const int E = a.num_experts, R = a.num_ranks, K = a.num_topk, El = a.experts_per_rank, A = a.expert_alignment;
    const int NW = EP_LAYOUT_THREADS / WAVE;
    const int b = blockIdx.x;
    int* s_tot = smem;                     // [El + R] totals of the local experts, then of the partitions
    int* s_we = s_tot + El + R;            // [NW][E] per-wave counts, then running slot counters
    int* s_wr = s_we + NW * E;             // [NW][R]
    int* s_tmp = s_wr + NW * R;            // [NW + 1]
    short* s_key = (short*)(s_tmp + NW + 1);
    short* s_rk = s_key + EP_TOKENS_PER_BLOCK * K;
    int* s_psum = (int*)(s_rk + EP_TOKENS_PER_BLOCK * K);      // [R + NW]  (receive side)
    const int tid = threadIdx.x, lane = lane_id(), w = wave_id();
    const int lo = a.rank_idx * El;
    const int ncols = El + R;              // column c < El: local expert lo + c; else partition c - El

    // The launch has one workgroup more than blocks of tokens.  It ranks nothing: it gets the totals like the others
    // (a single block: it counts that block's ids once more) and publishes them (handle tensors, inboxes, the host count
    // page with its two system-scope fences), so that no ranking workgroup has that on its way.
    const bool single = !FOLD && a.scan_mode == EP_LAYOUT_SINGLE;     // (the summing instance never runs alone)
    const bool publisher = b == a.num_blocks, worker = !publisher;
    const int kb = single ? 0 : b;         // the block whose ids this workgroup stages
    const int num_rows = layout_num_rows(a, s_psum, RECV);
    if (!publisher && b > 0 && b * EP_TOKENS_PER_BLOCK >= num_rows) return;      // nothing to rank here

    // ---- counts of the workgroups before this one (kept in registers) and totals over all of them ----
    int pre[EP_LAYOUT_MAX_COLS_PER_THREAD], tot[EP_LAYOUT_MAX_COLS_PER_THREAD];
#pragma unroll
    for (int k = 0; k < EP_LAYOUT_MAX_COLS_PER_THREAD; ++k) pre[k] = tot[k] = 0;
    if (!FOLD && a.scan_mode == EP_LAYOUT_SCANNED) {
#pragma unroll
        for (int k = 0; k < EP_LAYOUT_MAX_COLS_PER_THREAD; ++k) {
            const int c = tid + k * EP_LAYOUT_THREADS;
            if (c >= ncols) continue;
            if (worker) pre[k] = a.blk_cnt[(int64_t)b * a.cnt_stride + c];
            tot[k] = a.col_total[c];
        }
    }
    const int nkeys = EP_TOKENS_PER_BLOCK * K;
    const int64_t key_base = (int64_t)kb * nkeys, key_total = (int64_t)a.num_tokens * K;
    // EP_LAYOUT_RECOUNTED (one partition, a few blocks, send side): every workgroup reads the ids of all blocks in one
    // go: a histogram of all of them (the totals), one of the blocks before its own, its own block's ids staged on the
    // way.  With one partition the master of a token is its last valid position: the partition's column counts the
    // tokens that have a valid id at all (flags in LDS, counted by ballot).
    const bool recount = !FOLD && !RECV && a.scan_mode == EP_LAYOUT_RECOUNTED;
    if (recount) {
        int* s_rpre = s_psum + R + NW;                         // [ncols]
        int* s_rtot = s_rpre + ncols;                          // [ncols]
        int* s_any = s_rtot + ncols;                           // [num_blocks * EP_TOKENS_PER_BLOCK / 4] one byte a token
        unsigned char* s_anyb = (unsigned char*)s_any;
        const int ntok_all = a.num_blocks * EP_TOKENS_PER_BLOCK, n_all = a.num_blocks * nkeys;
        for (int i = tid; i < 2 * ncols + ntok_all / 4; i += blockDim.x) s_rpre[i] = 0;
        for (int i = tid; i < NW * (E + R); i += blockDim.x) s_we[i] = 0;
        for (int i = tid; i < nkeys; i += blockDim.x) s_key[i] = s_rk[i] = -1;
        __syncthreads();
        if (key_total > 0) {
            // (token and position of an id are carried along from load to load instead of divided out)
            const int tok_step = EP_LAYOUT_THREADS / K, pos_step = EP_LAYOUT_THREADS - tok_step * K;
            int tok = tid / K, pos = tid - tok * K;
            // all ids at once, in up to three goes of eight a thread (as many as there are blocks to read: the same in
            // every thread, so that a short launch neither asks for nor looks at the rest)
            constexpr int GO = EP_RECOUNT_DEPTH / 3;
            const int goes = (n_all + GO * EP_LAYOUT_THREADS - 1) / (GO * EP_LAYOUT_THREADS);      // 1..3 (the host's limit)
            int64_t v[3][GO];
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                if (c >= goes) break;
#pragma unroll
                for (int u = 0; u < GO; ++u) v[c][u] = a.topk_idx[min((int64_t)tid + (c * GO + u) * EP_LAYOUT_THREADS, key_total - 1)];
            }
            __builtin_amdgcn_sched_barrier(0);      // (every id is asked for before the first is looked at)
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                if (c >= goes) break;
#pragma unroll
                for (int u = 0; u < GO; ++u) {
                    const int i = tid + (c * GO + u) * EP_LAYOUT_THREADS;
                    const bool valid = i < n_all && i < key_total && v[c][u] >= 0 && v[c][u] < a.num_experts;
                    const int e = valid ? (int)v[c][u] : -1;
                    if (valid) {
                        atomicAdd(&s_rtot[e], 1);
                        if (i < b * nkeys) atomicAdd(&s_rpre[e], 1);
                        s_anyb[tok] = 1;
                    }
                    const int own = i - b * nkeys;
                    if (own >= 0 && own < nkeys) {
                        s_key[own] = (short)e;
                        s_rk[own] = (short)(valid ? 0 : -1);
                    }
                    tok += tok_step;
                    pos += pos_step;
                    if (pos >= K) { pos -= K; ++tok; }
                }
            }
        }
        __syncthreads();
        for (int t0 = 0; t0 < ntok_all; t0 += blockDim.x) {
            const int t = t0 + tid;
            const bool any = t < ntok_all && s_anyb[t] != 0;
            const int all = __popcll(__ballot(any)), before = __popcll(__ballot(any && t < b * EP_TOKENS_PER_BLOCK));
            if (lane == 0 && all > 0) {
                atomicAdd(&s_rtot[El], all);
                if (before > 0) atomicAdd(&s_rpre[El], before);
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < EP_LAYOUT_MAX_COLS_PER_THREAD; ++k) {
            const int c = tid + k * EP_LAYOUT_THREADS;
            if (c >= ncols) continue;
            pre[k] = s_rpre[c];
            tot[k] = s_rtot[c];
        }
    }
    // This workgroup's expert ids are asked for first (send side, up to four ids a thread).
    const bool folded = FOLD;
    const bool keys_early = folded && !RECV && nkeys <= 4 * EP_LAYOUT_THREADS && key_total > 0;
    // EP_LAYOUT_FOLDED: ep_layout_count has finished and left plain counts as 16-bit halves; the rows before this
    // workgroup's (and all rows) are summed here.  A thread takes 8 adjacent columns (one 16-byte load a row) of every
    // S-th row, EP_FOLD_DEPTH loads in flight, and adds them two columns an instruction: each half of the rows in flight
    // has 16-bit sums of its own (EP_FOLD_DEPTH / 2 rows of at most 4096 stay below 2^16), widened at its end; the S
    // partial sums of a column meet in LDS.  The rows come from memory (other XCDs wrote
    // them) and that trip is the longest wait of the kernel: the first turn's rows are asked for here and summed only
    // after the keys have been staged and counted per wave, which needs none of them.
    const int W = a.cnt_stride, FG = W >> 3;
    int* s_fpre = s_psum + R + NW;         // [W]  (EP_LAYOUT_FOLDED only)
    int* s_ftot = s_fpre + W;              // [W]
    const int nb = min(a.num_blocks, max(1, (num_rows + EP_TOKENS_PER_BLOCK - 1) / EP_TOKENS_PER_BLOCK));
    const int S = FG >= EP_LAYOUT_THREADS ? 1 : EP_LAYOUT_THREADS / FG;
    const int s0 = FG >= EP_LAYOUT_THREADS ? 0 : tid / FG;
    const int g0 = FG >= EP_LAYOUT_THREADS ? tid : tid - s0 * FG;
    // (rows are addressed by a 32-bit offset from the uniform base: two instructions a load)
    const unsigned row_bytes = (unsigned)W * 2u, step = (unsigned)S * row_bytes;
    auto fold_loads = [&](u32x4 (&v)[EP_FOLD_DEPTH], int r, int g) {
        const unsigned off = (unsigned)r * row_bytes + 16u * g, last = (unsigned)(nb - 1) * row_bytes + 16u * g;
        // unconditional loads (a row past the end re-reads the last one and is masked in the sums), so that all of
        // them are in flight before the first is waited for
#pragma unroll
        for (int u = 0; u < EP_FOLD_DEPTH; ++u) v[u] = *(const u32x4*)((const char*)a.blk_cnt + min(off + u * step, last));
        __builtin_amdgcn_sched_barrier(0);          // (the scheduler otherwise sums the first rows before it asks for the last)
    };
    auto fold_sums = [&](const u32x4 (&v)[EP_FOLD_DEPTH], int r, int (&p)[8], int (&t)[8]) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            // (a short launch has no rows in the second half of a turn: its adds are skipped)
            if (h == 1 && r + (EP_FOLD_DEPTH / 2) * S >= nb) break;
            u16x2 ts[4], ps[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) ts[q] = ps[q] = u16x2{0, 0};
#pragma unroll
            for (int u = h * (EP_FOLD_DEPTH / 2); u < (h + 1) * (EP_FOLD_DEPTH / 2); ++u) {
                const int rr = r + u * S;
                const unsigned mt = rr < nb ? ~0u : 0u, mp = rr < b ? ~0u : 0u;      // b <= nb - 1
                ts[0] += __builtin_bit_cast(u16x2, v[u].x & mt); ps[0] += __builtin_bit_cast(u16x2, v[u].x & mp);
                ts[1] += __builtin_bit_cast(u16x2, v[u].y & mt); ps[1] += __builtin_bit_cast(u16x2, v[u].y & mp);
                ts[2] += __builtin_bit_cast(u16x2, v[u].z & mt); ps[2] += __builtin_bit_cast(u16x2, v[u].z & mp);
                ts[3] += __builtin_bit_cast(u16x2, v[u].w & mt); ps[3] += __builtin_bit_cast(u16x2, v[u].w & mp);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                t[2 * q] += (int)ts[q].x;
                t[2 * q + 1] += (int)ts[q].y;
                p[2 * q] += (int)ps[q].x;
                p[2 * q + 1] += (int)ps[q].y;
            }
        }
    };
    // (Lanes are 8 columns apart: column 8 g + q lives at 8 g + ((q + g / 4) & 7), which spreads the 32 lanes of one
    //  add over the 32 banks instead of four.)
    auto fold_meet = [&](int g, const int (&p)[8], const int (&t)[8]) {
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const int at = 8 * g + ((q + (g >> 2)) & 7);
            atomicAdd(&s_fpre[at], p[q]);
            atomicAdd(&s_ftot[at], t[q]);
        }
    };
    // (the host sends shapes with more than 8 * EP_LAYOUT_THREADS count columns to the scan kernel: one column group a thread)
    const bool fold_mine = folded && s0 < S && g0 < FG;        // this thread sums rows

    // ---- A: stage this block's keys, clear the per-wave counters (and where the sums of the rows meet) ----
    // Every thread asks for rows and only the ones that sum look at what arrives; both ways through this phase leave
    // the same EP_FOLD_DEPTH loads in flight.  (The compiler counts the loads in flight along every path: with the
    // rows asked for on one path only, or under a per-thread condition, it waits for all of them at the next loop.)
    u32x4 v_first[EP_FOLD_DEPTH];
    auto clear_counters = [&]() {
        for (int i = tid; i < NW * (E + R); i += blockDim.x) s_we[i] = 0;
        if (folded)
            for (int i = tid; i < 2 * W; i += blockDim.x) s_fpre[i] = 0;
    };
    if (keys_early) {
        // ids first, rows behind them; the ids are staged while the rows are on their way
        int64_t pk[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) pk[u] = a.topk_idx[min(key_base + tid + u * EP_LAYOUT_THREADS, key_total - 1)];
        __builtin_amdgcn_sched_barrier(0);
        if (FOLD) fold_loads(v_first, s0, min(g0, FG - 1));
        clear_counters();
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = tid + u * EP_LAYOUT_THREADS;
            if (i >= nkeys) break;
            const int e = (key_base + i < key_total && pk[u] >= 0 && pk[u] < a.num_experts) ? (int)pk[u] : -1;
            s_key[i] = (short)e;
            s_rk[i] = (short)(e < 0 ? -1 : e / a.experts_per_rank);
        }
    } else if (!recount) {            // (recounted: the ids are staged and the counters clear already)
        clear_counters();
        layout_load_keys(a, s_key, s_rk, s_psum, num_rows, RECV, kb);
        if (FOLD) fold_loads(v_first, s0, min(g0, FG - 1));
    }
    __syncthreads();

    // ---- B: per-wave counts: wave w owns entries [w*epw, (w+1)*epw) of this block's chunk ----
    const int n = EP_TOKENS_PER_BLOCK * K;
    const int rounds = (n + EP_LAYOUT_THREADS - 1) / EP_LAYOUT_THREADS;
    const int epw = rounds * WAVE;
    // (token and position of this lane's entry of a round are carried along instead of divided out every round)
    const int tok0 = (w * epw + lane) / K, pos0 = (w * epw + lane) - tok0 * K;
    const int tok_step = WAVE / K, pos_step = WAVE - tok_step * K;
    for (int rd = 0, pos = pos0; rd < rounds; ++rd) {
        const int idx = w * epw + rd * WAVE + lane;
        if (idx < n) {
            const int e = s_key[idx];
            if (e >= 0) atomicAdd(&s_we[w * E + e], 1);
            const int mr = master_rank(s_rk, idx, pos, K);
            if (mr >= 0) {
                atomicAdd(&s_wr[w * R + mr], 1);
                s_key[idx] = (short)(e | EP_KEY_MASTER);        // remembered for the ranking (only this thread reads it)
            }
        }
        pos += pos_step;
        if (pos >= K) pos -= K;
    }

    // ---- the rows asked for at the top: counts of the workgroups before this one, totals over all ----
    if (fold_mine) {
        int p[8], t[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) p[q] = t[q] = 0;
        fold_sums(v_first, s0, p, t);
        for (int r = s0 + EP_FOLD_DEPTH * S; r < nb; r += EP_FOLD_DEPTH * S) {
            u32x4 v[EP_FOLD_DEPTH];
            fold_loads(v, r, g0);
            fold_sums(v, r, p, t);
        }
        fold_meet(g0, p, t);
    }
    __syncthreads();
    if (folded) {
#pragma unroll
        for (int k = 0; k < EP_LAYOUT_MAX_COLS_PER_THREAD; ++k) {
            const int c = tid + k * EP_LAYOUT_THREADS;
            if (c >= ncols) continue;
            const int at = (c & ~7) | ((c + (c >> 5)) & 7);
            pre[k] = s_fpre[at];
            tot[k] = s_ftot[at];
        }
    }

    // ---- C: totals over all workgroups into LDS (one workgroup: its own per-wave counts are the totals) ----
#pragma unroll
    for (int k = 0; k < EP_LAYOUT_MAX_COLS_PER_THREAD; ++k) {
        const int c = tid + k * EP_LAYOUT_THREADS;
        if (c >= ncols) continue;
        if (a.scan_mode == EP_LAYOUT_SINGLE) {
            const bool is_expert = c < El;
            const int* wc = is_expert ? s_we + lo + c : s_wr + (c - El);
            const int stride = is_expert ? E : R;
            int t = 0;
            for (int i = 0; i < NW; ++i) t += wc[i * stride];
            tot[k] = t;
        }
        s_tot[c] = tot[k];
    }
    __syncthreads();

    // ---- D + E: aligned exclusive scan over the local experts (totals are replaced in place by the
    //      first slot of each expert); the publishing workgroup writes the handle tensors and the host count page ----
    int* s_start = s_tot;
    const int per = (El + EP_LAYOUT_THREADS - 1) / EP_LAYOUT_THREADS;
    const int e0 = min(El, tid * per), e1 = min(El, e0 + per);
    int mine = 0;
    for (int e = e0; e < e1; ++e) mine += align_up(s_tot[e], A);
    const int incl = wave_inclusive_sum(mine);
    if (lane == WAVE - 1) s_tmp[w] = incl;
    __syncthreads();
    int wave_off = 0, grand = 0;
    for (int i = 0; i < NW; ++i) {
        if (i < w) wave_off += s_tmp[i];
        grand += s_tmp[i];
    }
    {
        int run = wave_off + incl - mine;
        for (int e = e0; e < e1; ++e) {
            const int c = s_tot[e];
            if (publisher && !a.send_only) {
                a.unaligned_expert[e] = c;
                a.psum_expert[e] = run + c;
                if (a.cumulative_stats != nullptr) atomicAdd(&a.cumulative_stats[e], c);
                if (a.notify_host) a.host_page[EP_HOST_EXPERT_OFF + e] = align_up(c, A);
            }
            s_start[e] = run;
            run += align_up(c, A);
        }
    }
    if (publisher && a.send_only) {
        // rows this partition sends to every partition, left in the receivers' inboxes: the count half of
        // the reference's cross-rank reduction (impls/ep/dispatch.hpp:469-545)
        // (a partition that is not connected to a node only has its own inbox)
        for (int r = tid; r < R; r += blockDim.x)
            if (a.connected || r == a.rank_idx)
                ((int*)(a.peer_arenas[r] + EP_WS_INBOX_OFF))[a.rank_idx] = min(s_tot[El + r], a.max_tokens);
    }
    if (publisher && !a.send_only) {
        // one partition: the receive stream is this partition's own routed tokens; several: the rows counted
        // in the inbox (csrc/buffers/ep.hpp:205-246 names the tensors)
        const int n_recv = RECV ? num_rows : s_tot[El + a.rank_idx];
        for (int r = tid; r < R; r += blockDim.x) {
            const int upto = RECV ? s_psum[r] : n_recv;
            const int from = RECV && r ? s_psum[r - 1] : 0;
            a.psum_rank[r] = upto;
            if (a.notify_host) a.host_page[EP_HOST_RANK_OFF + r] = upto - from;
        }
        if (a.notify_host) {
            __threadfence_system();
            __syncthreads();
            if (tid == 0) {
                a.host_page[1] = n_recv;
                a.host_page[2] = grand;
                __threadfence_system();
                __hip_atomic_store(&a.host_page[0], a.seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
            }
        }
    }
    if (!worker) return;
    __syncthreads();

    // ---- F: counts -> starting slots (global base + blocks before + waves before) ----
#pragma unroll
    for (int k = 0; k < EP_LAYOUT_MAX_COLS_PER_THREAD; ++k) {
        const int c = tid + k * EP_LAYOUT_THREADS;
        if (c >= ncols) continue;
        const bool is_expert = c < El;
        int* wc = is_expert ? s_we + lo + c : s_wr + (c - El);
        const int stride = is_expert ? E : R;
        int run = pre[k] + (is_expert ? s_start[c] : 0);
        for (int i = 0; i < NW; ++i) {
            const int cnt = wc[i * stride];
            wc[i * stride] = run;
            run += cnt;
        }
    }
    __syncthreads();

    // ---- G: stable ranking, 64 consecutive entries per wave per round ----
    const int ebits = 32 - __builtin_clz(E);       // keys+1 in [0, E]
    const int rbits = 32 - __builtin_clz(R);
    const uint64_t lt = (1ull << lane) - 1ull;
    const int64_t total = (int64_t)num_rows * K;
    for (int rd = 0, tok = tok0, pos = pos0; rd < rounds; ++rd) {
        const int idx = w * epw + rd * WAVE + lane;
        const bool in = idx < n;
        const int key = in ? s_key[idx] : -1;
        const int e = key < 0 ? -1 : key & (EP_KEY_MASTER - 1);
        const int le = e - lo;
        const bool local = e >= 0 && le >= 0 && le < El;
        const int mr = (key >= 0 && (key & EP_KEY_MASTER)) ? s_rk[idx] : -1;
        const uint64_t pe = match_any(local ? e + 1 : 0, ebits);
        const uint64_t pr = match_any(mr + 1, rbits);
        int eslot = -1, rslot = -1;
        if (local) {
            eslot = s_we[w * E + e] + __popcll(pe & lt);
            if ((pe >> lane) == 1ull) s_we[w * E + e] = eslot + 1;      // highest peer advances the counter
        }
        if (mr >= 0) {
            rslot = s_wr[w * R + mr] + __popcll(pr & lt);
            if ((pr >> lane) == 1ull) s_wr[w * R + mr] = rslot + 1;
        }
        const int64_t g = (int64_t)b * n + idx;
        if (in && g < total) {
            if (RECV) {
                const int64_t row = g / K;
                if (row < a.rows_cap) a.recv_src_metadata[row * (K + 2) + (g - row * K)] = eslot;
            } else {
                a.dst_buffer_slot_idx[g] = rslot;
                a.dst_gsge_idx[g] = -1;             // every copy is local: no transport descriptors
                if (!a.send_only) {
                    a.slot_map[g] = eslot;
                    if (mr == a.rank_idx) a.tok_row[b * EP_TOKENS_PER_BLOCK + tok] = rslot;
                }
            }
        }
        // the running counters of a wave are touched by that wave only and the LDS operations of a wave
        // complete in order: no block barrier (which would also wait for the stores above) is needed
        __builtin_amdgcn_wave_barrier();
        tok += tok_step;
        pos += pos_step;
        if (pos >= K) { pos -= K; ++tok; }
    }
    if (RECV) {
        // the two trailing columns of the metadata rows: source token and last local selection
        // (dispatch_copy_epilogue.hpp:514-522)
        for (int row = tid; row < EP_TOKENS_PER_BLOCK; row += blockDim.x) {
            const int g = b * EP_TOKENS_PER_BLOCK + row;
            if (g >= num_rows || g >= a.rows_cap) continue;
            int master = -1;
            for (int j = 0; j < K; ++j) {
                const int key = s_key[row * K + j];
                const int le = (key < 0 ? -1 : key & (EP_KEY_MASTER - 1)) - lo;
                if (key >= 0 && le >= 0 && le < El) master = j;
            }
            const int64_t pr = recv_packed_row(s_psum, R, a.max_tokens, g);
            int* m = a.recv_src_metadata + (int64_t)g * (K + 2);
            m[K] = *(const int*)(a.packed_base + pr * a.packed_row_bytes + a.src_off);
            m[K + 1] = master;
        }
    }
}

extern "C" __global__ __launch_bounds__(EP_LAYOUT_THREADS) void ep_layout_assign(EpLayoutArgs a) { layout_assign_body<false, false>(a); }
extern "C" __global__ __launch_bounds__(EP_LAYOUT_THREADS) void ep_layout_assign_fold(EpLayoutArgs a) { layout_assign_body<true, false>(a); }
extern "C" __global__ __launch_bounds__(EP_LAYOUT_THREADS) void ep_layout_assign_recv(EpLayoutArgs a) { layout_assign_body<false, true>(a); }
extern "C" __global__ __launch_bounds__(EP_LAYOUT_THREADS) void ep_layout_assign_fold_recv(EpLayoutArgs a) { layout_assign_body<true, true>(a); }

// ------------------------------------------------------------------------------------------------
// Scatter (dispatch copy epilogue): a wave task is one column part of one row (a token, or a row of the receive stream).
// Reference semantics: impls/ep/dispatch_copy_epilogue.hpp:450-545 (expand), :547-620 (zero padding).
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float bf16_lo(unsigned int u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(unsigned int u) { return __uint_as_float(u & 0xffff0000u); }

// Largest magnitude over the 16 lanes of a DPP row, result in every lane of the row.  The operands
// are the bit patterns of |x|: as unsigned integers they order like the floats, +inf above every
// finite value and NaN above +inf, so a NaN anywhere in the group comes out as the group's maximum,
// as it does from torch's amax (deep_ep/utils/math.py:36).
__device__ __forceinline__ unsigned row16_umax(unsigned x) {
    x = max(x, (unsigned)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x128, 0xf, 0xf, false));  // row_ror:8
    x = max(x, (unsigned)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x124, 0xf, 0xf, false));  // row_ror:4
    x = max(x, (unsigned)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x122, 0xf, 0xf, false));  // row_ror:2
    x = max(x, (unsigned)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x121, 0xf, 0xf, false));  // row_ror:1
    return x;
}

template <bool HW>
__device__ __forceinline__ u32x2 quant8(const float* f, float inv) {
    u32x2 o;
    if (HW) {
        int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0] * inv, f[1] * inv, 0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2] * inv, f[3] * inv, w0, true);
        int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4] * inv, f[5] * inv, 0, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6] * inv, f[7] * inv, w1, true);
        o.x = (unsigned)w0;
        o.y = (unsigned)w1;
    } else {
        unsigned b[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) b[i] = ep_f32_bits_to_e4m3fn(__float_as_uint(f[i] * inv));
        o.x = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
        o.y = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
    }
    return o;
}

struct RowCtx {
    int t;            // local token index of the row (expand and pack)
    int myslot;       // lane j < K: destination row of (row, j) or -1
    uint64_t mybase;  // lane j < K: first byte of the regions that row belongs to (pack)
    int64_t src_row;  // row of the source matrix holding the payload
};

// Stream row i of the receive side -> packed row of this partition's regions, with the inclusive row
// counts per source in global memory.  Every lane of the wave calls it.
__device__ __forceinline__ int64_t region_row_of_stream(const int* psum, int R, int max_tokens, int i) {
    const int lane = lane_id();
    int q = 0;                                         // sources whose rows all come before row i
    for (int r0 = 0; r0 < R; r0 += WAVE) {
        const bool before = r0 + lane < R && psum[r0 + lane] <= i;
        q += __popcll(__ballot(before));
    }
    q = min(q, R - 1);
    const int slot = min(i - (q ? psum[q - 1] : 0), max_tokens - 1);      // counts of a stale handle cannot lead outside
    return (int64_t)q * max_tokens + max(slot, 0);
}

// First byte of the rows that destination j of the task writes, and of their scales.
template <bool PACK>
__device__ __forceinline__ char* out_rows_of(const EpScatterArgs& a, const RowCtx& c, int j) {
    if (!PACK) return (char*)a.recv_x;
    const unsigned lo = (unsigned)readlane((int)(unsigned)c.mybase, j);
    const unsigned hi = (unsigned)readlane((int)(unsigned)(c.mybase >> 32), j);
    return (char*)(((uint64_t)hi << 32) | lo);
}
template <bool PACK>
__device__ __forceinline__ char* out_sf_of(const EpScatterArgs& a, char* rows) {
    return PACK ? rows + a.pack_sf_off : (char*)a.recv_sf;
}

// A wave task is (row, column part).  Resolves the row's token, its source row and its destination
// rows; the task of part 0 also writes the row's small items.  Three modes:
//   EP_SCATTER_EXPAND  rows are tokens (non-cached: slots from the slot map) or rows of the receive stream
//                      (cached: slots and token from the metadata row), payload read from x[token]; destinations
//                      are the expanded slots; part 0 writes the metadata row (non-cached) and the gate weights
//   EP_SCATTER_PACK    rows are tokens; destinations are rows of the partition-major regions
//                      (partition * max_tokens + slot of dst_buffer_slot_idx); part 0 writes the packed
//                      metadata [all K topk_idx | all K weights | src_token_global_idx] into each of them
//                      (impls/ep/dispatch.hpp:768-794, layout/ep/token.hpp:59-82)
//   EP_SCATTER_REGION  rows of the receive stream (the regions of every source partition in turn), payload,
//                      scales and weights read from the packed rows; destinations come from the metadata
//                      rows the receive-side layout wrote (dispatch_copy_epilogue.hpp:459-522)
template <bool PACK>
__device__ __forceinline__ bool scatter_row_prologue(const EpScatterArgs& a, int i, int part, RowCtx& c) {
    const int lane = lane_id();
    const int K = a.num_topk;
    int myslot = -1, t;
    float early_w = 0.0f;          // gate weight fetched ahead of its use (token-walking expand)
    if (PACK) {
        uint64_t mybase = 0;
        t = i;
        int64_t e = -1;
        if (lane < K) {
            e = a.topk_idx[(int64_t)t * K + lane];
            const int s = a.dst_slot_idx[(int64_t)t * K + lane];
            if (s >= 0 && s < a.max_tokens && e >= 0 && e < a.num_experts) {
                const int peer = (int)(e / a.experts_per_rank);
                myslot = (a.region_by_source ? a.rank_idx : peer) * a.max_tokens + s;
                mybase = (uint64_t)(a.peer_arenas[peer] + a.buffer_off);
            }
        }
        c.t = t;
        c.myslot = myslot;
        c.mybase = mybase;
        c.src_row = t;
        if (part == 0) {
            const float w = (a.topk_weights != nullptr && lane < K) ? a.topk_weights[(int64_t)t * K + lane] : 0.0f;
            for (int j = 0; j < K; ++j) {
                const int g = readlane(myslot, j);
                if (g < 0) continue;
                char* row = out_rows_of<PACK>(a, c, j) + (int64_t)g * a.out_row_bytes;
                if (lane < K) {
                    if (a.with_metadata) ((int64_t*)(row + a.idx_off))[lane] = e;
                    ((float*)(row + a.w_off))[lane] = w;
                }
                if (a.with_metadata && lane == 0) *(int*)(row + a.src_off) = a.rank_idx * a.max_tokens + t;
            }
        }
        return true;
    }
    c.mybase = 0;
    if (a.mode == EP_SCATTER_REGION) {
        // the metadata rows are complete before this kernel runs: written by the receive-side layout, or cached
        const int v = lane < K + 2 ? a.recv_src_metadata[(int64_t)i * (K + 2) + lane] : -1;
        if (i >= *a.num_recv_ptr) return false;          // (checked after the row's own load has been issued)
        if (lane < K && v >= 0 && v < a.num_out_rows) myslot = v;
        c.src_row = region_row_of_stream(a.psum_rank, a.num_ranks, a.max_tokens, i);
        if (part == 0 && a.recv_topk_weights != nullptr && myslot >= 0)
            a.recv_topk_weights[myslot] = ((const float*)((const char*)a.x + c.src_row * a.x_row_bytes + a.w_off))[lane];
        c.t = i;
        c.myslot = myslot;
        return true;
    }
    if (!a.cached) {
        // the tasks walk the tokens (nothing has to be looked up before the row of x can be fetched); the row of
        // the receive stream a token became is only needed for its metadata row
        t = i;
        if (lane < K) myslot = a.slot_map[(int64_t)t * K + lane];
        // the task that writes the token's metadata row and weights fetches what it needs for that in the same trip
        // (both are indexed by the token alone; tok_row holds nothing meaningful for a token nobody receives)
        int row = -1;
        if (part == 0) {
            row = a.tok_row[t];
            if (a.recv_topk_weights != nullptr && lane < K) early_w = a.topk_weights[(int64_t)t * K + lane];
        }
        const uint64_t vm = __ballot(myslot >= 0);
        if (vm == 0) return false;                       // a token nobody receives
        if (part == 0) {
            const int master = 63 - __builtin_clzll(vm);
            // [slot_0 .. slot_{K-1}, src_token_global_idx, last local j]  (dispatch_copy_epilogue.hpp:514-522)
            const int v = lane < K ? myslot : (lane == K ? a.rank_idx * a.max_tokens + t : master);
            if (lane < K + 2 && row >= 0 && row < a.num_meta_rows) a.recv_src_metadata[(int64_t)row * (K + 2) + lane] = v;
        }
    } else {
        const int v = lane < K + 2 ? a.recv_src_metadata[(int64_t)i * (K + 2) + lane] : -1;
        if (i >= *a.num_recv_ptr) return false;          // (checked after the row's own load has been issued)
        if (lane < K) myslot = v;
        t = readlane(v, K) - a.rank_idx * a.max_tokens;
        if (t < 0 || t >= a.num_tokens) return false;
    }
    if (lane < K && (myslot < 0 || myslot >= a.num_out_rows)) myslot = -1;
    c.src_row = (int64_t)t;
    if (part == 0 && a.recv_topk_weights != nullptr && lane < K && myslot >= 0)
        a.recv_topk_weights[myslot] = a.cached ? a.topk_weights[(int64_t)t * K + lane] : early_w;
    c.t = t;
    c.myslot = myslot;
    return true;
}

// Source row of task row i if it is known before the prologue has run, else -1.
template <bool PACK>
__device__ __forceinline__ int64_t scatter_guess_source_row(const EpScatterArgs& a, int i) {
    if (PACK) return i;                                            // rows are tokens
    if (a.mode == EP_SCATTER_EXPAND && (!a.cached || a.rows_are_tokens)) return i;
    return -1;
}

// The padding rows of an expert, [psum[e], align(psum[e], A)), are one contiguous span of each output:
// the workgroups that share it walk the span 4 KiB at a time, 16 bytes per lane
// (dispatch_copy_epilogue.hpp:547-620).
__device__ __forceinline__ void zero_span(char* base, int64_t nbytes, int part, int nparts) {
    const u32x4 z = {0u, 0u, 0u, 0u};
    const int64_t tid = (int64_t)part * EP_ROW_THREADS + threadIdx.x;     // among the threads sharing the span
    const int64_t nthreads = (int64_t)nparts * EP_ROW_THREADS;
    // 16-byte stores over the aligned body; the ends in 2-byte units (every element here is 2 or 4 bytes wide)
    const int64_t head = min((int64_t)((16 - ((uintptr_t)base & 15)) & 15), nbytes);
    const int64_t body = (nbytes - head) & ~(int64_t)15;
    for (int64_t o = tid * 16; o < body; o += nthreads * 16) stream_store<EP_PAD_ST_POL>((u32x4*)(base + head + o), z);
    for (int64_t o = tid * 2; o < head; o += nthreads * 2) *(unsigned short*)(base + o) = 0;
    for (int64_t o = head + body + tid * 2; o < nbytes; o += nthreads * 2) *(unsigned short*)(base + o) = 0;
}

__device__ __forceinline__ void zero_padding_rows(const EpScatterArgs& a) {
    const int pb = blockIdx.x - a.num_row_blocks;
    const int e = pb / a.pad_blocks_per_expert, part = pb % a.pad_blocks_per_expert;
    if (e >= a.num_local_experts) return;
    const int end = a.psum_expert[e];
    const int rows = min(align_up(end, a.expert_alignment), a.num_out_rows) - end;     // never past the outputs
    if (end < 0 || rows <= 0) return;
    zero_span((char*)a.recv_x + (int64_t)end * a.out_row_bytes, (int64_t)rows * a.out_row_bytes, part,
              a.pad_blocks_per_expert);
    if (a.recv_sf != nullptr && part == 0)
        zero_span((char*)a.recv_sf + (int64_t)end * a.out_sf_row_bytes, (int64_t)rows * a.out_sf_row_bytes, 0, 1);
    if (a.recv_topk_weights != nullptr && part == a.pad_blocks_per_expert - 1)
        zero_span((char*)(a.recv_topk_weights + end), (int64_t)rows * 4, 0, 1);
}

// Verbatim rows: BF16 payload, or FP8 payload with its 2-byte scale packs.  A task moves 1 KiB of
// the row (16 bytes per lane) to every slot; many short tasks keep far more loads in flight than
// one wave walking a whole row.
template <bool PACK>
__device__ __forceinline__ void scatter_copy_body(const EpScatterArgs& a) {
    if ((int)blockIdx.x >= a.num_row_blocks) {
        zero_padding_rows(a);
        return;
    }
    const int lane = lane_id();
    const int task = blockIdx.x * EP_ROWS_PER_BLOCK + wave_id();
    const int i = task / a.num_parts, part = task - i * a.num_parts;
    if (i >= a.num_rows_bound) return;
    const int K = a.num_topk;
    const int nvec = (int)(a.copy_bytes >> 4);
    // a task moves vecs_per_lane KiB of the row: 1 where a row fans out to several slots, more where
    // nearly every row has a single destination and the set-up above would outweigh the copy
    const int U = a.vecs_per_lane;
    u32x4 d[4];
    // Where the source row of a task is known up front (tokens are walked, or every token was received so that
    // row i of the receive stream is token i), its payload is fetched while the prologue looks up the slots;
    // a prologue that names another row after all fetches again.
    const int64_t guess = scatter_guess_source_row<PACK>(a, i);
    if (guess >= 0) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int v = (part * U + u) * WAVE + lane;
            if (u < U && v < nvec)
                d[u] = __builtin_nontemporal_load((const u32x4*)((const char*)a.x + guess * a.x_row_bytes) + v);
        }
    }
    RowCtx c;
    if (!scatter_row_prologue<PACK>(a, i, part, c)) return;
    if (c.src_row != guess) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int v = (part * U + u) * WAVE + lane;
            if (u < U && v < nvec)
                d[u] = __builtin_nontemporal_load((const u32x4*)((const char*)a.x + c.src_row * a.x_row_bytes) + v);
        }
    }
    for (int j = 0; j < K; ++j) {
        const int s = readlane(c.myslot, j);
        if (s < 0) continue;
        u32x4* row = (u32x4*)(out_rows_of<PACK>(a, c, j) + (int64_t)s * a.out_row_bytes);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int v = (part * U + u) * WAVE + lane;
            if (u < U && v < nvec) stream_store<EP_SCATTER_ST_POL>(row + v, d[u]);
        }
    }
    if (part == 0 && a.recv_sf != nullptr) {
        const int P = a.num_sf_packs;
        const char* sfrow = (const char*)a.sf + c.src_row * a.sf_token_stride_bytes;
        for (int p = lane; p < P; p += WAVE) {
            const unsigned short val = *(const unsigned short*)(sfrow + (int64_t)p * a.sf_pack_stride_bytes);
            for (int j = 0; j < K; ++j) {
                const int s = readlane(c.myslot, j);
                if (s < 0) continue;
                ((unsigned short*)(out_sf_of<PACK>(a, out_rows_of<PACK>(a, c, j)) + (int64_t)s * a.out_sf_row_bytes))[p] = val;
            }
        }
    }
}

// Fused BF16 -> e4m3fn quantisation (deep_ep/utils/math.py:30-38) + scatter.  A task owns 512
// channels of a row: a lane holds 8 of them, a 128-channel group is one DPP row of 16 lanes, so the
// task produces 512 payload bytes and 4 fp32 scales per slot.
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_scatter_copy(EpScatterArgs a) {
    scatter_copy_body<false>(a);
}
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_scatter_copy_pack(EpScatterArgs a) {
    scatter_copy_body<true>(a);
}

// (LOADS = false exists for the benchmarks' calibration code object only: the same tasks and stores with a
// made-up payload in place of the row of x.)
template <bool HW, bool PACK, bool LOADS = true>
__device__ __forceinline__ void scatter_quant_body(const EpScatterArgs& a) {
    if ((int)blockIdx.x >= a.num_row_blocks) {
        zero_padding_rows(a);
        return;
    }
    const int lane = lane_id();
    const int task = blockIdx.x * EP_ROWS_PER_BLOCK + wave_id();
    const int i = task / a.num_parts, part = task - i * a.num_parts;
    if (i >= a.num_rows_bound) return;
    const int K = a.num_topk;
    const int nvec = a.hidden >> 3;                      // 16-byte vectors of 8 BF16
    const int v = part * WAVE + lane;
    const bool live = v < nvec;
    u32x4 d = {0u, 0u, 0u, 0u};
    // the payload is fetched while the prologue looks up the slots wherever the source row is known up front
    const int64_t guess = scatter_guess_source_row<PACK>(a, i);
    if (live && LOADS && guess >= 0) d = __builtin_nontemporal_load((const u32x4*)((const char*)a.x + guess * a.x_row_bytes) + v);
    RowCtx c;
    if (!scatter_row_prologue<PACK>(a, i, part, c)) return;
    if (live && LOADS && c.src_row != guess)
        d = __builtin_nontemporal_load((const u32x4*)((const char*)a.x + c.src_row * a.x_row_bytes) + v);
    if (!LOADS) d = u32x4{0x3f803f80u + (unsigned)v, 0x40004000u, 0xbf80bf80u, 0x3f003f00u};
    float f[8] = {bf16_lo(d.x), bf16_hi(d.x), bf16_lo(d.y), bf16_hi(d.y),
                  bf16_lo(d.z), bf16_hi(d.z), bf16_lo(d.w), bf16_hi(d.w)};
    unsigned mbits = 0u;
#pragma unroll
    for (int q = 0; q < 8; ++q) mbits = max(mbits, __float_as_uint(f[q]) & 0x7fffffffu);
    const float m = __uint_as_float(row16_umax(mbits));
    const float amax = m < 1e-4f ? 1e-4f : m;       // clamp(min=1e-4): a NaN stays a NaN
    const float inv = (1.0f / amax) * 448.0f;       // torch evaluates `448.0 / t` as t.reciprocal() * 448.0
    const float scale = amax / 448.0f;
    u32x2 q8 = quant8<HW>(f, inv);
    if (amax != amax) q8 = u32x2{0x7f7f7f7fu, 0x7f7f7f7fu};   // every product is NaN: e4m3fn has one NaN, sign clear
    if (!live) return;
    const bool writes_scale = (lane & 15) == 0;
    for (int j = 0; j < K; ++j) {
        const int s = readlane(c.myslot, j);
        if (s < 0) continue;
        char* rows = out_rows_of<PACK>(a, c, j);
        stream_store<EP_SCATTER_ST_POL>((u32x2*)(rows + (int64_t)s * a.out_row_bytes) + v, q8);
        if (writes_scale) ((float*)(out_sf_of<PACK>(a, rows) + (int64_t)s * a.out_sf_row_bytes))[v >> 4] = scale;
    }
}

extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_scatter_quant(EpScatterArgs a) {
    scatter_quant_body<true, false>(a);
}
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_scatter_quant_sw(EpScatterArgs a) {
    scatter_quant_body<false, false>(a);
}
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_scatter_quant_pack(EpScatterArgs a) {
    scatter_quant_body<true, true>(a);
}
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_scatter_quant_sw_pack(EpScatterArgs a) {
    scatter_quant_body<false, true>(a);
}

// The quantiser alone (deep_ep/utils/math.py:30-38, what a caller runs before a dispatch of pre-quantised rows):
// the arithmetic of the fused kernel above, rows written in place of being scattered.
template <bool HW>
__device__ __forceinline__ void quant_rows_body(const EpQuantArgs& a) {
    const int lane = lane_id();
    const int task = blockIdx.x * EP_ROWS_PER_BLOCK + wave_id();
    const int t = task / a.num_parts, part = task - t * a.num_parts;
    if (t >= a.num_rows) return;
    const int nvec = a.hidden >> 3;
    const int v = part * WAVE + lane;
    const bool live = v < nvec;
    u32x4 d = {0u, 0u, 0u, 0u};
    if (live) d = __builtin_nontemporal_load((const u32x4*)((const char*)a.x + (int64_t)t * a.hidden * 2) + v);
    float f[8] = {bf16_lo(d.x), bf16_hi(d.x), bf16_lo(d.y), bf16_hi(d.y),
                  bf16_lo(d.z), bf16_hi(d.z), bf16_lo(d.w), bf16_hi(d.w)};
    unsigned mbits = 0u;
#pragma unroll
    for (int q = 0; q < 8; ++q) mbits = max(mbits, __float_as_uint(f[q]) & 0x7fffffffu);
    const float m = __uint_as_float(row16_umax(mbits));
    const float amax = m < 1e-4f ? 1e-4f : m;
    const float inv = (1.0f / amax) * 448.0f;
    u32x2 q8 = quant8<HW>(f, inv);
    if (amax != amax) q8 = u32x2{0x7f7f7f7fu, 0x7f7f7f7fu};
    if (!live) return;
    ((u32x2*)((char*)a.q + (int64_t)t * a.hidden))[v] = q8;
    if ((lane & 15) == 0) a.sf[(int64_t)t * ((a.hidden + 127) >> 7) + (v >> 4)] = amax / 448.0f;
}
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_quant_rows(EpQuantArgs a) {
    if (a.hw_convert) quant_rows_body<true>(a);
    else quant_rows_body<false>(a);
}

// Column-major scales (use_tma_aligned_col_major_sf): the copy kernels write scale rows, this
// kernel turns them into columns.  The reference does the same with a generic transposing copy
// (csrc/buffers/ep.hpp:379-381); writing columns straight from the copy kernel was measured and is
// slower, since every 4-byte scale then lands in a cache line of its own.
template <typename E>
__device__ __forceinline__ void sf_transpose_body(const EpSfTransposeArgs& a, unsigned (*tile)[EP_SF_TILE + 1]) {
    int n = a.num_rows;
    if (a.counted) n = min(n, align_up(a.psum_expert[a.num_local_experts - 1], a.expert_alignment));
    const int r0 = blockIdx.x * EP_SF_TILE;
    if (r0 >= n) return;
    const int tx = threadIdx.x % EP_SF_TILE, ty = threadIdx.x / EP_SF_TILE;
    constexpr int STEP = EP_LAYOUT_THREADS / EP_SF_TILE;
    const E* src = (const E*)a.src;
    E* dst = (E*)a.dst;
    for (int c0 = 0; c0 < a.num_cols; c0 += EP_SF_TILE) {
        for (int rr = ty; rr < EP_SF_TILE; rr += STEP)
            if (r0 + rr < n && c0 + tx < a.num_cols) tile[rr][tx] = src[(int64_t)(r0 + rr) * a.num_cols + c0 + tx];
        __syncthreads();
        for (int cc = ty; cc < EP_SF_TILE; cc += STEP)
            if (c0 + cc < a.num_cols && r0 + tx < n) dst[(int64_t)(c0 + cc) * n + r0 + tx] = (E)tile[tx][cc];
        __syncthreads();
    }
}

// 2-byte packs, two at a time: a thread reads two adjacent columns of a row as one 32-bit word and writes two
// adjacent rows of a column as one.  Needs an even column count (rows of the source start on 4 bytes) and an even
// row count (columns of the destination do); half the steps of the element-wise form.
__device__ __forceinline__ void sf_transpose_pairs(const EpSfTransposeArgs& a, int n, unsigned short (*tile)[EP_SF_TILE + 2]) {
    const int r0 = blockIdx.x * EP_SF_TILE;
    constexpr int HALF = EP_SF_TILE / 2;
    const int tx = threadIdx.x % HALF, ty = threadIdx.x / HALF;
    constexpr int STEP = EP_LAYOUT_THREADS / HALF;
    const unsigned* src = (const unsigned*)a.src;
    unsigned* dst = (unsigned*)a.dst;
    const int cols2 = a.num_cols >> 1, n2 = n >> 1;
    for (int c0 = 0; c0 < a.num_cols; c0 += EP_SF_TILE) {
        for (int rr = ty; rr < EP_SF_TILE; rr += STEP) {
            const int c = c0 + 2 * tx;
            if (r0 + rr < n && c < a.num_cols) {
                const unsigned v = src[(int64_t)(r0 + rr) * cols2 + (c >> 1)];
                tile[rr][2 * tx] = (unsigned short)v;
                tile[rr][2 * tx + 1] = (unsigned short)(v >> 16);
            }
        }
        __syncthreads();
        for (int cc = ty; cc < EP_SF_TILE; cc += STEP) {
            const int r = r0 + 2 * tx;
            if (c0 + cc < a.num_cols && r < n)
                dst[(int64_t)(c0 + cc) * n2 + (r >> 1)] = (unsigned)tile[2 * tx][cc] | ((unsigned)tile[2 * tx + 1][cc] << 16);
        }
        __syncthreads();
    }
}

extern "C" __global__ __launch_bounds__(EP_LAYOUT_THREADS) void ep_sf_transpose(EpSfTransposeArgs a) {
    __shared__ unsigned tile[EP_SF_TILE][EP_SF_TILE + 1];
    if (a.elem_bytes == 4) {
        sf_transpose_body<unsigned>(a, tile);
        return;
    }
    int n = a.num_rows;
    if (a.counted) n = min(n, align_up(a.psum_expert[a.num_local_experts - 1], a.expert_alignment));
    if ((n & 1) == 0 && (a.num_cols & 1) == 0 && (((uintptr_t)a.src | (uintptr_t)a.dst) & 3) == 0) {
        if ((int)blockIdx.x * EP_SF_TILE < n) sf_transpose_pairs(a, n, (unsigned short (*)[EP_SF_TILE + 2])tile);
        return;
    }
    sf_transpose_body<unsigned short>(a, tile);
}

// ------------------------------------------------------------------------------------------------
// Combine, single partition: gather the row's expanded slots, sum in fp32 in ascending slot
// order, round once to BF16, then add the biases the same way.
// Reference semantics: impls/ep/combine.hpp:291-324 + combine_utils.hpp:14-93 (owner side),
// combine_reduce_epilogue.hpp:96-154 (token side); with one partition each token has one partial.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ unsigned f32_to_bf16_bits(float f) {
    unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

__device__ __forceinline__ void unpack8(const u32x4& d, float* f) {
    f[0] = bf16_lo(d.x); f[1] = bf16_hi(d.x); f[2] = bf16_lo(d.y); f[3] = bf16_hi(d.y);
    f[4] = bf16_lo(d.z); f[5] = bf16_hi(d.z); f[6] = bf16_lo(d.w); f[7] = bf16_hi(d.w);
}

__device__ __forceinline__ u32x4 pack8(const float* f) {
    u32x4 o;
    o.x = f32_to_bf16_bits(f[0]) | (f32_to_bf16_bits(f[1]) << 16);
    o.y = f32_to_bf16_bits(f[2]) | (f32_to_bf16_bits(f[3]) << 16);
    o.z = f32_to_bf16_bits(f[4]) | (f32_to_bf16_bits(f[5]) << 16);
    o.w = f32_to_bf16_bits(f[6]) | (f32_to_bf16_bits(f[7]) << 16);
    return o;
}

// out = BF16(f32 b0 + f32 b1 + f32 partial), left to right; a single input is copied verbatim.
__device__ __forceinline__ u32x4 add_biases(const EpCombineArgs& a, int t, int v, bool have_partial, u32x4 partial) {
    const int64_t rowvec = a.hidden >> 3;
    float acc[8], g[8];
    int nin = 0;
    u32x4 last = {0u, 0u, 0u, 0u};
    const void* biases[2] = {a.bias_0, a.bias_1};
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        if (biases[b] == nullptr) continue;
        last = ((const u32x4*)biases[b])[(int64_t)t * rowvec + v];
        unpack8(last, g);
        if (nin == 0) { for (int q = 0; q < 8; ++q) acc[q] = g[q]; }
        else { for (int q = 0; q < 8; ++q) acc[q] = acc[q] + g[q]; }
        ++nin;
    }
    if (have_partial) {
        last = partial;
        unpack8(partial, g);
        if (nin == 0) { for (int q = 0; q < 8; ++q) acc[q] = g[q]; }
        else { for (int q = 0; q < 8; ++q) acc[q] = acc[q] + g[q]; }
        ++nin;
    }
    if (nin <= 1) return last;          // zero inputs -> zeros, one input -> verbatim
    return pack8(acc);
}

// The same with the bias vectors already in registers (fetched together with the rows): the biases that exist, in
// order, then the partial.  (Registers of their own and uniform flags: a run-time index into an array of loaded
// vectors would make the compiler wait for the loads where they are issued.)
__device__ __forceinline__ u32x4 add_loaded_biases(bool has0, u32x4 x0, bool has1, u32x4 x1, u32x4 partial) {
    if (!has0 && !has1) return partial;
    float acc[8], g[8];
    if (has0) {
        unpack8(x0, acc);
        if (has1) {
            unpack8(x1, g);
            for (int q = 0; q < 8; ++q) acc[q] = acc[q] + g[q];
        }
    } else {
        unpack8(x1, acc);
    }
    unpack8(partial, g);
    for (int q = 0; q < 8; ++q) acc[q] = acc[q] + g[q];
    return pack8(acc);
}

// Tokens with no valid slot are never received: their output is the bias sum (or zero).
__device__ __forceinline__ void combine_unrouted(const EpCombineArgs& a) {
    const int lane = lane_id();
    const int K = a.num_topk;
    const int tb = ((int)blockIdx.x - a.num_row_blocks) * EP_ROW_THREADS + wave_id() * WAVE;
    const int t = tb + lane;
    bool unrouted = false;
    if (t < a.num_tokens) {
        unrouted = true;
        for (int j = 0; j < K; ++j) {
            const int64_t e = a.topk_idx[(int64_t)t * K + j];
            if (e >= 0 && e < a.num_experts) unrouted = false;
        }
    }
    uint64_t m = __ballot(unrouted);
    const int nvec = a.hidden >> 3;
    const u32x4 z = {0u, 0u, 0u, 0u};
    while (m != 0) {
        const int l = __builtin_ctzll(m);
        m &= m - 1;
        const int tt = tb + l;
        for (int v = lane; v < nvec; v += WAVE)
            ((u32x4*)a.combined_x)[(int64_t)tt * nvec + v] = add_biases(a, tt, v, false, z);
        if (a.combined_topk_weights != nullptr && lane < K) a.combined_topk_weights[(int64_t)tt * K + lane] = 0.0f;
    }
}

// A wave task is (row, 1024-channel part): two 16-byte vectors per lane and input row, all loads
// issued before the first add.  MODE selects which reduction of the reference the task performs:
//   EP_COMBINE_FUSED    one partition: rows are the receive stream; out = BF16(sum_j f32 y[slot_j]), then
//                       BF16(f32 b0 + f32 b1 + f32 that) when biases are given (the two levels of
//                       combine.hpp:291-324 and combine_reduce_epilogue.hpp:114-140 for a single master)
//   EP_COMBINE_PARTIAL  owner side: same sum, stored with its K-wide weight vector in the combine buffer
//                       at [group * max_tokens + source token]            (combine.hpp:94-106,301-324)
//   EP_COMBINE_FINAL    token side: rows are tokens; inputs = b0, b1, then the partial of every master
//                       (last top-k position per destination partition) in ascending position, summed
//                       left to right in fp32 and rounded once; weight vectors OR-merged
//                       (combine_reduce_epilogue.hpp:96-153)
// LOADS / STORES: the benchmarks' calibration code object builds the single-partition kernel once without its row
// fetches and once without its stores (what each stream costs alone); the library's kernels have both.
template <int KT, int MODE, bool LOADS = true, bool STORES = true>
__device__ __forceinline__ void combine_body(const EpCombineArgs& a) {
    static_assert((LOADS && STORES) || (KT > 0 && MODE == EP_COMBINE_FUSED), "only the unrolled single-partition kernel is taken apart");
    if (MODE == EP_COMBINE_FUSED && (int)blockIdx.x >= a.num_row_blocks) {
        combine_unrouted(a);
        return;
    }
    const int lane = lane_id();
    const int K = KT > 0 ? KT : a.num_topk;
    const int task = blockIdx.x * EP_ROWS_PER_BLOCK + wave_id();
    const int i = task / a.num_parts, part = task - i * a.num_parts;
    if (i >= a.num_rows_bound) return;

    int myslot = -1, t, group = 0, src_rank = 0;
    if (MODE == EP_COMBINE_FINAL) {
        t = i;
        int r = -1;
        if (lane < K) {
            const int64_t e = a.topk_idx[(int64_t)t * K + lane];
            if (e >= 0 && e < a.num_experts) r = (int)(e / a.experts_per_rank);
        }
        bool master = r >= 0;
        for (int jj = 1; jj < K; ++jj) {
            const int rj = readlane(r, jj);
            if (lane < jj && rj == r) master = false;          // a later position goes to the same partition
        }
        if (master) myslot = (a.num_ranks < K ? r : lane) * a.max_tokens + t;
    } else {
        const int mv = lane < K + 2 ? a.recv_src_metadata[(int64_t)i * (K + 2) + lane] : -1;
        if (i >= *a.num_recv_ptr) return;                // (checked after the row's own load has been issued)
        if (lane < K && mv >= 0 && mv < a.num_in_rows) myslot = mv;
        const int src = readlane(mv, K);                        // source partition * max_tokens + its token
        if (MODE == EP_COMBINE_PARTIAL) {
            src_rank = src / a.max_tokens;
            if (src < 0 || src_rank >= a.num_ranks) return;
            t = src - src_rank * a.max_tokens;
        } else {
            t = src - a.rank_idx * a.max_tokens;
            if (t < 0 || t >= a.max_tokens || t >= a.num_tokens) return;
        }
        group = a.num_ranks < K ? a.rank_idx : readlane(mv, K + 1);
        if (MODE == EP_COMBINE_PARTIAL && (group < 0 || group >= a.num_groups)) return;
    }
    const int nvalid = __popcll(__ballot(myslot >= 0));
    // Owner side with whole rows per task: a received row mostly has a single slot among this partition's few
    // experts, and its partial is then that row verbatim: up to 16 vectors a lane in flight, no arithmetic.
    const bool verbatim = MODE == EP_COMBINE_PARTIAL && a.whole_rows && nvalid == 1;
    const int nvec = a.hidden >> 3;
    const int64_t yvec = a.y_row_bytes >> 4;
    const u32x4* y = (const u32x4*)a.y;
    // a partial goes to the combine buffer of the partition its token came from (impls/ep/combine.hpp:291-324)
    char* out_row = MODE == EP_COMBINE_PARTIAL
        ? a.peer_arenas[src_rank] + a.buffer_off + ((int64_t)group * a.max_tokens + t) * a.out_row_bytes
        : (char*)a.combined_x + (int64_t)t * a.out_row_bytes;

    // ---- gate weights ----
    float myw = 0.0f;
    if (MODE == EP_COMBINE_FINAL) {
        if (part == 0 && a.combined_topk_weights != nullptr) {
            unsigned acc = 0;
            if (KT > 0 && nvalid > 0) {
                // the weight vectors of all masters in one trip: no branch and no per-lane condition between the
                // loads (a position that is no master re-reads the first master's vector and is left out)
                const int s_any = readlane(myslot, (int)__builtin_ctzll(__ballot(myslot >= 0)));
                const int wl = min(lane, K - 1);
                unsigned wv[KT > 0 ? KT : 1];
#pragma unroll
                for (int j = 0; j < KT; ++j) {
                    const int s = readlane(myslot, j);
                    wv[j] = ((const unsigned*)((const char*)a.y + (int64_t)(s >= 0 ? s : s_any) * a.y_row_bytes + (a.hidden << 1)))[wl];
                }
#pragma unroll
                for (int j = 0; j < KT; ++j)
                    if (readlane(myslot, j) >= 0) acc |= wv[j];
            } else {
                for (int j = 0; j < K; ++j) {
                    const int s = readlane(myslot, j);
                    if (s < 0) continue;
                    if (lane < K) acc |= ((const unsigned*)((const char*)a.y + (int64_t)s * a.y_row_bytes + (a.hidden << 1)))[lane];
                }
            }
            if (lane < K) ((unsigned*)a.combined_topk_weights)[(int64_t)t * K + lane] = acc;
        }
    } else {
        const bool need_w = part == 0 || (MODE == EP_COMBINE_FUSED && a.weighted);
        if (LOADS && need_w && a.expanded_weights != nullptr && myslot >= 0) myw = a.expanded_weights[myslot];
        if (part == 0 && lane < K) {
            if (STORES && MODE == EP_COMBINE_FUSED && a.combined_topk_weights != nullptr)
                a.combined_topk_weights[(int64_t)t * K + lane] = myw;
            // (the verbatim path below stores them behind its row fetches, so that the two trips become one)
            if (MODE == EP_COMBINE_PARTIAL && a.expanded_weights != nullptr && !verbatim)
                ((float*)(out_row + (a.hidden << 1)))[lane] = myw;
        }
    }

    u32x4* out = (u32x4*)out_row;
    const bool has0 = a.bias_0 != nullptr, has1 = a.bias_1 != nullptr;
    const bool weighted = MODE == EP_COMBINE_FUSED && a.weighted;
    if (verbatim) {
        const int s1 = readlane(myslot, __builtin_ctzll(__ballot(myslot >= 0)));
        const u32x4* src = y + (int64_t)s1 * yvec;
        // (the loop counter is the same in every lane: a row shorter than the wave still gets its weights)
        for (int v0 = 0; v0 < nvec; v0 += 16 * WAVE) {
            const int vb = v0 + lane;
            u32x4 d[16];
#pragma unroll
            for (int u = 0; u < 16; ++u)
                if (vb + u * WAVE < nvec) d[u] = __builtin_nontemporal_load(src + vb + u * WAVE);
            if (v0 == 0 && lane < K && a.expanded_weights != nullptr) ((float*)(out_row + (a.hidden << 1)))[lane] = myw;
#pragma unroll
            for (int u = 0; u < 16; ++u)
                if (vb + u * WAVE < nvec) stream_store<EP_COMBINE_ST_POL>(out + vb + u * WAVE, d[u]);
        }
        return;
    }
    // a task is one 1024-channel part of its row, or (owner side, whole rows) all of them in turn
    const bool whole = MODE == EP_COMBINE_PARTIAL && a.whole_rows;
    const int part_end = whole ? (nvec + 2 * WAVE - 1) / (2 * WAVE) : part + 1;
    for (int cp = whole ? 0 : part; cp < part_end; ++cp) {
    const int v0 = cp * 2 * WAVE + lane, v1 = v0 + WAVE;
    const bool live0 = v0 < nvec, live1 = v1 < nvec;
    // the gate weights are scattered 4-byte loads: only the task that carries them back (part 0) or multiplies
    // by them has read them; the other tasks hold zeros
    const u32x4 zero = {0u, 0u, 0u, 0u};
    if (KT > 0) {
        // Every load of the task is issued before the first add: the biases of the token (not on the owner side), then
        // both 16-byte vectors of every input row.  The two vectors are then reduced one after the other, which
        // keeps the live registers at the loaded vectors plus one accumulator (72 VGPRs at K = 6: seven waves a SIMD).
        // No load depends on the lane being live: a lane past the end of the row fetches the row's last vector and
        // stores nothing.  (A load under a per-lane condition has to be merged with the register's old value when it
        // returns, and the compiler then waits for the first such load before it issues the next.)
        const int c0 = min(v0, nvec - 1), c1 = min(v1, nvec - 1);
        u32x4 d0[KT > 0 ? KT : 1], d1[KT > 0 ? KT : 1];
        // bias vectors: p0* of bias_0, p1* of bias_1, *a for the first vector of the task, *b for the second
        u32x4 p0a = zero, p0b = zero, p1a = zero, p1b = zero;
        if (MODE != EP_COMBINE_PARTIAL) {
            if (has0) {
                const u32x4* bp = (const u32x4*)a.bias_0 + (int64_t)t * nvec;
                p0a = __builtin_nontemporal_load(bp + c0);
                p0b = __builtin_nontemporal_load(bp + c1);
            }
            if (has1) {
                const u32x4* bp = (const u32x4*)a.bias_1 + (int64_t)t * nvec;
                p1a = __builtin_nontemporal_load(bp + c0);
                p1b = __builtin_nontemporal_load(bp + c1);
            }
        }
        // token side: the biases open the one accumulation; single partition: they are added to the rounded sum of
        // the rows in a second one (the two levels of the reference)
        const bool first0 = MODE == EP_COMBINE_FINAL && has0, first1 = MODE == EP_COMBINE_FINAL && has1;
        if (MODE == EP_COMBINE_PARTIAL) {
            // owner side: a received row has one or two of its K positions on this partition: fetch those only
#pragma unroll
            for (int j = 0; j < KT; ++j) {
                const int s = readlane(myslot, j);
                if (s < 0) continue;
                d0[j] = __builtin_nontemporal_load(y + (int64_t)s * yvec + c0);
                d1[j] = __builtin_nontemporal_load(y + (int64_t)s * yvec + c1);
            }
        } else if (!LOADS) {
            const u32x4 filler = {(unsigned)lane, (unsigned)i, 0x3f803f80u, 0x3f803f80u};
#pragma unroll
            for (int j = 0; j < KT; ++j) d0[j] = d1[j] = filler;
        } else if (nvalid > 0) {
            // nearly every position is valid: one straight run of 2 K loads with no branch in it, a position without
            // a row re-reads the first valid one (the same cache lines again) and is left out of the sum below
            const int s_any = readlane(myslot, (int)__builtin_ctzll(__ballot(myslot >= 0)));
#pragma unroll
            for (int j = 0; j < KT; ++j) {
                const int s = readlane(myslot, j);
                const int64_t row = (int64_t)(s >= 0 ? s : s_any) * yvec;
                d0[j] = __builtin_nontemporal_load(y + row + c0);
                d1[j] = __builtin_nontemporal_load(y + row + c1);
                // sixteen and more fetches a wave are better sent in two goes, the first row ahead of the others
                // (top-8 at 16384 / 32768 tokens: 354 / 707 us against 362 / 730 all at once; top-6 and below lose:
                // 277 against 272)
                if (KT >= 8 && j == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
        }
        // inputs in order: b0, b1, then the rows in ascending position; zero inputs -> zeros, one input -> verbatim
        // copy, more -> one rounding of the fp32 sum (a weighted single row is a product: rounded as well)
        auto reduce = [&](u32x4 x0, u32x4 x1, const u32x4* d) -> u32x4 {
            float acc[8], g[8];
            u32x4 first = zero;
            int nin = 0;
            if (first0) {
                unpack8(x0, acc);
                first = x0;
                ++nin;
            }
            if (first1) {
                unpack8(x1, g);
                if (nin == 0) { for (int q = 0; q < 8; ++q) acc[q] = g[q]; first = x1; }
                else { for (int q = 0; q < 8; ++q) acc[q] = acc[q] + g[q]; }
                ++nin;
            }
#pragma unroll
            for (int j = 0; j < KT; ++j) {
                const int s = readlane(myslot, j);
                if (s < 0) continue;
                unpack8(d[j], g);
                if (weighted) {
                    const float wj = __int_as_float(readlane(__float_as_int(myw), j));
                    for (int q = 0; q < 8; ++q) g[q] = g[q] * wj;
                }
                if (nin == 0) { for (int q = 0; q < 8; ++q) acc[q] = g[q]; first = d[j]; }
                else { for (int q = 0; q < 8; ++q) acc[q] = acc[q] + g[q]; }
                ++nin;
            }
            if (nin >= 2 || (weighted && nin == 1)) return pack8(acc);
            return first;
        };
        // (without stores the sums still have to be formed: they are stored under a condition that never holds)
        if (live0) {
            u32x4 res = reduce(p0a, p1a, d0);
            if (MODE == EP_COMBINE_FUSED) res = add_loaded_biases(has0, p0a, has1, p1a, res);
            if (STORES || ((res.x ^ res.y ^ res.z ^ res.w) == 0x9E3779B1u && a.num_in_rows < 0)) stream_store<EP_COMBINE_ST_POL>(out + v0, res);
        }
        if (live1) {
            u32x4 res = reduce(p0b, p1b, d1);
            if (MODE == EP_COMBINE_FUSED) res = add_loaded_biases(has0, p0b, has1, p1b, res);
            if (STORES || ((res.x ^ res.y ^ res.z ^ res.w) == 0x9E3779B1u && a.num_in_rows < 0)) stream_store<EP_COMBINE_ST_POL>(out + v1, res);
        }
        continue;
    }
    float acc0[8], acc1[8];
    u32x4 res0 = zero, res1 = zero;
    int nin = 0;                                              // inputs accumulated so far
    u32x4 p0a = zero, p0b = zero, p1a = zero, p1b = zero;     // single partition: biases fetched ahead of the rows
    if (MODE == EP_COMBINE_FUSED) {
        if (has0) {
            const u32x4* bp = (const u32x4*)a.bias_0 + (int64_t)t * nvec;
            if (live0) p0a = __builtin_nontemporal_load(bp + v0);
            if (live1) p0b = __builtin_nontemporal_load(bp + v1);
        }
        if (has1) {
            const u32x4* bp = (const u32x4*)a.bias_1 + (int64_t)t * nvec;
            if (live0) p1a = __builtin_nontemporal_load(bp + v0);
            if (live1) p1b = __builtin_nontemporal_load(bp + v1);
        }
    }
    if (MODE == EP_COMBINE_FINAL) {
        const void* biases[2] = {a.bias_0, a.bias_1};
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            if (biases[b] == nullptr) continue;
            const u32x4* bp = (const u32x4*)biases[b] + (int64_t)t * nvec;
            u32x4 e0 = zero, e1 = zero;
            if (live0) e0 = __builtin_nontemporal_load(bp + v0);
            if (live1) e1 = __builtin_nontemporal_load(bp + v1);
            float g0[8], g1[8];
            unpack8(e0, g0);
            unpack8(e1, g1);
            if (nin == 0) { for (int q = 0; q < 8; ++q) { acc0[q] = g0[q]; acc1[q] = g1[q]; } res0 = e0; res1 = e1; }
            else { for (int q = 0; q < 8; ++q) { acc0[q] = acc0[q] + g0[q]; acc1[q] = acc1[q] + g1[q]; } }
            ++nin;
        }
    }
    for (int j = 0; j < K; ++j) {
        const int s = readlane(myslot, j);
        if (s < 0) continue;
        u32x4 e0 = zero, e1 = zero;
        if (live0) e0 = __builtin_nontemporal_load(y + (int64_t)s * yvec + v0);
        if (live1) e1 = __builtin_nontemporal_load(y + (int64_t)s * yvec + v1);
        float g0[8], g1[8];
        unpack8(e0, g0);
        unpack8(e1, g1);
        if (weighted) {
            const float wj = __int_as_float(readlane(__float_as_int(myw), j));
            for (int q = 0; q < 8; ++q) { g0[q] = g0[q] * wj; g1[q] = g1[q] * wj; }
        }
        if (nin == 0) { for (int q = 0; q < 8; ++q) { acc0[q] = g0[q]; acc1[q] = g1[q]; } res0 = e0; res1 = e1; }
        else { for (int q = 0; q < 8; ++q) { acc0[q] = acc0[q] + g0[q]; acc1[q] = acc1[q] + g1[q]; } }
        ++nin;
    }
    // zero inputs -> zeros, one input -> verbatim copy, more -> one rounding of the fp32 sum
    if (nin >= 2 || (weighted && nvalid == 1)) {
        res0 = pack8(acc0);
        res1 = pack8(acc1);
    }
    if (live0) {
        if (MODE == EP_COMBINE_FUSED) res0 = add_loaded_biases(has0, p0a, has1, p1a, res0);
        stream_store<EP_COMBINE_ST_POL>(out + v0, res0);
    }
    if (live1) {
        if (MODE == EP_COMBINE_FUSED) res1 = add_loaded_biases(has0, p0b, has1, p1b, res1);
        stream_store<EP_COMBINE_ST_POL>(out + v1, res1);
    }
    }
}

#define EP_COMBINE_KERNELS(SUFFIX, MODE)                                                                                   \
    extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_combine##SUFFIX##_generic(EpCombineArgs a) { combine_body<0, MODE>(a); } \
    extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_combine##SUFFIX##_k2(EpCombineArgs a) { combine_body<2, MODE>(a); }     \
    extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_combine##SUFFIX##_k4(EpCombineArgs a) { combine_body<4, MODE>(a); }     \
    extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_combine##SUFFIX##_k6(EpCombineArgs a) { combine_body<6, MODE>(a); }     \
    extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_combine##SUFFIX##_k8(EpCombineArgs a) { combine_body<8, MODE>(a); }

EP_COMBINE_KERNELS(, EP_COMBINE_FUSED)
EP_COMBINE_KERNELS(_partial, EP_COMBINE_PARTIAL)
EP_COMBINE_KERNELS(_final, EP_COMBINE_FINAL)

// ------------------------------------------------------------------------------------------------
// Self-test: hardware e4m3fn conversion against the integer conversion over a range of fp32 bit
// patterns.  out[0] = number of mismatches, out[1] = first mismatching pattern (if any).
// ------------------------------------------------------------------------------------------------
extern "C" __global__ __launch_bounds__(256) void ep_fp8_selftest(EpFp8TestArgs a) {
    unsigned long long bad = 0, firstbad = ~0ull;
    for (unsigned long long k = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; k < a.count;
         k += (unsigned long long)gridDim.x * blockDim.x) {
        const unsigned bits = (unsigned)(a.first + k);
        const float f = __uint_as_float(bits);
        if (!(fabsf(f) <= a.limit)) continue;
        const unsigned hw = (unsigned)__builtin_amdgcn_cvt_pk_fp8_f32(f, 0.0f, 0, false) & 0xffu;
        const unsigned sw = ep_f32_bits_to_e4m3fn(bits);
        if (hw != sw) {
            ++bad;
            if (firstbad == ~0ull) firstbad = bits;
        }
    }
    if (bad != 0) {
        atomicAdd(&a.out[0], bad);
        atomicMin(&a.out[1], firstbad);
    }
}
