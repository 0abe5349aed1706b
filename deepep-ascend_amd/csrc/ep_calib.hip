// Calibration code object (ep_calib.hsaco): the measurement rig of the benchmarks, kept apart from the
// product's code object and library.  It compiles the product's device source once more (so the variants
// below run the very bodies the product runs) and adds kernels that price the memory system and the
// alternatives to the token-major copy kernel:
//
//   ep_calib_fill / _fill_shuffled     4 KiB chunks in address order / in a scrambled order
//   ep_calib_fronts                    many write fronts of whole rows advancing in lock step
//   ep_calib_mixed                     an address-ordered stream of reads and writes in a given ratio
//   ep_calib_read_rows                 the loads of the fused copy kernel alone (token-major, 16 bytes a lane)
//   ep_calib_scatter_stores_only       the fused copy kernel without its loads of x: same tasks, same stores
//   ep_calib_ordered_{flat,steered}*   the fused copy kernel with one task per DESTINATION row, the tasks in
//                                      destination order inside chunks of tokens (expert-major runs); steered:
//                                      all readers of a token on one XCD, so that x is fetched from memory once
//   ep_calib_quant_rows + ep_calib_copy_ordered_{flat,steered}   the same in two passes: quantise token-major,
//                                      then copy FP8 rows in destination order
//   ep_calib_combine_k6*               the single-partition combine at top-6: whole, its row fetches alone, its stores alone
#include "ep_kernels.hip"
#include "ep_calib_args.h"

extern "C" __global__ __launch_bounds__(256) void ep_calib_fill(EpCalibFillArgs a) {
    u32x4* p = (u32x4*)a.dst + (int64_t)blockIdx.x * 256 + threadIdx.x;
    const u32x4 v = {a.value, a.value, a.value, a.value};
    __builtin_nontemporal_store(v, p);
}
extern "C" __global__ __launch_bounds__(256) void ep_calib_fill_shuffled(EpCalibFillArgs a) {
    // units of unit_chunks consecutive chunks keep their inner order; the units are scrambled
    // (unit = odd multiplier * index modulo the number of units, a power of two)
    const unsigned unit = blockIdx.x / a.unit_chunks, in_unit = blockIdx.x - unit * a.unit_chunks;
    const unsigned num_units = a.num_chunks / a.unit_chunks;
    const unsigned chunk = ((unit * 0x9E3779B1u) & (num_units - 1u)) * a.unit_chunks + in_unit;
    u32x4* p = (u32x4*)a.dst + (int64_t)chunk * 256 + threadIdx.x;
    const u32x4 v = {a.value, a.value, a.value, a.value};
    __builtin_nontemporal_store(v, p);
}

// Scrambled order that keeps every chunk on the XCD address order would give it: workgroup b writes chunk
// scramble(b / unit_chunks) * unit_chunks + (b + shift) % unit_chunks, so that chunk index and workgroup index agree modulo
// unit_chunks up to the shift (consecutive workgroups go to consecutive XCDs: with unit_chunks a multiple of 8 and
// shift 0 an XCD writes the chunks it would write in address order, only at other times).
extern "C" __global__ __launch_bounds__(256) void ep_calib_fill_affine(EpCalibFillArgs a) {
    const unsigned unit = blockIdx.x / a.unit_chunks, in_unit = (blockIdx.x + a.pad) % a.unit_chunks;
    const unsigned num_units = a.num_chunks / a.unit_chunks;
    const unsigned chunk = ((unit * 0x9E3779B1u) & (num_units - 1u)) * a.unit_chunks + in_unit;
    u32x4* p = (u32x4*)a.dst + (int64_t)chunk * 256 + threadIdx.x;
    const u32x4 v = {a.value, a.value, a.value, a.value};
    __builtin_nontemporal_store(v, p);
}

// num_fronts regions filling up row by row at the same pace (what the expert regions of a gather-formulated
// dispatch look like to the memory): workgroup b writes row b / num_fronts of front b % num_fronts, one
// 16-byte store per thread (row_bytes / 16 threads).
extern "C" __global__ __launch_bounds__(1024) void ep_calib_fronts(EpCalibFrontsArgs a) {
    const unsigned f = blockIdx.x % a.num_fronts, n = blockIdx.x / a.num_fronts;
    char* p = (char*)a.dst + (int64_t)f * a.front_pitch_bytes + (int64_t)n * a.row_bytes + (int64_t)threadIdx.x * 16;
    const u32x4 v = {a.value, n, f, 0u};
    __builtin_nontemporal_store(v, (u32x4*)p);
}

// Address-ordered mixed stream: workgroup b writes 4 KiB chunk b of dst; reads_num of every reads_den
// consecutive workgroups also read one 4 KiB chunk of src (in address order too).  The loaded value reaches
// memory only under a condition that never holds.
extern "C" __global__ __launch_bounds__(256) void ep_calib_mixed(EpCalibMixedArgs a) {
    const unsigned b = blockIdx.x;
    const unsigned grp = b / a.reads_den, in_grp = b - grp * a.reads_den;
    u32x4 v = {a.value, a.value, a.value, a.value};
    if (in_grp < a.reads_num) {
        const unsigned rc = grp * a.reads_num + in_grp;
        if (rc < a.num_read_chunks) {
            const u32x4 r = __builtin_nontemporal_load((const u32x4*)a.src + (int64_t)rc * 256 + threadIdx.x);
            if ((r.x ^ r.y ^ r.z ^ r.w) == 0x9E3779B1u) v = r;       // keeps the load alive
        }
    }
    __builtin_nontemporal_store(v, (u32x4*)a.dst + (int64_t)b * 256 + threadIdx.x);
}

// The loads of the fused copy kernel alone: a wave task is (token, 512 channels), one 16-byte non-temporal
// load per lane, nothing in front of it; the result is stored only under a condition that never holds.
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_read_rows(EpScatterArgs a) {
    const int lane = lane_id();
    const int task = blockIdx.x * EP_ROWS_PER_BLOCK + wave_id();
    const int i = task / a.num_parts, part = task - i * a.num_parts;
    if (i >= a.num_rows_bound) return;
    const int nvec = a.hidden >> 3;
    const int v = part * WAVE + lane;
    if (v >= nvec) return;
    const u32x4 d = __builtin_nontemporal_load((const u32x4*)((const char*)a.x + (int64_t)i * a.x_row_bytes) + v);
    if ((d.x ^ d.y ^ d.z ^ d.w) == 0x9E3779B1u && a.num_out_rows < 0) *((u32x4*)a.recv_x + v) = d;
}

extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_scatter_stores_only(EpScatterArgs a) {
    scatter_quant_body<true, false, false>(a);
}
// (the product kernel from this code object, for a like-for-like figure in the same run)
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_scatter_token_major(EpScatterArgs a) {
    scatter_quant_body<true, false, true>(a);
}

// ---- one task per destination row, tasks in destination order ------------------------------------
// order[i] = (slot, token | position << 24), slot < 0 = hole.  Flat: entry = task / groups.  Steered: the
// entries come as lists, one per (chunk, XCD); workgroup w of a chunk serves list w % 8 (consecutive
// workgroups go to consecutive XCDs), so that every reader of a token's row runs on one XCD and only the
// first misses that XCD's L2.  A wave task is EP_CALIB_U consecutive 512-channel parts of its row.
#define EP_CALIB_U 7

template <bool STEERED, bool LOADS, bool STORES>
__device__ __forceinline__ void ordered_body(const EpCalibOrderedArgs& o) {
    const EpScatterArgs& a = o.s;
    if ((int)blockIdx.x >= a.num_row_blocks) {
        zero_padding_rows(a);
        return;
    }
    constexpr int U = EP_CALIB_U;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int groups = o.groups;
    int entry, grp_i;
    if (!STEERED) {
        const int task = blockIdx.x * EP_ROWS_PER_BLOCK + wave;
        entry = task / groups;
        grp_i = task - entry * groups;
        if (entry >= o.num_entries) return;
    } else {
        const int wg = blockIdx.x;
        const int chunk = wg / (8 * o.wgs_per_list), w = wg - chunk * 8 * o.wgs_per_list;
        const int wt = (w >> 3) * EP_ROWS_PER_BLOCK + wave;
        const int le = wt / groups;
        grp_i = wt - le * groups;
        if (le >= o.entries_per_list) return;
        entry = (chunk * 8 + (w & 7)) * o.entries_per_list + le;
        if (entry >= o.num_entries) return;
    }
    const int2 e = o.order[entry];
    const int s = e.x, t = e.y & 0xffffff, j = e.y >> 24;
    if (s < 0 || s >= a.num_out_rows || t >= a.num_tokens || j >= a.num_topk) return;
    const int nvec = a.hidden >> 3;
    const u32x4* src = (const u32x4*)((const char*)a.x + (int64_t)t * a.x_row_bytes);
    u32x4 d[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int v = min((grp_i * U + u) * WAVE + lane, nvec - 1);
        if (LOADS) d[u] = src[v];              // plain loads: the other readers of the row find it in the L2
        else d[u] = u32x4{0x3f803f80u + (unsigned)v, 0x40004000u, 0xbf80bf80u, 0x3f003f00u};
    }
    char* orow = (char*)a.recv_x + (int64_t)s * a.out_row_bytes;
    float* osf = (float*)((char*)a.recv_sf + (int64_t)s * a.out_sf_row_bytes);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int v = (grp_i * U + u) * WAVE + lane;
        float f[8] = {bf16_lo(d[u].x), bf16_hi(d[u].x), bf16_lo(d[u].y), bf16_hi(d[u].y),
                      bf16_lo(d[u].z), bf16_hi(d[u].z), bf16_lo(d[u].w), bf16_hi(d[u].w)};
        unsigned mbits = 0u;
#pragma unroll
        for (int q = 0; q < 8; ++q) mbits = max(mbits, __float_as_uint(f[q]) & 0x7fffffffu);
        const float m = __uint_as_float(row16_umax(mbits));
        const float amax = m < 1e-4f ? 1e-4f : m;
        const float inv = (1.0f / amax) * 448.0f;
        const float scale = amax / 448.0f;
        u32x2 q8 = quant8<true>(f, inv);
        if (amax != amax) q8 = u32x2{0x7f7f7f7fu, 0x7f7f7f7fu};
        // without stores the results still have to be "used": a condition that never holds
        if (STORES ? v < nvec : (q8.x == 0x9E3779B1u && scale == 3.0f)) {
            stream_store<EP_SCATTER_ST_POL>((u32x2*)orow + v, q8);
            if ((lane & 15) == 0) osf[v >> 4] = scale;
        }
    }
    if (STORES && grp_i == 0 && lane == 0 && a.recv_topk_weights != nullptr)
        a.recv_topk_weights[s] = a.topk_weights[(int64_t)t * a.num_topk + j];
}

extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_ordered_flat(EpCalibOrderedArgs o) { ordered_body<false, true, true>(o); }
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_ordered_flat_stores_only(EpCalibOrderedArgs o) { ordered_body<false, false, true>(o); }
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_ordered_steered(EpCalibOrderedArgs o) { ordered_body<true, true, true>(o); }
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_ordered_steered_stores_only(EpCalibOrderedArgs o) { ordered_body<true, false, true>(o); }
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_ordered_steered_loads_only(EpCalibOrderedArgs o) { ordered_body<true, true, false>(o); }

// ---- two passes ----------------------------------------------------------------------------------
// Pass 1: every token's row quantised once, in token order, into staging rows (plain stores: pass 2 reads
// them at once).  A wave task is (token, 512 channels), as in the fused kernel.
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_quant_rows(EpCalibOrderedArgs o) {
    const EpScatterArgs& a = o.s;
    const int lane = lane_id();
    const int task = blockIdx.x * EP_ROWS_PER_BLOCK + wave_id();
    const int t = task / a.num_parts, part = task - t * a.num_parts;
    if (t >= a.num_tokens) return;
    const int nvec = a.hidden >> 3, v = part * WAVE + lane;
    if (v >= nvec) return;
    const u32x4 d = __builtin_nontemporal_load((const u32x4*)((const char*)a.x + (int64_t)t * a.x_row_bytes) + v);
    float f[8] = {bf16_lo(d.x), bf16_hi(d.x), bf16_lo(d.y), bf16_hi(d.y), bf16_lo(d.z), bf16_hi(d.z), bf16_lo(d.w), bf16_hi(d.w)};
    unsigned mbits = 0u;
#pragma unroll
    for (int q = 0; q < 8; ++q) mbits = max(mbits, __float_as_uint(f[q]) & 0x7fffffffu);
    const float m = __uint_as_float(row16_umax(mbits));
    const float amax = m < 1e-4f ? 1e-4f : m;
    const float inv = (1.0f / amax) * 448.0f;
    u32x2 q8 = quant8<true>(f, inv);
    if (amax != amax) q8 = u32x2{0x7f7f7f7fu, 0x7f7f7f7fu};
    ((u32x2*)(o.q_rows + (int64_t)t * a.hidden))[v] = q8;
    if ((lane & 15) == 0) o.q_sf[(int64_t)t * a.num_sf_packs + (v >> 4)] = amax / 448.0f;
}

// Pass 2: a wave copies one staged FP8 row (16 bytes a lane, up to 7 vectors: rows up to 7168 bytes) and its
// scale row to the entry's slot.  Needs hidden % 16 == 0 and 16-byte aligned scale rows.
template <bool STEERED>
__device__ __forceinline__ void copy_ordered_body(const EpCalibOrderedArgs& o) {
    const EpScatterArgs& a = o.s;
    if ((int)blockIdx.x >= a.num_row_blocks) {
        zero_padding_rows(a);
        return;
    }
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    int entry;
    if (!STEERED) {
        entry = blockIdx.x * EP_ROWS_PER_BLOCK + wave;
    } else {
        const int wg = blockIdx.x;
        const int chunk = wg / (8 * o.wgs_per_list), w = wg - chunk * 8 * o.wgs_per_list;
        const int le = (w >> 3) * EP_ROWS_PER_BLOCK + wave;
        if (le >= o.entries_per_list) return;
        entry = (chunk * 8 + (w & 7)) * o.entries_per_list + le;
    }
    if (entry >= o.num_entries) return;
    const int2 e = o.order[entry];
    const int s = e.x, t = e.y & 0xffffff, j = e.y >> 24;
    if (s < 0 || s >= a.num_out_rows || t >= a.num_tokens || j >= a.num_topk) return;
    const int nvec = a.hidden >> 4;
    const u32x4* src = (const u32x4*)(o.q_rows + (int64_t)t * a.hidden);
    u32x4 d[7];
#pragma unroll
    for (int u = 0; u < 7; ++u) d[u] = src[min(u * WAVE + lane, nvec - 1)];
    const int sfvec = a.num_sf_packs >> 2;              // 16-byte vectors of a scale row
    u32x4 sc = {0u, 0u, 0u, 0u};
    if (lane < sfvec) sc = ((const u32x4*)(o.q_sf + (int64_t)t * a.num_sf_packs))[lane];
    u32x4* dst = (u32x4*)((char*)a.recv_x + (int64_t)s * a.out_row_bytes);
#pragma unroll
    for (int u = 0; u < 7; ++u) {
        const int v = u * WAVE + lane;
        if (v < nvec) stream_store<EP_SCATTER_ST_POL>(dst + v, d[u]);
    }
    if (lane < sfvec) stream_store<EP_SCATTER_ST_POL>((u32x4*)((char*)a.recv_sf + (int64_t)s * a.out_sf_row_bytes) + lane, sc);
    if (lane == 0 && a.recv_topk_weights != nullptr) a.recv_topk_weights[s] = a.topk_weights[(int64_t)t * a.num_topk + j];
}
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_copy_ordered_flat(EpCalibOrderedArgs o) { copy_ordered_body<false>(o); }
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_copy_ordered_steered(EpCalibOrderedArgs o) { copy_ordered_body<true>(o); }

// The single-partition combine at top-6 whole, without its stores, and without its row fetches: what the gather
// and the store stream of the product kernel cost alone.
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_combine_k6(EpCombineArgs a) {
    combine_body<6, EP_COMBINE_FUSED>(a);
}
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_combine_k6_loads_only(EpCombineArgs a) {
    combine_body<6, EP_COMBINE_FUSED, true, false>(a);
}
extern "C" __global__ __launch_bounds__(EP_ROW_THREADS) void ep_calib_combine_k6_stores_only(EpCombineArgs a) {
    combine_body<6, EP_COMBINE_FUSED, false, true>(a);
}
