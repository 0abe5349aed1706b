// Kernel argument blocks shared by the device code object (ep_kernels.hip) and the host
// runtime (ep_runtime.cpp).  Every kernel takes exactly one of these structs by value, so a
// launch through hipModuleLaunchKernel marshals a single parameter.
#pragma once
#include <stdint.h>

#define EP_MAX_RANKS 256          // reference: common/compiled.hpp:35
#define EP_MAX_EXPERTS 2048       // reference: common/compiled.hpp:36
#define EP_MAX_TOPK 32            // reference: csrc/kernels/ep/combine.hpp:85
#define EP_TOKENS_PER_BLOCK 128   // tokens owned by one layout workgroup
#define EP_LAYOUT_THREADS 256
#define EP_SCAN_THREADS 1024
#define EP_ROW_THREADS 256        // 4 waves, one row per wave
#define EP_ROWS_PER_BLOCK 4
#define EP_MAX_PAD_BLOCKS_PER_EXPERT 16

#define EP_LAYOUT_SCANNED 0
#define EP_LAYOUT_FOLDED 1
#define EP_LAYOUT_SINGLE 2
#define EP_LAYOUT_RECOUNTED 3     // no kernel in front: every workgroup counts the ids of all (few) blocks itself
#define EP_RECOUNT_DEPTH 24       // ids a thread of the slot assignment holds in flight for that (blocks x top-k <= 2 x this)

#define EP_SCATTER_EXPAND 0
#define EP_SCATTER_PACK 1
#define EP_SCATTER_REGION 2

#define EP_COMBINE_FUSED 0      // single partition: owner-side and token-side reduce in one pass
#define EP_COMBINE_PARTIAL 1    // owner side: per received row, partial into the combine buffer
#define EP_COMBINE_FINAL 2      // token side: biases + partials of the masters into combined_x

// Host-visible count page (pinned, mapped).  Written once per non-cached dispatch.
//   [0] ready sequence number (written last, release at system scope)
//   [1] number of received tokens   [2] number of expanded tokens (aligned)
//   [16 .. 16+R)                 received tokens per source rank
//   [16+EP_MAX_RANKS .. +El)     aligned received tokens per local expert
// Fixed header of every arena's workspace; the layout scratch is carved behind it.
//   [0, 4*EP_MAX_RANKS)                    inbox: rows each source partition put into this partition's regions
//   [EP_WS_PEERS_OFF, +8*EP_MAX_RANKS)     arena base of every partition of the node (own arena when not connected)
#define EP_WS_INBOX_OFF 0
#define EP_WS_PEERS_OFF 1024
#define EP_WS_HEADER_BYTES 4096

#define EP_HOST_RANK_OFF 16
#define EP_HOST_EXPERT_OFF (16 + EP_MAX_RANKS)
#define EP_HOST_PAGE_INTS (16 + EP_MAX_RANKS + EP_MAX_EXPERTS)

struct EpLayoutArgs {
    const int64_t* topk_idx;      // [T, K]
    int num_tokens, num_topk, num_experts, num_ranks;
    int rank_idx, expert_alignment, max_tokens, experts_per_rank;
    int num_blocks;               // ceil(T / EP_TOKENS_PER_BLOCK), at least 1
    int seq;                      // value the host waits for in host_page[0]
    int notify_host;              // do_cpu_sync
    int scan_mode;                // EP_LAYOUT_*: where ep_layout_assign finds the other blocks' counts
    // scratch (device)
    int* blk_cnt;                 // [num_blocks, cnt_stride]  per workgroup: entries per local expert (columns [0, El)),
                                  //   masters per partition (columns [El, El + R)), zeros up to the stride: 16-bit counts
                                  //   (EP_LAYOUT_FOLDED), or ints that ep_layout_scan replaces by the exclusive prefix
                                  //   over the workgroups (EP_LAYOUT_SCANNED)
    int* col_total;               // [cnt_stride]  column totals (written by ep_layout_scan)
    int cnt_stride;               // El + R rounded up to a multiple of 8 columns
    int* slot_map;                // [T, K]  expanded slot of (t, j) if its expert is local, else -1
    int* tok_row;                 // [T]  token -> its row of the receive stream (written for received tokens only)
    // handle tensors (device)
    int* dst_buffer_slot_idx;     // [T, K]
    int* dst_gsge_idx;            // [T, K]
    int* psum_rank;               // [R]
    int* psum_expert;             // [El]
    int* unaligned_expert;        // [El]
    int* cumulative_stats;        // [El] or null
    int* host_page;               // device view of the mapped host page
    // partitioned path (more than one partition)
    int send_only;                // send side: only dst_buffer_slot_idx / dst_gsge_idx and the peers' inboxes are written
    int recv_mode;                // receive side: the entries are the rows that arrived in this partition's regions
    char* const* peer_arenas;     // [R] arena bases (send side: whose inbox gets this partition's row counts)
    const int* inbox;             // [R] rows per source (receive side)
    const char* packed_base;      // this partition's regions of packed rows (receive side)
    int64_t packed_row_bytes;
    int idx_off, src_off;         // byte offsets of topk_idx and of the source token inside a packed row
    int* recv_src_metadata;       // [rows_cap, K+2]  (receive side: written here, there is no slot_map)
    int rows_cap;                 // rows the metadata tensor holds
    int connected;                // the peers are arenas of their own (a node), not this arena again
};

// One receive-stream row per wave: copy (or quantise) it into every expanded slot it owns.
struct EpScatterArgs {
    const void* x;                // [T, hidden] rows: BF16, or FP8 bytes when prequantised
    const void* sf;               // input scale factors (prequantised FP8) or null
    const float* topk_weights;    // [T, K] or null
    const int* slot_map;          // [T, K]   (non-cached)
    const int* tok_row;           // [T]      (non-cached)
    const int* num_recv_ptr;      // device scalar: psum_rank[R-1]  (modes whose rows are the receive stream)
    int* recv_src_metadata;       // [N, K+2]  written (non-cached) / read (cached)
    void* recv_x;                 // [N_exp, hidden] out
    void* recv_sf;                // out or null
    float* recv_topk_weights;     // [N_exp] out or null
    const int* psum_expert;       // [El]  (padding ranges)
    int64_t x_row_bytes;          // bytes per source row
    int64_t out_row_bytes;        // bytes per output row
    int64_t sf_token_stride_bytes, sf_pack_stride_bytes;   // input SF strides
    int64_t out_sf_row_bytes;
    int hidden;                   // channels per row
    int num_topk, num_rows_bound;     // grid covers rows [0, num_rows_bound)
    int rank_idx, max_tokens;
    int cached;                   // slots come from recv_src_metadata
    int num_sf_packs;             // 2-byte packs per row (prequantised) ; fused: hidden/128 floats
    int num_local_experts, expert_alignment;
    int num_meta_rows;            // rows recv_src_metadata holds
    int num_row_blocks;           // blocks [0, num_row_blocks) copy rows, the rest zero padding
    int num_tokens;               // T: bound of the token indices a row may name
    int num_parts;                // column parts per row; a wave task is (row, part)
    int mode;                     // EP_SCATTER_*
    // partitioned path (EP_SCATTER_PACK / EP_SCATTER_REGION)
    const int64_t* topk_idx;      // [T, K]            (pack)
    const int* dst_slot_idx;      // [T, K]            (pack)
    int64_t copy_bytes;           // payload bytes moved per row (verbatim kernel)
    int num_experts, experts_per_rank;
    int with_metadata;            // packed rows carry topk_idx and the source token (non-cached)
    int idx_off, w_off, src_off;  // byte offsets of the packed metadata inside a row
    int num_out_rows;             // rows of recv_x: slots outside are ignored
    int pad_blocks_per_expert;    // workgroups that share the zeroing of one expert's padding rows
    // where packed rows go (pack) and come from (region): partition p's regions start at
    // peer_arenas[p] + buffer_off; a row for partition r lands in region `region_by_source ? rank_idx : r`
    char* const* peer_arenas;
    const int* psum_rank;         // [R] inclusive row counts per source (region mode: stream row -> region, slot)
    int64_t buffer_off;
    int region_by_source;
    int num_ranks;
    int pack_sf_off;              // byte offset of the scales inside a packed row (pack mode)
    int vecs_per_lane;            // verbatim kernel: 16-byte vectors a lane moves per task (1..4)
    int rows_are_tokens;          // cached expand: every token was received, so row i of the receive stream is token i
};

// recv_sf layouts: rows of scales, or columns of scales whose stride is the row count of recv_sf
// (EP_SF_COL_MAJOR) or the expanded row count the layout pass produced (EP_SF_COL_MAJOR_COUNTED:
// the host does not know it yet when the kernel is enqueued).
#define EP_SF_ROW_MAJOR 0
#define EP_SF_COL_MAJOR 1
#define EP_SF_COL_MAJOR_COUNTED 2
#define EP_SF_TILE 64

// Row-major scale rows -> column-major, 64 x 64 tiles through LDS.
struct EpSfTransposeArgs {
    const void* src;              // [num_rows, num_cols] row-major
    void* dst;                    // column c starts at element c * (row count)
    const int* psum_expert;       // [El]: the expanded row count is its last entry, aligned (counted layout)
    int num_rows, num_cols;
    int elem_bytes;               // 2 or 4
    int counted;                  // row count and column stride come from psum_expert
    int num_local_experts, expert_alignment;
};

// Fused single-partition combine: one receive-stream row per wave.
struct EpCombineArgs {
    const void* y;                // [N_exp, hidden] BF16 expert outputs
    const float* expanded_weights;// [N_exp] or null
    const void* bias_0;           // [T, hidden] BF16 or null
    const void* bias_1;
    const int* recv_src_metadata; // [N, K+2]
    const int* num_recv_ptr;      // device scalar
    const int64_t* topk_idx;      // [T, K]
    void* combined_x;             // [T, hidden] BF16 out
    float* combined_topk_weights; // [T, K] out or null
    int hidden, num_topk, num_tokens, num_rows_bound;
    int rank_idx, max_tokens;
    int weighted;                 // opt-in: multiply by the gate weight before summing
    int num_row_blocks;           // blocks [0, num_row_blocks) reduce rows, the rest handle unrouted tokens
    int num_experts;
    int num_parts;                // 1024-channel parts per row; a wave task is (row, part)
    int64_t y_row_bytes;          // stride of the rows being gathered (hidden*2, or a combine-buffer token)
    int64_t out_row_bytes;        // stride of the rows being written
    int num_ranks, experts_per_rank;
    int num_in_rows;              // rows of y: slots outside are ignored
    int num_groups;               // partial groups of the combine buffer: min(K, R)
    // owner-side reduce: the partial of a row goes to the combine buffer of the partition its token came from
    char* const* peer_arenas;
    int64_t buffer_off;
    int whole_rows;               // owner-side reduce: a task is a whole row (num_parts == 1), not a 1024-channel part
};

// Caller-side quantiser: rows of BF16 -> rows of e4m3fn bytes + one fp32 scale per row and 128 channels.
struct EpQuantArgs {
    const void* x;                // [num_rows, hidden] BF16
    void* q;                      // [num_rows, hidden] e4m3fn out
    float* sf;                    // [num_rows, ceil(hidden / 128)] out
    int num_rows, hidden;
    int num_parts;                // 512-channel parts per row; a wave task is (row, part)
    int hw_convert;               // 1: v_cvt_pk_fp8_f32, 0: integer conversion
};

// Hardware vs integer e4m3fn conversion over fp32 bit patterns [first, first+count).
struct EpFp8TestArgs {
    unsigned long long first, count;
    unsigned long long* out;      // [0] mismatches, [1] first mismatching pattern
    float limit;                  // only |x| <= limit is compared (NaN patterns are skipped)
    int pad;
};
