/* C ABI of libdeep_ep_hip.so -- the MI355X (gfx950) implementation of the EPBuffer
 * dispatch/combine hot path.  Plain pointers, sizes and a hipStream_t (passed as void*); no
 * torch types.  Each entry point names the reference interface it replaces (paths relative to
 * the reference checkout).
 *
 * Conventions
 *   - every function returning int returns 0 on success; on failure it returns non-zero and
 *     ep_last_error() gives a thread-local message.  Contract violations read
 *     "Assertion exception (<file>:<line>): <condition>", the text the reference's EP_HOST_ASSERT
 *     produces (deep_ep/include/deep_ep/common/exception.hpp:14-35).
 *   - all device pointers belong to the device that was current when the buffer was created;
 *     all kernels are enqueued on the `stream` argument and nothing synchronises unless said.
 *   - an ep_tensor_t with data == NULL means "absent".
 *   - a buffer is driven by one host thread at a time; different buffers may be used from
 *     different threads (ep_last_error is per thread).
 *   - none of the launch functions allocates, frees, memsets or synchronises: they only validate
 *     and enqueue kernels, so they can be recorded into a HIP graph.
 */
#ifndef DEEP_EP_HIP_H
#define DEEP_EP_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ep_buffer ep_buffer_t;

enum ep_dtype {
    EP_DTYPE_NONE = 0,
    EP_DTYPE_BF16 = 1,
    EP_DTYPE_FP8_E4M3 = 2,
    EP_DTYPE_I16 = 3,     /* any 2-byte element: the reference's sf_pack_t */
    EP_DTYPE_I32 = 4,
    EP_DTYPE_I64 = 5,
    EP_DTYPE_F32 = 6,
    EP_DTYPE_U8 = 7
};

typedef struct ep_tensor {
    void* data;
    int32_t dtype;        /* enum ep_dtype */
    int32_t ndim;         /* 1 or 2 */
    int64_t size[2];
    int64_t stride[2];    /* in elements */
} ep_tensor_t;

/* ---- library ------------------------------------------------------------------------------- */

/* Loads the ahead-of-time built gfx950 code object `<dir>/ep_kernels.hsaco` (dir == NULL: the
 * directory holding this library).  Replaces init_jit (csrc/runtime/jit.hpp:74-82,110-112). */
int ep_init(const char* dir);
const char* ep_last_error(void);

/* csrc/python_api.cpp:64-73 */
int64_t ep_get_num_allocation_alignment(void);   /* 2 MiB */
int64_t ep_get_num_tma_alignment(void);          /* 32 */
int64_t ep_get_num_rdma_alignment(void);         /* 32 */
/* Compute-unit count of the current device; stands where get_num_ai_cores does
 * (csrc/runtime/jit.hpp:89-91). */
int ep_get_num_compute_units(void);

/* EPBuffer::calculate_buffer_size (csrc/buffers/ep.hpp:581-605).  Returns -1 on a contract
 * violation. */
int64_t ep_calculate_buffer_size(int num_ranks, int num_max_tokens_per_rank, int hidden, int num_topk,
                                 int use_fp8_dispatch);
/* EPBuffer::get_dispatch_buffer_size / get_combine_buffer_size (csrc/buffers/ep.hpp:560-579). */
int64_t ep_get_dispatch_buffer_size(int num_max_tokens_per_rank, int hidden, int num_sf_packs, int num_topk,
                                    int element_size, int num_ranks);
int64_t ep_get_combine_buffer_size(int num_ranks, int num_max_tokens_per_rank, int hidden, int num_topk);

/* fp32 -> e4m3fn on the host with the integer algorithm the device fallback uses. */
void ep_host_f32_to_e4m3fn(const float* src, uint8_t* dst, int64_t n);
/* Compares the hardware conversion with the integer one over fp32 bit patterns
 * [first, first+count) with |x| <= limit.  out[0] = mismatches, out[1] = first mismatching
 * pattern.  Synchronises. */
int ep_fp8_selftest(uint64_t first, uint64_t count, float limit, uint64_t out[2]);
/* 1: hardware v_cvt_pk_fp8_f32 (default), 0: integer conversion. */
void ep_set_fp8_hw_convert(int enable);

/* The caller-side quantiser per_token_cast_to_fp8 (deep_ep/utils/math.py:30-38) on the device: x [T,H] BF16
 * (H a multiple of 8) -> q [T,H] e4m3fn bytes and sf [T, ceil(H/128)] fp32 with, per token and per group of 128
 * channels, sf = max(|x|, 1e-4) / 448 and q = e4m3fn(x * (448 / amax)), bit for bit what torch computes for that
 * formula on the CPU, and what ep_dispatch_epilogue_launch with fused_fp8_quant writes into the slots. */
int ep_per_token_cast_to_fp8(const ep_tensor_t* x, const ep_tensor_t* q, const ep_tensor_t* sf, void* stream);

/* ---- buffer ---------------------------------------------------------------------------------- */

/* One hipMalloc'd, zero-filled arena = workspace || buffer (num_bytes) || lb storage
 * (num_lb_bytes), plus a pinned mapped page for the receive counts.  Replaces the EPBuffer
 * constructor and its comm::Context / SymmetricMemory (csrc/buffers/ep.hpp:36-59,
 * csrc/kernels/comm/api.hpp:34-64, csrc/kernels/comm/symmetric.hpp:11-29). */
int ep_buffer_create(int rank_idx, int num_ranks, int64_t num_bytes, int64_t num_lb_bytes,
                     int num_cpu_timeout_secs, int num_gpu_timeout_secs, ep_buffer_t** out);
/* Makes bufs[0..n) the n partitions of one node living in this process: bufs[i] must be partition i
 * of n, all on the current device with equal buffer sizes.  From then on a dispatch of partition s
 * stores the packed rows for partition r straight into region s of r's arena and leaves the row
 * count in r's inbox, and the owner-side combine stores each partial into the arena of the
 * partition its token came from: what the reference does through symmetric memory
 * (csrc/kernels/comm/symmetric.hpp:11-29, impls/ep/dispatch.hpp:768-794, impls/ep/combine.hpp:291-324),
 * with plain device pointers standing where peer-mapped ones would on several GPUs.  There are no
 * cross-partition waits: the caller orders the launches (every partition's ep_dispatch_launch
 * before any ep_dispatch_recv_launch; every copy epilogue before any combine; every combine phase 0
 * before any phase 1), e.g. by enqueueing them in that order on one stream; the library counts
 * the phases of every partition and fails a call that comes before its peers' previous phase.
 * Destroying a
 * partition disconnects the others.  Synchronises.  No counterpart call in the reference, whose
 * ranks find each other through the process group. */
int ep_buffer_connect(ep_buffer_t** bufs, int n);
/* The same connection, one partition at a time and by address: arena_bases[i] is where partition i's
 * arena (what ep_buffer_region(peer, 0, ..) returns in the process that owns it) can be reached from
 * this process -- the pointer itself for a buffer of this process, or the mapping of that
 * allocation obtained otherwise (hipIpcOpenMemHandle in a process per GPU).  arena_bases[rank] must
 * be this buffer's own arena; all arenas must have been created with the same sizes.  The caller
 * keeps the mappings alive while the buffer is connected; arena_bases == NULL disconnects.
 * Synchronises. */
int ep_buffer_set_peers(ep_buffer_t* buf, void* const* arena_bases, int n);
/* EPBuffer::destroy (csrc/buffers/ep.hpp:65-73). */
int ep_buffer_destroy(ep_buffer_t* buf);
/* which: 0 workspace, 1 buffer, 2 lb storage (csrc/buffers/ep.hpp:50-53). */
void* ep_buffer_region(ep_buffer_t* buf, int which, int64_t* num_bytes);
/* BufferBase::print_memory_usage (csrc/buffers/base.hpp:37-49). */
int ep_buffer_print_memory_usage(ep_buffer_t* buf);

/* ---- dispatch -------------------------------------------------------------------------------- */

typedef struct ep_dispatch_args {
    /* inputs: x [T,H] BF16, or FP8 with sf [T,P] of 2-byte packs (either stride 1);
     * topk_idx [T,K] int64 (-1 = no selection); topk_weights [T,K] fp32 (optional);
     * cumulative_local_expert_recv_stats [E/R] int32 (optional).  csrc/buffers/ep.hpp:134-187 */
    ep_tensor_t x, sf, topk_idx, topk_weights, cumulative_local_expert_recv_stats;
    /* handle tensors: written in non-cached mode, only checked in cached mode (ep.hpp:205-246) */
    ep_tensor_t psum_num_recv_tokens_per_rank;          /* [R] int32 */
    ep_tensor_t psum_num_recv_tokens_per_expert;        /* [E/R] int32 */
    ep_tensor_t num_unaligned_recv_tokens_per_expert;   /* [E/R] int32 */
    ep_tensor_t dst_buffer_slot_idx;                    /* [T,K] int32 */
    ep_tensor_t dst_gsge_idx;                           /* [T,K] int32 */
    int32_t num_max_tokens_per_rank, num_experts, expert_alignment;
    int32_t cached_mode, do_cpu_sync;
    int32_t fused_fp8_quant;    /* extension: x is BF16 and is quantised to e4m3fn on the way */
    void* stream;
} ep_dispatch_args_t;

/* Validates like EPBuffer::dispatch (csrc/buffers/ep.hpp:113-246) and enqueues the layout
 * kernels: replaces launch_dispatch (csrc/kernels/ep/dispatch.hpp:20-82).  With more than one
 * partition this is the send side (dst_buffer_slot_idx, dst_gsge_idx, packed rows, inbox counts)
 * and ep_dispatch_recv_launch writes the other handle tensors. */
int ep_dispatch_launch(ep_buffer_t* buf, const ep_dispatch_args_t* args);

typedef struct ep_dispatch_recv_args {
    /* handle tensors, written here (csrc/buffers/ep.hpp:205-246) */
    ep_tensor_t psum_num_recv_tokens_per_rank;          /* [R] int32 */
    ep_tensor_t psum_num_recv_tokens_per_expert;        /* [E/R] int32 */
    ep_tensor_t num_unaligned_recv_tokens_per_expert;   /* [E/R] int32 */
    ep_tensor_t cumulative_local_expert_recv_stats;     /* [E/R] int32 (optional) */
    ep_tensor_t recv_src_metadata;                      /* [>= rows that can arrive, K+2] int32 out */
    int32_t hidden_bytes, num_sf_packs;                 /* payload bytes and 2-byte scale packs of a packed row */
    int32_t num_topk, num_max_tokens_per_rank, num_experts, expert_alignment;
    int32_t do_cpu_sync, reserved;
    void* stream;
    int64_t dispatch_stamp;                             /* ep_dispatch_stamp() taken after this dispatch's ep_dispatch_launch */
} ep_dispatch_recv_args_t;

/* Stamp of the buffer's latest non-cached ep_dispatch_launch (0: none): hand it to that dispatch's
 * ep_dispatch_recv_launch / ep_dispatch_epilogue_launch.  No counterpart in the reference, which leaves
 * the order of deferred epilogues to the caller. */
int64_t ep_dispatch_stamp(ep_buffer_t* buf);

/* Tuning: number of layout workgroups (128 tokens each) up to which the slot-assignment kernel sums the
 * per-workgroup histograms itself instead of a scan kernel running in between (default 256; quoted for count rows of
 * 264 columns, 256 local experts + one partition: with narrower rows the limit grows in proportion).  Results do
 * not depend on it. */
void ep_set_layout_fold_max_blocks(int num_blocks);

/* Tuning: with one partition and few layout blocks (blocks x top-k up to this limit; default and most 48, 0 turns it
 * off) the histogram kernel is not launched: every workgroup of the slot assignment counts the ids of all blocks itself.
 * Results do not depend on it. */
void ep_set_layout_recount_limit(int blocks_times_topk);

/* Tuning: workgroups (of 4 waves) of the single-partition combine kernel that a compute unit holds at once;
 * 0 lifts the cap, a negative value lets the library choose by top-k (the default: 3 at top-6 and top-8,
 * 4 at top-4, none at top-2 and for launches too small to fill the machine twice).  The cap is enforced through
 * an LDS allocation: the smallest one that can be enforced is 2 (a request for 1 is served as 2), and values from
 * 160 on mean no cap.  Results do not depend on it. */
void ep_set_combine_blocks_per_cu(int num_blocks);

/* More than one partition, non-cached dispatch: the receive side of launch_dispatch and the slot
 * assignment of the copy epilogue (impls/ep/dispatch.hpp:469-545,
 * impls/ep/dispatch_copy_epilogue.hpp:130-174,397-423,471-488,514-522).  Walks the rows that
 * arrived in this partition's regions (source partitions in turn, each up to its inbox count),
 * ranks them per local expert and writes the handle tensors, the metadata rows and, with
 * do_cpu_sync, the host counts.  Rows can arrive from n * num_max_tokens_per_rank tokens in a
 * node, from the dispatched tokens otherwise.  A no-op with one partition.  Call it after
 * ep_dispatch_launch (of every partition of a node) and before ep_dispatch_wait_counts /
 * ep_dispatch_epilogue_launch. */
int ep_dispatch_recv_launch(ep_buffer_t* buf, const ep_dispatch_recv_args_t* args);

/* Host wait for the counts of the last non-cached do_cpu_sync dispatch, with the buffer's CPU
 * timeout ("reduction timeout").  per_expert receives E/R aligned counts.  Replaces the
 * reduction::host::wait_ready loop of csrc/buffers/ep.hpp:295-315. */
int ep_dispatch_wait_counts(ep_buffer_t* buf, int* num_recv_tokens, int* num_expanded_tokens, int* per_expert);
/* Worst-case sizes without a host sync (csrc/buffers/ep.hpp:288,316-320).  buf == NULL: one partition. */
int ep_dispatch_worst_case_sizes(ep_buffer_t* buf, int num_max_tokens_per_rank, int num_topk, int num_experts,
                                 int expert_alignment, int* num_recv_tokens, int* num_expanded_tokens);

/* recv_sf_layout of ep_dispatch_epilogue_args_t */
enum ep_sf_layout {
    EP_SF_LAYOUT_ROW_MAJOR = 0,
    EP_SF_LAYOUT_COL_MAJOR = 1,
    EP_SF_LAYOUT_COL_MAJOR_COUNTED = 2
};

typedef struct ep_dispatch_epilogue_args {
    ep_tensor_t x, sf, topk_weights;                    /* as given to ep_dispatch_launch */
    ep_tensor_t psum_num_recv_tokens_per_rank, psum_num_recv_tokens_per_expert;
    ep_tensor_t recv_x;                                 /* [N_exp,H] out, dtype of x (FP8 if fused) */
    ep_tensor_t recv_sf;                                /* [N_exp,P] out, laid out as recv_sf_layout says */
    ep_tensor_t recv_sf_staging;                        /* [N_exp,P] row-major scratch; layouts 1 and 2 only */
    ep_tensor_t recv_topk_weights;                      /* [N_exp] fp32 out (optional) */
    ep_tensor_t recv_src_metadata;                      /* [N_recv,K+2] int32: out, or in when cached */
    int32_t num_topk, num_max_tokens_per_rank, num_experts, expert_alignment;
    int32_t cached_mode, do_zero_padding, fused_fp8_quant;
    /* 0: rows of scales, strides (P,1) (ep.hpp:328-336).  1: columns of scales, strides (1,N_exp): the
     * layout the reference reaches with a transposing copy after its epilogue (ep.hpp:379-381); here
     * the copy kernel writes scale rows into recv_sf_staging and a tiled kernel turns them into
     * recv_sf.  2: as 1, but recv_sf describes storage for an upper bound of rows and the column
     * stride is the expanded row count of this dispatch, read on the device: the result is the
     * tensor of shape (N_exp,P), strides (1,N_exp) at the start of that storage. */
    int32_t recv_sf_layout;
    void* stream;
    /* non-cached mode: ep_dispatch_stamp() taken after this dispatch's ep_dispatch_launch.  The slot map the
     * epilogue reads lives in the buffer's workspace, which the next ep_dispatch_launch overwrites: an epilogue
     * whose stamp is not the latest fails with an Assertion exception instead of scattering one dispatch's
     * rows with another's slots (the usage contract of csrc/buffers/ep.hpp:284-286,396-408, enforced). */
    int64_t dispatch_stamp;
} ep_dispatch_epilogue_args_t;

/* Expands every received row into its expert-major slots and zeroes the alignment padding:
 * replaces launch_dispatch_copy_epilogue (csrc/kernels/ep/dispatch.hpp:84-139). */
int ep_dispatch_epilogue_launch(ep_buffer_t* buf, const ep_dispatch_epilogue_args_t* args);

/* A whole single-partition dispatch without a host sync (ep_dispatch_launch followed by
 * ep_dispatch_epilogue_launch, non-cached, do_cpu_sync = 0) that needs no ep_buffer and allocates
 * nothing: the layout scratch lives in a device array inside the library (ep_dispatch_static_scratch_capacity()
 * bytes, 4 MiB) instead of a buffer's arena.  It has no counterpart in the reference; it is for callers that
 * cannot allocate (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * ep_init must have run on the device before the first such call: loading the code object and looking up the
 * array's address do allocate, and ep_init is where they happen.  The caller passes every input and output, the
 * outputs sized by ep_dispatch_worst_case_sizes(NULL, ...); epilogue_args->dispatch_stamp is ignored.  Fails
 * with a clear message when the scratch the shape needs, ep_dispatch_static_scratch_bytes(T, K, E) =
 * 4096 + 4 * (a64(W) + a64(B * W) + a64(T * K) + a64(T)) with W = E + 1 rounded up to 8, B = ceil(T / 128) (at
 * least 1) and a64 rounding up to a multiple of 64, exceeds the array.  Results equal those of the two calls it
 * stands for.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (different streams,
 * or host threads) race; calls on one stream are ordered and safe. */
int64_t ep_dispatch_static_scratch_bytes(int num_tokens, int num_topk, int num_experts);
int64_t ep_dispatch_static_scratch_capacity(void);
int ep_dispatch_static_launch(const ep_dispatch_args_t* args, const ep_dispatch_epilogue_args_t* epilogue_args);

/* ---- combine --------------------------------------------------------------------------------- */

typedef struct ep_combine_args {
    ep_tensor_t x;                      /* [N_exp,H] BF16 */
    ep_tensor_t topk_weights;           /* [N_exp] fp32 (optional) */
    ep_tensor_t bias_0, bias_1;         /* [T,H] BF16 (optional) */
    ep_tensor_t src_metadata;           /* [N_recv,K+2] int32 */
    ep_tensor_t combined_topk_idx;      /* [T,K] int64 */
    ep_tensor_t psum_num_recv_tokens_per_rank;   /* [R] int32 */
    ep_tensor_t combined_x;             /* [T,H] BF16 out */
    ep_tensor_t combined_topk_weights;  /* [T,K] fp32 out (iff topk_weights) */
    int32_t num_experts, num_max_tokens_per_rank;
    int32_t apply_weights;              /* extension: multiply rows by their gate weight */
    void* stream;
} ep_combine_args_t;

/* Validates like EPBuffer::combine (csrc/buffers/ep.hpp:426-481).  Replaces launch_combine and
 * launch_combine_reduce_epilogue (csrc/kernels/ep/combine.hpp:18-112); `phase` selects which
 * half of the reference's two launches is enqueued: 0 = owner-side reduce, 1 = token-side
 * reduce into combined_x.  With one partition the whole reduction runs in phase 1.  Phase 1 of a
 * buffer that is one partition of several reads, for every token, one partial per destination
 * partition from this buffer's combine region: in a connected node the peers' phase 0 put them there;
 * a partition used alone (not connected) holds only its own partials after phase 0, the caller
 * places the others (what a transport would deliver) before phase 1. */
int ep_combine_launch(ep_buffer_t* buf, const ep_combine_args_t* args, int phase);

#ifdef __cplusplus
}
#endif
#endif /* DEEP_EP_HIP_H */
