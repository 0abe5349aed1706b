/* C ABI of libdeep_ep_calib.so -- the measurement rig of the benchmarks for the MI355X EP dispatch path.
 * It is NOT part of the product: libdeep_ep_hip.so neither links nor loads it, and nothing in it has a
 * counterpart in the reference.  It owns a code object of its own (ep_calib.hsaco, next to the library)
 * with pure-write patterns, the product's fused copy kernel and its combine kernel with their loads or their
 * stores taken out, and the destination-ordered and two-pass formulations of the copy kernel, so that every figure a benchmark
 * quotes for "what the memory system allows" comes from a committed kernel run in the same process.
 * Every function returns 0 on success; otherwise ep_calib_last_error() holds a thread-local message.
 * Nothing here allocates or synchronises; all kernels are enqueued on `stream`. */
#ifndef DEEP_EP_CALIB_H
#define DEEP_EP_CALIB_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Loads `<dir>/ep_calib.hsaco` (dir == NULL: the directory holding this library). */
int ep_calib_init(const char* dir);
const char* ep_calib_last_error(void);

/* num_bytes / 4096 workgroups each write one 4 KiB chunk of dst with one 16-byte non-temporal store per
 * thread: in address order (shuffled = 0), or with runs of `shuffled` consecutive chunks kept together and
 * the runs in a scrambled order (shuffled and the chunk count powers of two). */
int ep_calib_fill(void* dst, int64_t num_bytes, int shuffled, unsigned value, void* stream);

/* The chunks in a scrambled order again, but workgroup b writes a chunk whose index equals b + shift modulo
 * `modulus` (a power of two, as the chunk count): consecutive workgroups go to consecutive XCDs, so with a modulus
 * that is a multiple of 8 and shift 0 every XCD writes exactly the chunks it writes in address order, only at
 * other times; a shift moves every chunk to another XCD. */
int ep_calib_fill_affine(void* dst, int64_t num_bytes, int modulus, int shift, unsigned value, void* stream);

/* num_fronts regions, front_pitch_bytes apart, filling up row by row in lock step: workgroup b writes row
 * b / num_fronts of front b % num_fronts (row_bytes a multiple of 16, at most 16384). */
int ep_calib_fronts(void* dst, int num_fronts, int rows_per_front, int row_bytes, int64_t front_pitch_bytes,
                    unsigned value, void* stream);

/* An address-ordered stream of 4 KiB chunks: every chunk of dst (write_bytes) is written, and reads_num of
 * every reads_den workgroups also read a chunk of src (which must hold write_bytes * reads_num / reads_den
 * bytes, rounded up to 4 KiB). */
int ep_calib_mixed(const void* src, void* dst, int64_t write_bytes, int reads_num, int reads_den, unsigned value,
                   void* stream);

enum ep_calib_variant {
    EP_CALIB_TOKEN_MAJOR = 0,           /* the product's fused copy kernel body, cached-replay form */
    EP_CALIB_STORES_ONLY = 1,           /* ... without its loads of x (outputs hold arbitrary payload) */
    EP_CALIB_READ_ROWS = 2,             /* ... its loads of x alone (nothing is written) */
    EP_CALIB_ORDERED_FLAT = 3,          /* one task per destination row, destination order inside chunks */
    EP_CALIB_ORDERED_FLAT_STORES_ONLY = 4,
    EP_CALIB_ORDERED_STEERED = 5,       /* ... the readers of a token steered to one XCD */
    EP_CALIB_ORDERED_STEERED_STORES_ONLY = 6,
    EP_CALIB_ORDERED_STEERED_LOADS_ONLY = 7,
    EP_CALIB_QUANT_ROWS = 8,            /* two passes, pass 1: x -> q_rows, q_sf in token order */
    EP_CALIB_COPY_ORDERED_FLAT = 9,     /* two passes, pass 2: staged rows -> slots in destination order */
    EP_CALIB_COPY_ORDERED_STEERED = 10
};

typedef struct ep_calib_scatter {
    /* a single-partition fused-FP8 dispatch as its cached replay sees it */
    const void* x;                      /* [T, H] BF16 */
    const float* topk_weights;          /* [T, K] or NULL */
    const int32_t* recv_src_metadata;   /* [num_recv_rows, K + 2] of the dispatch handle */
    const int32_t* num_recv;            /* device scalar: received rows */
    const int32_t* psum_expert;         /* [E] psum_num_recv_tokens_per_expert of the handle */
    void* recv_x;                       /* [num_out_rows, H] FP8 out */
    float* recv_sf;                     /* [num_out_rows, H / 128] out */
    float* recv_topk_weights;           /* [num_out_rows] out, or NULL */
    /* destination-ordered variants: (slot, token | position << 24) pairs, a negative slot is a hole.
     * Flat: num_entries pairs, sorted by slot inside each chunk of tokens.  Steered: num_lists lists of
     * entries_per_list pairs each, list (chunk * 8 + x) holding the chunk's entries of the tokens with
     * token % 8 == x, sorted by slot, padded with holes. */
    const int32_t* order;
    void* q_rows;                       /* two passes: [T, H] bytes of staging */
    float* q_sf;                        /* two passes: [T, H / 128] */
    int32_t num_tokens, hidden, num_topk, num_experts, expert_alignment;
    int32_t num_recv_rows, num_out_rows;
    int32_t do_zero_padding;
    int32_t num_entries, entries_per_list, num_lists;
    void* stream;
} ep_calib_scatter_t;

/* Enqueues one variant.  H must be a multiple of 128 (a multiple of 512 and at most 7168 for the two-pass
 * variants), T at most 2^24 - 1, K at most 32. */
int ep_calib_scatter(int variant, const ep_calib_scatter_t* args);

enum ep_calib_combine_variant {
    EP_CALIB_COMBINE = 0,               /* the product's single-partition combine body at top-6 */
    EP_CALIB_COMBINE_LOADS_ONLY = 1,    /* ... its row fetches and sums alone (nothing is written) */
    EP_CALIB_COMBINE_STORES_ONLY = 2    /* ... its stores alone (rows of filler values; nothing is fetched but the slots) */
};

typedef struct ep_calib_combine {
    /* a single-partition BF16 combine at top-6 without biases, as the product's kernel takes it */
    const void* y;                      /* [num_in_rows, H] BF16 expert outputs */
    const float* expanded_weights;      /* [num_in_rows] or NULL */
    const int32_t* recv_src_metadata;   /* [num_recv_rows, K + 2] of the dispatch handle */
    const int32_t* num_recv;            /* device scalar: received rows */
    const int64_t* topk_idx;            /* [T, K] */
    void* combined_x;                   /* [T, H] BF16 out */
    float* combined_topk_weights;       /* [T, K] out, or NULL (iff expanded_weights is NULL) */
    int32_t num_tokens, hidden, num_topk, num_experts;
    int32_t num_recv_rows, num_in_rows;
    int32_t blocks_per_cu;              /* workgroups a compute unit holds at once (0: no cap); the library's own choice at top-6 is 3 */
    int32_t reserved;
    void* stream;
} ep_calib_combine_t;

/* Enqueues one variant.  K must be 6, H a multiple of 8. */
int ep_calib_combine(int variant, const ep_calib_combine_t* args);

#ifdef __cplusplus
}
#endif
#endif /* DEEP_EP_CALIB_H */
