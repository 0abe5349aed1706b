/* A caller of libdeep_ep_hip.so written in plain C: no torch, no C++, device memory from hipMalloc.
 * It sends 64 tokens of small integers to 2 of 8 experts each, checks the layout the library
 * reports against counts made here, lets the "experts" be the identity and checks that the combine
 * returns exactly twice every token (two copies of a small integer sum exactly in fp32 and round
 * exactly to BF16) with the gate weights carried back.  Exit status 0 and "abi_client: ok" on success.
 *
 * Built by deep_ep/_build.py with gcc; run by the GPU tests. */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/deep_ep_hip.h"

#define T 64
#define H 256
#define E 8
#define K 2
#define A 4

#define CHECK_HIP(call)                                                              \
    do {                                                                             \
        hipError_t e_ = (call);                                                      \
        if (e_ != hipSuccess) {                                                      \
            fprintf(stderr, "abi_client: %s -> %s\n", #call, hipGetErrorString(e_)); \
            return 2;                                                                \
        }                                                                            \
    } while (0)
#define CHECK_EP(call)                                                          \
    do {                                                                        \
        if ((call) != 0) {                                                      \
            fprintf(stderr, "abi_client: %s -> %s\n", #call, ep_last_error()); \
            return 3;                                                           \
        }                                                                       \
    } while (0)
#define EXPECT(cond)                                                \
    do {                                                            \
        if (!(cond)) {                                              \
            fprintf(stderr, "abi_client: expected %s\n", #cond);   \
            return 4;                                               \
        }                                                           \
    } while (0)

static uint16_t bf16_of_small_int(int v) {      /* |v| < 256: exact */
    float f = (float)v;
    uint32_t u;
    memcpy(&u, &f, 4);
    return (uint16_t)(u >> 16);
}

static ep_tensor_t tensor(void* data, int dtype, int ndim, int64_t n0, int64_t n1) {
    ep_tensor_t t;
    memset(&t, 0, sizeof t);
    t.data = data;
    t.dtype = dtype;
    t.ndim = ndim;
    t.size[0] = n0;
    t.size[1] = ndim == 2 ? n1 : 0;
    t.stride[0] = ndim == 2 ? n1 : 1;
    t.stride[1] = ndim == 2 ? 1 : 0;
    return t;
}

static void* dev_alloc(size_t n) {
    void* p = NULL;
    if (hipMalloc(&p, n ? n : 16) != hipSuccess) return NULL;
    return p;
}

int main(void) {
    static uint16_t x[T][H], out[T][H];
    static int64_t topk[T][K];
    static float w[T][K], wout[T][K];
    int count[E] = {0};
    for (int t = 0; t < T; ++t) {
        for (int h = 0; h < H; ++h) x[t][h] = bf16_of_small_int((t * 7 + h) % 13 - 6);
        topk[t][0] = t % E;
        topk[t][1] = (t + 3) % E;
        for (int j = 0; j < K; ++j) {
            w[t][j] = 0.25f + (float)j + (float)t / 128.0f;
            ++count[topk[t][j]];
        }
    }
    int expanded = 0;
    for (int e = 0; e < E; ++e) expanded += (count[e] + A - 1) / A * A;

    CHECK_EP(ep_init(NULL));
    const int64_t bytes = ep_calculate_buffer_size(1, T, H, K, 0);
    EXPECT(bytes > 0 && bytes % ep_get_num_allocation_alignment() == 0);
    ep_buffer_t* buf = NULL;
    CHECK_EP(ep_buffer_create(0, 1, bytes, 0, 30, 30, &buf));

    void *d_x = dev_alloc(sizeof x), *d_topk = dev_alloc(sizeof topk), *d_w = dev_alloc(sizeof w);
    void *d_psum_rank = dev_alloc(4), *d_psum_expert = dev_alloc(4 * E), *d_unaligned = dev_alloc(4 * E);
    void *d_slot = dev_alloc(4 * T * K), *d_gsge = dev_alloc(4 * T * K);
    EXPECT(d_x && d_topk && d_w && d_psum_rank && d_psum_expert && d_unaligned && d_slot && d_gsge);
    CHECK_HIP(hipMemcpy(d_x, x, sizeof x, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_topk, topk, sizeof topk, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_w, w, sizeof w, hipMemcpyHostToDevice));
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));

    ep_dispatch_args_t a;
    memset(&a, 0, sizeof a);
    a.x = tensor(d_x, EP_DTYPE_BF16, 2, T, H);
    a.topk_idx = tensor(d_topk, EP_DTYPE_I64, 2, T, K);
    a.topk_weights = tensor(d_w, EP_DTYPE_F32, 2, T, K);
    a.psum_num_recv_tokens_per_rank = tensor(d_psum_rank, EP_DTYPE_I32, 1, 1, 0);
    a.psum_num_recv_tokens_per_expert = tensor(d_psum_expert, EP_DTYPE_I32, 1, E, 0);
    a.num_unaligned_recv_tokens_per_expert = tensor(d_unaligned, EP_DTYPE_I32, 1, E, 0);
    a.dst_buffer_slot_idx = tensor(d_slot, EP_DTYPE_I32, 2, T, K);
    a.dst_gsge_idx = tensor(d_gsge, EP_DTYPE_I32, 2, T, K);
    a.num_max_tokens_per_rank = T;
    a.num_experts = E;
    a.expert_alignment = A;
    a.do_cpu_sync = 1;
    a.stream = stream;
    CHECK_EP(ep_dispatch_launch(buf, &a));

    int n_recv = -1, n_exp = -1, per_expert[E];
    CHECK_EP(ep_dispatch_wait_counts(buf, &n_recv, &n_exp, per_expert));
    EXPECT(n_recv == T && n_exp == expanded);
    for (int e = 0; e < E; ++e) EXPECT(per_expert[e] == (count[e] + A - 1) / A * A);

    void *d_recv_x = dev_alloc((size_t)n_exp * H * 2), *d_recv_w = dev_alloc((size_t)n_exp * 4);
    void* d_meta = dev_alloc((size_t)n_recv * (K + 2) * 4);
    EXPECT(d_recv_x && d_recv_w && d_meta);
    ep_dispatch_epilogue_args_t e;
    memset(&e, 0, sizeof e);
    e.x = a.x;
    e.topk_weights = a.topk_weights;
    e.psum_num_recv_tokens_per_rank = a.psum_num_recv_tokens_per_rank;
    e.psum_num_recv_tokens_per_expert = a.psum_num_recv_tokens_per_expert;
    e.recv_x = tensor(d_recv_x, EP_DTYPE_BF16, 2, n_exp, H);
    e.recv_topk_weights = tensor(d_recv_w, EP_DTYPE_F32, 1, n_exp, 0);
    e.recv_src_metadata = tensor(d_meta, EP_DTYPE_I32, 2, n_recv, K + 2);
    e.num_topk = K;
    e.num_max_tokens_per_rank = T;
    e.num_experts = E;
    e.expert_alignment = A;
    e.do_zero_padding = 1;
    e.stream = stream;
    e.dispatch_stamp = ep_dispatch_stamp(buf);
    EXPECT(e.dispatch_stamp > 0);
    CHECK_EP(ep_dispatch_epilogue_launch(buf, &e));

    /* identity experts: the expanded rows go straight back */
    void *d_out = dev_alloc(sizeof out), *d_wout = dev_alloc(sizeof wout);
    EXPECT(d_out && d_wout);
    ep_combine_args_t c;
    memset(&c, 0, sizeof c);
    c.x = e.recv_x;
    c.topk_weights = e.recv_topk_weights;
    c.src_metadata = e.recv_src_metadata;
    c.combined_topk_idx = a.topk_idx;
    c.psum_num_recv_tokens_per_rank = a.psum_num_recv_tokens_per_rank;
    c.combined_x = tensor(d_out, EP_DTYPE_BF16, 2, T, H);
    c.combined_topk_weights = tensor(d_wout, EP_DTYPE_F32, 2, T, K);
    c.num_experts = E;
    c.num_max_tokens_per_rank = T;
    c.stream = stream;
    CHECK_EP(ep_combine_launch(buf, &c, 0));
    CHECK_EP(ep_combine_launch(buf, &c, 1));
    CHECK_HIP(hipStreamSynchronize(stream));

    int meta[T][K + 2];
    int psum_expert[E];
    CHECK_HIP(hipMemcpy(out, d_out, sizeof out, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(wout, d_wout, sizeof wout, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(meta, d_meta, sizeof meta, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(psum_expert, d_psum_expert, sizeof psum_expert, hipMemcpyDeviceToHost));
    int start = 0;
    for (int ex = 0; ex < E; ++ex) {                 /* aligned starts, valid rows first */
        EXPECT(psum_expert[ex] == start + count[ex]);
        start += (count[ex] + A - 1) / A * A;
    }
    for (int i = 0; i < T; ++i) {                    /* all tokens are routed: the stream is the token order */
        EXPECT(meta[i][K] == i && meta[i][K + 1] == K - 1);
        for (int j = 0; j < K; ++j) EXPECT(meta[i][j] >= 0 && meta[i][j] < n_exp);
    }
    for (int t = 0; t < T; ++t) {
        for (int h = 0; h < H; ++h) EXPECT(out[t][h] == bf16_of_small_int(2 * ((t * 7 + h) % 13 - 6)));
        for (int j = 0; j < K; ++j) EXPECT(wout[t][j] == w[t][j]);
    }

    CHECK_EP(ep_buffer_destroy(buf));
    printf("abi_client: ok (%d tokens, %d expanded rows)\n", n_recv, n_exp);
    return 0;
}
