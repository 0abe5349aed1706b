// Host runtime behind the C ABI of include/deep_ep_hip.h: argument contracts, the pooled arena,
// the mapped count page and the launches of the ahead-of-time built gfx950 kernels through
// hipModuleLaunchKernel.  It stands where the reference has csrc/buffers/ep.hpp (host class),
// csrc/kernels/ep/*.hpp (launchers) and csrc/runtime/jit.hpp (run-time compiler).
#include <hip/hip_runtime.h>

#include <dlfcn.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/deep_ep_hip.h"
#include "ep_args.h"
#include "ep_fp8.h"

void ep_static_scratch_init();      // looks up this device's copy of the static scratch (end of this file)

namespace {

constexpr int64_t kAllocAlign = 2097152;       // reference: common/compiled.hpp:48
constexpr int kUbAlign = 32;                   // reference: common/compiled.hpp:39
constexpr int64_t kWorkspaceBytes = 16 * 1024 * 1024;

thread_local std::string g_err;

struct EpError {
    std::string msg;
};

std::string format(const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    return buf;
}

#define EP_HOST_ASSERT(cond)                                                                        \
    do {                                                                                            \
        if (!(cond)) throw EpError{format("Assertion exception (%s:%d): %s", __FILE_NAME__, __LINE__, #cond)}; \
    } while (0)

#define EP_HOST_UNREACHABLE(reason) \
    throw EpError { format("Assertion exception (%s:%d): %s", __FILE_NAME__, __LINE__, reason) }

#define HIP_CHECK(cmd)                                                                              \
    do {                                                                                            \
        const hipError_t e_ = (cmd);                                                                \
        if (e_ != hipSuccess)                                                                       \
            throw EpError{format("HIP runtime exception (%s:%d): Error code: %d, detail: %s", __FILE_NAME__, \
                                 __LINE__, (int)e_, hipGetErrorString(e_))};                        \
    } while (0)

template <class F>
int guarded(F&& f) {
    try {
        f();
        return 0;
    } catch (const EpError& e) {
        g_err = e.msg;
        return 1;
    } catch (const std::exception& e) {
        g_err = e.what();
        return 1;
    }
}

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
int64_t align_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// ---- token layout (reference: layout/ep/token.hpp:9-83) -------------------------------------
int64_t token_bytes(int hidden_bytes, int sf_bytes, int topk, bool with_metadata) {
    int64_t meta = (int64_t)topk * 4 + (with_metadata ? align_up((int64_t)topk * 8, kUbAlign) + 4 : 0);
    int64_t n = hidden_bytes;
    if (sf_bytes > 0) n += align_up(sf_bytes, kUbAlign);
    return n + align_up(meta, kUbAlign);
}

// Byte offsets inside a packed token (reference: layout/ep/token.hpp:59-82).
struct PackedToken {
    int64_t bytes;
    int sf_off, idx_off, w_off, src_off;
};

PackedToken packed_token(int hidden_bytes, int sf_bytes, int topk, bool with_metadata) {
    PackedToken p{};
    p.bytes = token_bytes(hidden_bytes, sf_bytes, topk, with_metadata);
    p.sf_off = (int)align_up(hidden_bytes, kUbAlign);
    p.idx_off = sf_bytes > 0 ? p.sf_off + (int)align_up(sf_bytes, kUbAlign) : hidden_bytes;
    p.w_off = p.idx_off + (with_metadata ? (int)align_up((int64_t)topk * 8, kUbAlign) : 0);
    p.src_off = p.w_off + topk * 4;
    return p;
}

int64_t dispatch_buffer_size(int max_tokens, int hidden, int sf_packs, int topk, int elem, int ranks) {
    return (int64_t)ranks * max_tokens * token_bytes(hidden * elem, sf_packs * 2, topk, true);
}

int64_t combine_buffer_size(int ranks, int max_tokens, int hidden, int topk) {
    return (int64_t)std::min(topk, ranks) * max_tokens * token_bytes(hidden * 2, 0, topk, false);
}

// ---- code object ------------------------------------------------------------------------------
struct Kernels {
    hipModule_t module = nullptr;
    hipFunction_t layout_count, layout_scan, layout_assign[2][2];      // [sums the counts itself][receive side]
    hipFunction_t scatter_copy, scatter_quant, scatter_quant_sw, sf_transpose;
    hipFunction_t scatter_copy_pack, scatter_quant_pack, scatter_quant_sw_pack;
    hipFunction_t combine[3][5];     // [mode][generic, k2, k4, k6, k8]
    hipFunction_t fp8_selftest, quant_rows;
    int device = -1;
};

std::mutex g_mutex;
Kernels g_k;
std::atomic<bool> g_fp8_hw{true};
// Workgroups of the single-partition combine kernel a CU holds at once, enforced through an unused dynamic LDS
// allocation (0: no cap, the registers decide: 5 to 8; negative: chosen by top-k, below).  The gather is fastest
// with about 150 KiB of row fetches in flight a CU (a wave fetches top-k x 2 KiB): more waves queue more fetches
// than the memory keeps open.  Measured at 16384 tokens x 7168 (microseconds at 2/3/4/5 workgroups and uncapped):
//   top-2  175 140 126 120 120      top-4  233 201 194 199 200
//   top-6  297 272 286 289 291      top-8  385 354 377 378 376
// and for the kernel that takes any top-k: top-1 best uncapped, top-3 at 6, top-5 at 5, top-7 to top-16 at 4.
// A bias row is one more row a wave fetches: top-6 with one / two biases 326 311 329 336 / 358 350 373 377 at 2/3/4/5.
// The two-phase kernels of the partitioned path do not react to it.
std::atomic<int> g_combine_blocks_per_cu{-1};
constexpr unsigned kLdsBytesPerCu = 160 * 1024;
unsigned combine_lds_cap(int num_topk, bool specialised, int num_row_blocks, int hidden) {     // num_topk: rows a wave fetches, biases included
    int n = g_combine_blocks_per_cu;
    if (n < 0) {
        // a launch that fills the machine less than about twice over wants every wave it can get
        // (1024 tokens, top-6: 23.8 us uncapped, 25.4 at four workgroups; from 4096 tokens on the cap costs nothing),
        // and so do short rows (hidden 512 / 1536, top-8: 113 / 160 us uncapped, 124 / 170 at three; from 2048 on the
        // cap wins)
        if (num_row_blocks < 4096 or hidden < 2048) n = 0;
        else if (specialised) n = num_topk <= 2 ? 0 : num_topk <= 4 ? 4 : 3;
        else n = num_topk <= 2 ? 0 : num_topk == 3 ? 6 : num_topk <= 5 ? 5 : 4;
    }
    // a workgroup can ask for 64 KiB at most, which lets two of them into a CU: a cap of one cannot be enforced this
    // way (it is served as two), and from 160 workgroups on a share of the LDS is too small to mean anything (no cap)
    if (n <= 0) return 0;
    const unsigned share = kLdsBytesPerCu / (unsigned)n;
    if (share <= 1024u) return 0;
    return std::min(64u * 1024u, share - 1024u);       // n of them fit a CU, n + 1 do not
}
std::atomic<int> g_recount_limit{2 * EP_RECOUNT_DEPTH};   // blocks x top-k up to which one partition's slot assignment counts all ids itself
std::atomic<int> g_fold_max_blocks{256};    // up to this many layout workgroups the slot assignment sums the block counts itself

std::string library_dir() {
    Dl_info info;
    if (dladdr((void*)&library_dir, &info) == 0 || info.dli_fname == nullptr) return ".";
    std::string p = info.dli_fname;
    const auto pos = p.find_last_of('/');
    return pos == std::string::npos ? "." : p.substr(0, pos);
}

void load_kernels(const char* dir) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_k.module != nullptr) return;
    const std::string path = (dir != nullptr ? std::string(dir) : library_dir()) + "/ep_kernels.hsaco";
    FILE* f = fopen(path.c_str(), "rb");
    if (f == nullptr) throw EpError{"cannot open the gfx950 code object " + path + " (build it first)"};
    fclose(f);
    int ndev = 0;
    HIP_CHECK(hipGetDeviceCount(&ndev));
    if (ndev <= 0) throw EpError{"no HIP device visible: the EP kernels only run on a gfx950 GPU"};
    HIP_CHECK(hipGetDevice(&g_k.device));
    hipModule_t m;
    HIP_CHECK(hipModuleLoad(&m, path.c_str()));
    auto get = [&](hipFunction_t& fn, const char* name) { HIP_CHECK(hipModuleGetFunction(&fn, m, name)); };
    get(g_k.layout_count, "ep_layout_count");
    get(g_k.layout_scan, "ep_layout_scan");
    get(g_k.layout_assign[0][0], "ep_layout_assign");
    get(g_k.layout_assign[1][0], "ep_layout_assign_fold");
    get(g_k.layout_assign[0][1], "ep_layout_assign_recv");
    get(g_k.layout_assign[1][1], "ep_layout_assign_fold_recv");
    get(g_k.scatter_copy, "ep_scatter_copy");
    get(g_k.scatter_quant, "ep_scatter_quant");
    get(g_k.scatter_quant_sw, "ep_scatter_quant_sw");
    get(g_k.scatter_copy_pack, "ep_scatter_copy_pack");
    get(g_k.scatter_quant_pack, "ep_scatter_quant_pack");
    get(g_k.scatter_quant_sw_pack, "ep_scatter_quant_sw_pack");
    get(g_k.sf_transpose, "ep_sf_transpose");
    const char* modes[3] = {"", "_partial", "_final"};
    const char* ks[5] = {"_generic", "_k2", "_k4", "_k6", "_k8"};
    for (int mode = 0; mode < 3; ++mode)
        for (int k = 0; k < 5; ++k)
            get(g_k.combine[mode][k], (std::string("ep_combine") + modes[mode] + ks[k]).c_str());
    get(g_k.fp8_selftest, "ep_fp8_selftest");
    get(g_k.quant_rows, "ep_quant_rows");
    g_k.module = m;
}

template <class A>
void launch(hipFunction_t fn, unsigned grid, unsigned block, unsigned smem, void* stream, A& args) {
    void* params[] = {&args};
    HIP_CHECK(hipModuleLaunchKernel(fn, grid, 1, 1, block, 1, 1, smem, (hipStream_t)stream, params, nullptr));
}

// ---- tensor contracts -------------------------------------------------------------------------
bool present(const ep_tensor_t& t) { return t.data != nullptr; }

int elem_size(int dtype) {
    switch (dtype) {
        case EP_DTYPE_BF16: case EP_DTYPE_I16: return 2;
        case EP_DTYPE_FP8_E4M3: case EP_DTYPE_U8: return 1;
        case EP_DTYPE_I32: case EP_DTYPE_F32: return 4;
        case EP_DTYPE_I64: return 8;
        default: return 0;
    }
}

bool contiguous(const ep_tensor_t& t) {
    int64_t expect = 1;
    for (int d = t.ndim - 1; d >= 0; --d) {
        if (t.size[d] != 1 && t.stride[d] != expect) return false;
        expect *= t.size[d];
    }
    return true;
}

}  // namespace

struct ep_buffer {
    int rank_idx = 0, num_ranks = 1;
    int64_t num_buffer_bytes = 0, num_lb_bytes = 0;
    int cpu_timeout_secs = 300, gpu_timeout_secs = 100;
    char* arena = nullptr;       // workspace || buffer || lb storage
    int* host_page = nullptr;    // pinned + mapped
    int* host_page_dev = nullptr;
    int seq = 0;                 // sequence number of the last non-cached dispatch
    int64_t launch_stamp = 0;    // counts the non-cached ep_dispatch_launch calls; the latest one owns the workspace
    int64_t workspace_bytes = kWorkspaceBytes;
    bool is_static = false;      // a view over the library's static scratch: no arena, no count page, one partition
    bool destroyed = false;
    int device = 0;
    // node of partitions living in this process (ep_buffer_connect): every partition's arena is a peer
    bool connected = false;
    std::vector<ep_buffer*> peers;
    // how often each phase has been enqueued: the partitions of a node move in lockstep, which lets the
    // host catch a phase enqueued before the peers' previous phase (nothing on the device waits for it)
    int64_t num_sends = 0, num_expands = 0, num_partials = 0;
    // state handed from ep_dispatch_launch to ep_dispatch_epilogue_launch
    struct {
        bool valid = false;
        int64_t stamp = 0;
        int num_tokens = 0, num_topk = 0, num_experts = 0, alignment = 0, max_tokens = 0;
        int* slot_map = nullptr;
        int* tok_row = nullptr;
        bool notified = false;
        bool recv_done = false;     // more than one partition: the receive-side layout has been enqueued
    } last;

    char* const* peer_table() const { return (char* const*)(arena + EP_WS_PEERS_OFF); }
    const int* inbox() const { return (const int*)(arena + EP_WS_INBOX_OFF); }
    // rows the receive stream of this partition can hold
    int64_t recv_rows_bound(int num_tokens, int max_tokens) const {
        return connected ? (int64_t)num_ranks * max_tokens : num_tokens;
    }

    char* workspace() const { return arena; }
    char* buffer() const { return arena + workspace_bytes; }
    char* lb() const { return arena + workspace_bytes + num_buffer_bytes; }
};

namespace {
// LDS of the layout kernels: histograms / per-wave counters, the staged keys, the per-source row counts
unsigned layout_key_bytes(int K) { return 2u * EP_TOKENS_PER_BLOCK * K * sizeof(short); }
unsigned layout_count_lds(int E, int R, int K) {
    return (unsigned)(E + R + R + EP_LAYOUT_THREADS / 64) * sizeof(int) + layout_key_bytes(K);
}
// (cnt_stride > 0: the assignment sums the count rows itself and needs two rows of ints where the partial sums meet)
unsigned layout_assign_lds(int E, int R, int K, int cnt_stride) {
    const unsigned nw = EP_LAYOUT_THREADS / 64;
    return (unsigned)(E / R + R + nw * (E + R) + nw + 1 + R + nw + 2 * cnt_stride) * sizeof(int) + layout_key_bytes(K);
}

// The layout pass: per-block histograms, then the slot assignment.  One block needs no histogram pass; up
// to g_fold_max_blocks blocks the assignment kernel sums the histograms of the blocks before it itself;
// beyond that a scan kernel turns them into prefixes first.
void launch_layout(EpLayoutArgs& la, int num_blocks, void* stream) {
    const int E = la.num_experts, R = la.num_ranks, K = la.num_topk;
    // (the few shapes with more count columns than the summing instance has threads for, or whose LDS would not hold
    //  the rows where its sums meet, take the scan kernel at any size)
    // (what the summing costs is rows a thread: blocks x column groups of 8 / threads.  The limit is quoted in blocks at
    //  the headline's 264 columns, 33 groups; narrower rows, as the 40 columns of an EP32 partition, sum that many more)
    const bool fold = (int64_t)num_blocks * (la.cnt_stride / 8) <= (int64_t)g_fold_max_blocks * 33 and
                      la.cnt_stride <= 8 * EP_LAYOUT_THREADS and layout_assign_lds(E, R, K, la.cnt_stride) <= 64 * 1024;
    // a few blocks of one partition (send side): the slot assignment counts the ids of all blocks itself, a launch less
    // (two histograms of El + R ints and a byte a token on top of its LDS)
    const unsigned recount_extra = (unsigned)(2 * (E / R + R)) * sizeof(int) + (unsigned)num_blocks * EP_TOKENS_PER_BLOCK;
    const bool recount = R == 1 and not la.recv_mode and not la.send_only and num_blocks >= 2 and
                         (int64_t)num_blocks * K <= std::min(g_recount_limit.load(), 2 * EP_RECOUNT_DEPTH) and
                         layout_assign_lds(E, R, K, 0) + recount_extra <= 64 * 1024;
    la.scan_mode = num_blocks == 1 ? EP_LAYOUT_SINGLE
                   : recount       ? EP_LAYOUT_RECOUNTED
                   : fold          ? EP_LAYOUT_FOLDED
                                   : EP_LAYOUT_SCANNED;
    const unsigned smem_assign = layout_assign_lds(E, R, K, la.scan_mode == EP_LAYOUT_FOLDED ? la.cnt_stride : 0) +
                                 (la.scan_mode == EP_LAYOUT_RECOUNTED ? recount_extra : 0u);
    EP_HOST_ASSERT(smem_assign <= 64 * 1024);
    if (la.scan_mode == EP_LAYOUT_FOLDED or la.scan_mode == EP_LAYOUT_SCANNED)
        launch(g_k.layout_count, num_blocks, EP_LAYOUT_THREADS, layout_count_lds(E, R, K), stream, la);
    if (la.scan_mode == EP_LAYOUT_SCANNED)
        launch(g_k.layout_scan, (unsigned)ceil_div(la.cnt_stride, 16), EP_SCAN_THREADS, 0, stream, la);
    // (one workgroup more than blocks: it publishes the totals and ranks nothing)
    launch(g_k.layout_assign[la.scan_mode == EP_LAYOUT_FOLDED][la.recv_mode != 0], (unsigned)num_blocks + 1u, EP_LAYOUT_THREADS,
           smem_assign, stream, la);
}

void write_peer_table(ep_buffer* b, const std::vector<char*>& arenas) {
    std::vector<char*> table(EP_MAX_RANKS, nullptr);
    for (size_t i = 0; i < arenas.size(); ++i) table[i] = arenas[i];
    HIP_CHECK(hipMemcpy(b->arena + EP_WS_PEERS_OFF, table.data(), sizeof(char*) * EP_MAX_RANKS, hipMemcpyHostToDevice));
}

void disconnect(ep_buffer* b) {
    write_peer_table(b, std::vector<char*>(b->num_ranks, b->arena));
    // the row counts the other partitions left while connected describe rows nobody will refresh
    HIP_CHECK(hipMemset(b->arena + EP_WS_INBOX_OFF, 0, sizeof(int) * EP_MAX_RANKS));
    b->connected = false;
    b->peers.clear();
}

// Phase order inside a node (ep_buffer_connect): `ready(peer)` must hold for every partition.
template <class F>
void check_peers(const ep_buffer* b, F&& ready, const char* what) {
    for (const ep_buffer* p : b->peers)
        if (not ready(*p)) throw EpError{format("Assertion exception (%s): partition %d of the node: %s", __FILE_NAME__, p->rank_idx, what)};
}

// The code object is loaded on one device and the arena lives there: calls must come with that
// device current.
void check_buffer(const ep_buffer* b) {
    EP_HOST_ASSERT(b != nullptr);
    EP_HOST_ASSERT(not b->destroyed);
    int dev = -1;
    HIP_CHECK(hipGetDevice(&dev));
    EP_HOST_ASSERT(dev == b->device and "the buffer belongs to another device");
}
}  // namespace

extern "C" {

const char* ep_last_error(void) { return g_err.c_str(); }

int ep_init(const char* dir) {
    return guarded([&] {
        load_kernels(dir);
        ep_static_scratch_init();      // the address of the static scratch on this device
    });
}

int64_t ep_get_num_allocation_alignment(void) { return kAllocAlign; }
int64_t ep_get_num_tma_alignment(void) { return 32; }
int64_t ep_get_num_rdma_alignment(void) { return 32; }

int ep_get_num_compute_units(void) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    return n;
}

int64_t ep_get_dispatch_buffer_size(int max_tokens, int hidden, int sf_packs, int topk, int elem, int ranks) {
    return dispatch_buffer_size(max_tokens, hidden, sf_packs, topk, elem, ranks);
}

int64_t ep_get_combine_buffer_size(int ranks, int max_tokens, int hidden, int topk) {
    return combine_buffer_size(ranks, max_tokens, hidden, topk);
}

int64_t ep_calculate_buffer_size(int num_ranks, int max_tokens, int hidden, int num_topk, int use_fp8) {
    int64_t out = -1;
    const int rc = guarded([&] {
        EP_HOST_ASSERT(num_ranks > 0);
        EP_HOST_ASSERT(max_tokens > 0);
        EP_HOST_ASSERT(hidden > 0);
        EP_HOST_ASSERT(num_topk >= 0);
        const int topk = num_topk == 0 ? 32 : num_topk;            // room for the largest top-k
        const int sf_packs = use_fp8 ? (int)ceil_div(hidden, 32) : 0;   // the hint never sees the SF tensor
        const int64_t d = dispatch_buffer_size(max_tokens, hidden, sf_packs, topk, use_fp8 ? 1 : 2, num_ranks);
        const int64_t c = combine_buffer_size(num_ranks, max_tokens, hidden, topk);
        out = align_up(std::max(d, c), kAllocAlign);
    });
    return rc == 0 ? out : -1;
}

void ep_host_f32_to_e4m3fn(const float* src, uint8_t* dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        uint32_t b;
        memcpy(&b, src + i, 4);
        dst[i] = (uint8_t)ep_f32_bits_to_e4m3fn(b);
    }
}

void ep_set_fp8_hw_convert(int enable) { g_fp8_hw = enable != 0; }

int ep_fp8_selftest(uint64_t first, uint64_t count, float limit, uint64_t out[2]) {
    return guarded([&] {
        load_kernels(nullptr);
        unsigned long long* dev = nullptr;
        HIP_CHECK(hipMalloc((void**)&dev, 16));
        const unsigned long long init[2] = {0ull, ~0ull};
        HIP_CHECK(hipMemcpy(dev, init, 16, hipMemcpyHostToDevice));
        EpFp8TestArgs args = {first, count, dev, limit, 0};
        launch(g_k.fp8_selftest, 4096, 256, 0, nullptr, args);
        HIP_CHECK(hipDeviceSynchronize());
        unsigned long long res[2];
        HIP_CHECK(hipMemcpy(res, dev, 16, hipMemcpyDeviceToHost));
        HIP_CHECK(hipFree(dev));
        out[0] = res[0];
        out[1] = res[1];
    });
}

int ep_per_token_cast_to_fp8(const ep_tensor_t* px, const ep_tensor_t* pq, const ep_tensor_t* psf, void* stream) {
    return guarded([&] {
        load_kernels(nullptr);
        EP_HOST_ASSERT(px != nullptr and pq != nullptr and psf != nullptr);
        const ep_tensor_t &x = *px, &q = *pq, &sf = *psf;
        EP_HOST_ASSERT(present(x) and x.ndim == 2 and x.dtype == EP_DTYPE_BF16 and contiguous(x));
        const int64_t rows = x.size[0], hidden = x.size[1];
        EP_HOST_ASSERT(hidden > 0 and hidden % 8 == 0 and hidden <= 16384);
        EP_HOST_ASSERT(present(q) and q.ndim == 2 and q.size[0] == rows and q.size[1] == hidden and contiguous(q));
        EP_HOST_ASSERT(q.dtype == EP_DTYPE_FP8_E4M3 or q.dtype == EP_DTYPE_U8);
        EP_HOST_ASSERT(present(sf) and sf.ndim == 2 and sf.size[0] == rows and sf.size[1] == ceil_div(hidden, 128));
        EP_HOST_ASSERT(sf.dtype == EP_DTYPE_F32 and contiguous(sf));
        EP_HOST_ASSERT(((uintptr_t)x.data & 15) == 0 and ((uintptr_t)q.data & 7) == 0);
        EpQuantArgs qa{};
        qa.x = x.data;
        qa.q = q.data;
        qa.sf = (float*)sf.data;
        qa.num_rows = (int)rows;
        qa.hidden = (int)hidden;
        qa.num_parts = (int)ceil_div(hidden, 512);
        qa.hw_convert = g_fp8_hw ? 1 : 0;
        const int64_t blocks = ceil_div(rows * qa.num_parts, EP_ROWS_PER_BLOCK);
        EP_HOST_ASSERT(rows <= INT32_MAX and blocks <= INT32_MAX);
        if (blocks > 0) launch(g_k.quant_rows, (unsigned)blocks, EP_ROW_THREADS, 0, stream, qa);
    });
}

// ---- buffer -----------------------------------------------------------------------------------
int ep_buffer_create(int rank_idx, int num_ranks, int64_t num_bytes, int64_t num_lb_bytes, int cpu_timeout_secs,
                     int gpu_timeout_secs, ep_buffer_t** out) {
    return guarded([&] {
        EP_HOST_ASSERT(out != nullptr);
        EP_HOST_ASSERT(num_bytes >= 0 and num_bytes % kAllocAlign == 0);
        EP_HOST_ASSERT(num_lb_bytes >= 0 and num_lb_bytes % kAllocAlign == 0);
        EP_HOST_ASSERT(num_ranks > 0 and num_ranks <= EP_MAX_RANKS and rank_idx >= 0 and rank_idx < num_ranks);
        EP_HOST_ASSERT(cpu_timeout_secs > 0 and gpu_timeout_secs > 0);
        load_kernels(nullptr);
        int cur = -1;
        HIP_CHECK(hipGetDevice(&cur));
        EP_HOST_ASSERT(cur == g_k.device and "the kernels were loaded on another device");
        auto* b = new ep_buffer();
        b->rank_idx = rank_idx;
        b->num_ranks = num_ranks;
        b->num_buffer_bytes = num_bytes;
        b->num_lb_bytes = num_lb_bytes;
        b->cpu_timeout_secs = cpu_timeout_secs;
        b->gpu_timeout_secs = gpu_timeout_secs;
        try {
            HIP_CHECK(hipGetDevice(&b->device));
            const int64_t total = kWorkspaceBytes + num_bytes + num_lb_bytes;
            HIP_CHECK(hipMalloc((void**)&b->arena, (size_t)total));
            HIP_CHECK(hipMemset(b->arena, 0, (size_t)total));
            HIP_CHECK(hipHostMalloc((void**)&b->host_page, EP_HOST_PAGE_INTS * sizeof(int), hipHostMallocMapped));
            memset(b->host_page, 0, EP_HOST_PAGE_INTS * sizeof(int));
            HIP_CHECK(hipHostGetDevicePointer((void**)&b->host_page_dev, b->host_page, 0));
            write_peer_table(b, std::vector<char*>(num_ranks, b->arena));    // not connected: every peer is this arena
            HIP_CHECK(hipDeviceSynchronize());
        } catch (...) {
            if (b->arena != nullptr) (void)hipFree(b->arena);
            if (b->host_page != nullptr) (void)hipHostFree(b->host_page);
            delete b;
            throw;
        }
        *out = b;
    });
}

int ep_buffer_connect(ep_buffer_t** bufs, int n) {
    return guarded([&] {
        EP_HOST_ASSERT(bufs != nullptr and n > 1);
        std::vector<char*> arenas(n);
        for (int i = 0; i < n; ++i) {
            check_buffer(bufs[i]);
            EP_HOST_ASSERT(bufs[i]->num_ranks == n and bufs[i]->rank_idx == i);
            EP_HOST_ASSERT(bufs[i]->num_buffer_bytes == bufs[0]->num_buffer_bytes);
            EP_HOST_ASSERT(not bufs[i]->connected);
            arenas[i] = bufs[i]->arena;
        }
        HIP_CHECK(hipDeviceSynchronize());
        for (int i = 0; i < n; ++i) {
            write_peer_table(bufs[i], arenas);
            bufs[i]->connected = true;
            bufs[i]->peers.assign(bufs, bufs + n);
        }
    });
}

int ep_buffer_set_peers(ep_buffer_t* b, void* const* arena_bases, int n) {
    return guarded([&] {
        check_buffer(b);
        HIP_CHECK(hipDeviceSynchronize());
        if (arena_bases == nullptr) {
            disconnect(b);
            return;
        }
        EP_HOST_ASSERT(n == b->num_ranks and n > 1);
        std::vector<char*> arenas(n);
        for (int i = 0; i < n; ++i) {
            EP_HOST_ASSERT(arena_bases[i] != nullptr);
            arenas[i] = (char*)arena_bases[i];
        }
        EP_HOST_ASSERT(arenas[b->rank_idx] == b->arena and "a partition's own entry is its own arena");
        write_peer_table(b, arenas);
        b->connected = true;
        b->peers.clear();           // arenas the caller mapped: theirs to keep alive and to disconnect
    });
}

int ep_buffer_destroy(ep_buffer_t* b) {
    return guarded([&] {
        EP_HOST_ASSERT(b != nullptr);
        EP_HOST_ASSERT(not b->destroyed);
        HIP_CHECK(hipDeviceSynchronize());
        // the other partitions of a node must not keep pointers into this arena
        const std::vector<ep_buffer*> peers = b->peers;
        for (ep_buffer* p : peers)
            if (p != b) disconnect(p);
        b->peers.clear();
        HIP_CHECK(hipFree(b->arena));
        HIP_CHECK(hipHostFree(b->host_page));
        b->arena = nullptr;
        b->host_page = nullptr;
        b->destroyed = true;
        delete b;
    });
}

void* ep_buffer_region(ep_buffer_t* b, int which, int64_t* num_bytes) {
    if (b == nullptr || b->destroyed) return nullptr;
    switch (which) {
        case 0: if (num_bytes) *num_bytes = kWorkspaceBytes; return b->workspace();
        case 1: if (num_bytes) *num_bytes = b->num_buffer_bytes; return b->buffer();
        case 2: if (num_bytes) *num_bytes = b->num_lb_bytes; return b->lb();
        default: return nullptr;
    }
}

int ep_buffer_print_memory_usage(ep_buffer_t* b) {
    return guarded([&] {
        EP_HOST_ASSERT(b != nullptr and not b->destroyed);
        const double gib = 1 << 30;
        printf("[DeepEP memory usage] rank_idx=%d, num_ranks=%d, GPU total %.3f GiB "
               "(workspace %.3f GiB, buffer %.3f GiB, RDMA storage %.3f GiB), CPU total %.3f GiB\n",
               b->rank_idx, b->num_ranks, (kWorkspaceBytes + b->num_buffer_bytes + b->num_lb_bytes) / gib,
               kWorkspaceBytes / gib, b->num_buffer_bytes / gib, b->num_lb_bytes / gib, 0.0);
        fflush(stdout);
    });
}

// ---- dispatch ---------------------------------------------------------------------------------
int ep_dispatch_launch(ep_buffer_t* b, const ep_dispatch_args_t* pa) {
    return guarded([&] {
        EP_HOST_ASSERT(pa != nullptr);
        check_buffer(b);
        const ep_dispatch_args_t& a = *pa;
        const bool cached_mode = a.cached_mode != 0;
        const bool do_cpu_sync = a.do_cpu_sync != 0;
        EP_HOST_ASSERT(not b->is_static or (not cached_mode and not do_cpu_sync and b->num_ranks == 1));
        if (cached_mode) {
            EP_HOST_ASSERT(not do_cpu_sync and "Cannot do CPU sync with cached mode");
            EP_HOST_ASSERT(not present(a.cumulative_local_expert_recv_stats));
        }

        // data tensor
        EP_HOST_ASSERT(present(a.x));
        EP_HOST_ASSERT(a.x.ndim == 2);
        const int num_tokens = (int)a.x.size[0];
        const int hidden = (int)a.x.size[1];
        const int num_ranks = b->num_ranks;
        EP_HOST_ASSERT(a.num_experts > 0 and a.num_experts <= EP_MAX_EXPERTS);
        EP_HOST_ASSERT(a.num_experts % num_ranks == 0);
        const int num_experts_per_rank = a.num_experts / num_ranks;
        EP_HOST_ASSERT(contiguous(a.x));
        EP_HOST_ASSERT(num_tokens <= a.num_max_tokens_per_rank);
        EP_HOST_ASSERT(a.num_max_tokens_per_rank > 0);
        EP_HOST_ASSERT(a.expert_alignment > 0);

        int num_sf_packs = 0;
        if (present(a.sf)) {
            EP_HOST_ASSERT(not a.fused_fp8_quant);
            EP_HOST_ASSERT(a.x.dtype == EP_DTYPE_FP8_E4M3);
            EP_HOST_ASSERT(a.sf.ndim == 2 and a.sf.size[0] == num_tokens);
            EP_HOST_ASSERT(elem_size(a.sf.dtype) == 2);
            EP_HOST_ASSERT(a.sf.stride[0] == 1 or a.sf.stride[1] == 1);
            EP_HOST_ASSERT(a.sf.stride[0] <= INT32_MAX and a.sf.stride[1] <= INT32_MAX);
            num_sf_packs = (int)a.sf.size[1];
        } else {
            EP_HOST_ASSERT(a.x.dtype == EP_DTYPE_BF16);
        }
        const int x_elem = elem_size(a.x.dtype);
        EP_HOST_ASSERT((int64_t)hidden * x_elem % 16 == 0);
        if (a.fused_fp8_quant) {
            EP_HOST_ASSERT(hidden % 8 == 0 and hidden <= 16384);
        }

        // top-k
        EP_HOST_ASSERT(present(a.topk_idx) and a.topk_idx.ndim == 2);
        const int num_topk = (int)a.topk_idx.size[1];
        EP_HOST_ASSERT(a.topk_idx.size[0] == num_tokens);
        EP_HOST_ASSERT(a.topk_idx.dtype == EP_DTYPE_I64);
        EP_HOST_ASSERT(contiguous(a.topk_idx));
        EP_HOST_ASSERT(num_topk > 0 and num_topk <= EP_MAX_TOPK);
        if (present(a.topk_weights)) {
            EP_HOST_ASSERT(a.topk_weights.ndim == 2);
            EP_HOST_ASSERT(a.topk_weights.size[0] == num_tokens and a.topk_weights.size[1] == num_topk);
            EP_HOST_ASSERT(contiguous(a.topk_weights));
            EP_HOST_ASSERT(a.topk_weights.dtype == EP_DTYPE_F32);
        }
        if (present(a.cumulative_local_expert_recv_stats)) {
            const auto& s = a.cumulative_local_expert_recv_stats;
            EP_HOST_ASSERT(s.ndim == 1 and s.size[0] == num_experts_per_rank);
            EP_HOST_ASSERT(contiguous(s));
            EP_HOST_ASSERT(s.dtype == EP_DTYPE_I32);
        }

        // buffer size (the packed regions of csrc/buffers/ep.hpp:196-198)
        const int packed_elem = a.fused_fp8_quant ? 1 : x_elem;
        const int packed_sf = a.fused_fp8_quant ? 2 * (int)ceil_div(hidden, 128) : num_sf_packs;
        // (the static view has no buffer: with one partition the packed regions are never materialised)
        EP_HOST_ASSERT(b->is_static or dispatch_buffer_size(a.num_max_tokens_per_rank, hidden, packed_sf, num_topk, packed_elem,
                                                            num_ranks) <= b->num_buffer_bytes);
        // packed rows put the scales at the next multiple of 32 bytes behind the payload while the row size adds the
        // payload unaligned (layout/ep/token.hpp:36-43,59-61, whose own check of this is commented out :29): rows
        // would overlap their neighbours
        EP_HOST_ASSERT(num_ranks == 1 or packed_sf == 0 or (int64_t)hidden * packed_elem % kUbAlign == 0);

        // handle tensors
        const auto& psum_rank = a.psum_num_recv_tokens_per_rank;
        const auto& psum_expert = a.psum_num_recv_tokens_per_expert;
        const auto& unaligned = a.num_unaligned_recv_tokens_per_expert;
        EP_HOST_ASSERT(present(psum_rank) and present(psum_expert) and present(unaligned));
        EP_HOST_ASSERT(present(a.dst_buffer_slot_idx) and present(a.dst_gsge_idx));
        EP_HOST_ASSERT(psum_rank.ndim == 1 and psum_rank.size[0] == num_ranks);
        EP_HOST_ASSERT(psum_expert.ndim == 1 and psum_expert.size[0] == num_experts_per_rank);
        EP_HOST_ASSERT(unaligned.ndim == 1 and unaligned.size[0] == num_experts_per_rank);
        EP_HOST_ASSERT(a.dst_buffer_slot_idx.ndim == 2 and a.dst_buffer_slot_idx.size[0] == num_tokens and
                       a.dst_buffer_slot_idx.size[1] == num_topk);
        EP_HOST_ASSERT(a.dst_gsge_idx.ndim == 2 and a.dst_gsge_idx.size[0] == num_tokens and
                       a.dst_gsge_idx.size[1] == num_topk);
        EP_HOST_ASSERT(contiguous(psum_rank) and contiguous(psum_expert) and contiguous(unaligned));
        EP_HOST_ASSERT(contiguous(a.dst_buffer_slot_idx) and contiguous(a.dst_gsge_idx));
        EP_HOST_ASSERT(psum_rank.dtype == EP_DTYPE_I32 and psum_expert.dtype == EP_DTYPE_I32);
        EP_HOST_ASSERT(unaligned.dtype == EP_DTYPE_I32);
        EP_HOST_ASSERT(a.dst_buffer_slot_idx.dtype == EP_DTYPE_I32 and a.dst_gsge_idx.dtype == EP_DTYPE_I32);

        // geometry of the packed rows of the partition-major regions (only materialised when R > 1)
        const PackedToken pk = packed_token(hidden * packed_elem, packed_sf * 2, num_topk, not cached_mode);
        auto launch_pack = [&]() {
            EpScatterArgs sa{};
            sa.mode = EP_SCATTER_PACK;
            sa.x = a.x.data;
            sa.sf = a.sf.data;
            sa.topk_weights = (const float*)a.topk_weights.data;
            sa.topk_idx = (const int64_t*)a.topk_idx.data;
            sa.dst_slot_idx = (const int*)a.dst_buffer_slot_idx.data;
            sa.recv_x = b->buffer();
            sa.recv_sf = packed_sf > 0 ? b->buffer() + pk.sf_off : nullptr;
            sa.x_row_bytes = (int64_t)hidden * x_elem;
            sa.copy_bytes = sa.x_row_bytes;
            sa.out_row_bytes = pk.bytes;
            sa.out_sf_row_bytes = pk.bytes;
            if (present(a.sf)) {
                sa.sf_token_stride_bytes = a.sf.stride[0] * 2;
                sa.sf_pack_stride_bytes = a.sf.stride[1] * 2;
            }
            sa.hidden = hidden;
            sa.num_topk = num_topk;
            sa.num_rows_bound = num_tokens;
            sa.num_tokens = num_tokens;
            sa.rank_idx = b->rank_idx;
            sa.max_tokens = a.num_max_tokens_per_rank;
            sa.num_sf_packs = num_sf_packs;
            sa.num_experts = a.num_experts;
            sa.experts_per_rank = num_experts_per_rank;
            sa.with_metadata = cached_mode ? 0 : 1;
            sa.idx_off = pk.idx_off;
            sa.w_off = pk.w_off;
            sa.src_off = pk.src_off;
            sa.num_out_rows = num_ranks * a.num_max_tokens_per_rank;
            // unconnected: the regions of this arena, one per destination; in a node: region `rank_idx` of
            // the destination's own arena, where its receive side will look for them
            sa.peer_arenas = b->peer_table();
            sa.buffer_off = b->workspace_bytes;
            sa.region_by_source = b->connected ? 1 : 0;
            sa.num_ranks = num_ranks;
            sa.pack_sf_off = pk.sf_off;
            sa.vecs_per_lane = 1;
            sa.num_parts = (int)std::max<int64_t>(1, a.fused_fp8_quant ? ceil_div(hidden, 512) : ceil_div(sa.copy_bytes, 1024));
            sa.num_row_blocks = (int)ceil_div((int64_t)num_tokens * sa.num_parts, EP_ROWS_PER_BLOCK);
            if (sa.num_row_blocks == 0) return;
            hipFunction_t fn = a.fused_fp8_quant ? (g_fp8_hw ? g_k.scatter_quant_pack : g_k.scatter_quant_sw_pack)
                                                 : g_k.scatter_copy_pack;
            launch(fn, (unsigned)sa.num_row_blocks, EP_ROW_THREADS, 0, a.stream, sa);
        };

        if (num_ranks > 1) {
            // the rows about to be packed overwrite what the peers received last time
            check_peers(b, [&](const ep_buffer& p) { return p.num_expands >= b->num_sends; },
                        "has not run the copy epilogue of the previous dispatch yet");
            ++b->num_sends;
        }
        if (cached_mode) {
            // the cached handle already holds the whole layout: only the packed regions are refreshed
            b->last.valid = false;
            if (num_ranks > 1) launch_pack();
            return;
        }

        // scratch carved from the workspace
        const int E = a.num_experts, R = num_ranks, K = num_topk;
        const int num_blocks = std::max<int>(1, (int)ceil_div(num_tokens, EP_TOKENS_PER_BLOCK));
        int* ws = (int*)b->workspace();
        int64_t off = EP_WS_HEADER_BYTES / sizeof(int);
        auto carve = [&](int64_t n) {
            int* p = ws + off;
            off += align_up(std::max<int64_t>(n, 1), 64);
            return p;
        };
        EpLayoutArgs la{};
        la.cnt_stride = (int)align_up(E / R + R, 8);
        la.col_total = carve(la.cnt_stride);
        la.blk_cnt = carve((int64_t)num_blocks * la.cnt_stride);
        if (R == 1) {
            la.slot_map = carve((int64_t)num_tokens * K);
            la.tok_row = carve(num_tokens);
        }
        if (b->is_static and off * (int64_t)sizeof(int) > b->workspace_bytes)
            throw EpError{format("Assertion exception (%s:%d): the layout scratch of %d tokens x top-%d over %d experts (%lld bytes) "
                                 "exceeds the library's static scratch of %lld bytes", __FILE_NAME__, __LINE__, num_tokens, K, E,
                                 (long long)(off * (int64_t)sizeof(int)), (long long)b->workspace_bytes)};
        EP_HOST_ASSERT(off * (int64_t)sizeof(int) <= b->workspace_bytes);
        // more than one partition: this launch is the send side only (slots in the destinations' regions, row
        // counts into their inboxes); the receive side is ep_dispatch_recv_launch
        la.send_only = R > 1 ? 1 : 0;
        la.peer_arenas = b->peer_table();
        la.connected = b->connected ? 1 : 0;

        la.topk_idx = (const int64_t*)a.topk_idx.data;
        la.num_tokens = num_tokens;
        la.num_topk = K;
        la.num_experts = E;
        la.num_ranks = R;
        la.rank_idx = b->rank_idx;
        la.expert_alignment = a.expert_alignment;
        la.max_tokens = a.num_max_tokens_per_rank;
        la.experts_per_rank = num_experts_per_rank;
        la.num_blocks = num_blocks;
        la.seq = R == 1 ? ++b->seq : 0;
        la.notify_host = do_cpu_sync and R == 1 ? 1 : 0;
        la.dst_buffer_slot_idx = (int*)a.dst_buffer_slot_idx.data;
        la.dst_gsge_idx = (int*)a.dst_gsge_idx.data;
        la.psum_rank = (int*)psum_rank.data;
        la.psum_expert = (int*)psum_expert.data;
        la.unaligned_expert = (int*)unaligned.data;
        la.cumulative_stats = (int*)a.cumulative_local_expert_recv_stats.data;
        la.host_page = b->host_page_dev;

        launch_layout(la, num_blocks, a.stream);

        if (num_ranks > 1) launch_pack();

        b->last.valid = true;
        b->last.stamp = ++b->launch_stamp;
        b->last.num_tokens = num_tokens;
        b->last.num_topk = K;
        b->last.num_experts = E;
        b->last.alignment = a.expert_alignment;
        b->last.max_tokens = a.num_max_tokens_per_rank;
        b->last.slot_map = la.slot_map;
        b->last.tok_row = la.tok_row;
        b->last.notified = do_cpu_sync and R == 1;
        b->last.recv_done = false;
    });
}

int64_t ep_dispatch_stamp(ep_buffer_t* b) {
    return (b == nullptr || b->destroyed || !b->last.valid) ? 0 : b->last.stamp;
}

void ep_set_layout_fold_max_blocks(int num_blocks) { g_fold_max_blocks = num_blocks; }

void ep_set_layout_recount_limit(int blocks_times_topk) { g_recount_limit = blocks_times_topk; }

void ep_set_combine_blocks_per_cu(int num_blocks) { g_combine_blocks_per_cu = num_blocks; }

int ep_dispatch_recv_launch(ep_buffer_t* b, const ep_dispatch_recv_args_t* pa) {
    return guarded([&] {
        EP_HOST_ASSERT(pa != nullptr);
        check_buffer(b);
        const ep_dispatch_recv_args_t& a = *pa;
        const int R = b->num_ranks;
        if (R == 1) return;             // one partition: ep_dispatch_launch has produced the whole layout
        EP_HOST_ASSERT(b->last.valid and not b->last.recv_done and "follows this buffer's own ep_dispatch_launch");
        EP_HOST_ASSERT(a.dispatch_stamp == b->last.stamp and "the receive side belongs to the latest dispatch launch of this buffer");
        check_peers(b, [&](const ep_buffer& p) { return p.num_sends >= b->num_sends; },
                    "its ep_dispatch_launch comes before any receive side");
        const int K = a.num_topk, E = a.num_experts;
        EP_HOST_ASSERT(K == b->last.num_topk and E == b->last.num_experts);
        EP_HOST_ASSERT(a.expert_alignment == b->last.alignment and a.num_max_tokens_per_rank == b->last.max_tokens);
        const int El = E / R;
        const auto& psum_rank = a.psum_num_recv_tokens_per_rank;
        const auto& psum_expert = a.psum_num_recv_tokens_per_expert;
        const auto& unaligned = a.num_unaligned_recv_tokens_per_expert;
        EP_HOST_ASSERT(present(psum_rank) and psum_rank.ndim == 1 and psum_rank.size[0] == R);
        EP_HOST_ASSERT(present(psum_expert) and psum_expert.ndim == 1 and psum_expert.size[0] == El);
        EP_HOST_ASSERT(present(unaligned) and unaligned.ndim == 1 and unaligned.size[0] == El);
        EP_HOST_ASSERT(psum_rank.dtype == EP_DTYPE_I32 and psum_expert.dtype == EP_DTYPE_I32);
        EP_HOST_ASSERT(unaligned.dtype == EP_DTYPE_I32);
        EP_HOST_ASSERT(contiguous(psum_rank) and contiguous(psum_expert) and contiguous(unaligned));
        if (present(a.cumulative_local_expert_recv_stats)) {
            const auto& st = a.cumulative_local_expert_recv_stats;
            EP_HOST_ASSERT(st.ndim == 1 and st.size[0] == El and contiguous(st) and st.dtype == EP_DTYPE_I32);
        }
        const auto& meta = a.recv_src_metadata;
        EP_HOST_ASSERT(present(meta) and meta.ndim == 2 and meta.size[1] == K + 2);
        EP_HOST_ASSERT(contiguous(meta) and meta.dtype == EP_DTYPE_I32);
        const int64_t rows_bound = b->recv_rows_bound(b->last.num_tokens, a.num_max_tokens_per_rank);
        EP_HOST_ASSERT(meta.size[0] >= rows_bound and "room for every row that can arrive");
        EP_HOST_ASSERT(rows_bound <= INT32_MAX);
        EP_HOST_ASSERT(a.hidden_bytes > 0 and a.num_sf_packs >= 0);
        const PackedToken pk = packed_token(a.hidden_bytes, a.num_sf_packs * 2, K, true);
        EP_HOST_ASSERT((int64_t)R * a.num_max_tokens_per_rank * pk.bytes <= b->num_buffer_bytes);
        EP_HOST_ASSERT(a.num_sf_packs == 0 or a.hidden_bytes % kUbAlign == 0);      // see ep_dispatch_launch

        const int num_blocks = std::max<int>(1, (int)ceil_div(rows_bound, EP_TOKENS_PER_BLOCK));
        int* ws = (int*)b->workspace();
        int64_t off = EP_WS_HEADER_BYTES / sizeof(int);
        auto carve = [&](int64_t n) {
            int* p = ws + off;
            off += align_up(std::max<int64_t>(n, 1), 64);
            return p;
        };
        EpLayoutArgs la{};
        la.cnt_stride = (int)align_up(E / R + R, 8);
        la.col_total = carve(la.cnt_stride);
        la.blk_cnt = carve((int64_t)num_blocks * la.cnt_stride);
        EP_HOST_ASSERT(off * (int64_t)sizeof(int) <= b->workspace_bytes and "layout scratch of the receive stream fits the workspace");
        la.recv_mode = 1;
        la.num_tokens = (int)rows_bound;
        la.num_topk = K;
        la.num_experts = E;
        la.num_ranks = R;
        la.rank_idx = b->rank_idx;
        la.expert_alignment = a.expert_alignment;
        la.max_tokens = a.num_max_tokens_per_rank;
        la.experts_per_rank = El;
        la.num_blocks = num_blocks;
        la.seq = ++b->seq;
        la.notify_host = a.do_cpu_sync ? 1 : 0;
        la.psum_rank = (int*)psum_rank.data;
        la.psum_expert = (int*)psum_expert.data;
        la.unaligned_expert = (int*)unaligned.data;
        la.cumulative_stats = (int*)a.cumulative_local_expert_recv_stats.data;
        la.host_page = b->host_page_dev;
        la.peer_arenas = b->peer_table();
        la.connected = b->connected ? 1 : 0;
        la.inbox = b->inbox();
        la.packed_base = b->buffer();
        la.packed_row_bytes = pk.bytes;
        la.idx_off = pk.idx_off;
        la.src_off = pk.src_off;
        la.recv_src_metadata = (int*)meta.data;
        la.rows_cap = (int)std::min<int64_t>(meta.size[0], INT32_MAX);
        launch_layout(la, num_blocks, a.stream);
        b->last.recv_done = true;
        b->last.notified = a.do_cpu_sync != 0;
    });
}

int ep_dispatch_wait_counts(ep_buffer_t* b, int* num_recv_tokens, int* num_expanded_tokens, int* per_expert) {
    return guarded([&] {
        EP_HOST_ASSERT(b != nullptr and not b->destroyed);
        EP_HOST_ASSERT(b->last.valid);
        EP_HOST_ASSERT(b->last.notified and "the last dispatch was launched with do_cpu_sync (nothing else publishes the counts)");
        const auto deadline = std::chrono::steady_clock::now() + std::chrono::seconds(b->cpu_timeout_secs);
        volatile int* page = b->host_page;
        while (__atomic_load_n(&page[0], __ATOMIC_ACQUIRE) != b->seq) {
            if (std::chrono::steady_clock::now() >= deadline) EP_HOST_UNREACHABLE("reduction timeout");
        }
        if (num_recv_tokens != nullptr) *num_recv_tokens = page[1];
        if (num_expanded_tokens != nullptr) *num_expanded_tokens = page[2];
        if (per_expert != nullptr) {
            const int El = b->last.num_experts / b->num_ranks;
            for (int e = 0; e < El; ++e) per_expert[e] = page[EP_HOST_EXPERT_OFF + e];
        }
    });
}

int ep_dispatch_worst_case_sizes(ep_buffer_t* b, int max_tokens, int num_topk, int num_experts, int alignment,
                                 int* num_recv_tokens, int* num_expanded_tokens) {
    return guarded([&] {
        EP_HOST_ASSERT(b == nullptr or not b->destroyed);
        const int num_ranks = b == nullptr ? 1 : b->num_ranks;      // no buffer: one partition
        EP_HOST_ASSERT(num_experts % num_ranks == 0 and alignment > 0);
        const int El = num_experts / num_ranks;
        int64_t n = (int64_t)num_ranks * max_tokens * std::min(num_topk, El);
        n += (int64_t)(alignment - 1) * El;
        n = align_up(n, alignment);
        EP_HOST_ASSERT(n <= INT32_MAX);
        *num_recv_tokens = num_ranks * max_tokens;
        *num_expanded_tokens = (int)n;
    });
}

int ep_dispatch_epilogue_launch(ep_buffer_t* b, const ep_dispatch_epilogue_args_t* pa) {
    return guarded([&] {
        EP_HOST_ASSERT(pa != nullptr);
        check_buffer(b);
        const ep_dispatch_epilogue_args_t& a = *pa;
        const bool cached_mode = a.cached_mode != 0;
        EP_HOST_ASSERT(present(a.x) and a.x.ndim == 2 and contiguous(a.x));
        const int num_tokens = (int)a.x.size[0];
        const int hidden = (int)a.x.size[1];
        const int K = a.num_topk;
        const int R = b->num_ranks;
        EP_HOST_ASSERT(K > 0 and K <= EP_MAX_TOPK);
        EP_HOST_ASSERT(a.num_experts % R == 0);
        const int El = a.num_experts / R;
        const bool fused = a.fused_fp8_quant != 0;
        // the same input contract as ep_dispatch_launch: this entry point may be called on its own
        if (present(a.sf)) {
            EP_HOST_ASSERT(not fused and a.x.dtype == EP_DTYPE_FP8_E4M3);
            EP_HOST_ASSERT(a.sf.ndim == 2 and a.sf.size[0] == num_tokens and elem_size(a.sf.dtype) == 2);
            EP_HOST_ASSERT(a.sf.stride[0] == 1 or a.sf.stride[1] == 1);
            EP_HOST_ASSERT(a.sf.stride[0] <= INT32_MAX and a.sf.stride[1] <= INT32_MAX);
        } else {
            EP_HOST_ASSERT(a.x.dtype == EP_DTYPE_BF16);
        }
        EP_HOST_ASSERT(not fused or (hidden % 8 == 0 and hidden <= 16384));
        EP_HOST_ASSERT(a.num_max_tokens_per_rank > 0 and num_tokens <= a.num_max_tokens_per_rank);
        EP_HOST_ASSERT(a.expert_alignment > 0);
        EP_HOST_ASSERT(present(a.recv_x) and a.recv_x.ndim == 2 and a.recv_x.size[1] == hidden);
        EP_HOST_ASSERT(contiguous(a.recv_x));
        EP_HOST_ASSERT(a.recv_x.dtype == (fused ? (int)EP_DTYPE_FP8_E4M3 : a.x.dtype));
        const int64_t num_expanded = a.recv_x.size[0];
        const bool has_sf = present(a.sf) or fused;
        int num_sf_packs = 0;
        if (has_sf) {
            EP_HOST_ASSERT(present(a.recv_sf) and a.recv_sf.ndim == 2 and a.recv_sf.size[0] == num_expanded);
            if (fused) {
                EP_HOST_ASSERT(a.recv_sf.dtype == EP_DTYPE_F32 and a.recv_sf.size[1] == ceil_div(hidden, 128));
            } else {
                EP_HOST_ASSERT(elem_size(a.recv_sf.dtype) == 2 and a.recv_sf.size[1] == a.sf.size[1]);
                num_sf_packs = (int)a.sf.size[1];
            }
            // row-major scale rows (csrc/kernels/ep/dispatch.hpp:112-113), or the column-major result of
            // the reference's transposing pass (csrc/buffers/ep.hpp:379-381) written in place
            EP_HOST_ASSERT(a.recv_sf_layout >= EP_SF_ROW_MAJOR and a.recv_sf_layout <= EP_SF_COL_MAJOR_COUNTED);
            if (a.recv_sf_layout == EP_SF_ROW_MAJOR) {
                EP_HOST_ASSERT(a.recv_sf.stride[1] == 1 and a.recv_sf.stride[0] == a.recv_sf.size[1]);
            } else {
                EP_HOST_ASSERT(a.recv_sf.stride[0] == 1 and a.recv_sf.stride[1] == a.recv_sf.size[0]);
                // the copy kernel writes scale rows into the staging tensor, a second kernel turns them
                const ep_tensor_t& st = a.recv_sf_staging;
                EP_HOST_ASSERT(present(st) and st.ndim == 2 and st.dtype == a.recv_sf.dtype);
                EP_HOST_ASSERT(st.size[0] == a.recv_sf.size[0] and st.size[1] == a.recv_sf.size[1]);
                EP_HOST_ASSERT(st.stride[1] == 1 and st.stride[0] == st.size[1] and st.data != a.recv_sf.data);
            }
        }
        if (present(a.topk_weights)) {
            EP_HOST_ASSERT(present(a.recv_topk_weights) and a.recv_topk_weights.ndim == 1);
            EP_HOST_ASSERT(a.recv_topk_weights.size[0] == num_expanded and a.recv_topk_weights.dtype == EP_DTYPE_F32);
            EP_HOST_ASSERT(a.topk_weights.ndim == 2 and a.topk_weights.size[0] == num_tokens and a.topk_weights.size[1] == K);
            EP_HOST_ASSERT(contiguous(a.topk_weights) and a.topk_weights.dtype == EP_DTYPE_F32);
            EP_HOST_ASSERT(contiguous(a.recv_topk_weights));
        }
        EP_HOST_ASSERT(present(a.recv_src_metadata) and a.recv_src_metadata.ndim == 2);
        EP_HOST_ASSERT(a.recv_src_metadata.size[1] == K + 2);
        EP_HOST_ASSERT(contiguous(a.recv_src_metadata));
        EP_HOST_ASSERT(a.recv_src_metadata.dtype == EP_DTYPE_I32);
        for (const ep_tensor_t* ps : {&a.psum_num_recv_tokens_per_rank, &a.psum_num_recv_tokens_per_expert})
            EP_HOST_ASSERT(present(*ps) and ps->ndim == 1 and contiguous(*ps) and ps->dtype == EP_DTYPE_I32);
        EP_HOST_ASSERT(a.psum_num_recv_tokens_per_rank.size[0] == R and a.psum_num_recv_tokens_per_expert.size[0] == El);
        if (not cached_mode) {
            EP_HOST_ASSERT(b->last.valid and "the copy epilogue follows its own dispatch launch");
            // the slot map and the receive order live in the workspace, which every dispatch launch overwrites
            EP_HOST_ASSERT(a.dispatch_stamp == b->last.stamp and "the copy epilogue belongs to the latest dispatch launch of this buffer");
            EP_HOST_ASSERT(b->last.num_tokens == num_tokens and b->last.num_topk == K);
            EP_HOST_ASSERT((R == 1 or b->last.recv_done) and "the receive-side layout comes before the copy");
        }
        if (R > 1) {
            check_peers(b, [&](const ep_buffer& p) { return p.num_sends >= b->num_sends; },
                        "its ep_dispatch_launch comes before any copy epilogue");
            b->num_expands = b->num_sends;
        }

        EpScatterArgs sa{};
        sa.topk_weights = (const float*)a.topk_weights.data;
        sa.slot_map = b->last.slot_map;
        sa.tok_row = b->last.tok_row;
        sa.num_recv_ptr = (const int*)a.psum_num_recv_tokens_per_rank.data + (R - 1);
        sa.recv_src_metadata = (int*)a.recv_src_metadata.data;
        sa.recv_x = a.recv_x.data;
        const bool sf_columns = has_sf and a.recv_sf_layout != EP_SF_ROW_MAJOR;
        sa.recv_sf = has_sf ? (sf_columns ? a.recv_sf_staging.data : a.recv_sf.data) : nullptr;
        sa.recv_topk_weights = present(a.topk_weights) ? (float*)a.recv_topk_weights.data : nullptr;
        sa.psum_expert = (const int*)a.psum_num_recv_tokens_per_expert.data;
        sa.out_row_bytes = (int64_t)hidden * elem_size(a.recv_x.dtype);
        sa.out_sf_row_bytes = has_sf ? a.recv_sf.size[1] * elem_size(a.recv_sf.dtype) : 0;
        sa.hidden = hidden;
        sa.num_topk = K;
        // never walk past the rows the metadata tensor holds
        sa.num_rows_bound = (int)std::min<int64_t>(b->recv_rows_bound(num_tokens, a.num_max_tokens_per_rank),
                                                   a.recv_src_metadata.size[0]);
        sa.num_meta_rows = (int)std::min<int64_t>(a.recv_src_metadata.size[0], INT32_MAX);
        sa.num_tokens = num_tokens;
        sa.rank_idx = b->rank_idx;
        sa.max_tokens = a.num_max_tokens_per_rank;
        sa.cached = cached_mode ? 1 : 0;
        sa.num_local_experts = El;
        sa.expert_alignment = a.expert_alignment;
        sa.num_out_rows = (int)std::min<int64_t>(num_expanded, INT32_MAX);
        bool quantise_here = fused;
        if (R == 1) {
            // one partition: the packed intermediate is skipped, rows come straight from x
            sa.mode = EP_SCATTER_EXPAND;
            if (not cached_mode) {
                // the tasks walk the tokens, not the receive stream: no device count bounds them
                sa.num_recv_ptr = nullptr;
                sa.num_rows_bound = num_tokens;
            }
            // a cached handle that holds one metadata row per token: row i is token i (the rows ascend with the token)
            sa.rows_are_tokens = cached_mode and a.recv_src_metadata.size[0] == num_tokens ? 1 : 0;
            sa.x = a.x.data;
            sa.sf = a.sf.data;
            sa.x_row_bytes = (int64_t)hidden * elem_size(a.x.dtype);
            sa.copy_bytes = sa.x_row_bytes;
            if (present(a.sf)) {
                sa.sf_token_stride_bytes = a.sf.stride[0] * 2;
                sa.sf_pack_stride_bytes = a.sf.stride[1] * 2;
            }
            sa.num_sf_packs = num_sf_packs;
        } else {
            // expand this partition's own region of the packed rows written by ep_dispatch_launch
            const int payload_elem = fused ? 1 : elem_size(a.x.dtype);
            const int sf_packs = fused ? 2 * (int)ceil_div(hidden, 128) : num_sf_packs;
            const PackedToken pk = packed_token(hidden * payload_elem, sf_packs * 2, K, not cached_mode);
            EP_HOST_ASSERT((int64_t)R * a.num_max_tokens_per_rank * pk.bytes <= b->num_buffer_bytes);
            EP_HOST_ASSERT(sf_packs == 0 or (int64_t)hidden * payload_elem % kUbAlign == 0);   // see ep_dispatch_launch
            sa.mode = EP_SCATTER_REGION;
            sa.psum_rank = (const int*)a.psum_num_recv_tokens_per_rank.data;
            sa.num_ranks = R;
            sa.x = b->buffer();
            sa.x_row_bytes = pk.bytes;
            sa.copy_bytes = (int64_t)hidden * payload_elem;
            sa.sf = sf_packs > 0 ? b->buffer() + pk.sf_off : nullptr;
            sa.sf_token_stride_bytes = pk.bytes;
            sa.sf_pack_stride_bytes = 2;
            sa.num_sf_packs = sf_packs;
            sa.w_off = pk.w_off;
            quantise_here = false;
        }
        // a wave task covers 1 KiB of a verbatim row (4 KiB of a packed row, which mostly has one destination
        // among this partition's few experts), or 512 channels of a row being quantised
        sa.vecs_per_lane = sa.mode == EP_SCATTER_REGION ? 4 : 1;
        sa.num_parts = (int)std::max<int64_t>(
            1, quantise_here ? ceil_div(hidden, 512) : ceil_div(sa.copy_bytes, 1024 * sa.vecs_per_lane));
        const int64_t row_blocks = ceil_div((int64_t)sa.num_rows_bound * sa.num_parts, EP_ROWS_PER_BLOCK);
        EP_HOST_ASSERT(row_blocks <= INT32_MAX / 2);
        sa.num_row_blocks = (int)row_blocks;
        // rows are read in 16-byte vectors; the verbatim kernel writes them so, the quantising one 8 bytes a lane
        EP_HOST_ASSERT(sa.x_row_bytes % 16 == 0 and sa.out_row_bytes % (quantise_here ? 8 : 16) == 0);
        // an expert has at most alignment - 1 padding rows: about one workgroup per 8 of them (measured: 16 a
        // expert at alignment 128 and 32 or 64 give the same time; one per 4 KiB chunk, 223 a expert, is 10-20 %
        // slower: every workgroup first waits for the expert's row count)
        sa.pad_blocks_per_expert = std::max(1, std::min(EP_MAX_PAD_BLOCKS_PER_EXPERT, a.expert_alignment / 8));
        const unsigned pad_blocks = a.do_zero_padding ? (unsigned)(El * sa.pad_blocks_per_expert) : 0u;
        const unsigned grid = (unsigned)sa.num_row_blocks + pad_blocks;
        if (grid > 0) {
            hipFunction_t fn = quantise_here ? (g_fp8_hw ? g_k.scatter_quant : g_k.scatter_quant_sw) : g_k.scatter_copy;
            launch(fn, grid, EP_ROW_THREADS, 0, a.stream, sa);
        }
        if (sf_columns and num_expanded > 0) {
            EpSfTransposeArgs ta{};
            ta.src = a.recv_sf_staging.data;
            ta.dst = a.recv_sf.data;
            ta.psum_expert = sa.psum_expert;
            ta.num_rows = sa.num_out_rows;
            ta.num_cols = (int)a.recv_sf.size[1];
            ta.elem_bytes = elem_size(a.recv_sf.dtype);
            ta.counted = a.recv_sf_layout == EP_SF_COL_MAJOR_COUNTED ? 1 : 0;
            ta.num_local_experts = El;
            ta.expert_alignment = a.expert_alignment;
            launch(g_k.sf_transpose, (unsigned)ceil_div(ta.num_rows, EP_SF_TILE), EP_LAYOUT_THREADS, 0, a.stream, ta);
        }
    });
}

// ---- combine ----------------------------------------------------------------------------------
int ep_combine_launch(ep_buffer_t* b, const ep_combine_args_t* pa, int phase) {
    return guarded([&] {
        EP_HOST_ASSERT(pa != nullptr);
        check_buffer(b);
        const ep_combine_args_t& a = *pa;
        const int R = b->num_ranks;
        EP_HOST_ASSERT(a.num_experts > 0 and a.num_experts % R == 0);

        EP_HOST_ASSERT(present(a.x) and a.x.ndim == 2);
        const int num_tokens = (int)a.x.size[0];
        const int hidden = (int)a.x.size[1];
        EP_HOST_ASSERT(contiguous(a.x));
        EP_HOST_ASSERT(a.x.dtype == EP_DTYPE_BF16);
        EP_HOST_ASSERT(hidden % 8 == 0);

        EP_HOST_ASSERT(present(a.combined_topk_idx) and a.combined_topk_idx.ndim == 2);
        const int num_combined_tokens = (int)a.combined_topk_idx.size[0];
        const int K = (int)a.combined_topk_idx.size[1];
        EP_HOST_ASSERT(K > 0 and K <= EP_MAX_TOPK);
        EP_HOST_ASSERT(num_combined_tokens <= a.num_max_tokens_per_rank);
        EP_HOST_ASSERT(contiguous(a.combined_topk_idx));
        EP_HOST_ASSERT(a.combined_topk_idx.dtype == EP_DTYPE_I64);
        EP_HOST_ASSERT(present(a.src_metadata) and a.src_metadata.ndim == 2 and a.src_metadata.size[1] == K + 2);
        EP_HOST_ASSERT(a.src_metadata.size[0] <= (int64_t)R * a.num_max_tokens_per_rank);
        EP_HOST_ASSERT(contiguous(a.src_metadata));
        EP_HOST_ASSERT(a.src_metadata.dtype == EP_DTYPE_I32);
        const auto& psum_rank = a.psum_num_recv_tokens_per_rank;
        EP_HOST_ASSERT(present(psum_rank) and psum_rank.ndim == 1);
        EP_HOST_ASSERT(psum_rank.size[0] == R);
        EP_HOST_ASSERT(contiguous(psum_rank));
        EP_HOST_ASSERT(psum_rank.dtype == EP_DTYPE_I32);

        if (present(a.topk_weights)) {
            EP_HOST_ASSERT(a.topk_weights.ndim == 1 and a.topk_weights.size[0] == num_tokens);
            EP_HOST_ASSERT(contiguous(a.topk_weights));
            EP_HOST_ASSERT(a.topk_weights.dtype == EP_DTYPE_F32);
        }
        EP_HOST_ASSERT(not a.apply_weights or present(a.topk_weights));
        const ep_tensor_t* biases[2] = {&a.bias_0, &a.bias_1};
        for (const ep_tensor_t* bias : biases) {
            if (present(*bias)) {
                EP_HOST_ASSERT(bias->ndim == 2);
                EP_HOST_ASSERT(bias->size[0] == num_combined_tokens and bias->size[1] == hidden);
                EP_HOST_ASSERT(contiguous(*bias));
                EP_HOST_ASSERT(bias->dtype == a.x.dtype);
            }
        }
        EP_HOST_ASSERT(combine_buffer_size(R, a.num_max_tokens_per_rank, hidden, K) <= b->num_buffer_bytes);
        EP_HOST_ASSERT(phase == 0 or phase == 1);
        EP_HOST_ASSERT(not a.apply_weights or R == 1);
        const int kidx = K == 2 ? 1 : K == 4 ? 2 : K == 6 ? 3 : K == 8 ? 4 : 0;
        const int64_t combine_token = token_bytes(hidden * 2, 0, K, false);

        EpCombineArgs ca{};
        ca.expanded_weights = (const float*)a.topk_weights.data;
        ca.recv_src_metadata = (const int*)a.src_metadata.data;
        ca.topk_idx = (const int64_t*)a.combined_topk_idx.data;
        ca.hidden = hidden;
        ca.num_topk = K;
        ca.num_tokens = num_combined_tokens;
        ca.rank_idx = b->rank_idx;
        ca.max_tokens = a.num_max_tokens_per_rank;
        ca.num_parts = (int)std::max<int64_t>(1, ceil_div(hidden, 1024));
        ca.num_experts = a.num_experts;
        ca.num_ranks = R;
        ca.experts_per_rank = a.num_experts / R;
        ca.num_groups = std::min(K, R);

        if (phase == 0) {
            if (R == 1) return;     // single partition: the whole reduction is one token-side launch
            // the partials land where the peers' packed rows are
            check_peers(b, [&](const ep_buffer& p) { return p.num_expands >= p.num_sends and p.num_sends >= b->num_sends; },
                        "runs its copy epilogue before any combine");
            ++b->num_partials;
            // owner side: one partial per received row into this GPU's combine buffer
            ca.y = a.x.data;
            ca.y_row_bytes = (int64_t)hidden * 2;
            ca.num_in_rows = num_tokens;
            ca.num_recv_ptr = (const int*)psum_rank.data + (R - 1);
            ca.num_rows_bound = (int)a.src_metadata.size[0];
            ca.combined_x = b->buffer();
            ca.peer_arenas = b->peer_table();
            ca.buffer_off = b->workspace_bytes;
            ca.out_row_bytes = combine_token;
            // a received row mostly has one slot among a partition's few experts: whole rows per wave task once
            // there are enough rows to fill the machine that way (a few thousand rows are spread part by part)
            if (ca.num_rows_bound >= 16384) {
                ca.whole_rows = 1;
                ca.num_parts = 1;
            }
            ca.num_row_blocks = (int)ceil_div((int64_t)ca.num_rows_bound * ca.num_parts, EP_ROWS_PER_BLOCK);
            if (ca.num_row_blocks == 0) return;
            launch(g_k.combine[EP_COMBINE_PARTIAL][kidx], (unsigned)ca.num_row_blocks, EP_ROW_THREADS, 0, a.stream, ca);
            return;
        }

        EP_HOST_ASSERT(present(a.combined_x) and a.combined_x.ndim == 2);
        EP_HOST_ASSERT(a.combined_x.size[0] == num_combined_tokens and a.combined_x.size[1] == hidden);
        EP_HOST_ASSERT(contiguous(a.combined_x) and a.combined_x.dtype == EP_DTYPE_BF16);
        if (present(a.topk_weights)) {
            const auto& w = a.combined_topk_weights;
            EP_HOST_ASSERT(present(w) and w.ndim == 2 and w.size[0] == num_combined_tokens and w.size[1] == K);
            EP_HOST_ASSERT(contiguous(w) and w.dtype == EP_DTYPE_F32);
        }
        ca.bias_0 = a.bias_0.data;
        ca.bias_1 = a.bias_1.data;
        ca.combined_x = a.combined_x.data;
        ca.combined_topk_weights = present(a.topk_weights) ? (float*)a.combined_topk_weights.data : nullptr;
        ca.out_row_bytes = (int64_t)hidden * 2;
        if (R == 1) {
            ca.y = a.x.data;
            ca.y_row_bytes = (int64_t)hidden * 2;
            ca.num_in_rows = num_tokens;
            ca.num_recv_ptr = (const int*)psum_rank.data + (R - 1);
            ca.num_rows_bound = (int)a.src_metadata.size[0];
            ca.weighted = a.apply_weights ? 1 : 0;
            ca.num_row_blocks = (int)ceil_div((int64_t)ca.num_rows_bound * ca.num_parts, EP_ROWS_PER_BLOCK);
            const unsigned grid = (unsigned)ca.num_row_blocks + (unsigned)ceil_div(num_combined_tokens, EP_ROW_THREADS);
            if (grid == 0) return;
            launch(g_k.combine[EP_COMBINE_FUSED][kidx], grid, EP_ROW_THREADS, combine_lds_cap(K + (ca.bias_0 != nullptr) + (ca.bias_1 != nullptr), kidx != 0, ca.num_row_blocks, hidden), a.stream, ca);
        } else {
            check_peers(b, [&](const ep_buffer& p) { return p.num_partials >= b->num_partials; },
                        "its owner-side reduce (phase 0) comes before any token-side reduce");
            // token side: biases + the partial of every master, read from the combine buffer
            ca.y = b->buffer();
            ca.y_row_bytes = combine_token;
            ca.num_in_rows = ca.num_groups * a.num_max_tokens_per_rank;
            ca.num_recv_ptr = nullptr;
            ca.num_rows_bound = num_combined_tokens;
            ca.num_row_blocks = (int)ceil_div((int64_t)ca.num_rows_bound * ca.num_parts, EP_ROW_THREADS / 64);
            if (ca.num_row_blocks == 0) return;
            launch(g_k.combine[EP_COMBINE_FINAL][kidx], (unsigned)ca.num_row_blocks, EP_ROW_THREADS, 0, a.stream, ca);
        }
    });
}

}  // extern "C"

// ---- dispatch without any allocation ------------------------------------------------------------
// For callers that cannot call hipMalloc (code under HIP graph capture, serving loops, harnesses that
// forbid it): the layout scratch that ep_dispatch_launch carves from a buffer's arena lives in a
// file-scope device array instead, so no ep_buffer (whose creation allocates) is needed at all.  Every
// GPU holds its own copy of the array until the process ends; its device address is looked up once per
// device and kept.  The kernels take that address as an argument, exactly as they take the arena's
// workspace.  Every call on a GPU shares the array: calls that overlap on one GPU race.  Nothing in it
// has to start at zero (every word the kernels read was written earlier in the same call).
#define EP_STATIC_SCRATCH_BYTES (4 * 1024 * 1024)
static __device__ __align__(256) unsigned char scratch[EP_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
ep_buffer g_static_view[kMaxDevices];       // host-side views: arena = the device's copy of `scratch`
std::mutex g_static_mutex;

ep_buffer* static_view_of_current_device() {
    int dev = -1;
    HIP_CHECK(hipGetDevice(&dev));
    EP_HOST_ASSERT(dev >= 0 and dev < kMaxDevices);
    EP_HOST_ASSERT(dev == g_k.device and "the kernels were loaded on another device");
    std::lock_guard<std::mutex> lock(g_static_mutex);
    ep_buffer* v = &g_static_view[dev];
    if (v->arena == nullptr) {
        void* ptr = nullptr;
        HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));     // this device's copy; never the array's name
        EP_HOST_ASSERT(ptr != nullptr);
        v->arena = (char*)ptr;
        v->device = dev;
        v->rank_idx = 0;
        v->num_ranks = 1;
        v->num_buffer_bytes = 0;
        v->workspace_bytes = EP_STATIC_SCRATCH_BYTES;
        v->is_static = true;
    }
    return v;
}
}  // namespace

void ep_static_scratch_init() { (void)static_view_of_current_device(); }

// Bytes of the static scratch a single-partition dispatch of this shape carves: the header, then the column
// totals, the count matrix, the slot map and the token -> row map, each rounded up to 64 ints (what
// ep_dispatch_launch carves from a workspace, restated).
extern "C" int64_t ep_dispatch_static_scratch_bytes(int num_tokens, int num_topk, int num_experts) {
    if (num_tokens < 0 or num_topk <= 0 or num_experts <= 0) return -1;
    auto a64 = [](int64_t n) { return align_up(std::max<int64_t>(n, 1), 64); };
    const int64_t W = align_up((int64_t)num_experts + 1, 8);
    const int64_t B = std::max<int64_t>(1, ceil_div(num_tokens, EP_TOKENS_PER_BLOCK));
    return EP_WS_HEADER_BYTES + 4 * (a64(W) + a64(B * W) + a64((int64_t)num_tokens * num_topk) + a64(num_tokens));
}
extern "C" int64_t ep_dispatch_static_scratch_capacity(void) { return EP_STATIC_SCRATCH_BYTES; }

extern "C" int ep_dispatch_static_launch(const ep_dispatch_args_t* d, const ep_dispatch_epilogue_args_t* e) {
    int rc = guarded([&] {
        EP_HOST_ASSERT(d != nullptr and e != nullptr);
        load_kernels(nullptr);
        EP_HOST_ASSERT(not d->cached_mode and not d->do_cpu_sync and not e->cached_mode);
        EP_HOST_ASSERT(d->stream == e->stream);
    });
    if (rc != 0) return rc;
    ep_buffer* v = nullptr;
    rc = guarded([&] { v = static_view_of_current_device(); });
    if (rc != 0) return rc;
    rc = ep_dispatch_launch(v, d);
    if (rc != 0) return rc;
    ep_dispatch_epilogue_args_t ee = *e;
    ee.dispatch_stamp = v->last.stamp;
    return ep_dispatch_epilogue_launch(v, &ee);
}
