// Host side of libdeep_ep_calib.so (include/deep_ep_calib.h): loads the calibration code object and
// launches its kernels through hipModuleLaunchKernel.  Benchmarks load it; the product library does not.
#include <hip/hip_runtime.h>

#include <dlfcn.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <string>

#include "../../include/deep_ep_calib.h"
#include "ep_calib_args.h"

namespace {

thread_local std::string g_err;

struct CalibError {
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

#define CALIB_ASSERT(cond)                                                                                          \
    do {                                                                                                            \
        if (!(cond)) throw CalibError{format("Assertion exception (%s:%d): %s", __FILE_NAME__, __LINE__, #cond)};   \
    } while (0)

#define HIP_CHECK(cmd)                                                                                              \
    do {                                                                                                            \
        const hipError_t e_ = (cmd);                                                                                \
        if (e_ != hipSuccess)                                                                                       \
            throw CalibError{format("HIP runtime exception (%s:%d): Error code: %d, detail: %s", __FILE_NAME__,     \
                                    __LINE__, (int)e_, hipGetErrorString(e_))};                                     \
    } while (0)

template <class F>
int guarded(F&& f) {
    try {
        f();
        return 0;
    } catch (const CalibError& e) {
        g_err = e.msg;
        return 1;
    } catch (const std::exception& e) {
        g_err = e.what();
        return 1;
    }
}

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

constexpr int kNumVariants = 11;
const char* const kVariantKernels[kNumVariants] = {
    "ep_calib_scatter_token_major", "ep_calib_scatter_stores_only", "ep_calib_read_rows",
    "ep_calib_ordered_flat", "ep_calib_ordered_flat_stores_only",
    "ep_calib_ordered_steered", "ep_calib_ordered_steered_stores_only", "ep_calib_ordered_steered_loads_only",
    "ep_calib_quant_rows", "ep_calib_copy_ordered_flat", "ep_calib_copy_ordered_steered"};

constexpr int kNumCombineVariants = 3;
const char* const kCombineKernels[kNumCombineVariants] = {"ep_calib_combine_k6", "ep_calib_combine_k6_loads_only",
                                                          "ep_calib_combine_k6_stores_only"};

struct Kernels {
    hipModule_t module = nullptr;
    hipFunction_t fill, fill_shuffled, fill_affine, fronts, mixed;
    hipFunction_t variant[kNumVariants];
    hipFunction_t combine[kNumCombineVariants];
    int device = -1;
};
std::mutex g_mutex;
Kernels g_k;

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
    const std::string path = (dir != nullptr ? std::string(dir) : library_dir()) + "/ep_calib.hsaco";
    FILE* f = fopen(path.c_str(), "rb");
    if (f == nullptr) throw CalibError{"cannot open the calibration code object " + path + " (build it first)"};
    fclose(f);
    HIP_CHECK(hipGetDevice(&g_k.device));
    hipModule_t m;
    HIP_CHECK(hipModuleLoad(&m, path.c_str()));
    auto get = [&](hipFunction_t& fn, const char* name) { HIP_CHECK(hipModuleGetFunction(&fn, m, name)); };
    get(g_k.fill, "ep_calib_fill");
    get(g_k.fill_shuffled, "ep_calib_fill_shuffled");
    get(g_k.fill_affine, "ep_calib_fill_affine");
    get(g_k.fronts, "ep_calib_fronts");
    get(g_k.mixed, "ep_calib_mixed");
    for (int i = 0; i < kNumVariants; ++i) get(g_k.variant[i], kVariantKernels[i]);
    for (int i = 0; i < kNumCombineVariants; ++i) get(g_k.combine[i], kCombineKernels[i]);
    g_k.module = m;
}

template <class A>
void launch(hipFunction_t fn, unsigned grid, unsigned block, void* stream, A& args, unsigned lds_bytes = 0) {
    void* params[] = {&args};
    HIP_CHECK(hipModuleLaunchKernel(fn, grid, 1, 1, block, 1, 1, lds_bytes, (hipStream_t)stream, params, nullptr));
}

void check_device() {
    int dev = -1;
    HIP_CHECK(hipGetDevice(&dev));
    CALIB_ASSERT(dev == g_k.device and "the calibration kernels were loaded on another device");
}

}  // namespace

extern "C" {

const char* ep_calib_last_error(void) { return g_err.c_str(); }

int ep_calib_init(const char* dir) {
    return guarded([&] { load_kernels(dir); });
}

int ep_calib_fill(void* dst, int64_t num_bytes, int shuffled, unsigned value, void* stream) {
    return guarded([&] {
        load_kernels(nullptr);
        check_device();
        CALIB_ASSERT(dst != nullptr and ((uintptr_t)dst & 15) == 0);
        CALIB_ASSERT(num_bytes > 0 and num_bytes % 4096 == 0 and num_bytes / 4096 <= INT32_MAX);
        const unsigned chunks = (unsigned)(num_bytes / 4096);
        CALIB_ASSERT(shuffled >= 0 and (shuffled & (shuffled - 1)) == 0);
        CALIB_ASSERT(not shuffled or ((chunks & (chunks - 1)) == 0 and (unsigned)shuffled <= chunks));     // powers of two
        EpCalibFillArgs a = {dst, chunks, value, (unsigned)std::max(1, shuffled), 0u};
        launch(shuffled ? g_k.fill_shuffled : g_k.fill, chunks, 256, stream, a);
    });
}

int ep_calib_fill_affine(void* dst, int64_t num_bytes, int modulus, int shift, unsigned value, void* stream) {
    return guarded([&] {
        load_kernels(nullptr);
        check_device();
        CALIB_ASSERT(dst != nullptr and ((uintptr_t)dst & 15) == 0);
        CALIB_ASSERT(num_bytes > 0 and num_bytes % 4096 == 0 and num_bytes / 4096 <= INT32_MAX);
        const unsigned chunks = (unsigned)(num_bytes / 4096);
        CALIB_ASSERT(modulus > 0 and (modulus & (modulus - 1)) == 0 and (chunks & (chunks - 1)) == 0 and (unsigned)modulus <= chunks);
        CALIB_ASSERT(shift >= 0);
        EpCalibFillArgs a = {dst, chunks, value, (unsigned)modulus, (unsigned)shift};
        launch(g_k.fill_affine, chunks, 256, stream, a);
    });
}

int ep_calib_fronts(void* dst, int num_fronts, int rows_per_front, int row_bytes, int64_t front_pitch_bytes,
                    unsigned value, void* stream) {
    return guarded([&] {
        load_kernels(nullptr);
        check_device();
        CALIB_ASSERT(dst != nullptr and ((uintptr_t)dst & 15) == 0);
        CALIB_ASSERT(num_fronts > 0 and rows_per_front > 0);
        CALIB_ASSERT(row_bytes > 0 and row_bytes % 16 == 0 and row_bytes <= 16384);
        CALIB_ASSERT(front_pitch_bytes >= (int64_t)rows_per_front * row_bytes and front_pitch_bytes % 16 == 0);
        CALIB_ASSERT((int64_t)num_fronts * rows_per_front <= INT32_MAX);
        EpCalibFrontsArgs a = {dst, front_pitch_bytes, (unsigned)num_fronts, (unsigned)row_bytes, value, 0u};
        launch(g_k.fronts, (unsigned)(num_fronts * rows_per_front), (unsigned)(row_bytes / 16), stream, a);
    });
}

int ep_calib_mixed(const void* src, void* dst, int64_t write_bytes, int reads_num, int reads_den, unsigned value,
                   void* stream) {
    return guarded([&] {
        load_kernels(nullptr);
        check_device();
        CALIB_ASSERT(dst != nullptr and ((uintptr_t)dst & 15) == 0);
        CALIB_ASSERT(write_bytes > 0 and write_bytes % 4096 == 0 and write_bytes / 4096 <= INT32_MAX);
        CALIB_ASSERT(reads_den > 0 and reads_num >= 0 and reads_num <= reads_den);
        CALIB_ASSERT(reads_num == 0 or (src != nullptr and ((uintptr_t)src & 15) == 0));
        const unsigned chunks = (unsigned)(write_bytes / 4096);
        // chunks of src the launch reads: what the caller was told to provide
        const unsigned read_chunks = (unsigned)ceil_div((int64_t)chunks * reads_num, reads_den);
        EpCalibMixedArgs a = {src, dst, read_chunks, (unsigned)reads_num, (unsigned)reads_den, value};
        launch(g_k.mixed, chunks, 256, stream, a);
    });
}

int ep_calib_scatter(int variant, const ep_calib_scatter_t* pa) {
    return guarded([&] {
        load_kernels(nullptr);
        check_device();
        CALIB_ASSERT(pa != nullptr);
        CALIB_ASSERT(variant >= 0 and variant < kNumVariants);
        const ep_calib_scatter_t& c = *pa;
        const int T = c.num_tokens, H = c.hidden, K = c.num_topk, E = c.num_experts;
        CALIB_ASSERT(T > 0 and T < (1 << 24) and K > 0 and K <= EP_MAX_TOPK and E > 0 and E <= EP_MAX_EXPERTS);
        CALIB_ASSERT(H > 0 and H % 128 == 0 and H <= 16384);
        CALIB_ASSERT(c.expert_alignment > 0 and c.num_out_rows > 0);
        CALIB_ASSERT(c.x != nullptr and c.recv_x != nullptr and c.recv_sf != nullptr and c.psum_expert != nullptr);
        CALIB_ASSERT(((uintptr_t)c.x & 15) == 0 and ((uintptr_t)c.recv_x & 15) == 0 and ((uintptr_t)c.recv_sf & 15) == 0);
        CALIB_ASSERT(c.recv_topk_weights == nullptr or c.topk_weights != nullptr);

        EpScatterArgs sa{};
        sa.x = c.x;
        sa.topk_weights = c.topk_weights;
        sa.recv_src_metadata = const_cast<int*>(c.recv_src_metadata);      // read only: the cached-replay form
        sa.num_recv_ptr = c.num_recv;
        sa.recv_x = c.recv_x;
        sa.recv_sf = c.recv_sf;
        sa.recv_topk_weights = c.recv_topk_weights;
        sa.psum_expert = c.psum_expert;
        sa.x_row_bytes = (int64_t)H * 2;
        sa.out_row_bytes = H;
        sa.out_sf_row_bytes = (int64_t)(H / 128) * 4;
        sa.hidden = H;
        sa.num_topk = K;
        sa.max_tokens = T;
        sa.cached = 1;
        sa.num_sf_packs = H / 128;
        sa.num_local_experts = E;
        sa.expert_alignment = c.expert_alignment;
        sa.num_tokens = T;
        sa.num_parts = (int)ceil_div(H, 512);
        sa.mode = EP_SCATTER_EXPAND;
        sa.num_out_rows = c.num_out_rows;
        sa.pad_blocks_per_expert = std::max(1, std::min(EP_MAX_PAD_BLOCKS_PER_EXPERT, c.expert_alignment / 8));
        const unsigned pad_blocks = c.do_zero_padding ? (unsigned)(E * sa.pad_blocks_per_expert) : 0u;

        if (variant <= EP_CALIB_READ_ROWS) {
            // the product's cached replay: rows of the receive stream, row i = token i when every token was received
            CALIB_ASSERT(c.recv_src_metadata != nullptr and c.num_recv != nullptr);
            CALIB_ASSERT(c.num_recv_rows > 0 and c.num_recv_rows <= T);
            sa.num_rows_bound = variant == EP_CALIB_READ_ROWS ? T : c.num_recv_rows;
            sa.num_meta_rows = c.num_recv_rows;
            sa.rows_are_tokens = c.num_recv_rows == T ? 1 : 0;
            sa.num_row_blocks = (int)ceil_div((int64_t)sa.num_rows_bound * sa.num_parts, EP_ROWS_PER_BLOCK);
            const unsigned grid = (unsigned)sa.num_row_blocks + (variant == EP_CALIB_READ_ROWS ? 0u : pad_blocks);
            launch(g_k.variant[variant], grid, EP_ROW_THREADS, c.stream, sa);
            return;
        }

        EpCalibOrderedArgs oa{};
        oa.order = (const ep_calib_entry_t*)c.order;
        oa.q_rows = (unsigned char*)c.q_rows;
        oa.q_sf = c.q_sf;
        oa.num_entries = c.num_entries;
        const bool two_pass = variant >= EP_CALIB_QUANT_ROWS;
        if (two_pass) {
            CALIB_ASSERT(c.q_rows != nullptr and c.q_sf != nullptr and ((uintptr_t)c.q_rows & 15) == 0 and ((uintptr_t)c.q_sf & 15) == 0);
            // pass 2 moves a row as at most 7 vectors of 16 bytes a lane and a scale row as 16-byte vectors
            CALIB_ASSERT(H % 512 == 0 and H <= 7168);
        }
        if (variant == EP_CALIB_QUANT_ROWS) {
            oa.s = sa;
            launch(g_k.variant[variant], (unsigned)ceil_div((int64_t)T * sa.num_parts, EP_ROWS_PER_BLOCK), EP_ROW_THREADS, c.stream, oa);
            return;
        }
        CALIB_ASSERT(c.order != nullptr and c.num_entries > 0);
        oa.groups = two_pass ? 1 : (int)ceil_div(sa.num_parts, 7);            // EP_CALIB_U parts a wave task
        const bool steered = variant == EP_CALIB_ORDERED_STEERED or variant == EP_CALIB_ORDERED_STEERED_STORES_ONLY or
                             variant == EP_CALIB_ORDERED_STEERED_LOADS_ONLY or variant == EP_CALIB_COPY_ORDERED_STEERED;
        int64_t row_blocks;
        if (steered) {
            CALIB_ASSERT(c.entries_per_list > 0 and c.num_lists > 0 and c.num_lists % 8 == 0);
            CALIB_ASSERT((int64_t)c.entries_per_list * c.num_lists == c.num_entries);
            oa.entries_per_list = c.entries_per_list;
            oa.wgs_per_list = (int)ceil_div((int64_t)c.entries_per_list * oa.groups, EP_ROWS_PER_BLOCK);
            row_blocks = (int64_t)c.num_lists * oa.wgs_per_list;
        } else {
            row_blocks = ceil_div((int64_t)c.num_entries * oa.groups, EP_ROWS_PER_BLOCK);
        }
        CALIB_ASSERT(row_blocks > 0 and row_blocks <= INT32_MAX / 2);
        sa.num_row_blocks = (int)row_blocks;
        oa.s = sa;
        const bool writes = variant != EP_CALIB_ORDERED_STEERED_LOADS_ONLY;
        launch(g_k.variant[variant], (unsigned)row_blocks + (writes ? pad_blocks : 0u), EP_ROW_THREADS, c.stream, oa);
    });
}

int ep_calib_combine(int variant, const ep_calib_combine_t* pa) {
    return guarded([&] {
        load_kernels(nullptr);
        check_device();
        CALIB_ASSERT(pa != nullptr);
        CALIB_ASSERT(variant >= 0 and variant < kNumCombineVariants);
        const ep_calib_combine_t& c = *pa;
        const int T = c.num_tokens, H = c.hidden, K = c.num_topk;
        CALIB_ASSERT(K == 6 and T > 0 and H > 0 and H % 8 == 0 and c.num_experts > 0 and c.num_experts <= EP_MAX_EXPERTS);
        CALIB_ASSERT(c.num_recv_rows > 0 and c.num_recv_rows <= T and c.num_in_rows > 0);
        CALIB_ASSERT(c.y != nullptr and c.recv_src_metadata != nullptr and c.num_recv != nullptr and c.topk_idx != nullptr);
        CALIB_ASSERT(c.combined_x != nullptr and ((uintptr_t)c.y & 15) == 0 and ((uintptr_t)c.combined_x & 15) == 0);
        CALIB_ASSERT((c.expanded_weights == nullptr) == (c.combined_topk_weights == nullptr));
        CALIB_ASSERT(c.blocks_per_cu >= 0);

        EpCombineArgs ca{};
        ca.y = c.y;
        ca.expanded_weights = c.expanded_weights;
        ca.recv_src_metadata = c.recv_src_metadata;
        ca.num_recv_ptr = c.num_recv;
        ca.topk_idx = c.topk_idx;
        ca.combined_x = c.combined_x;
        ca.combined_topk_weights = c.combined_topk_weights;
        ca.hidden = H;
        ca.num_topk = K;
        ca.num_tokens = T;
        ca.num_rows_bound = c.num_recv_rows;
        ca.rank_idx = 0;
        ca.max_tokens = T;
        ca.num_experts = c.num_experts;
        ca.num_parts = (int)std::max<int64_t>(1, ceil_div(H, 1024));
        ca.y_row_bytes = (int64_t)H * 2;
        ca.out_row_bytes = (int64_t)H * 2;
        ca.num_ranks = 1;
        ca.experts_per_rank = c.num_experts;
        ca.num_in_rows = c.num_in_rows;
        ca.num_groups = 1;
        ca.num_row_blocks = (int)ceil_div((int64_t)ca.num_rows_bound * ca.num_parts, EP_ROWS_PER_BLOCK);
        const unsigned grid = (unsigned)ca.num_row_blocks + (unsigned)ceil_div(T, EP_ROW_THREADS);
        // an unused LDS allocation caps the workgroups a compute unit holds (160 KiB of LDS a CU), as the library does
        unsigned lds = 0;
        if (c.blocks_per_cu >= 2 and c.blocks_per_cu < 160) lds = std::min(64u * 1024u, 160u * 1024u / (unsigned)c.blocks_per_cu - 1024u);
        launch(g_k.combine[variant], grid, EP_ROW_THREADS, c.stream, ca, lds);
    });
}

}  // extern "C"
