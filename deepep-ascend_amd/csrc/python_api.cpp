// Compiled Python binding of the EP hot calls: `EPBuffer.dispatch(27 args)` / `.combine(14 args)` as the
// reference's pybind module exports them (csrc/python_api.cpp:18-74, csrc/buffers/ep.hpp:88-112,411-425),
// over the C ABI of include/deep_ep_hip.h.  Torch is plumbing here: this layer allocates the outputs,
// fills the plain-pointer descriptors, passes the current HIP stream and builds the result tuples; every
// contract and every launch lives behind the C ABI in libdeep_ep_hip.so.
#include <torch/extension.h>

#include <ATen/hip/EmptyTensor.h>
#include <c10/hip/HIPStream.h>

#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/deep_ep_hip.h"

namespace py = pybind11;

namespace {

struct EpPyError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

inline void check(int rc) {
    if (rc != 0) throw EpPyError(ep_last_error());
}

#define EP_PY_ASSERT(cond)                                                                     \
    do {                                                                                       \
        if (!(cond)) throw EpPyError("Assertion exception (python_api.cpp): " #cond);          \
    } while (0)

using OptTensor = std::optional<at::Tensor>;

int dtype_code(const at::Tensor& t, bool two_byte_packs) {
    if (two_byte_packs && t.element_size() == 2) return EP_DTYPE_I16;
    switch (t.scalar_type()) {
        case at::kBFloat16: return EP_DTYPE_BF16;
        case at::kFloat8_e4m3fn: return EP_DTYPE_FP8_E4M3;
        case at::kShort: return EP_DTYPE_I16;
        case at::kInt: return EP_DTYPE_I32;
        case at::kLong: return EP_DTYPE_I64;
        case at::kFloat: return EP_DTYPE_F32;
        case at::kByte: return EP_DTYPE_U8;
        default: return EP_DTYPE_NONE;
    }
}

// Empty tensors have a null data pointer while the ABI reads null as "absent": they get the address of a
// small per-device allocation instead (never dereferenced: their sizes are zero).
void* nonnull_ptr(const at::Tensor& t) {
    // (never destroyed: at process exit torch's allocator may be gone before the statics of this module)
    static auto* dummy = new std::vector<at::Tensor>(64);
    const int dev = t.device().has_index() ? t.device().index() : 0;
    EP_PY_ASSERT(dev >= 0 && dev < 64);
    if (!(*dummy)[dev].defined()) (*dummy)[dev] = at::zeros({64}, at::TensorOptions().dtype(at::kByte).device(t.device()));
    return (*dummy)[dev].data_ptr();
}

ep_tensor_t desc(const at::Tensor& t, bool two_byte_packs = false) {
    if (!t.is_cuda()) throw EpPyError("every tensor handed to the EP kernels must live on the GPU");
    ep_tensor_t d{};
    d.data = t.data_ptr();
    if (d.data == nullptr) d.data = nonnull_ptr(t);
    d.dtype = dtype_code(t, two_byte_packs);
    const int nd = (int)t.dim();
    EP_PY_ASSERT(nd == 1 || nd == 2);
    d.ndim = nd;
    d.size[0] = t.size(0);
    d.stride[0] = t.stride(0);
    if (nd == 2) {
        d.size[1] = t.size(1);
        d.stride[1] = t.stride(1);
    }
    return d;
}

ep_tensor_t desc(const OptTensor& t, bool two_byte_packs = false) {
    return t.has_value() ? desc(*t, two_byte_packs) : ep_tensor_t{};
}

void* current_stream() { return (void*)c10::hip::getCurrentHIPStream().stream(); }

py::object new_event() {
    // (never destroyed: the interpreter is finalised before the statics of this module are)
    static auto* cls = new py::object(py::module_::import("deep_ep._C").attr("EventHandle"));
    return (*cls)();
}

// Uninitialised device tensors straight from torch's caching allocator (what at::empty reaches through its
// dispatcher).
at::Tensor alloc(at::IntArrayRef shape, at::ScalarType dtype, const at::Device& dev) {
    return at::Tensor(at::detail::empty_cuda(shape, dtype, dev, std::nullopt));
}
at::Tensor empty_i32(std::initializer_list<int64_t> shape, const at::Device& dev) { return alloc(shape, at::kInt, dev); }

// What a dispatch call keeps until its copy epilogue has been enqueued (the descriptors hold raw pointers:
// the tensors stay referenced here).
struct DispatchState {
    ep_buffer_t* buf;
    int num_ranks;
    bool connected;
    at::Tensor x, topk_idx;
    OptTensor sf, topk_weights, stats;
    at::Tensor psum_rank, psum_expert, unaligned, dst_slot, dst_gsge;
    OptTensor cached_meta;
    py::object cached_list;
    int64_t cached_num_recv = 0, cached_num_expanded = 0;
    ep_dispatch_args_t a{};
    int64_t stamp = 0;
    int num_tokens, hidden, num_topk, num_local_experts;
    int num_max_tokens_per_rank, num_experts, expert_alignment;
    bool cached_mode, do_cpu_sync, do_zero_padding, use_col_major_sf, fused;
    bool exact_sync_sizes = false;
};

py::tuple run_dispatch_epilogue(DispatchState& s) {
    const at::Device dev = s.x.device();
    const int K = s.num_topk, El = s.num_local_experts, A = s.expert_alignment, T = s.num_tokens, H = s.hidden;
    const bool partitioned = s.num_ranks > 1;
    const int64_t rows_bound = s.connected ? (int64_t)s.num_ranks * s.num_max_tokens_per_rank : T;
    at::Tensor meta;
    bool have_meta = false;
    if (partitioned && !s.cached_mode) {
        // receive side: count and rank the rows that arrived in this partition's regions
        int c_recv = 0, c_exp = 0;
        check(ep_dispatch_worst_case_sizes(s.buf, s.num_max_tokens_per_rank, K, s.num_experts, A, &c_recv, &c_exp));
        meta = empty_i32({s.do_cpu_sync ? rows_bound : (int64_t)c_recv, K + 2}, dev);
        have_meta = true;
        ep_dispatch_recv_args_t r{};
        r.psum_num_recv_tokens_per_rank = s.a.psum_num_recv_tokens_per_rank;
        r.psum_num_recv_tokens_per_expert = s.a.psum_num_recv_tokens_per_expert;
        r.num_unaligned_recv_tokens_per_expert = s.a.num_unaligned_recv_tokens_per_expert;
        r.cumulative_local_expert_recv_stats = s.a.cumulative_local_expert_recv_stats;
        r.recv_src_metadata = desc(meta);
        r.hidden_bytes = H * (s.fused ? 1 : (int)s.x.element_size());
        r.num_sf_packs = s.fused ? 2 * ((H + 127) / 128) : (s.sf.has_value() ? (int)s.sf->size(1) : 0);
        r.num_topk = K;
        r.num_max_tokens_per_rank = s.num_max_tokens_per_rank;
        r.num_experts = s.num_experts;
        r.expert_alignment = A;
        r.do_cpu_sync = s.do_cpu_sync ? 1 : 0;
        r.dispatch_stamp = s.stamp;
        r.stream = current_stream();
        check(ep_dispatch_recv_launch(s.buf, &r));
    }

    int num_recv = -1, num_expanded = -1;
    std::vector<int> per_expert((size_t)std::max(1, El));
    auto wait_counts = [&]() {
        int rc;
        {
            py::gil_scoped_release release;
            rc = ep_dispatch_wait_counts(s.buf, &num_recv, &num_expanded, per_expert.data());
        }
        check(rc);
    };
    bool counts_known = true, counts_from_host = false;
    int64_t alloc_recv, alloc_expanded;
    if (s.cached_mode) {
        num_recv = (int)s.cached_num_recv;
        num_expanded = (int)s.cached_num_expanded;
        alloc_recv = num_recv;
        alloc_expanded = num_expanded;
    } else if (s.do_cpu_sync && (s.connected || s.exact_sync_sizes)) {
        // a node: the bound over every partition's tokens is far above what arrives; wait for the counts
        // (one partition, on request: outputs of exactly the counted sizes, as the reference allocates them, at the
        // price of an idle GPU between the layout kernels and the copy)
        wait_counts();
        counts_from_host = true;
        alloc_recv = num_recv;
        alloc_expanded = num_expanded;
        if (have_meta) meta = meta.narrow(0, 0, num_recv);
    } else if (s.do_cpu_sync) {
        // Exact sizes come from the host count page, but waiting for it here would leave the GPU idle between the
        // layout kernels and the copy.  Allocate for this call's upper bound, enqueue the copy, and read the counts
        // while it runs; the results are narrowed below.
        alloc_recv = T;
        alloc_expanded = (int64_t)T * std::min(K, El) + (int64_t)(A - 1) * El;
        alloc_expanded = (alloc_expanded + A - 1) / A * A;
        counts_known = false;
    } else {
        int c_recv = 0, c_exp = 0;
        check(ep_dispatch_worst_case_sizes(s.buf, s.num_max_tokens_per_rank, K, s.num_experts, A, &c_recv, &c_exp));
        num_recv = c_recv;
        num_expanded = c_exp;
        alloc_recv = c_recv;
        alloc_expanded = c_exp;
    }

    at::Tensor recv_x = alloc({alloc_expanded, H}, s.fused ? at::kFloat8_e4m3fn : s.x.scalar_type(), dev);
    OptTensor recv_sf, sf_staging, sf_storage, recv_w;
    int64_t sf_cols = 0;
    const bool has_sf = s.fused || s.sf.has_value();
    if (has_sf) {
        sf_cols = s.fused ? (H + 127) / 128 : s.sf->size(1);
        const at::ScalarType sf_type = s.fused ? at::kFloat : s.sf->scalar_type();
        if (s.use_col_major_sf) {
            // scale rows go to a staging tensor, a tiled kernel of the library turns them into columns
            sf_staging = alloc({alloc_expanded, sf_cols}, sf_type, dev);
            sf_storage = alloc({sf_cols * alloc_expanded}, sf_type, dev);
            recv_sf = sf_storage->as_strided({alloc_expanded, sf_cols}, {1, alloc_expanded});
        } else {
            recv_sf = alloc({alloc_expanded, sf_cols}, sf_type, dev);
        }
    }
    if (s.topk_weights.has_value()) recv_w = alloc({alloc_expanded}, s.topk_weights->scalar_type(), dev);
    if (s.cached_mode) {
        meta = *s.cached_meta;
        if (meta.dim() != 2 || meta.size(0) != num_recv)
            throw EpPyError("Assertion exception (python_api.cpp): recv_src_metadata.size(0) == num_recv_tokens");
    } else if (!have_meta) {
        meta = empty_i32({alloc_recv, K + 2}, dev);
    }

    ep_dispatch_epilogue_args_t e{};
    e.x = s.a.x;
    e.sf = s.a.sf;
    e.topk_weights = s.a.topk_weights;
    e.psum_num_recv_tokens_per_rank = s.a.psum_num_recv_tokens_per_rank;
    e.psum_num_recv_tokens_per_expert = s.a.psum_num_recv_tokens_per_expert;
    e.recv_x = desc(recv_x);
    e.recv_sf = desc(recv_sf, !s.fused);
    if (recv_sf.has_value()) e.recv_sf_staging = desc(sf_staging, !s.fused);
    e.recv_topk_weights = desc(recv_w);
    e.recv_src_metadata = desc(meta);
    e.num_topk = K;
    e.num_max_tokens_per_rank = s.num_max_tokens_per_rank;
    e.num_experts = s.num_experts;
    e.expert_alignment = A;
    e.cached_mode = s.cached_mode ? 1 : 0;
    e.do_zero_padding = s.do_zero_padding ? 1 : 0;
    e.fused_fp8_quant = s.fused ? 1 : 0;
    // sizes still unknown on the host: the column stride is the row count the device computed
    e.recv_sf_layout = s.use_col_major_sf ? (counts_known ? EP_SF_LAYOUT_COL_MAJOR : EP_SF_LAYOUT_COL_MAJOR_COUNTED)
                                          : EP_SF_LAYOUT_ROW_MAJOR;
    e.stream = current_stream();
    e.dispatch_stamp = s.stamp;
    check(ep_dispatch_epilogue_launch(s.buf, &e));

    if (!counts_known) {
        wait_counts();
        counts_from_host = true;
        if (num_recv > alloc_recv || num_expanded > alloc_expanded)
            throw EpPyError("Assertion exception (python_api.cpp): received counts exceed this call's bound");
        recv_x = recv_x.narrow(0, 0, num_expanded);
        if (recv_sf.has_value() && s.use_col_major_sf)
            recv_sf = sf_storage->as_strided({(int64_t)num_expanded, sf_cols}, {1, (int64_t)num_expanded});
        else if (recv_sf.has_value())
            recv_sf = recv_sf->narrow(0, 0, num_expanded);
        if (recv_w.has_value()) recv_w = recv_w->narrow(0, 0, num_expanded);
        meta = meta.narrow(0, 0, num_recv);
    }

    py::object list_obj;
    if (s.cached_mode) {
        list_obj = s.cached_list;
    } else {
        py::list l;
        if (counts_from_host)
            for (int i = 0; i < El; ++i) l.append(per_expert[(size_t)i]);
        list_obj = std::move(l);
    }
    return py::make_tuple(recv_x, recv_sf, recv_w, num_recv, num_expanded, list_obj, s.psum_rank, s.psum_expert,
                          s.unaligned, meta, s.dst_slot, s.dst_gsge);
}

struct CombineState {
    ep_buffer_t* buf;
    at::Tensor x, src_metadata, combined_topk_idx, psum_rank;
    OptTensor topk_weights, bias_0, bias_1;
    ep_combine_args_t c{};
    int64_t num_combined_tokens, hidden, num_topk;
};

py::tuple run_combine_epilogue(CombineState& s) {
    at::Tensor combined_x = alloc({s.num_combined_tokens, s.hidden}, s.x.scalar_type(), s.x.device());
    OptTensor combined_w;
    if (s.topk_weights.has_value())
        combined_w = alloc({s.num_combined_tokens, s.num_topk}, s.topk_weights->scalar_type(), s.x.device());
    s.c.combined_x = desc(combined_x);
    s.c.combined_topk_weights = desc(combined_w);
    s.c.stream = current_stream();
    check(ep_combine_launch(s.buf, &s.c, 1));            // token side
    return py::make_tuple(combined_x, combined_w);
}

class NativeBuffer {
public:
    NativeBuffer(uintptr_t handle, int rank_idx, int num_ranks)
        : buf_((ep_buffer_t*)handle), rank_idx_(rank_idx), num_ranks_(num_ranks) {}

    void set_connected(bool c) { connected_ = c; }
    void set_exact_sync_sizes(bool e) { exact_sync_sizes_ = e; }
    void invalidate() { buf_ = nullptr; }

    // argument order of csrc/buffers/ep.hpp:89-112
    py::tuple dispatch(const at::Tensor& x, const OptTensor& sf, const at::Tensor& topk_idx, const OptTensor& topk_weights,
                       const OptTensor& cumulative_local_expert_recv_stats, const std::optional<int64_t>& cached_num_recv_tokens,
                       const std::optional<int64_t>& cached_num_expanded_tokens, const py::object& cached_list,
                       const OptTensor& cached_psum_rank, const OptTensor& cached_psum_expert, const OptTensor& cached_unaligned,
                       const OptTensor& cached_dst_slot, const OptTensor& cached_dst_gsge, const OptTensor& cached_meta,
                       int num_max_tokens_per_rank, int num_experts, int expert_alignment, int num_ai_cores,
                       const py::object& previous_event, bool async_with_compute_stream, bool allocate_on_comm_stream,
                       bool do_handle_copy, bool do_cpu_sync, bool do_expand, bool do_zero_padding, bool use_col_major_sf,
                       bool defer_epilogue, bool fused_fp8_quant) {
        (void)allocate_on_comm_stream;
        if (buf_ == nullptr) throw EpPyError("Assertion exception (python_api.cpp): not destroyed");
        if (!previous_event.is_none()) previous_event.attr("current_stream_wait")();     // the launches below are ordered behind it
        EP_PY_ASSERT(do_expand);
        EP_PY_ASSERT(not do_handle_copy);
        EP_PY_ASSERT(num_ai_cores > 0);
        const bool cached_mode = cached_num_recv_tokens.has_value();
        if (cached_mode) {
            if (!cached_num_expanded_tokens.has_value() || cached_list.is_none() || !cached_psum_rank.has_value() ||
                !cached_psum_expert.has_value() || !cached_unaligned.has_value() || !cached_dst_slot.has_value() ||
                !cached_dst_gsge.has_value() || !cached_meta.has_value())
                throw EpPyError("Assertion exception (python_api.cpp): cached handle field has a value");
        }
        if (x.dim() != 2 || topk_idx.dim() != 2)
            throw EpPyError("Assertion exception (python_api.cpp): x.dim() == 2 and topk_idx.dim() == 2");
        if (!x.is_cuda()) throw EpPyError("every tensor handed to the EP kernels must live on the GPU");
        auto st = std::make_shared<DispatchState>();
        DispatchState& s = *st;
        s.buf = buf_;
        s.num_ranks = num_ranks_;
        s.connected = connected_;
        s.exact_sync_sizes = exact_sync_sizes_;
        s.x = x;
        s.sf = sf;
        s.topk_idx = topk_idx;
        s.topk_weights = topk_weights;
        s.stats = cumulative_local_expert_recv_stats;
        s.num_tokens = (int)x.size(0);
        s.hidden = (int)x.size(1);
        s.num_topk = (int)topk_idx.size(1);
        s.num_local_experts = num_experts / num_ranks_;
        s.num_max_tokens_per_rank = num_max_tokens_per_rank;
        s.num_experts = num_experts;
        s.expert_alignment = expert_alignment;
        s.cached_mode = cached_mode;
        s.do_cpu_sync = do_cpu_sync;
        s.do_zero_padding = do_zero_padding;
        s.use_col_major_sf = use_col_major_sf;
        s.fused = fused_fp8_quant;
        const at::Device dev = x.device();
        if (cached_mode) {
            s.psum_rank = *cached_psum_rank;
            s.psum_expert = *cached_psum_expert;
            s.unaligned = *cached_unaligned;
            s.dst_slot = *cached_dst_slot;
            s.dst_gsge = *cached_dst_gsge;
            s.cached_meta = cached_meta;
            s.cached_list = cached_list;
            s.cached_num_recv = *cached_num_recv_tokens;
            s.cached_num_expanded = *cached_num_expanded_tokens;
        } else {
            // the three count vectors share one allocation (each starts on a multiple of 64 bytes)
            const int64_t r16 = (num_ranks_ + 15) / 16 * 16, e16 = (s.num_local_experts + 15) / 16 * 16;
            at::Tensor counts = empty_i32({r16 + 2 * e16}, dev);
            s.psum_rank = counts.narrow(0, 0, num_ranks_);
            s.psum_expert = counts.narrow(0, r16, s.num_local_experts);
            s.unaligned = counts.narrow(0, r16 + e16, s.num_local_experts);
            s.dst_slot = empty_i32({s.num_tokens, s.num_topk}, dev);
            s.dst_gsge = empty_i32({s.num_tokens, s.num_topk}, dev);
        }
        ep_dispatch_args_t& a = s.a;
        a.x = desc(x);
        a.sf = desc(sf, true);
        a.topk_idx = desc(topk_idx);
        a.topk_weights = desc(topk_weights);
        a.cumulative_local_expert_recv_stats = desc(cumulative_local_expert_recv_stats);
        a.psum_num_recv_tokens_per_rank = desc(s.psum_rank);
        a.psum_num_recv_tokens_per_expert = desc(s.psum_expert);
        a.num_unaligned_recv_tokens_per_expert = desc(s.unaligned);
        a.dst_buffer_slot_idx = desc(s.dst_slot);
        a.dst_gsge_idx = desc(s.dst_gsge);
        a.num_max_tokens_per_rank = num_max_tokens_per_rank;
        a.num_experts = num_experts;
        a.expert_alignment = expert_alignment;
        a.cached_mode = cached_mode ? 1 : 0;
        a.do_cpu_sync = do_cpu_sync ? 1 : 0;
        a.fused_fp8_quant = fused_fp8_quant ? 1 : 0;
        a.stream = current_stream();
        check(ep_dispatch_launch(buf_, &a));
        // the epilogue below belongs to this launch: the library refuses it once a later dispatch has taken over
        // the buffer's workspace
        s.stamp = ep_dispatch_stamp(buf_);

        if (defer_epilogue) {
            if (!async_with_compute_stream) throw EpPyError("Assertion exception (python_api.cpp): async_with_compute_stream");
            py::object ev = new_event();
            py::cpp_function epilogue([st]() { return run_dispatch_epilogue(*st); });
            return py::make_tuple(py::none(), ev, epilogue);
        }
        py::tuple result = run_dispatch_epilogue(s);
        py::object ev = async_with_compute_stream ? new_event() : py::object(py::none());
        return py::make_tuple(result, ev, py::none());
    }

    // argument order of csrc/buffers/ep.hpp:412-425
    py::tuple combine(const at::Tensor& x, const OptTensor& topk_weights, const OptTensor& bias_0, const OptTensor& bias_1,
                      const at::Tensor& src_metadata, const at::Tensor& combined_topk_idx,
                      const at::Tensor& psum_num_recv_tokens_per_rank, int num_experts, int num_max_tokens_per_rank, int num_sms,
                      const py::object& previous_event, bool async_with_compute_stream, bool allocate_on_comm_stream,
                      bool defer_epilogue, bool apply_weights) {
        (void)allocate_on_comm_stream;
        if (buf_ == nullptr) throw EpPyError("Assertion exception (python_api.cpp): not destroyed");
        if (!previous_event.is_none()) previous_event.attr("current_stream_wait")();
        EP_PY_ASSERT(num_sms > 0);
        if (x.dim() != 2 || combined_topk_idx.dim() != 2)
            throw EpPyError("Assertion exception (python_api.cpp): x.dim() == 2 and combined_topk_idx.dim() == 2");
        if (!x.is_cuda()) throw EpPyError("every tensor handed to the EP kernels must live on the GPU");
        auto st = std::make_shared<CombineState>();
        CombineState& s = *st;
        s.buf = buf_;
        s.x = x;
        s.topk_weights = topk_weights;
        s.bias_0 = bias_0;
        s.bias_1 = bias_1;
        s.src_metadata = src_metadata;
        s.combined_topk_idx = combined_topk_idx;
        s.psum_rank = psum_num_recv_tokens_per_rank;
        s.hidden = x.size(1);
        s.num_combined_tokens = combined_topk_idx.size(0);
        s.num_topk = combined_topk_idx.size(1);
        ep_combine_args_t& c = s.c;
        c.x = desc(x);
        c.topk_weights = desc(topk_weights);
        c.bias_0 = desc(bias_0);
        c.bias_1 = desc(bias_1);
        c.src_metadata = desc(src_metadata);
        c.combined_topk_idx = desc(combined_topk_idx);
        c.psum_num_recv_tokens_per_rank = desc(psum_num_recv_tokens_per_rank);
        c.num_experts = num_experts;
        c.num_max_tokens_per_rank = num_max_tokens_per_rank;
        c.apply_weights = apply_weights ? 1 : 0;
        c.stream = current_stream();
        // owner side; with one partition it only validates, which the token side below repeats: then it is called
        // only where the token side is deferred, so that a bad argument still fails at the call
        if (num_ranks_ > 1 || defer_epilogue) check(ep_combine_launch(buf_, &c, 0));

        if (defer_epilogue) {
            if (!async_with_compute_stream) throw EpPyError("Assertion exception (python_api.cpp): async_with_compute_stream");
            py::object ev = new_event();
            py::cpp_function epilogue([st]() { return run_combine_epilogue(*st); });
            return py::make_tuple(py::none(), ev, epilogue);
        }
        py::tuple result = run_combine_epilogue(s);
        py::object ev = async_with_compute_stream ? new_event() : py::object(py::none());
        return py::make_tuple(result, ev, py::none());
    }

private:
    ep_buffer_t* buf_;
    int rank_idx_, num_ranks_;
    bool connected_ = false;
    bool exact_sync_sizes_ = false;
};

}  // namespace

PYBIND11_MODULE(_native, m) {
    m.doc() = "compiled binding of the EP dispatch/combine calls over the C ABI of libdeep_ep_hip.so";
    py::register_exception<EpPyError>(m, "EPException", PyExc_RuntimeError);
    py::class_<NativeBuffer>(m, "Buffer")
        .def(py::init<uintptr_t, int, int>())
        .def("set_connected", &NativeBuffer::set_connected)
        .def("set_exact_sync_sizes", &NativeBuffer::set_exact_sync_sizes)
        .def("invalidate", &NativeBuffer::invalidate)
        .def("dispatch", &NativeBuffer::dispatch, py::arg("x"), py::arg("sf"), py::arg("topk_idx"), py::arg("topk_weights"),
             py::arg("cumulative_local_expert_recv_stats"), py::arg("cached_num_recv_tokens"),
             py::arg("cached_num_expanded_tokens"), py::arg("cached_num_recv_tokens_per_expert_list"),
             py::arg("cached_psum_num_recv_tokens_per_rank"), py::arg("cached_psum_num_recv_tokens_per_expert"),
             py::arg("cached_num_unaligned_recv_tokens_per_expert"), py::arg("cached_dst_buffer_slot_idx"),
             py::arg("cached_dst_gsge_idx"), py::arg("cached_recv_src_metadata"), py::arg("num_max_tokens_per_rank"),
             py::arg("num_experts"), py::arg("expert_alignment"), py::arg("num_ai_cores"), py::arg("previous_event"),
             py::arg("async_with_compute_stream"), py::arg("allocate_on_comm_stream"), py::arg("do_handle_copy"),
             py::arg("do_cpu_sync"), py::arg("do_expand"), py::arg("do_zero_padding"), py::arg("use_col_major_sf"),
             py::arg("defer_epilogue"), py::arg("fused_fp8_quant") = false)
        .def("combine", &NativeBuffer::combine, py::arg("x"), py::arg("topk_weights"), py::arg("bias_0"), py::arg("bias_1"),
             py::arg("src_metadata"), py::arg("combined_topk_idx"), py::arg("psum_num_recv_tokens_per_rank"),
             py::arg("num_experts"), py::arg("num_max_tokens_per_rank"), py::arg("num_sms"), py::arg("previous_event"),
             py::arg("async_with_compute_stream"), py::arg("allocate_on_comm_stream"), py::arg("defer_epilogue"),
             py::arg("apply_weights") = false);
}
