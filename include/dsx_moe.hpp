// dsx_moe.hpp -- C++ host side of the deepstrix MoE feed-forward path, above the C ABI of
// libdsx_moe.so (dsx_moe.h).
//
// The reference's host side is Rust: typed launch wrappers over caller-owned device buffers that
// check every length before anything is launched and hand back a Result.  This header is the
// same layer in C++17, name for name, so that a test or an engine written against the reference
// reads the same here:
//
//   reference (paths relative to the reference tree)                      here
//   crates/v4flash-hip/src/error.rs:10-78      HipError -> eyre::Report    dsx::Status
//   crates/v4flash-hip/src/stream.rs           Stream                      dsx::Stream
//   crates/v4flash-hip/src/buffer.rs:19-35     DeviceBuffer<T>             dsx::DeviceBuffer<T>
//   crates/v4flash-hip/src/buffer.rs:106-125   slice_view (non-owning)     dsx::DeviceSlice<T>
//   crates/v4flash-kernels/src/router_topk.rs:245-364   RouterTopk         dsx::RouterTopk
//   crates/v4flash-kernels/src/q8_k.rs:33-104           Q8KQuantize        dsx::Q8KQuantize
//   crates/v4flash-kernels/src/moe_group_builder.rs:72-260  MoeGroupBuilder  dsx::MoeGroupBuilder
//   crates/v4flash-kernels/src/het/dispatch.rs:26-185,450-454,534-620      dsx::dispatch::*
//   crates/v4flash-kernels/src/q2_k.rs:454-500  launch_reduce_partials     dsx::dispatch::reduce_partials
//   crates/v4flash-kernels/src/het/remote_experts.rs:7266-7325,7432-7443  MoeExecutor  dsx::MoeExecutor
//
// Conventions kept from the reference: nothing throws and nothing panics across a call -- every
// operation returns a Status ([[nodiscard]]); lengths and divisibility are checked on the host
// before the C entry point is called (crates/v4flash-kernels/src/mxfp4.rs:416-424), and the
// C entry point checks again; buffers are owned by the caller; launches are asynchronous on the
// given stream and safe inside a HIP graph capture.  The header needs the HIP runtime only for
// memory and streams.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "dsx_moe.h"

namespace dsx {

// ---- errors --------------------------------------------------------------------------------
// code: 0 ok, > 0 a hipError_t, < 0 a DSX_ERR_* argument error (raised before any launch).
struct [[nodiscard]] Status {
    int code = 0;
    std::string message;
    bool ok() const { return code == 0; }
    explicit operator bool() const { return ok(); }
    static Status success() { return {}; }
    static Status invalid(std::string msg) { return {DSX_ERR_INVALID_ARG, std::move(msg)}; }
    static Status shape(std::string msg) { return {DSX_ERR_SHAPE, std::move(msg)}; }
    // wraps the return value of a C entry point; context names the wrapper, like
    // HipError::context (crates/v4flash-hip/src/error.rs:10-30)
    static Status from_c(int rc, const char *context) {
        if (rc == 0) return {};
        const char *m = dsx_last_error();
        return {rc, std::string(context) + ": " + (m != nullptr && *m ? m : "error")};
    }
    static Status from_hip(hipError_t e, const char *context) {
        if (e == hipSuccess) return {};
        return {(int)e, std::string(context) + ": " + hipGetErrorName(e) + ": " + hipGetErrorString(e)};
    }
};

#define DSX_TRY(expr)                          \
    do {                                       \
        ::dsx::Status dsx_try_st_ = (expr);    \
        if (!dsx_try_st_.ok()) return dsx_try_st_; \
    } while (0)

namespace detail {
inline Status need(const char *what, size_t have, size_t want) {
    if (have >= want) return {};
    return Status::invalid(std::string(what) + " len: have " + std::to_string(have) + ", need " +
                           std::to_string(want));
}
}  // namespace detail

// ---- stream --------------------------------------------------------------------------------
class Stream {
   public:
    Stream() = default;
    Stream(const Stream &) = delete;
    Stream &operator=(const Stream &) = delete;
    Stream(Stream &&o) noexcept : s_(o.s_), owned_(o.owned_) { o.s_ = nullptr; o.owned_ = false; }
    ~Stream() {
        if (owned_ && s_ != nullptr) (void)hipStreamDestroy(s_);
    }
    // a new stream at the default priority, ordered with the null stream (the synchronous
    // copies and fills of DeviceBuffer run there)
    static Status create(Stream &out) {
        hipStream_t s = nullptr;
        DSX_TRY(Status::from_hip(hipStreamCreate(&s), "Stream::create"));
        out = Stream(s, true);
        return {};
    }
    // a stream somebody else owns (null = the default stream)
    static Stream borrowed(hipStream_t s) { return Stream(s, false); }
    Stream &operator=(Stream &&o) noexcept {
        if (this != &o) {
            if (owned_ && s_ != nullptr) (void)hipStreamDestroy(s_);
            s_ = o.s_; owned_ = o.owned_; o.s_ = nullptr; o.owned_ = false;
        }
        return *this;
    }
    Status synchronize() const { return Status::from_hip(hipStreamSynchronize(s_), "Stream::synchronize"); }
    hipStream_t raw() const { return s_; }

   private:
    Stream(hipStream_t s, bool owned) : s_(s), owned_(owned) {}
    hipStream_t s_ = nullptr;
    bool owned_ = false;
};

// ---- device memory ---------------------------------------------------------------------------
// Non-owning view of device memory: what slice_view hands out, and what every wrapper takes, so
// that sub-ranges of one allocation can be passed like whole buffers.
template <typename T>
class DeviceSlice {
   public:
    DeviceSlice() = default;
    DeviceSlice(T *ptr, size_t len) : ptr_(ptr), len_(len) {}
    template <typename U, typename = std::enable_if_t<std::is_same<const U, T>::value>>
    DeviceSlice(const DeviceSlice<U> &o) : ptr_(o.ptr()), len_(o.len()) {}
    T *ptr() const { return ptr_; }
    size_t len() const { return len_; }
    size_t byte_len() const { return len_ * sizeof(T); }
    bool empty() const { return len_ == 0; }
    // elements [offset, offset + len); an out-of-range request yields an empty slice
    DeviceSlice slice_view(size_t offset, size_t len) const {
        if (offset > len_ || len > len_ - offset) return {};
        return {ptr_ + offset, len};
    }

   private:
    T *ptr_ = nullptr;
    size_t len_ = 0;
};

template <typename T>
class DeviceBuffer {
   public:
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept : ptr_(o.ptr_), len_(o.len_) { o.ptr_ = nullptr; o.len_ = 0; }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept {
        if (this != &o) {
            release();
            ptr_ = o.ptr_; len_ = o.len_; o.ptr_ = nullptr; o.len_ = 0;
        }
        return *this;
    }
    ~DeviceBuffer() { release(); }

    static Status alloc(DeviceBuffer &out, size_t len) {
        void *p = nullptr;
        if (len != 0) DSX_TRY(Status::from_hip(hipMalloc(&p, len * sizeof(T)), "DeviceBuffer::alloc"));
        out.release();
        out.ptr_ = (T *)p;
        out.len_ = len;
        return {};
    }
    static Status zeroed(DeviceBuffer &out, size_t len) {
        DSX_TRY(alloc(out, len));
        if (len == 0) return {};
        DSX_TRY(Status::from_hip(hipMemset(out.ptr_, 0, len * sizeof(T)), "DeviceBuffer::zeroed"));
        // a fill may return before it has run; set-up code wants it done
        return Status::from_hip(hipDeviceSynchronize(), "DeviceBuffer::zeroed");
    }
    static Status from_host(DeviceBuffer &out, const T *host, size_t len) {
        DSX_TRY(alloc(out, len));
        return out.copy_from_host(host, len);
    }
    static Status from_host(DeviceBuffer &out, const std::vector<T> &host) {
        return from_host(out, host.data(), host.size());
    }
    // synchronous copies (set-up and checking; not for the timed path)
    Status copy_from_host(const T *host, size_t len) {
        DSX_TRY(detail::need("copy_from_host dst", len_, len));
        if (len == 0) return {};
        return Status::from_hip(hipMemcpy(ptr_, host, len * sizeof(T), hipMemcpyHostToDevice),
                                "DeviceBuffer::copy_from_host");
    }
    Status copy_to_host(std::vector<T> &host) const {
        host.resize(len_);
        if (len_ == 0) return {};
        return Status::from_hip(hipMemcpy(host.data(), ptr_, len_ * sizeof(T), hipMemcpyDeviceToHost),
                                "DeviceBuffer::copy_to_host");
    }

    T *ptr() const { return ptr_; }
    size_t len() const { return len_; }
    size_t byte_len() const { return len_ * sizeof(T); }
    DeviceSlice<T> view() { return {ptr_, len_}; }
    DeviceSlice<const T> view() const { return {ptr_, len_}; }
    DeviceSlice<T> slice_view(size_t offset, size_t len) { return view().slice_view(offset, len); }
    DeviceSlice<const T> slice_view(size_t offset, size_t len) const { return view().slice_view(offset, len); }
    operator DeviceSlice<T>() { return view(); }
    operator DeviceSlice<const T>() const { return view(); }

   private:
    void release() {
        if (ptr_ != nullptr) (void)hipFree(ptr_);
        ptr_ = nullptr;
        len_ = 0;
    }
    T *ptr_ = nullptr;
    size_t len_ = 0;
};

template <typename T> using In = DeviceSlice<const T>;
template <typename T> using Out = DeviceSlice<T>;

// ggml type ids as the reference's GgufType carries them (crates/v4flash-core/src/gguf.rs:569-592)
enum class GgufType : int { Q8_0 = DSX_FMT_Q8_0, MXFP4 = DSX_FMT_MXFP4 };
enum class RouterMode : uint32_t {
    SqrtSoftplus = DSX_ROUTER_SQRT_SOFTPLUS,
    Sigmoid = DSX_ROUTER_SIGMOID,
    Softmax = DSX_ROUTER_SOFTMAX,
};

// Bytes of one activation row of k elements in front of a matrix of format dt: Q8_K blocks for
// MXFP4 (292 per 256), [k int8][k/32 f32] for Q8_0.
inline size_t act_row_bytes(GgufType dt, uint32_t k) {
    return dt == GgufType::MXFP4 ? (size_t)(k / 256u) * DSX_Q8K_BLOCK_BYTES : (size_t)k + k / 8u;
}
// Bytes of one weight row of k elements (crates/v4flash-kernels/src/weight_contract.rs:146-158).
inline size_t weight_row_bytes(GgufType dt, uint32_t k) {
    return dt == GgufType::MXFP4 ? (size_t)(k / 256u) * DSX_MXFP4_SUPER_BYTES : (size_t)(k / 32u) * 34u;
}

// Every wrapper of the reference is built with for_arch(arch) and refuses an architecture it has
// no code object for; here there is one architecture and the check is the library's.
inline Status for_arch(const std::string &arch) {
    if (arch.rfind("gfx950", 0) != 0) return {DSX_ERR_DEVICE, "no kernels for " + arch + " (gfx950 only)"};
    return Status::from_c(dsx_init(), "for_arch");
}

// ---- RouterTopk (crates/v4flash-kernels/src/router_topk.rs:245-364) -------------------------
struct RouterTopk {
    static Status launch_batched_ex(const Stream &s, Out<int32_t> selected, Out<float> weights,
                                    In<float> logits, In<float> bias /* may be empty */,
                                    uint32_t n_expert, uint32_t n_used, float scale, float eps, uint32_t b,
                                    RouterMode mode, uint32_t n_group = 1, uint32_t topk_group = 1) {
        DSX_TRY(detail::need("router_topk logits", logits.len(), (size_t)b * n_expert));
        DSX_TRY(detail::need("router_topk selected", selected.len(), (size_t)b * n_used));
        DSX_TRY(detail::need("router_topk weights", weights.len(), (size_t)b * n_used));
        if (!bias.empty()) DSX_TRY(detail::need("router_topk bias", bias.len(), n_expert));
        return Status::from_c(
            dsx_router_topk(s.raw(), selected.ptr(), weights.ptr(), logits.ptr(), bias.ptr(), n_expert, n_used,
                            scale, eps, b, (uint32_t)mode, n_group, topk_group),
            "RouterTopk::launch_batched_ex");
    }
};

// ---- Q8KQuantize (crates/v4flash-kernels/src/q8_k.rs:33-104) --------------------------------
struct Q8KQuantize {
    static Status launch(const Stream &s, Out<uint8_t> out, In<float> x, uint32_t n_blocks) {
        DSX_TRY(detail::need("q8_k_quantize x", x.len(), (size_t)n_blocks * 256u));
        DSX_TRY(detail::need("q8_k_quantize out bytes", out.byte_len(), (size_t)n_blocks * DSX_Q8K_BLOCK_BYTES));
        return Status::from_c(dsx_q8k_quantize(s.raw(), out.ptr(), x.ptr(), n_blocks), "Q8KQuantize::launch");
    }
};

// Activation rows in front of a matrix of format dt (Q8_K for MXFP4, per-32 int8 for Q8_0):
// what the reference's executor does with q8k.launch / q8.quantize_input before each product.
inline Status quantize_rows(const Stream &s, GgufType dt, Out<uint8_t> out, In<float> x, uint32_t rows,
                            uint32_t k) {
    DSX_TRY(detail::need("quantize_rows x", x.len(), (size_t)rows * k));
    DSX_TRY(detail::need("quantize_rows out bytes", out.byte_len(), (size_t)rows * act_row_bytes(dt, k)));
    if (dt == GgufType::MXFP4) {
        if (k % 256u != 0) return Status::shape("quantize_rows: k must be a multiple of 256 for Q8_K");
        return Status::from_c(dsx_q8k_quantize(s.raw(), out.ptr(), x.ptr(), rows * (k / 256u)), "quantize_rows");
    }
    return Status::from_c(dsx_q8_0_quantize_rows(s.raw(), out.ptr(), x.ptr(), rows, k), "quantize_rows");
}

// ---- MoeGroupBuilder (crates/v4flash-kernels/src/moe_group_builder.rs:72-260) ----------------
// The token -> expert inversion and its work items.  One object holds the five tables, sized
// once for the largest batch like the executor's (remote_experts.rs:7266-7325).
struct MoeGroups {
    DeviceBuffer<int32_t> group_count, group_offset, expert_members, work_items, n_work_items;
    uint32_t n_expert = 0, max_members = 0;
    static Status alloc(MoeGroups &g, uint32_t n_expert, uint32_t max_members) {
        DSX_TRY(DeviceBuffer<int32_t>::zeroed(g.group_count, n_expert));
        DSX_TRY(DeviceBuffer<int32_t>::zeroed(g.group_offset, (size_t)n_expert + 1));
        DSX_TRY(DeviceBuffer<int32_t>::zeroed(g.expert_members, max_members));
        DSX_TRY(DeviceBuffer<int32_t>::zeroed(g.work_items, (size_t)max_members + n_expert));
        DSX_TRY(DeviceBuffer<int32_t>::zeroed(g.n_work_items, 1));
        g.n_expert = n_expert;
        g.max_members = max_members;
        return {};
    }
};

struct MoeGroupBuilder {
    // launch + launch_work_items in one call; selected entries outside [0, n_expert) are skipped,
    // which is how a het-split side (dispatch::hetsplit_select) leaves out the other side's picks.
    static Status launch(const Stream &s, MoeGroups &g, In<int32_t> selected, uint32_t b, uint32_t n_used,
                         uint32_t n_expert, uint32_t chunk) {
        DSX_TRY(detail::need("group_build selected", selected.len(), (size_t)b * n_used));
        DSX_TRY(detail::need("group_build group_count", g.group_count.len(), n_expert));
        DSX_TRY(detail::need("group_build group_offset", g.group_offset.len(), (size_t)n_expert + 1));
        DSX_TRY(detail::need("group_build expert_members", g.expert_members.len(), (size_t)b * n_used));
        DSX_TRY(detail::need("group_build work_items", g.work_items.len(), (size_t)b * n_used + n_expert));
        DSX_TRY(detail::need("group_build n_work_items", g.n_work_items.len(), 1));
        return Status::from_c(
            dsx_moe_group_build(s.raw(), g.group_count.ptr(), g.group_offset.ptr(), g.expert_members.ptr(),
                                g.work_items.ptr(), g.n_work_items.ptr(), selected.ptr(), b, n_used, n_expert,
                                chunk),
            "MoeGroupBuilder::launch");
    }
};

// ---- HcPost (crates/v4flash-kernels/src/head.rs:269-500) ---------------------------------------
// The hyper-connection combine behind the FFN; the names are the reference wrapper's.
struct HcPost {
    // launch / launch_batched (head.rs:286-345): separate post [b, n_hc] and comb [b, n_hc, n_hc]
    static Status launch_batched(const Stream &s, Out<float> out_hc, In<float> block_out, In<float> residual_hc,
                                 In<float> post, In<float> comb, uint32_t n_embd, uint32_t n_hc, uint32_t batch) {
        DSX_TRY(detail::need("hc_post out_hc", out_hc.len(), (size_t)batch * n_hc * n_embd));
        DSX_TRY(detail::need("hc_post block_out", block_out.len(), (size_t)batch * n_embd));
        DSX_TRY(detail::need("hc_post residual_hc", residual_hc.len(), (size_t)batch * n_hc * n_embd));
        DSX_TRY(detail::need("hc_post post", post.len(), (size_t)batch * n_hc));
        DSX_TRY(detail::need("hc_post comb", comb.len(), (size_t)batch * n_hc * n_hc));
        const dsx_hc_post_desc d{out_hc.ptr(), residual_hc.ptr(), post.ptr(), comb.ptr(), n_hc, n_hc, n_hc * n_hc};
        return Status::from_c(dsx_hc_post(s.raw(), &d, block_out.ptr(), nullptr, nullptr, n_embd, batch),
                              "HcPost::launch_batched");
    }
    static Status launch(const Stream &s, Out<float> out_hc, In<float> block_out, In<float> residual_hc,
                         In<float> post, In<float> comb, uint32_t n_embd, uint32_t n_hc) {
        return launch_batched(s, out_hc, block_out, residual_hc, post, comb, n_embd, n_hc, 1u);
    }
    // launch_from_split_batched / _add / _add2 (head.rs:347-455): post and comb inside the packed
    // rows split[batch, n_w + n_hc + n_hc * n_hc]; add1 / add2 may be empty (add2 only with add1):
    // block = (block_out + add1) + add2
    static Status launch_from_split_batched_add2(const Stream &s, Out<float> out_hc, In<float> block_out,
                                                 In<float> add1, In<float> add2, In<float> residual_hc,
                                                 In<float> split, uint32_t n_w, uint32_t n_embd, uint32_t n_hc,
                                                 uint32_t batch) {
        const uint32_t stride = n_w + n_hc + n_hc * n_hc;
        DSX_TRY(detail::need("hc_post out_hc", out_hc.len(), (size_t)batch * n_hc * n_embd));
        DSX_TRY(detail::need("hc_post block_out", block_out.len(), (size_t)batch * n_embd));
        DSX_TRY(detail::need("hc_post residual_hc", residual_hc.len(), (size_t)batch * n_hc * n_embd));
        DSX_TRY(detail::need("hc_post split", split.len(), (size_t)batch * stride));
        if (!add1.empty()) DSX_TRY(detail::need("hc_post add1", add1.len(), (size_t)batch * n_embd));
        if (!add2.empty()) DSX_TRY(detail::need("hc_post add2", add2.len(), (size_t)batch * n_embd));
        const dsx_hc_post_desc d{out_hc.ptr(), residual_hc.ptr(), split.ptr() + n_w, split.ptr() + n_w + n_hc,
                                 n_hc, stride, stride};
        return Status::from_c(dsx_hc_post(s.raw(), &d, block_out.ptr(), add1.ptr(), add2.ptr(), n_embd, batch),
                              "HcPost::launch_from_split_batched");
    }
    static Status launch_from_split_batched(const Stream &s, Out<float> out_hc, In<float> block_out,
                                            In<float> residual_hc, In<float> split, uint32_t n_w, uint32_t n_embd,
                                            uint32_t n_hc, uint32_t batch) {
        return launch_from_split_batched_add2(s, out_hc, block_out, In<float>(), In<float>(), residual_hc, split,
                                              n_w, n_embd, n_hc, batch);
    }
};

// ---- het::dispatch (crates/v4flash-kernels/src/het/dispatch.rs) ------------------------------
namespace dispatch {

// dispatch.rs:450-454
inline uint32_t moe_wi_upper_bound(size_t members, uint32_t groups, uint32_t chunk, size_t cap) {
    const size_t m = members;
    const size_t g = m < groups ? m : (size_t)groups;
    const size_t c = chunk != 0 ? chunk : 1;
    size_t v = g + (m + c - 1) / c;
    v = v < m ? v : m;
    v = v < cap ? v : cap;
    return (uint32_t)v;
}

// dispatch.rs:26-66 -- one token: mid[slot, row] = swiglu(gate_e[row] . xq, up_e[row] . xq) * ew[slot]
inline Status moe_gate_up_batch(GgufType dt, const Stream &s, Out<float> mid, In<uint8_t> gate, In<uint8_t> up,
                                In<uint8_t> xq, In<float> ew, In<int32_t> selected, uint64_t gbpe,
                                uint64_t ubpe, uint32_t n_used, float clamp, uint32_t n_rows,
                                uint32_t n_blocks) {
    DSX_TRY(detail::need("moe_gate_up_batch mid", mid.len(), (size_t)n_used * n_rows));
    DSX_TRY(detail::need("moe_gate_up_batch ew", ew.len(), n_used));
    DSX_TRY(detail::need("moe_gate_up_batch selected", selected.len(), n_used));
    const uint32_t k = dt == GgufType::MXFP4 ? n_blocks * 256u : n_blocks * 32u;
    DSX_TRY(detail::need("moe_gate_up_batch xq bytes", xq.byte_len(), act_row_bytes(dt, k)));
    if (gbpe < (uint64_t)n_rows * weight_row_bytes(dt, k) || ubpe < (uint64_t)n_rows * weight_row_bytes(dt, k))
        return Status::shape("moe_gate_up_batch: bytes per expert smaller than n_rows rows");
    DSX_TRY(detail::need("moe_gate_up_batch gate bytes", gate.byte_len(), gbpe));
    DSX_TRY(detail::need("moe_gate_up_batch up bytes", up.byte_len(), ubpe));
    return Status::from_c(dsx_moe_gate_up_batch(s.raw(), (int)dt, mid.ptr(), gate.ptr(), up.ptr(), xq.ptr(),
                                                ew.ptr(), selected.ptr(), gbpe, ubpe, n_used, clamp, n_rows,
                                                n_blocks),
                          "dispatch::moe_gate_up_batch");
}

// dispatch.rs:121-150 -- one token: out[row] = sum over slots, in slot order, of down_e[row] . midq[slot]
inline Status moe_down_batched(GgufType dt, const Stream &s, Out<float> out, In<uint8_t> down, In<uint8_t> midq,
                               In<int32_t> selected, uint64_t dbpe, uint32_t xq_slot_stride, uint32_t n_used,
                               uint32_t n_rows, uint32_t n_blocks_in) {
    DSX_TRY(detail::need("moe_down_batched out", out.len(), n_rows));
    DSX_TRY(detail::need("moe_down_batched selected", selected.len(), n_used));
    DSX_TRY(detail::need("moe_down_batched midq bytes", midq.byte_len(), (size_t)n_used * xq_slot_stride));
    DSX_TRY(detail::need("moe_down_batched down bytes", down.byte_len(), dbpe));
    return Status::from_c(dsx_moe_down_batched(s.raw(), (int)dt, out.ptr(), down.ptr(), midq.ptr(),
                                               selected.ptr(), dbpe, xq_slot_stride, n_used, n_rows,
                                               n_blocks_in),
                          "dispatch::moe_down_batched");
}

// dispatch.rs:534-570 -- by expert: mid[b, n_used, n_rows]
inline Status moe_gate_up_chunked_rows(GgufType dt, const Stream &s, Out<float> mid, In<uint8_t> gate,
                                       In<uint8_t> up, In<uint8_t> xq, In<float> ew, const MoeGroups &g,
                                       uint32_t max_work_items, uint64_t gbpe, uint64_t ubpe, uint32_t n_used,
                                       uint32_t chunk, float clamp, uint32_t n_rows, uint32_t n_blocks,
                                       uint32_t rows) {
    const uint32_t k = dt == GgufType::MXFP4 ? n_blocks * 256u : n_blocks * 32u;
    DSX_TRY(detail::need("moe_gate_up_chunked_rows mid", mid.len(), (size_t)rows * n_used * n_rows));
    DSX_TRY(detail::need("moe_gate_up_chunked_rows ew", ew.len(), (size_t)rows * n_used));
    DSX_TRY(detail::need("moe_gate_up_chunked_rows xq bytes", xq.byte_len(), (size_t)rows * act_row_bytes(dt, k)));
    DSX_TRY(detail::need("moe_gate_up_chunked_rows work_items", g.work_items.len(), max_work_items));
    DSX_TRY(detail::need("moe_gate_up_chunked_rows gate bytes", gate.byte_len(), gbpe));
    DSX_TRY(detail::need("moe_gate_up_chunked_rows up bytes", up.byte_len(), ubpe));
    return Status::from_c(
        dsx_moe_gate_up_chunked_rows(s.raw(), (int)dt, mid.ptr(), gate.ptr(), up.ptr(), xq.ptr(), ew.ptr(),
                                     g.group_count.ptr(), g.group_offset.ptr(), g.expert_members.ptr(),
                                     g.work_items.ptr(), g.n_work_items.ptr(), max_work_items, gbpe, ubpe,
                                     n_used, chunk, clamp, n_rows, n_blocks),
        "dispatch::moe_gate_up_chunked_rows");
}

// dispatch.rs:580-620 -- by expert: partials[(t * n_used + slot) * n_rows + row]
inline Status moe_down_mxfp4(GgufType dt, const Stream &s, Out<float> partials, In<uint8_t> down,
                             In<uint8_t> midq, const MoeGroups &g, uint32_t max_work_items, uint64_t dbpe,
                             uint32_t xq_slot_stride, uint32_t n_used, uint32_t chunk, uint32_t n_rows,
                             uint32_t n_blocks_in, uint32_t rows) {
    DSX_TRY(detail::need("moe_down partials", partials.len(), (size_t)rows * n_used * n_rows));
    DSX_TRY(detail::need("moe_down midq bytes", midq.byte_len(), (size_t)rows * n_used * xq_slot_stride));
    DSX_TRY(detail::need("moe_down work_items", g.work_items.len(), max_work_items));
    DSX_TRY(detail::need("moe_down down bytes", down.byte_len(), dbpe));
    return Status::from_c(
        dsx_moe_down_by_expert(s.raw(), (int)dt, partials.ptr(), down.ptr(), midq.ptr(), g.group_count.ptr(),
                               g.group_offset.ptr(), g.expert_members.ptr(), g.work_items.ptr(),
                               g.n_work_items.ptr(), max_work_items, dbpe, xq_slot_stride, n_used, chunk,
                               n_rows, n_blocks_in),
        "dispatch::moe_down_mxfp4");
}

// Q2KAccumulateMatvec::launch_reduce_partials (crates/v4flash-kernels/src/q2_k.rs:454-500):
// out[t, row] = sum over slots in slot order; slots whose pick is < 0 are skipped.
inline Status reduce_partials(const Stream &s, Out<float> out, In<float> partials, In<int32_t> selected,
                              uint32_t n_used, uint32_t n_rows, uint32_t b) {
    DSX_TRY(detail::need("reduce_partials out", out.len(), (size_t)b * n_rows));
    DSX_TRY(detail::need("reduce_partials partials", partials.len(), (size_t)b * n_used * n_rows));
    if (!selected.empty()) DSX_TRY(detail::need("reduce_partials selected", selected.len(), (size_t)b * n_used));
    return Status::from_c(
        dsx_moe_reduce_partials(s.raw(), out.ptr(), partials.ptr(), selected.ptr(), n_used, n_rows, b),
        "dispatch::reduce_partials");
}

// The ownership rule of the *_hetsplit variants (dispatch.rs:68-119,152-185), applied once:
// selected_side is what the side passes as `selected` to every call above.
inline Status hetsplit_select(const Stream &s, Out<int32_t> selected_side, In<int32_t> selected,
                              In<int32_t> remap, uint32_t mode, uint32_t cap, uint32_t n_used, uint32_t b) {
    DSX_TRY(detail::need("hetsplit_select selected", selected.len(), (size_t)b * n_used));
    DSX_TRY(detail::need("hetsplit_select selected_side", selected_side.len(), (size_t)b * n_used));
    return Status::from_c(dsx_moe_hetsplit_select(s.raw(), selected_side.ptr(), selected.ptr(), remap.ptr(), mode,
                                                  cap, n_used, (uint32_t)remap.len(), b),
                          "dispatch::hetsplit_select");
}

// VecAddInplace::launch (crates/v4flash-kernels/src/ffn.rs:135-153)
inline Status vec_add_inplace(const Stream &s, Out<float> out, In<float> rhs, uint64_t n) {
    DSX_TRY(detail::need("vec_add out", out.len(), n));
    DSX_TRY(detail::need("vec_add rhs", rhs.len(), n));
    return Status::from_c(dsx_vec_add_inplace(s.raw(), out.ptr(), rhs.ptr(), n), "dispatch::vec_add_inplace");
}

}  // namespace dispatch

// ---- MoeExecutor (crates/v4flash-kernels/src/het/remote_experts.rs:7266-7325,7432-7443) ------
// Owns the layer handle and the scratch for up to max_tokens tokens (the reference's executor
// owns mid / midq / partials / group tables the same way); weights stay the caller's.
class MoeExecutor {
   public:
    MoeExecutor() = default;
    MoeExecutor(const MoeExecutor &) = delete;
    MoeExecutor &operator=(const MoeExecutor &) = delete;
    ~MoeExecutor() {
        if (layer_ != nullptr) dsx_moe_layer_destroy(layer_);
    }
    static Status create(MoeExecutor &out, const dsx_moe_layer_desc &desc, uint32_t max_tokens) {
        if (out.layer_ != nullptr) return Status::invalid("MoeExecutor::create: already created");
        if (max_tokens == 0) return Status::invalid("MoeExecutor::create: max_tokens is 0");
        DSX_TRY(Status::from_c(dsx_moe_layer_create(&desc, &out.layer_), "MoeExecutor::create"));
        out.desc_ = desc;
        out.max_tokens_ = max_tokens;
        return DeviceBuffer<uint8_t>::zeroed(out.workspace_, dsx_moe_layer_workspace_bytes(out.layer_, max_tokens));
    }
    uint32_t max_tokens() const { return max_tokens_; }
    const dsx_moe_layer_desc &desc() const { return desc_; }

    // out[t, :] = sum over the token's picks of expert(x[t]) + shared(x[t]), routing from logits.
    // selected_out / weights_out may be empty.
    Status run(const Stream &s, Out<float> out, In<float> x, In<float> logits, uint32_t n_tokens,
               Out<int32_t> selected_out = {}, Out<float> weights_out = {}) {
        DSX_TRY(check(out, x, n_tokens));
        DSX_TRY(detail::need("MoeExecutor::run logits", logits.len(), (size_t)n_tokens * desc_.n_expert));
        if (!selected_out.empty())
            DSX_TRY(detail::need("MoeExecutor::run selected_out", selected_out.len(), (size_t)n_tokens * desc_.n_used));
        if (!weights_out.empty())
            DSX_TRY(detail::need("MoeExecutor::run weights_out", weights_out.len(), (size_t)n_tokens * desc_.n_used));
        return Status::from_c(
            dsx_moe_layer_forward(layer_, s.raw(), out.ptr(), x.ptr(), logits.ptr(), n_tokens, workspace_.ptr(),
                                  workspace_.byte_len(), selected_out.ptr(), weights_out.ptr(), nullptr, nullptr),
            "MoeExecutor::run");
    }
    // The same with the picks given (the reference's run(): the router ran elsewhere).
    Status run_selected(const Stream &s, Out<float> out, In<float> x, In<int32_t> selected, In<float> weights,
                        uint32_t n_tokens) {
        DSX_TRY(check(out, x, n_tokens));
        DSX_TRY(detail::need("MoeExecutor::run_selected selected", selected.len(), (size_t)n_tokens * desc_.n_used));
        DSX_TRY(detail::need("MoeExecutor::run_selected weights", weights.len(), (size_t)n_tokens * desc_.n_used));
        return Status::from_c(
            dsx_moe_layer_forward(layer_, s.raw(), out.ptr(), x.ptr(), nullptr, n_tokens, workspace_.ptr(),
                                  workspace_.byte_len(), nullptr, nullptr, selected.ptr(), weights.ptr()),
            "MoeExecutor::run_selected");
    }

   private:
    Status check(Out<float> out, In<float> x, uint32_t n_tokens) const {
        if (layer_ == nullptr) return Status::invalid("MoeExecutor: not created");
        if (n_tokens > max_tokens_)
            return Status::invalid("MoeExecutor: " + std::to_string(n_tokens) + " tokens, sized for " +
                                   std::to_string(max_tokens_));
        DSX_TRY(detail::need("MoeExecutor x", x.len(), (size_t)n_tokens * desc_.hidden));
        return detail::need("MoeExecutor out", out.len(), (size_t)n_tokens * desc_.hidden);
    }
    dsx_moe_layer *layer_ = nullptr;
    dsx_moe_layer_desc desc_{};
    uint32_t max_tokens_ = 0;
    DeviceBuffer<uint8_t> workspace_;
};

}  // namespace dsx
