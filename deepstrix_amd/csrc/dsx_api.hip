// dsx_api.hip -- the C ABI of libdsx_moe.so (see include/dsx_moe.h): argument validation,
// grid/block selection and the layer-level sequencing.  Nothing here synchronizes,
// allocates device memory or reads back, so every entry point can be captured in a graph.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>

#include "../../include/dsx_moe.h"
#include "dsx_decode_fused.hpp"
#include "dsx_expert_kernels.hpp"
#include "dsx_gemm_kernels.hpp"
#include "dsx_misc_kernels.hpp"
#include "dsx_q8_0_kernels.hpp"

using namespace dsx;

namespace {

thread_local char g_err[512] = "";
int g_num_cu = 256;  // refreshed by dsx_init

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

int launched(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, "%s: %s", what, hipGetErrorString(e));
    return DSX_OK;
}

hipStream_t S(dsx_stream_t s) { return (hipStream_t)s; }

bool aligned(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }

// Kernels whose dynamic LDS may exceed the 64 KiB default get their limit raised once.
template <typename K>
void allow_lds(K kernel) {
    (void)hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              160 * 1024 - 16 * 1024);
}

// Scratch of the one entry point that takes no workspace (dsx_moe_layer_forward_noalloc): a
// fixed array in the code object instead of caller memory.  Host code never uses this name as
// an address -- it is a host-side stand-in; dsx_init asks the runtime for each device's copy.
constexpr size_t kStaticScratchBytes = DSX_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Per-device state set up by dsx_init with that device current: function attributes belong to
// a device, and every device holds its own copy of `scratch` at its own address.
constexpr int kMaxDevices = 64;
std::mutex g_init_mutex;
std::atomic<bool> g_dev_ready[kMaxDevices];
void *g_scratch_ptr[kMaxDevices] = {};

// Entry points that launch kernels with raised LDS limits refuse to run before dsx_init: raising
// the limits lazily would put API calls inside a caller's stream capture.
int need_init(const char *who) {
    int dev = 0;
    const hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail((int)e, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(DSX_ERR_DEVICE, "%s: device %d out of range", who, dev);
    if (!g_dev_ready[dev].load(std::memory_order_acquire))
        return fail(DSX_ERR_DEVICE, "%s: call dsx_init() with device %d current first", who, dev);
    return DSX_OK;
}

void raise_lds_limits() {
    {
        allow_lds(k_mxfp4_gate_up<1, false, false, false>);
        allow_lds(k_mxfp4_gate_up<1, false, true, true>);
        allow_lds(k_mxfp4_gate_up<1, true, false, false>);
        allow_lds(k_mxfp4_gate_up<2, true, false, false>);
        allow_lds(k_mxfp4_gate_up<4, true, false, false>);
        allow_lds(k_mxfp4_gate_up<8, true, false, false>);
        allow_lds(k_mxfp4_gate_up_be4<1>);
        allow_lds(k_mxfp4_gate_up_be4<2>);
        allow_lds(k_mxfp4_gate_up_be4<4>);
        allow_lds(k_mxfp4_gate_up_be4<8>);
        allow_lds(k_mxfp4_decode_fused<8, false>);
        allow_lds(k_mxfp4_decode_fused<0, false>);
        allow_lds(k_mxfp4_decode_fused<8, true>);
        allow_lds(k_mxfp4_decode_fused<0, true>);
        allow_lds(k_mxfp4_decode_fused<8, false, true>);
        allow_lds(k_mxfp4_decode_fused<0, false, true>);
        allow_lds(k_mxfp4_decode_fused<8, true, true>);
        allow_lds(k_mxfp4_decode_fused<0, true, true>);
        allow_lds(k_mxfp4_gemm<true, kGemmMT>);
        allow_lds(k_mxfp4_gemm<false, kGemmMT>);
        allow_lds(k_mxfp4_gemm<true, kGemmMTNarrow>);
        allow_lds(k_mxfp4_gemm<false, kGemmMTNarrow>);
        allow_lds(k_mxfp4_gemm<true, kGemmMT, true>);
        allow_lds(k_mxfp4_gemm<false, kGemmMT, true>);
        allow_lds(k_mxfp4_gemm<true, kGemmMTNarrow, true>);
        allow_lds(k_mxfp4_gemm<false, kGemmMTNarrow, true>);
        allow_lds(k_mxfp4_relayout<true>);
        allow_lds(k_mxfp4_relayout<false>);
        allow_lds(k_mxfp4_down_decode<false>);
        allow_lds(k_mxfp4_down_decode<true>);
        allow_lds(k_mxfp4_down_decode<true, 9>);
        allow_lds(k_mxfp4_down_by_expert<1, false>);
        allow_lds(k_mxfp4_down_by_expert<2, false>);
        allow_lds(k_mxfp4_down_by_expert<4, false>);
        allow_lds(k_mxfp4_down_by_expert<8, false>);
        allow_lds(k_mxfp4_down_by_expert<16, false>);
        allow_lds(k_mxfp4_down_be4<1>);
        allow_lds(k_mxfp4_down_be4<2>);
        allow_lds(k_mxfp4_down_be4<4>);
        allow_lds(k_mxfp4_down_be4<8>);
        allow_lds(k_mxfp4_down_be4<16>);
        q8_0_raise_lds_limits();
        q8_0_gemm_raise_lds_limits();
    }
}

constexpr size_t kLdsBudget = 140 * 1024;  // dynamic LDS a workgroup may ask for

int pick_nt(uint32_t chunk) {
    if (chunk <= 1) return 1;
    if (chunk <= 2) return 2;
    if (chunk <= 4) return 4;
    if (chunk <= 8) return 8;
    return 16;
}

// max_wi work items, p.n_sub workgroups along grid.y for each
template <int NT>
static void launch_gate_up_be(hipStream_t st, const GateUpParams &p, uint32_t max_wi, size_t lds,
                              bool staged) {
    const dim3 grid(p.n_rows / 16, max_wi * p.n_sub);
    if (staged)   // (four row tiles per workgroup)
        hipLaunchKernelGGL((k_mxfp4_gate_up_be4<NT>), dim3((p.n_rows / 16 + kGuBeTiles - 1) / kGuBeTiles, grid.y),
                           dim3(kGuWaves * 64), lds, st, p);
    else
        hipLaunchKernelGGL((k_mxfp4_gate_up<NT, true, false, false>), grid, dim3(kGuWaves * 64), lds, st, p);
}

template <int NT>
static void launch_down_be(hipStream_t st, const DownByExpertParams &p, uint32_t max_wi, size_t lds,
                           bool staged) {
    const dim3 grid(p.n_rows / 16, max_wi * p.n_sub);
    if (staged)   // (four row tiles per workgroup)
        hipLaunchKernelGGL((k_mxfp4_down_be4<NT>), dim3((p.n_rows / 16 + kBe4Waves - 1) / kBe4Waves, grid.y),
                           dim3(kBe4Waves * 64), lds, st, p);
    else
        hipLaunchKernelGGL((k_mxfp4_down_by_expert<NT, false>), grid, dim3(kDownBeWaves * 64), lds, st, p);
}

// Columns per workgroup for a work item of `chunk` members: the largest power of two (at most
// `cap`) whose activation tiles fit LDS; a larger chunk is served by several workgroups per item.
static int fit_nt(uint32_t chunk, uint32_t n_blocks, int cap) {
    int nt = std::min(pick_nt(chunk), cap);
    while (nt > 1 && (size_t)n_blocks * 512 * nt + (size_t)n_blocks * nt * 4 > kLdsBudget) nt /= 2;
    return nt;
}


// Group tables in one launch (a workgroup per group places its members, one more makes the counts,
// offsets and work items: 3.5 us of kernel time up to a thousand picks, 10 us at 32768), with an
// optional extra group `n_expert` that holds every token (slot n_used).
int group_build_big(hipStream_t st, int32_t *group_count, int32_t *group_offset, int32_t *members,
                    int32_t *work_items, int32_t *n_work_items, const int32_t *selected, uint32_t b,
                    uint32_t n_used, uint32_t n_expert, uint32_t chunk, bool extra) {
    hipLaunchKernelGGL(k_group_tables, dim3(n_expert + (extra ? 1u : 0u) + 1u), dim3(kGbThreads), 0, st,
                       group_count, group_offset, members, work_items, n_work_items, selected, b, n_used,
                       n_expert, chunk, extra ? 1u : 0u);
    return launched("group_tables");
}

// Grouped GEMM launch; max_wi bounds the number of work items, MT is the chunk they were built
// with (kGemmMT or kGemmMTNarrow).
// planar: the weights are in the planar form.
template <bool PAIR, int MT = kGemmMT>
int launch_gemm(hipStream_t st, const GemmParams &p, uint32_t max_wi, bool planar = false) {
    if (max_wi == 0) return DSX_OK;
    const uint32_t per_xcd = (max_wi + 7u) / 8u;
    const uint64_t grid = (uint64_t)8u * per_xcd * p.n_row_tiles;
    if (grid > 0x7FFFFFFFull) return fail(DSX_ERR_INVALID_ARG, "gemm: grid too large");
    // the kernel addresses weights and activations with 32-bit byte offsets from their bases
    const uint64_t act_rows = (uint64_t)p.n_tokens * (p.n_used + 1u);
    if ((uint64_t)p.n_rows * p.n_sb * kSuperBytes > 0xFFFFFFFFull ||
        act_rows * p.act_row_bytes > 0xFFFFFFFFull)
        return fail(DSX_ERR_INVALID_ARG, "gemm: a weight matrix or the activation rows exceed 4 GiB");
    if (planar) {
        hipLaunchKernelGGL((k_mxfp4_gemm<PAIR, MT, true>), dim3((uint32_t)grid), dim3(kGemmWaves * 64),
                           gemm_lds_bytes(MT, true), st, p);
        return launched(PAIR ? "gate_up gemm" : "down gemm");
    }
    hipLaunchKernelGGL((k_mxfp4_gemm<PAIR, MT>), dim3((uint32_t)grid), dim3(kGemmWaves * 64),
                       gemm_lds_bytes(MT, false), st, p);
    return launched(PAIR ? "gate_up gemm" : "down gemm");
}

}  // namespace

int dsx::q8_0_fail(int code, const char *what, const char *why) {
    return fail(code, "%s: %s", what, why);
}

extern "C" {

int dsx_abi_version(void) { return DSX_ABI_VERSION; }

const char *dsx_last_error(void) { return g_err; }

int dsx_init(void) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail((int)e, "dsx_init: hipGetDevice: %s", hipGetErrorString(e));
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess)
        return fail((int)e, "dsx_init: hipGetDeviceProperties: %s", hipGetErrorString(e));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(DSX_ERR_DEVICE, "dsx_init: device %d is %s; this library is built for gfx950",
                    dev, prop.gcnArchName);
    if (dev < 0 || dev >= kMaxDevices) return fail(DSX_ERR_DEVICE, "dsx_init: device %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_dev_ready[dev].load(std::memory_order_acquire)) return DSX_OK;
    g_num_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    raise_lds_limits();
    e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, "dsx_init: hipFuncSetAttribute: %s", hipGetErrorString(e));
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
        return fail(e != hipSuccess ? (int)e : DSX_ERR_DEVICE, "dsx_init: hipGetSymbolAddress(scratch): %s",
                    hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
    g_dev_ready[dev].store(true, std::memory_order_release);
    return DSX_OK;
}

// ---- router -------------------------------------------------------------------------
int dsx_router_topk(dsx_stream_t stream, int32_t *selected, float *weights, const float *logits,
                    const float *bias, uint32_t n_expert, uint32_t n_used, float scale, float eps,
                    uint32_t b, uint32_t mode, uint32_t n_group, uint32_t topk_group) {
    if (b == 0) return DSX_OK;
    if (!selected || !weights || !logits) return fail(DSX_ERR_INVALID_ARG, "router_topk: null pointer");
    if (n_expert == 0 || n_expert > DSX_MAX_EXPERTS)
        return fail(DSX_ERR_INVALID_ARG, "router_topk: n_expert=%u not in 1..%d", n_expert,
                    DSX_MAX_EXPERTS);
    if (n_used == 0 || n_used > DSX_MAX_USED || n_used > n_expert)
        return fail(DSX_ERR_INVALID_ARG, "router_topk: n_used=%u not in 1..%d", n_used, DSX_MAX_USED);
    if (mode > 2) return fail(DSX_ERR_INVALID_ARG, "router_topk: mode=%u", mode);
    if (n_group > 1) {
        if (n_group > 64 || n_expert % n_group != 0 || topk_group == 0)
            return fail(DSX_ERR_SHAPE, "router_topk: n_group=%u topk_group=%u n_expert=%u", n_group,
                        topk_group, n_expert);
    }
    hipLaunchKernelGGL(k_router_topk, dim3(b), dim3(kRouterThreads), 0, S(stream), selected, weights, logits,
                       bias, n_expert, n_used, scale, eps, mode, n_group, topk_group);
    return launched("router_topk");
}

int dsx_router_hash_select(dsx_stream_t stream, int32_t *selected, float *weights,
                           const float *logits, const int32_t *tid2eid, const int32_t *token_ids,
                           uint32_t n_expert, uint32_t n_used, uint32_t vocab, float scale,
                           float eps, uint32_t b) {
    if (b == 0) return DSX_OK;
    if (!selected || !weights || !logits || !tid2eid || !token_ids)
        return fail(DSX_ERR_INVALID_ARG, "router_hash_select: null pointer");
    if (n_expert == 0 || vocab == 0)
        return fail(DSX_ERR_INVALID_ARG, "router_hash_select: n_expert=%u vocab=%u", n_expert, vocab);
    if (n_used == 0 || n_used > DSX_MAX_USED)
        return fail(DSX_ERR_INVALID_ARG, "router_hash_select: n_used=%u not in 1..%d", n_used, DSX_MAX_USED);
    hipLaunchKernelGGL(k_router_hash_select, dim3((b + 255) / 256), dim3(256), 0, S(stream), selected,
                       weights, logits, tid2eid, token_ids, n_expert, n_used, vocab, scale, eps, b);
    return launched("router_hash_select");
}

int dsx_moe_hetsplit_select(dsx_stream_t stream, int32_t *selected_side, const int32_t *selected,
                            const int32_t *remap, uint32_t mode, uint32_t cap, uint32_t n_used,
                            uint32_t n_expert, uint32_t b) {
    if (b == 0) return DSX_OK;
    if (!selected_side || !selected || !remap)
        return fail(DSX_ERR_INVALID_ARG, "moe_hetsplit_select: null pointer");
    if (mode > 1) return fail(DSX_ERR_INVALID_ARG, "moe_hetsplit_select: mode=%u", mode);
    if (n_used == 0 || n_expert == 0)
        return fail(DSX_ERR_INVALID_ARG, "moe_hetsplit_select: n_used=%u n_expert=%u", n_used, n_expert);
    hipLaunchKernelGGL(k_hetsplit_select, dim3((b + 255) / 256), dim3(256), 0, S(stream),
                       selected_side, selected, remap, mode, cap, n_used, n_expert, b);
    return launched("moe_hetsplit_select");
}

// ---- quantizers -----------------------------------------------------------------------
int dsx_q8k_quantize(dsx_stream_t stream, uint8_t *out, const float *x, uint32_t n_blocks) {
    if (n_blocks == 0) return DSX_OK;
    if (!out || !x) return fail(DSX_ERR_INVALID_ARG, "q8k_quantize: null pointer");
    if (!aligned(x, 16) || !aligned(out, 4))
        return fail(DSX_ERR_SHAPE, "q8k_quantize: x must be 16-byte and out 4-byte aligned");
    hipLaunchKernelGGL(k_q8k_quantize, dim3((n_blocks + 3) / 4), dim3(256), 0, S(stream), out, x,
                       n_blocks);
    return launched("q8k_quantize");
}

int dsx_q8_0_quantize(dsx_stream_t stream, int8_t *xq, float *xscale, const float *x,
                      uint32_t blocks) {
    if (blocks == 0) return DSX_OK;
    if (!xq || !xscale || !x) return fail(DSX_ERR_INVALID_ARG, "q8_0_quantize: null pointer");
    if (!aligned(x, 16) || !aligned(xq, 4))
        return fail(DSX_ERR_SHAPE, "q8_0_quantize: x must be 16-byte and xq 4-byte aligned");
    hipLaunchKernelGGL(k_q8_0_quantize, dim3((blocks * 8 + 255) / 256), dim3(256), 0, S(stream), xq,
                       xscale, x, blocks);
    return launched("q8_0_quantize");
}

int dsx_q8_0_quantize_rows(dsx_stream_t stream, uint8_t *out, const float *x, uint32_t rows,
                           uint32_t k) {
    if (rows == 0) return DSX_OK;
    if (!out || !x) return fail(DSX_ERR_INVALID_ARG, "q8_0_quantize_rows: null pointer");
    if (k == 0 || k % 32 != 0) return fail(DSX_ERR_SHAPE, "q8_0_quantize_rows: k=%u must be a multiple of 32", k);
    if (!aligned(x, 16) || !aligned(out, 4))
        return fail(DSX_ERR_SHAPE, "q8_0_quantize_rows: x must be 16-byte and out 4-byte aligned");
    const uint64_t threads = (uint64_t)rows * (k / 32) * 8;
    hipLaunchKernelGGL(k_q8_0_quantize_rows, dim3((uint32_t)((threads + 255) / 256)), dim3(256), 0,
                       S(stream), out, x, rows, k);
    return launched("q8_0_quantize_rows");
}

// ---- decode ---------------------------------------------------------------------------
// staged != 0: xq is a staged row, midp receives the fused quantization of mid, and mid must hold
// kMidUnwritten everywhere on entry (the front kernel of the layer writes it).
static int gate_up_decode_impl(hipStream_t st, int dtype, float *mid, const uint8_t *gate,
                               const uint8_t *up, const uint8_t *xq, const float *ew,
                               const int32_t *selected, const uint8_t *sh_gate,
                               const uint8_t *sh_up, float sh_clamp, uint64_t gbpe, uint64_t ubpe,
                               uint32_t n_used, float clamp, uint32_t n_rows, uint32_t n_blocks,
                               bool staged = false, uint8_t *midp = nullptr,
                               uint32_t n_tokens = 1, uint32_t *status = nullptr,
                               uint32_t spin_limit = 0) {
    if (n_used == 0 && !sh_gate) return DSX_OK;
    if (!mid || !gate || !up || !xq || !ew || !selected)
        return fail(DSX_ERR_INVALID_ARG, "moe_gate_up_batch: null pointer");
    if (n_used > DSX_MAX_USED) return fail(DSX_ERR_INVALID_ARG, "moe_gate_up_batch: n_used=%u", n_used);
    if (dtype == DSX_FMT_Q8_0)
        return q8_0_gate_up_decode(st, mid, gate, up, xq, ew, selected, sh_gate, sh_up, sh_clamp,
                                   gbpe, ubpe, n_used, clamp, n_rows, n_blocks);
    const bool planar = dtype == DSX_FMT_MXFP4_PLANAR;
    if (dtype != DSX_FMT_MXFP4 && !planar)
        return fail(DSX_ERR_UNSUPPORTED, "moe_gate_up_batch: no kernel for dtype %d", dtype);
    if (n_rows == 0 || n_rows % 16 != 0)
        return fail(DSX_ERR_SHAPE, "moe_gate_up_batch: n_rows=%u must be a multiple of 16", n_rows);
    if (n_blocks == 0) return fail(DSX_ERR_INVALID_ARG, "moe_gate_up_batch: n_blocks=0");
    if (gbpe % 8 || ubpe % 8 || !aligned(gate, 8) || !aligned(up, 8) || !aligned(xq, 4))
        return fail(DSX_ERR_SHAPE, "moe_gate_up_batch: weights must be 8-byte aligned, xq 4-byte");
    const size_t lds = (size_t)n_blocks * 512 + (size_t)n_blocks * 4;
    if (lds > kLdsBudget)
        return fail(DSX_ERR_UNSUPPORTED, "moe_gate_up_batch: n_blocks=%u exceeds LDS staging", n_blocks);
    if (int rc_init = need_init("gate_up_decode_impl")) return rc_init;
    GateUpParams p{};
    p.mid = mid; p.gate = gate; p.up = up; p.xq = xq; p.ew = ew; p.selected = selected;
    p.sh_gate = sh_gate; p.sh_up = sh_up; p.gbpe = gbpe; p.ubpe = ubpe; p.n_used = n_used;
    p.chunk = 1; p.clamp = clamp; p.sh_clamp = sh_clamp; p.n_rows = n_rows; p.n_blocks = n_blocks;
    p.xq_row_bytes = staged ? staged_row_bytes(n_blocks) : n_blocks * kQ8kBytes;
    p.planar = planar ? 1u : 0u;
    const uint32_t n_slots = n_used + (sh_gate ? 1u : 0u);
    if (staged) {
        if (n_rows % 256 != 0 || !midp || !aligned(xq, 16))
            return fail(DSX_ERR_SHAPE, "moe_gate_up_batch: fused mid quantization needs n_rows %% 256 == 0");
        p.midp = midp;
        p.status = status;
        p.spin_limit = spin_limit;
        p.midp_row_bytes = staged_row_bytes(n_rows / 256);
        hipLaunchKernelGGL((k_mxfp4_gate_up<1, false, true, true>),
                           dim3(n_rows / 16, n_slots * n_tokens), dim3(kGuWaves * 64), lds, st, p);
    } else {
        hipLaunchKernelGGL((k_mxfp4_gate_up<1, false, false, false>),
                           dim3(n_rows / 16, n_slots * n_tokens), dim3(kGuWaves * 64), lds, st, p);
    }
    return launched("moe_gate_up_batch");
}

int dsx_moe_gate_up_batch(dsx_stream_t stream, int dtype, float *mid, const uint8_t *gate,
                          const uint8_t *up, const uint8_t *xq, const float *ew,
                          const int32_t *selected, uint64_t gbpe, uint64_t ubpe, uint32_t n_used,
                          float clamp, uint32_t n_rows, uint32_t n_blocks) {
    return gate_up_decode_impl(S(stream), dtype, mid, gate, up, xq, ew, selected, nullptr, nullptr,
                               0.0f, gbpe, ubpe, n_used, clamp, n_rows, n_blocks);
}

static int down_decode_impl(hipStream_t st, int dtype, float *out, const uint8_t *down,
                            const uint8_t *xq, const int32_t *selected, const uint8_t *sh_down,
                            uint64_t dbpe, uint32_t xq_slot_stride, uint32_t n_used,
                            uint32_t n_rows, uint32_t n_blocks_in, bool staged = false,
                            uint32_t n_tokens = 1, const float *residual = nullptr) {
    if (!out || !down || !xq || !selected)
        return fail(DSX_ERR_INVALID_ARG, "moe_down_batched: null pointer");
    if (n_used > DSX_MAX_USED) return fail(DSX_ERR_INVALID_ARG, "moe_down_batched: n_used=%u", n_used);
    if (dtype == DSX_FMT_Q8_0)
        return q8_0_down_decode(st, out, down, xq, selected, sh_down, dbpe, xq_slot_stride, n_used,
                                n_rows, n_blocks_in);
    const bool planar = dtype == DSX_FMT_MXFP4_PLANAR;
    if (dtype != DSX_FMT_MXFP4 && !planar)
        return fail(DSX_ERR_UNSUPPORTED, "moe_down_batched: no kernel for dtype %d", dtype);
    if (n_rows == 0 || n_rows % 16 != 0)
        return fail(DSX_ERR_SHAPE, "moe_down_batched: n_rows=%u must be a multiple of 16", n_rows);
    if (n_blocks_in == 0) return fail(DSX_ERR_INVALID_ARG, "moe_down_batched: n_blocks_in=0");
    if (xq_slot_stride < n_blocks_in * (staged ? 516u : (uint32_t)kQ8kBytes) ||
        xq_slot_stride % (staged ? 16 : 4))
        return fail(DSX_ERR_SHAPE, "moe_down_batched: xq_slot_stride=%u", xq_slot_stride);
    if (dbpe % 8 || !aligned(down, 8) || !aligned(xq, staged ? 16 : 4))
        return fail(DSX_ERR_SHAPE, "moe_down_batched: weights must be 8-byte aligned, xq 4-byte");
    const uint32_t n_slots = n_used + (sh_down ? 1u : 0u);
    const size_t units = (size_t)n_slots * n_blocks_in;
    const size_t lds = units * 512 + units * 4;
    if (lds > kLdsBudget)
        return fail(DSX_ERR_UNSUPPORTED, "moe_down_batched: %zu (slot, block) tiles exceed LDS", units);
    if (int rc_init = need_init("down_decode_impl")) return rc_init;
    DownDecodeParams p{};
    p.out = out; p.down = down; p.xq = xq; p.selected = selected; p.sh_down = sh_down;
    p.residual = residual;
    p.dbpe = dbpe; p.xq_slot_stride = xq_slot_stride; p.n_used = n_used; p.n_slots = n_slots;
    p.n_rows = n_rows; p.n_blocks_in = n_blocks_in; p.planar = planar ? 1u : 0u;
    // two workgroups of 8 waves per CU, all resident at once and of equal size where the row
    // count allows (7168 rows on 256 CUs: 512 workgroups of 14 rows)
    const uint32_t even = (n_rows + 2u * g_num_cu - 1u) / (2u * g_num_cu);
    p.rows_per_wg = std::min(16u, std::max(8u, even));
    const uint32_t gx = (n_rows + p.rows_per_wg - 1u) / p.rows_per_wg;
    if (staged && units == 9u * kDownWaves)  // the V3 shape: 9 slots x 8 super-blocks, 9 units per wave
        hipLaunchKernelGGL((k_mxfp4_down_decode<true, 9>), dim3(gx, n_tokens), dim3(kDownWaves * 64), lds, st, p);
    else if (staged)
        hipLaunchKernelGGL(k_mxfp4_down_decode<true>, dim3(gx, n_tokens), dim3(kDownWaves * 64), lds, st, p);
    else
        hipLaunchKernelGGL(k_mxfp4_down_decode<false>, dim3(gx, n_tokens), dim3(kDownWaves * 64), lds, st, p);
    return launched("moe_down_batched");
}

int dsx_moe_down_batched(dsx_stream_t stream, int dtype, float *out, const uint8_t *down,
                         const uint8_t *xq, const int32_t *selected, uint64_t dbpe,
                         uint32_t xq_slot_stride, uint32_t n_used, uint32_t n_rows,
                         uint32_t n_blocks_in) {
    if (n_used == 0) return fail(DSX_ERR_INVALID_ARG, "moe_down_batched: n_used=0");
    return down_decode_impl(S(stream), dtype, out, down, xq, selected, nullptr, dbpe,
                            xq_slot_stride, n_used, n_rows, n_blocks_in);
}

// ---- by-expert ------------------------------------------------------------------------
// extra: also build group n_expert that holds every token (slot n_used)
static int group_build_impl(hipStream_t st, int32_t *group_count, int32_t *group_offset,
                            int32_t *expert_members, int32_t *work_items, int32_t *n_work_items,
                            const int32_t *selected, uint32_t b, uint32_t n_used, uint32_t n_expert,
                            uint32_t chunk, bool extra) {
    if (!group_count || !group_offset || !expert_members || !work_items || !n_work_items || !selected)
        return fail(DSX_ERR_INVALID_ARG, "moe_group_build: null pointer");
    if (n_expert == 0 || n_expert > DSX_MAX_EXPERTS)
        return fail(DSX_ERR_INVALID_ARG, "moe_group_build: n_expert=%u", n_expert);
    if (b >= 65536 || n_used == 0 || n_used >= 65536)
        return fail(DSX_ERR_INVALID_ARG, "moe_group_build: b=%u n_used=%u must be below 65536", b, n_used);
    if (chunk == 0 || chunk > 128) return fail(DSX_ERR_INVALID_ARG, "moe_group_build: chunk=%u not in 1..128", chunk);
    return group_build_big(st, group_count, group_offset, expert_members, work_items, n_work_items,
                           selected, b, n_used, n_expert, chunk, extra);
}

int dsx_moe_group_build(dsx_stream_t stream, int32_t *group_count, int32_t *group_offset,
                        int32_t *expert_members, int32_t *work_items, int32_t *n_work_items,
                        const int32_t *selected, uint32_t b, uint32_t n_used, uint32_t n_expert,
                        uint32_t chunk) {
    if (chunk > 64) return fail(DSX_ERR_INVALID_ARG, "moe_group_build: chunk=%u not in 1..64", chunk);
    return group_build_impl(S(stream), group_count, group_offset, expert_members, work_items,
                            n_work_items, selected, b, n_used, n_expert, chunk, false);
}

static int gate_up_be_impl(dsx_stream_t stream, int dtype, float *mid, const uint8_t *gate,
                                 const uint8_t *up, const uint8_t *xq, const float *ew,
                                 const int32_t *group_count, const int32_t *group_offset,
                                 const int32_t *expert_members, const int32_t *work_items,
                                 const int32_t *n_work_items, uint32_t max_work_items,
                                 uint64_t gbpe, uint64_t ubpe, uint32_t n_used, uint32_t chunk,
                                 float clamp, uint32_t n_rows, uint32_t n_blocks, bool staged,
                                 const uint8_t *sh_gate = nullptr, const uint8_t *sh_up = nullptr,
                                 float sh_clamp = 0.0f, uint32_t n_expert = 0, uint32_t n_tokens = 0) {
    if (max_work_items == 0) return DSX_OK;
    if (!mid || !gate || !up || !xq || !ew || !group_count || !group_offset || !expert_members ||
        !work_items || !n_work_items)
        return fail(DSX_ERR_INVALID_ARG, "moe_gate_up_chunked_rows: null pointer");
    if (max_work_items > 65535)
        return fail(DSX_ERR_INVALID_ARG, "moe_gate_up_chunked_rows: max_work_items=%u", max_work_items);
    if (chunk == 0 || chunk > 64)
        return fail(DSX_ERR_INVALID_ARG, "moe_gate_up_chunked_rows: chunk=%u not in 1..64", chunk);
    if (dtype == DSX_FMT_Q8_0)
        return q8_0_gate_up_by_expert(S(stream), mid, gate, up, xq, ew, group_count, group_offset,
                                      expert_members, work_items, n_work_items, max_work_items,
                                      gbpe, ubpe, n_used, chunk, clamp, n_rows, n_blocks, sh_gate, sh_up,
                                      sh_clamp, n_expert, n_tokens);
    const bool planar = dtype == DSX_FMT_MXFP4_PLANAR;
    if (dtype != DSX_FMT_MXFP4 && !planar)
        return fail(DSX_ERR_UNSUPPORTED, "moe_gate_up_chunked_rows: no kernel for dtype %d", dtype);
    if (n_rows == 0 || n_rows % 16 != 0)
        return fail(DSX_ERR_SHAPE, "moe_gate_up_chunked_rows: n_rows=%u must be a multiple of 16", n_rows);
    if (n_blocks == 0) return fail(DSX_ERR_INVALID_ARG, "moe_gate_up_chunked_rows: n_blocks=0");
    if (gbpe % 8 || ubpe % 8 || !aligned(gate, 8) || !aligned(up, 8) || !aligned(xq, staged ? 16 : 4))
        return fail(DSX_ERR_SHAPE, "moe_gate_up_chunked_rows: weights must be 8-byte aligned, xq 4-byte");
    if (staged && !aligned(mid, 16))   // (the staged-row kernels store four rows of a column at a time)
        return fail(DSX_ERR_SHAPE, "moe_gate_up_chunked_rows: mid must be 16-byte aligned");
    const int nt = fit_nt(chunk, n_blocks, 8);
    const size_t lds = (size_t)n_blocks * 512 * nt + (size_t)n_blocks * nt * 4;
    if (lds > kLdsBudget)
        return fail(DSX_ERR_UNSUPPORTED, "moe_gate_up_chunked_rows: n_blocks=%u needs %zu B of LDS",
                    n_blocks, lds);
    const uint32_t n_sub = (chunk + (uint32_t)nt - 1u) / (uint32_t)nt;
    if ((uint64_t)max_work_items * n_sub > 65535u)
        return fail(DSX_ERR_INVALID_ARG, "moe_gate_up_chunked_rows: %u work items x %u sub-chunks exceed the grid",
                    max_work_items, n_sub);
    if (int rc_init = need_init("gate_up_be_impl")) return rc_init;
    GateUpParams p{};
    p.mid = mid; p.gate = gate; p.up = up; p.xq = xq; p.ew = ew;
    p.group_count = group_count; p.group_offset = group_offset; p.members = expert_members;
    p.work_items = work_items; p.n_work_items = n_work_items;
    p.gbpe = gbpe; p.ubpe = ubpe; p.n_used = n_used; p.chunk = chunk; p.clamp = clamp;
    p.n_rows = n_rows; p.n_blocks = n_blocks;
    p.xq_row_bytes = staged ? staged_row_bytes(n_blocks) : n_blocks * kQ8kBytes;
    p.sh_gate = sh_gate; p.sh_up = sh_up; p.sh_clamp = sh_clamp; p.n_expert = n_expert; p.n_tokens = n_tokens;
    p.n_sub = n_sub; p.planar = planar ? 1u : 0u;
    hipStream_t st = S(stream);
    switch (nt) {
        case 1: launch_gate_up_be<1>(st, p, max_work_items, lds, staged); break;
        case 2: launch_gate_up_be<2>(st, p, max_work_items, lds, staged); break;
        case 4: launch_gate_up_be<4>(st, p, max_work_items, lds, staged); break;
        default: launch_gate_up_be<8>(st, p, max_work_items, lds, staged); break;
    }
    return launched("moe_gate_up_chunked_rows");
}

int dsx_moe_gate_up_chunked_rows(dsx_stream_t stream, int dtype, float *mid, const uint8_t *gate,
                                 const uint8_t *up, const uint8_t *xq, const float *ew,
                                 const int32_t *group_count, const int32_t *group_offset,
                                 const int32_t *expert_members, const int32_t *work_items,
                                 const int32_t *n_work_items, uint32_t max_work_items,
                                 uint64_t gbpe, uint64_t ubpe, uint32_t n_used, uint32_t chunk,
                                 float clamp, uint32_t n_rows, uint32_t n_blocks) {
    return gate_up_be_impl(stream, dtype, mid, gate, up, xq, ew, group_count, group_offset,
                           expert_members, work_items, n_work_items, max_work_items, gbpe, ubpe,
                           n_used, chunk, clamp, n_rows, n_blocks, false);
}

static int down_be_impl(dsx_stream_t stream, int dtype, float *partials, const uint8_t *down,
                           const uint8_t *xq, const int32_t *group_count,
                           const int32_t *group_offset, const int32_t *expert_members,
                           const int32_t *work_items, const int32_t *n_work_items,
                           uint32_t max_work_items, uint64_t dbpe, uint32_t xq_slot_stride,
                           uint32_t n_used, uint32_t chunk, uint32_t n_rows, uint32_t n_blocks_in,
                           bool staged, const uint8_t *sh_down = nullptr, uint32_t n_expert = 0,
                           uint32_t n_tokens = 0) {
    if (max_work_items == 0) return DSX_OK;
    if (!partials || !down || !xq || !group_count || !group_offset || !expert_members ||
        !work_items || !n_work_items)
        return fail(DSX_ERR_INVALID_ARG, "moe_down_by_expert: null pointer");
    if (max_work_items > 65535)
        return fail(DSX_ERR_INVALID_ARG, "moe_down_by_expert: max_work_items=%u", max_work_items);
    if (chunk == 0 || chunk > 64)
        return fail(DSX_ERR_INVALID_ARG, "moe_down_by_expert: chunk=%u not in 1..64", chunk);
    if (dtype == DSX_FMT_Q8_0)
        return q8_0_down_by_expert(S(stream), partials, down, xq, group_count, group_offset,
                                   expert_members, work_items, n_work_items, max_work_items, dbpe,
                                   xq_slot_stride, n_used, chunk, n_rows, n_blocks_in, sh_down, n_expert,
                                   n_tokens);
    const bool planar = dtype == DSX_FMT_MXFP4_PLANAR;
    if (dtype != DSX_FMT_MXFP4 && !planar)
        return fail(DSX_ERR_UNSUPPORTED, "moe_down_by_expert: no kernel for dtype %d", dtype);
    if (n_rows == 0 || n_rows % 16 != 0)
        return fail(DSX_ERR_SHAPE, "moe_down_by_expert: n_rows=%u must be a multiple of 16", n_rows);
    if (n_blocks_in == 0) return fail(DSX_ERR_INVALID_ARG, "moe_down_by_expert: n_blocks_in=0");
    if (xq_slot_stride < n_blocks_in * (staged ? 516u : (uint32_t)kQ8kBytes) ||
        xq_slot_stride % (staged ? 16 : 4))
        return fail(DSX_ERR_SHAPE, "moe_down_by_expert: xq_slot_stride=%u", xq_slot_stride);
    if (dbpe % 8 || !aligned(down, 8) || !aligned(xq, staged ? 16 : 4))
        return fail(DSX_ERR_SHAPE, "moe_down_by_expert: weights must be 8-byte aligned, xq 4-byte");
    if (staged && !aligned(partials, 16))
        return fail(DSX_ERR_SHAPE, "moe_down_by_expert: partials must be 16-byte aligned");
    const int nt = fit_nt(chunk, n_blocks_in, 16);
    const size_t lds = (size_t)n_blocks_in * 512 * nt + (size_t)n_blocks_in * nt * 4;
    if (lds > kLdsBudget)
        return fail(DSX_ERR_UNSUPPORTED, "moe_down_by_expert: n_blocks_in=%u needs %zu B of LDS",
                    n_blocks_in, lds);
    const uint32_t n_sub = (chunk + (uint32_t)nt - 1u) / (uint32_t)nt;
    if ((uint64_t)max_work_items * n_sub > 65535u)
        return fail(DSX_ERR_INVALID_ARG, "moe_down_by_expert: %u work items x %u sub-chunks exceed the grid",
                    max_work_items, n_sub);
    if (int rc_init = need_init("down_be_impl")) return rc_init;
    DownByExpertParams p{};
    p.partials = partials; p.down = down; p.xq = xq;
    p.group_count = group_count; p.group_offset = group_offset; p.members = expert_members;
    p.work_items = work_items; p.n_work_items = n_work_items;
    p.dbpe = dbpe; p.xq_slot_stride = xq_slot_stride; p.n_used = n_used; p.chunk = chunk;
    p.n_rows = n_rows; p.n_blocks_in = n_blocks_in;
    p.sh_down = sh_down; p.n_expert = n_expert; p.n_tokens = n_tokens;
    p.n_sub = n_sub; p.planar = planar ? 1u : 0u;
    hipStream_t st = S(stream);
    switch (nt) {
        case 1: launch_down_be<1>(st, p, max_work_items, lds, staged); break;
        case 2: launch_down_be<2>(st, p, max_work_items, lds, staged); break;
        case 4: launch_down_be<4>(st, p, max_work_items, lds, staged); break;
        case 8: launch_down_be<8>(st, p, max_work_items, lds, staged); break;
        default: launch_down_be<16>(st, p, max_work_items, lds, staged); break;
    }
    return launched("moe_down_by_expert");
}

int dsx_moe_down_by_expert(dsx_stream_t stream, int dtype, float *partials, const uint8_t *down,
                           const uint8_t *xq, const int32_t *group_count,
                           const int32_t *group_offset, const int32_t *expert_members,
                           const int32_t *work_items, const int32_t *n_work_items,
                           uint32_t max_work_items, uint64_t dbpe, uint32_t xq_slot_stride,
                           uint32_t n_used, uint32_t chunk, uint32_t n_rows, uint32_t n_blocks_in) {
    return down_be_impl(stream, dtype, partials, down, xq, group_count, group_offset,
                        expert_members, work_items, n_work_items, max_work_items, dbpe,
                        xq_slot_stride, n_used, chunk, n_rows, n_blocks_in, false);
}

static int reduce_impl(hipStream_t st, float *out, const float *partials, const int32_t *selected,
                       const float *add, uint32_t n_used, uint32_t n_rows, uint32_t b,
                       const HcPost &hc = HcPost{}) {
    if (b == 0) return DSX_OK;
    if ((!out && !hc.n_hc) || !partials) return fail(DSX_ERR_INVALID_ARG, "moe_reduce_partials: null pointer");
    if (n_rows == 0 || n_rows % 4 != 0 || !aligned(out, 16) || !aligned(partials, 16) ||
        (add && !aligned(add, 16)))
        return fail(DSX_ERR_SHAPE, "moe_reduce_partials: n_rows=%u must be a multiple of 4, buffers 16-byte aligned", n_rows);
    const uint64_t n4 = (uint64_t)b * (n_rows / 4);
    hipLaunchKernelGGL(k_reduce_partials, dim3((uint32_t)((n4 + 255) / 256)), dim3(256), 0, st, out,
                       partials, selected, add, n_used, n_rows, b, hc);
    return launched("moe_reduce_partials");
}

int dsx_moe_reduce_partials(dsx_stream_t stream, float *out, const float *partials,
                            const int32_t *selected, uint32_t n_used, uint32_t n_rows, uint32_t b) {
    return reduce_impl(S(stream), out, partials, selected, nullptr, n_used, n_rows, b);
}

extern "C++" {
namespace {
constexpr uint32_t kRouterTiledMinTokens = 16;  // from here on the router matvec runs as a tiled GEMM
template <typename WT>
int router_logits_impl(dsx_stream_t stream, float *logits, const WT *router_w, const float *x,
                       uint32_t n_expert, uint32_t hidden, uint32_t n_tokens) {
    if (n_tokens == 0) return DSX_OK;
    if (!logits || !router_w || !x) return fail(DSX_ERR_INVALID_ARG, "router_logits: null pointer");
    if (n_expert == 0 || hidden == 0) return fail(DSX_ERR_INVALID_ARG, "router_logits: n_expert=%u hidden=%u", n_expert, hidden);
    if (!aligned(router_w, 16) || !aligned(x, 16))
        return fail(DSX_ERR_SHAPE, "router_logits: router_w and x must be 16-byte aligned");
    if (n_tokens >= kRouterTiledMinTokens && hidden % 16 == 0 && n_expert % 4 == 0 && aligned(logits, 16)) {
        // many tokens: tiles of 32 experts x 32 tokens on the f32 matrix instruction
        hipLaunchKernelGGL((k_router_logits_tiled<WT>), dim3((n_expert + 31) / 32, (n_tokens + 31) / 32),
                           dim3(256), 0, S(stream), logits, router_w, x, n_expert, hidden, n_tokens);
        return launched("router_logits");
    }
    hipLaunchKernelGGL((k_router_logits<false, WT>), dim3(n_expert), dim3(256), 0, S(stream), logits,
                       (float *)nullptr, router_w, x, (const float *)nullptr, 0.0f, n_expert, hidden,
                       n_tokens);
    return launched("router_logits");
}
}  // namespace
}  // extern "C++"

int dsx_router_logits(dsx_stream_t stream, float *logits, const float *router_w, const float *x,
                      uint32_t n_expert, uint32_t hidden, uint32_t n_tokens) {
    return router_logits_impl(stream, logits, router_w, x, n_expert, hidden, n_tokens);
}

int dsx_router_logits_f16(dsx_stream_t stream, float *logits, const uint16_t *router_w,
                          const float *x, uint32_t n_expert, uint32_t hidden, uint32_t n_tokens) {
    return router_logits_impl(stream, logits, (const __half *)router_w, x, n_expert, hidden, n_tokens);
}

// ---- hyper-connection combine --------------------------------------------------------------
// Checks a caller's descriptor and turns it into the kernels' (0 = ok).
static int hc_post_args(const char *who, const dsx_hc_post_desc *d, uint32_t n_embd, HcPost *out) {
    if (!d || !d->out_hc || !d->residual_hc || !d->post || !d->comb)
        return fail(DSX_ERR_INVALID_ARG, "%s: null pointer in the hc_post descriptor", who);
    if (d->n_hc == 0 || d->n_hc > kMaxHc)
        return fail(DSX_ERR_INVALID_ARG, "%s: n_hc=%u not in 1..%u", who, d->n_hc, kMaxHc);
    if (n_embd == 0 || n_embd % 4 != 0 || !aligned(d->out_hc, 16) || !aligned(d->residual_hc, 16))
        return fail(DSX_ERR_SHAPE, "%s: n_embd=%u must be a multiple of 4, out_hc / residual_hc 16-byte aligned", who, n_embd);
    *out = HcPost{d->out_hc, d->residual_hc, d->post, d->comb, d->n_hc, d->post_stride, d->comb_stride};
    return DSX_OK;
}

static int add_rows_impl(hipStream_t st, float *out, const float *a, const float *b, const float *c,
                         uint32_t n_embd, uint32_t n_tokens, const HcPost &hc) {
    const uint64_t n4 = (uint64_t)n_tokens * (n_embd / 4u);
    hipLaunchKernelGGL(k_add_rows, dim3((uint32_t)((n4 + 255u) / 256u)), dim3(256), 0, st, out, a, b, c,
                       n_embd, n_tokens, hc);
    return launched("add_rows");
}

int dsx_hc_post(dsx_stream_t stream, const dsx_hc_post_desc *desc, const float *block_out,
                const float *add1, const float *add2, uint32_t n_embd, uint32_t b) {
    if (b == 0) return DSX_OK;
    if (!block_out) return fail(DSX_ERR_INVALID_ARG, "hc_post: null block_out");
    if (add2 && !add1) return fail(DSX_ERR_INVALID_ARG, "hc_post: add2 without add1");
    HcPost hc{};
    if (int rc = hc_post_args("hc_post", desc, n_embd, &hc)) return rc;
    if (!aligned(block_out, 16) || (add1 && !aligned(add1, 16)) || (add2 && !aligned(add2, 16)))
        return fail(DSX_ERR_SHAPE, "hc_post: block_out / add1 / add2 must be 16-byte aligned");
    if ((uint64_t)b * (n_embd / 4u) > 0xFFFFFFFFull * 256ull) return fail(DSX_ERR_INVALID_ARG, "hc_post: too many rows");
    return add_rows_impl(S(stream), nullptr, block_out, add1, add2, n_embd, b, hc);
}

// ---- element-wise -----------------------------------------------------------------------
int dsx_vec_add_inplace(dsx_stream_t stream, float *out, const float *rhs, uint64_t n) {
    if (n == 0) return DSX_OK;
    if (!out || !rhs) return fail(DSX_ERR_INVALID_ARG, "vec_add_inplace: null pointer");
    hipLaunchKernelGGL(k_vec_add_inplace, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, S(stream),
                       out, rhs, n);
    return launched("vec_add_inplace");
}

int dsx_rms_norm(dsx_stream_t stream, float *out, const float *x, const float *weight, uint32_t n,
                 float eps, uint32_t rows) {
    if (rows == 0) return DSX_OK;
    if (!out || !x || !weight || n == 0) return fail(DSX_ERR_INVALID_ARG, "rms_norm: null pointer or n=0");
    hipLaunchKernelGGL(k_rms_norm, dim3(rows), dim3(256), 0, S(stream), out, x, weight, n, eps);
    return launched("rms_norm");
}

int dsx_swiglu_clamp_weighted(dsx_stream_t stream, float *mid, const float *gate, const float *up,
                              const float *expert_w, float clamp, uint32_t ff, uint32_t n_experts) {
    if (ff == 0 || n_experts == 0) return DSX_OK;
    if (!mid || !gate || !up || !expert_w)
        return fail(DSX_ERR_INVALID_ARG, "swiglu_clamp_weighted: null pointer");
    hipLaunchKernelGGL(k_swiglu_clamp_weighted, dim3((ff + 255) / 256, n_experts), dim3(256), 0,
                       S(stream), mid, gate, up, expert_w, clamp, ff);
    return launched("swiglu_clamp_weighted");
}

// ---- weight pipeline ----------------------------------------------------------------------
int dsx_mxfp4_repack_hf_to_v2(dsx_stream_t stream, uint8_t *dst, const uint8_t *packed,
                              const uint8_t *scale, uint32_t out, uint32_t nb) {
    if (out == 0 || nb == 0) return DSX_OK;
    if (!dst || !packed || !scale) return fail(DSX_ERR_INVALID_ARG, "mxfp4_repack: null pointer");
    if (nb % 8 != 0) return fail(DSX_ERR_SHAPE, "mxfp4_repack: nb=%u must be a multiple of 8", nb);
    if (!aligned(dst, 8) || !aligned(packed, 8))
        return fail(DSX_ERR_SHAPE, "mxfp4_repack: dst and packed must be 8-byte aligned");
    const uint64_t n = (uint64_t)out * nb;
    hipLaunchKernelGGL(k_mxfp4_repack, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, S(stream),
                       dst, packed, scale, out, nb);
    return launched("mxfp4_repack");
}

static int mxfp4_relayout(hipStream_t st, bool to_planar, uint8_t *w, uint32_t n_rows, uint32_t cols,
                          uint32_t n_matrices, uint64_t stride) {
    const char *who = to_planar ? "mxfp4_rows_to_planar" : "mxfp4_planar_to_rows";
    if (n_matrices == 0 || n_rows == 0 || cols == 0) return DSX_OK;
    if (!w) return fail(DSX_ERR_INVALID_ARG, "%s: null pointer", who);
    if (n_rows % 16 != 0 || cols % 256 != 0)
        return fail(DSX_ERR_SHAPE, "%s: n_rows=%u must be a multiple of 16, cols=%u of 256", who, n_rows, cols);
    const uint32_t n_sb = cols / 256;
    const uint64_t mat_bytes = (uint64_t)n_rows * n_sb * kSuperBytes;
    if (stride < mat_bytes || stride % 8 != 0 || !aligned(w, 8))
        return fail(DSX_ERR_SHAPE, "%s: matrices must be 8-byte aligned and at least %llu bytes apart", who,
                    (unsigned long long)mat_bytes);
    const size_t lds = (size_t)16 * n_sb * kSuperBytes;   // one 16-row tile
    if (lds > kLdsBudget)
        return fail(DSX_ERR_UNSUPPORTED, "%s: cols=%u: a 16-row tile exceeds LDS", who, cols);
    if (int rc_init = need_init(who)) return rc_init;
    for (uint32_t m0 = 0; m0 < n_matrices; m0 += 65535u) {
        const uint32_t m = std::min(65535u, n_matrices - m0);
        uint8_t *first = w + (uint64_t)m0 * stride;
        if (to_planar)
            hipLaunchKernelGGL(k_mxfp4_relayout<true>, dim3(n_rows / 16, m), dim3(256), lds, st, first, n_sb, stride);
        else
            hipLaunchKernelGGL(k_mxfp4_relayout<false>, dim3(n_rows / 16, m), dim3(256), lds, st, first, n_sb, stride);
        if (int rc = launched(who)) return rc;
    }
    return DSX_OK;
}

int dsx_mxfp4_rows_to_planar(dsx_stream_t stream, uint8_t *w, uint32_t n_rows, uint32_t cols,
                             uint32_t n_matrices, uint64_t stride) {
    return mxfp4_relayout(S(stream), true, w, n_rows, cols, n_matrices, stride);
}

int dsx_mxfp4_planar_to_rows(dsx_stream_t stream, uint8_t *w, uint32_t n_rows, uint32_t cols,
                             uint32_t n_matrices, uint64_t stride) {
    return mxfp4_relayout(S(stream), false, w, n_rows, cols, n_matrices, stride);
}

int dsx_q8_0_weights_from_hf(dsx_stream_t stream, uint8_t *dst, const void *src,
                             const uint8_t *scale, uint32_t src_dtype, uint32_t out_rows,
                             uint32_t in_cols, uint32_t scale_rows, uint32_t scale_cols,
                             uint32_t split_rows) {
    if (out_rows == 0 || in_cols == 0) return DSX_OK;
    if (!dst || !src) return fail(DSX_ERR_INVALID_ARG, "q8_0_weights_from_hf: null pointer");
    if (in_cols % 32 != 0)
        return fail(DSX_ERR_SHAPE, "q8_0_weights_from_hf: in_cols=%u must be a multiple of 32", in_cols);
    if (!aligned(dst, 2)) return fail(DSX_ERR_SHAPE, "q8_0_weights_from_hf: dst must be 2-byte aligned");
    uint32_t br = 1, bc = 1;
    const uint64_t groups = (uint64_t)out_rows * (in_cols / 32) * 8;
    const dim3 grid((uint32_t)((groups + 255) / 256));
    if (groups > 0xFFFFFFFFull * 256ull) return fail(DSX_ERR_SHAPE, "q8_0_weights_from_hf: matrix too large");
    switch (src_dtype) {
    case DSX_SRC_F32:
        if (!aligned(src, 16)) return fail(DSX_ERR_SHAPE, "q8_0_weights_from_hf: f32 src must be 16-byte aligned");
        hipLaunchKernelGGL(k_q8_0_weights<kSrcF32>, grid, dim3(256), 0, S(stream), dst, src, scale,
                           out_rows, in_cols, br, bc, 1u, split_rows);
        break;
    case DSX_SRC_BF16:
        if (!aligned(src, 8)) return fail(DSX_ERR_SHAPE, "q8_0_weights_from_hf: bf16 src must be 8-byte aligned");
        hipLaunchKernelGGL(k_q8_0_weights<kSrcBF16>, grid, dim3(256), 0, S(stream), dst, src, scale,
                           out_rows, in_cols, br, bc, 1u, split_rows);
        break;
    case DSX_SRC_F8E4M3:
        if (!scale) return fail(DSX_ERR_INVALID_ARG, "q8_0_weights_from_hf: fp8 weight without a scale tensor");
        if (scale_rows == 0 || scale_cols == 0 || out_rows % scale_rows != 0 || in_cols % scale_cols != 0)
            return fail(DSX_ERR_SHAPE,
                        "q8_0_weights_from_hf: fp8 scale grid %ux%u does not exactly tile %ux%u",
                        scale_rows, scale_cols, out_rows, in_cols);
        if (!aligned(src, 4)) return fail(DSX_ERR_SHAPE, "q8_0_weights_from_hf: fp8 src must be 4-byte aligned");
        br = out_rows / scale_rows;
        bc = in_cols / scale_cols;
        hipLaunchKernelGGL(k_q8_0_weights<kSrcF8E4M3>, grid, dim3(256), 0, S(stream), dst, src, scale,
                           out_rows, in_cols, br, bc, scale_cols, split_rows);
        break;
    default:
        return fail(DSX_ERR_INVALID_ARG, "q8_0_weights_from_hf: cannot Q8_0-quantise source dtype %u", src_dtype);
    }
    return launched("q8_0_weights_from_hf");
}

int dsx_q8_0_repack_rows(dsx_stream_t stream, uint8_t *dst, const uint8_t *src, uint32_t num_rows,
                         uint32_t blocks_per_row) {
    if (num_rows == 0 || blocks_per_row == 0) return DSX_OK;
    if (!dst || !src) return fail(DSX_ERR_INVALID_ARG, "q8_0_repack_rows: null pointer");
    if (dst == src) return fail(DSX_ERR_INVALID_ARG, "q8_0_repack_rows: cannot repack in place");
    if (!aligned(dst, 2) || !aligned(src, 2))
        return fail(DSX_ERR_SHAPE, "q8_0_repack_rows: dst and src must be 2-byte aligned");
    const uint64_t groups = (uint64_t)num_rows * blocks_per_row * 8;
    if (groups > 0xFFFFFFFFull * 256ull) return fail(DSX_ERR_SHAPE, "q8_0_repack_rows: matrix too large");
    hipLaunchKernelGGL(k_q8_0_repack_rows, dim3((uint32_t)((groups + 255) / 256)), dim3(256), 0,
                       S(stream), dst, src, num_rows, blocks_per_row);
    return launched("q8_0_repack_rows");
}

int dsx_dequant_rows(dsx_stream_t stream, int dtype, float *y, const uint8_t *rows, uint32_t n_rows,
                     uint32_t cols) {
    if (n_rows == 0 || cols == 0) return DSX_OK;
    if (!y || !rows) return fail(DSX_ERR_INVALID_ARG, "dequant_rows: null pointer");
    if (dtype == DSX_FMT_MXFP4) {
        if (cols % 256) return fail(DSX_ERR_SHAPE, "dequant_rows: cols=%u must be a multiple of 256", cols);
        const uint64_t nb = (uint64_t)n_rows * (cols / 32);
        hipLaunchKernelGGL(k_mxfp4_dequant, dim3((uint32_t)((nb + 255) / 256)), dim3(256), 0,
                           S(stream), y, rows, nb);
    } else if (dtype == DSX_FMT_Q8_0) {
        if (cols % 32) return fail(DSX_ERR_SHAPE, "dequant_rows: cols=%u must be a multiple of 32", cols);
        const uint64_t nb = (uint64_t)n_rows * (cols / 32);
        hipLaunchKernelGGL(k_q8_0_dequant, dim3((uint32_t)((nb + 255) / 256)), dim3(256), 0,
                           S(stream), y, rows, n_rows, cols / 32);
    } else {
        return fail(DSX_ERR_UNSUPPORTED, "dequant_rows: dtype %d", dtype);
    }
    return launched("dequant_rows");
}

}  // extern "C"

#include "dsx_layer.inc"

// ---- the layer for callers that cannot allocate ---------------------------------------------
// Same sequencing and kernels as dsx_moe_layer_forward; the workspace is this device's copy of
// the file-scope `scratch` array, whose address dsx_init resolved (g_scratch_ptr).  Nothing in
// the workspace has to start at zero: every region is written before it is read within a call
// (the front kernel fills `mid` with its "unwritten" pattern, the group builders zero their
// own counters), exactly as with a caller's uninitialised workspace.
extern "C" int dsx_moe_layer_forward_noalloc(dsx_moe_layer *layer, dsx_stream_t stream, float *out,
                                             const float *x, const float *logits, uint32_t n_tokens,
                                             int32_t *selected_out, float *weights_out,
                                             const int32_t *selected_in, const float *weights_in) {
    if (n_tokens == 0) return DSX_OK;
    if (!layer) return fail(DSX_ERR_INVALID_ARG, "moe_layer_forward_noalloc: null layer");
    if (int rc_init = need_init("moe_layer_forward_noalloc")) return rc_init;
    int dev = 0;
    (void)hipGetDevice(&dev);  // checked by need_init
    void *ws = g_scratch_ptr[dev];
    const size_t need = dsx_moe_layer_workspace_bytes(layer, n_tokens);
    if (need > kStaticScratchBytes)
        return fail(DSX_ERR_UNSUPPORTED,
                    "moe_layer_forward_noalloc: %u tokens need %zu B of scratch, the built-in array "
                    "holds %zu B; use dsx_moe_layer_forward with a workspace",
                    n_tokens, need, kStaticScratchBytes);
    return layer_forward_impl(layer, stream, out, x, logits, n_tokens, ws, kStaticScratchBytes,
                              selected_out, weights_out, selected_in, weights_in, nullptr);
}
