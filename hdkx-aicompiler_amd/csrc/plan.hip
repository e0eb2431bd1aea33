// plan.hip -- launch plan: the body of one compiled function as a list of kernel launches on one
// stream.  Fills the gap the reference leaves in its execution plan, whose executor only copies
// buffers (src/base/disco/executor.cc:122-157): every node here is a real launch, named by a
// kernel_symbol as KernelExecNode would carry it (include/base/execution_plan.h:42-50).
// Intermediates live in ONE workspace allocated at finalize time (the CPU backend mallocs and frees
// every intermediate on every call, src/codegen/codegen_llvm.cc:578-623).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <sstream>
#include <string>
#include <memory>
#include <utility>
#include <vector>

#include "common.h"

using namespace kxc_hip;

namespace {

enum class NodeKind {
    kConv2D, kPool2D, kGlobalAvgPool, kGemm, kBinary, kRelu, kCopy,
    kQConv2D, kQuantize, kMaxPoolI8, kGlobalAvgPoolI8, kQDense, kModuleKernel, kI8Layout
};
constexpr NodeKind kLastNodeKind = NodeKind::kI8Layout;

struct Node {
    NodeKind kind;
    std::string symbol;
    kxc_hip_buf bufs[6];
    kxc_hip_conv2d_desc conv;
    kxc_hip_qconv2d_desc qconv;
    kxc_hip_pool2d_desc pool;
    int64_t dims[4];
    float f[2];
    int32_t i32[4];
    int64_t a_shape[6], b_shape[6];
    // concurrency: lane 1 = runs on the plan's side stream, concurrently with the main-lane nodes enqueued
    // after it; `join` = this (main-lane) node first waits for every side-lane node enqueued before it
    int32_t lane = 0, join = 0;
    hipEvent_t fork_event = nullptr, done_event = nullptr;
    // chain > 0: the node belongs to an independent chain of nodes (one share of the batch) that runs on its own
    // stream from the start of the run to its end, in plan order, beside the main lane and the other chains
    int32_t chain = 0;
    // Winograd convolution (i32[0] == 1 on a kConv2D node): the weight pointer whose transform bufs[5] holds
    const void* transformed_from = nullptr;
    // convolution launches resolved at finalize (kernel, tile shape, grid, split, environment switches)
    std::shared_ptr<kxc_hip::PreparedConv> prepared_conv;
    std::shared_ptr<kxc_hip::PreparedWinograd> prepared_wino;
    // module kernel
    void* function = nullptr;
    uint32_t grid[3], block[3], shared_bytes = 0;
    std::vector<kxc_hip_buf> params;
};

// A weight tensor that is packed for its kernel at the start of a run (kxc_hip_plan_add_qconv_weight_pack).
struct PackJob {
    int32_t kind = 0;                     // KXC_HIP_QPACK_*
    kxc_hip_qconv2d_desc desc;
    kxc_hip_buf w, wp;
    int32_t every_run = 0;
    const void* packed_from = nullptr;    // the weight pointer whose packed form wp holds
};

int64_t PoolOutDim(const kxc_hip_pool2d_desc& d, int64_t in, int64_t k, int64_t s, int64_t p0, int64_t p1) {
    const int64_t span = in + p0 + p1 - k;
    if (span < 0 || s <= 0) return 0;
    return (d.ceil_mode ? (span + s - 1) / s : span / s) + 1;      // as the pooling entry points size their output
}

// Bytes of every operand whose size follows from the node's geometry (module kernels' parameters are checked by
// offset only).
void OperandExtents(const Node& n, std::vector<std::pair<kxc_hip_buf, size_t>>* out) {
    auto add = [&](const kxc_hip_buf& b, int64_t elems, size_t elem_bytes = 4) {
        if (b.kind != KXC_HIP_BUF_NONE && elems > 0) out->emplace_back(b, static_cast<size_t>(elems) * elem_bytes);
    };
    switch (n.kind) {
        case NodeKind::kConv2D: {
            const kxc_hip_conv2d_desc& d = n.conv;
            const int64_t oh = (static_cast<int64_t>(d.h) + 2 * d.pad_h - (static_cast<int64_t>(d.dil_h) * (d.kh - 1) + 1)) / d.stride_h + 1;
            const int64_t ow = (static_cast<int64_t>(d.w) + 2 * d.pad_w - (static_cast<int64_t>(d.dil_w) * (d.kw - 1) + 1)) / d.stride_w + 1;
            // (KXC_HIP_CONV_HPOOL: the output is pooled along W, half as wide)
            const int64_t y = static_cast<int64_t>(d.n) * d.o * oh * ((d.flags & KXC_HIP_CONV_HPOOL) ? ow / 2 : ow);
            add(n.bufs[0], static_cast<int64_t>(d.n) * d.c * d.h * d.w);
            add(n.bufs[1], static_cast<int64_t>(d.o) * d.c * d.kh * d.kw);
            add(n.bufs[2], d.o);
            add(n.bufs[3], y);
            add(n.bufs[4], y);
            if (n.i32[0] == 1) {
                size_t u = 0;
                if (kxc_hip_conv2d_winograd_weight_bytes(&d, &u) == KXC_HIP_OK) add(n.bufs[5], static_cast<int64_t>(u), 1);
            }
            if (n.i32[0] == 2 && n.params.size() == 3) {
                add(n.params[0], static_cast<int64_t>(d.o) * d.c);
                add(n.params[1], d.o);
                add(n.params[2], y);
            }
            break;
        }
        case NodeKind::kPool2D: {
            const kxc_hip_pool2d_desc& d = n.pool;
            add(n.bufs[0], static_cast<int64_t>(d.n) * d.c * d.h * d.w);
            add(n.bufs[1], static_cast<int64_t>(d.n) * d.c * PoolOutDim(d, d.h, d.kh, d.stride_h, d.pad_top, d.pad_bottom) *
                               PoolOutDim(d, d.w, d.kw, d.stride_w, d.pad_left, d.pad_right));
            break;
        }
        case NodeKind::kMaxPoolI8: {
            // i32[0] == 1: channel-blocked (16 bytes per position and block of 16 channels)
            const kxc_hip_pool2d_desc& d = n.pool;
            const int64_t cbytes = n.i32[0] == 1 ? (static_cast<int64_t>(d.c) + 15) / 16 * 16 : d.c;
            add(n.bufs[0], static_cast<int64_t>(d.n) * cbytes * d.h * d.w, 1);
            add(n.bufs[1], static_cast<int64_t>(d.n) * cbytes * PoolOutDim(d, d.h, d.kh, d.stride_h, d.pad_top, d.pad_bottom) *
                               PoolOutDim(d, d.w, d.kw, d.stride_w, d.pad_left, d.pad_right), 1);
            break;
        }
        case NodeKind::kGlobalAvgPoolI8: {
            const int64_t cbytes = n.i32[0] == 1 ? (n.dims[1] + 15) / 16 * 16 : n.dims[1];
            add(n.bufs[0], n.dims[0] * cbytes * n.dims[2] * n.dims[3], 1);
            add(n.bufs[1], n.dims[0] * cbytes, 1);
            break;
        }
        case NodeKind::kQuantize:
            if (n.i32[0] == 0) {
                add(n.bufs[0], n.dims[0]);
                add(n.bufs[1], n.dims[0], 1);
            } else {
                // dims = {n, c, h*w}; i32[0] == 1: c16 output, 2: c4 output
                add(n.bufs[0], n.dims[0] * n.dims[1] * n.dims[2]);
                add(n.bufs[1], n.dims[0] * (n.i32[0] == 1 ? (n.dims[1] + 15) / 16 * 16 : 4) * n.dims[2], 1);
            }
            break;
        case NodeKind::kI8Layout: {
            // dims = {n, c, h*w}; i32[0] != 0: NCHW -> c16
            const int64_t plain = n.dims[0] * n.dims[1] * n.dims[2], blocked = n.dims[0] * ((n.dims[1] + 15) / 16 * 16) * n.dims[2];
            add(n.bufs[0], n.i32[0] ? plain : blocked, 1);
            add(n.bufs[1], n.i32[0] ? blocked : plain, 1);
            break;
        }
        case NodeKind::kQDense:
            add(n.bufs[0], n.dims[0] * n.dims[2], 1);
            add(n.bufs[1], n.dims[1] * n.dims[2], 1);
            add(n.bufs[2], n.dims[1]);
            add(n.bufs[3], n.dims[1]);
            add(n.bufs[4], n.dims[0] * n.dims[1]);
            break;
        case NodeKind::kQConv2D: {
            // i32[0]: 0 NCHW, 1 c16, 2 c4 input / c16 output, 3 c16 with a second output (params),
            // 4 c4 input / c16 output max-pooled 3x3 / 2 / 1 in the same kernel
            const kxc_hip_qconv2d_desc& d = n.qconv;
            if (d.stride_h <= 0 || d.stride_w <= 0) break;
            const int64_t oh = (static_cast<int64_t>(d.h) + 2 * d.pad_h - d.kh) / d.stride_h + 1;
            const int64_t ow = (static_cast<int64_t>(d.w) + 2 * d.pad_w - d.kw) / d.stride_w + 1;
            const int mode = n.i32[0];
            const int64_t ob = mode == 0 ? d.o : (static_cast<int64_t>(d.o) + 15) / 16 * 16;
            const int64_t y = mode == 4 ? static_cast<int64_t>(d.n) * ob * ((oh - 1) / 2 + 1) * ((ow - 1) / 2 + 1)
                                        : static_cast<int64_t>(d.n) * ob * oh * ow;
            const int64_t xc = mode == 0 ? d.c : (mode == 2 || mode == 4) ? 4 : (static_cast<int64_t>(d.c) + 15) / 16 * 16;
            add(n.bufs[0], static_cast<int64_t>(d.n) * xc * d.h * d.w, 1);
            size_t wbytes = static_cast<size_t>(d.o) * d.c * d.kh * d.kw;
            if (mode == 1 || mode == 3) { if (kxc_hip_qconv2d_c16_packed_bytes(&d, &wbytes) != KXC_HIP_OK) wbytes = 0; }
            if (mode == 2 || mode == 4) { if (kxc_hip_qconv2d_c4_packed_bytes(&d, &wbytes) != KXC_HIP_OK) wbytes = 0; }
            add(n.bufs[1], static_cast<int64_t>(wbytes), 1);
            add(n.bufs[2], d.o);
            add(n.bufs[3], d.o);
            add(n.bufs[4], y, 1);
            add(n.bufs[5], y, 1);
            if (mode == 3 && n.params.size() == 4) {
                size_t w2 = 0;
                if (kxc_hip_qconv2d_c16_pair_packed_bytes(&d, &w2) == KXC_HIP_OK) add(n.params[0], static_cast<int64_t>(w2), 1);
                add(n.params[1], d.o);
                add(n.params[2], d.o);
                add(n.params[3], y, 1);
            }
            break;
        }
        case NodeKind::kGlobalAvgPool:
            add(n.bufs[0], n.dims[0] * n.dims[1] * n.dims[2] * n.dims[3]);
            add(n.bufs[1], n.dims[0] * n.dims[1]);
            break;
        case NodeKind::kGemm:
            add(n.bufs[0], n.dims[0] * n.dims[2]);
            add(n.bufs[1], n.dims[1] * n.dims[2]);
            add(n.bufs[2], n.dims[3]);
            add(n.bufs[3], n.dims[0] * n.dims[1]);
            break;
        case NodeKind::kBinary: {
            int64_t a = 1, b = 1;
            for (int i = 0; i < n.i32[1]; ++i) a *= n.a_shape[i];
            for (int i = 0; i < n.i32[2]; ++i) b *= n.b_shape[i];
            add(n.bufs[0], a);
            add(n.bufs[1], b);
            add(n.bufs[2], a > b ? a : b);      // (the broadcast result is at least as large as either operand)
            break;
        }
        case NodeKind::kRelu:
            add(n.bufs[0], n.dims[0]);
            add(n.bufs[1], n.dims[0]);
            break;
        case NodeKind::kCopy:
            add(n.bufs[0], n.dims[0], 1);
            add(n.bufs[1], n.dims[0], 1);
            break;
        default:
            break;
    }
}

}  // namespace

constexpr int32_t kMaxChains = 7;

struct kxc_hip_plan {
    int32_t device_id = 0;
    int32_t num_args = 0;
    std::vector<Node> nodes;
    std::vector<PackJob> packs;
    void* workspace = nullptr;
    size_t workspace_bytes = 0;
    bool finalized = false;
    hipStream_t side_stream = nullptr;     // created at finalize when a node uses lane 1 (default priority)
    // chains (kxc_hip_plan_set_chain): one stream and one end-of-chain event each, one fork event for all
    hipStream_t chain_streams[kMaxChains] = {};
    hipEvent_t chain_done[kMaxChains] = {};
    hipEvent_t chain_fork = nullptr;
    int32_t num_chains = 0;
    // number of equal launches the convolution variants were chosen for (the chains run side by side)
    int32_t select_lanes = 1;
    // HIP graph replay (kxc_hip_plan_enable_graph): the run after the first one on a capturable stream is
    // captured; later runs with the same argument pointers launch the instantiated graph
    bool graph_enabled = false;
    int eager_runs = 0;
    hipStream_t eager_stream = nullptr;   // stream of the last eager run (scratch buffers are per stream)
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    std::vector<void*> graph_args;
    hipStream_t graph_stream = nullptr;   // the graph is replayed only on the stream it was captured on
    // Constants of Winograd nodes and of the int8 matrix-core convolutions (packs).  Default: the filter transforms
    // of all such nodes run at the start of EVERY run (one launch each kind), so weights rewritten in place -- or another tensor at the same address -- are seen, as
    // with the CPU backend, which re-reads every constant on every call.  Frozen (kxc_hip_plan_freeze_constants):
    // transformed when first seen or when another pointer arrives; constants_ready orders runs on other streams
    // after the stream the transforms were enqueued on.
    bool constants_frozen = false;
    hipEvent_t constants_ready = nullptr;
    bool constants_recorded = false;
    hipStream_t constants_stream = nullptr;
};

namespace {

int32_t CheckBuf(const kxc_hip_plan* p, kxc_hip_buf b, bool optional, const char* who) {
    if (b.kind == KXC_HIP_BUF_NONE) {
        KXC_HIP_REQUIRE(optional, "%s: a required operand is absent", who);
        return KXC_HIP_OK;
    }
    if (b.kind == KXC_HIP_BUF_ARG) {
        KXC_HIP_REQUIRE(b.index_or_offset >= 0 && b.index_or_offset < p->num_args,
                        "%s: packed argument index %lld out of range [0,%d)", who,
                        static_cast<long long>(b.index_or_offset), p->num_args);
        return KXC_HIP_OK;
    }
    if (b.kind == KXC_HIP_BUF_ARG_OFFSET) {
        const int64_t arg = b.index_or_offset >> 48, off = b.index_or_offset & ((int64_t{1} << 48) - 1);
        KXC_HIP_REQUIRE(b.index_or_offset >= 0 && arg < p->num_args, "%s: packed argument index %lld out of range [0,%d)", who,
                        static_cast<long long>(arg), p->num_args);
        KXC_HIP_REQUIRE(off % 16 == 0, "%s: the byte offset into a packed argument must be a multiple of 16", who);
        return KXC_HIP_OK;
    }
    KXC_HIP_REQUIRE(b.kind == KXC_HIP_BUF_WORKSPACE, "%s: bad buffer kind %d", who, b.kind);
    KXC_HIP_REQUIRE(b.index_or_offset >= 0 && (b.index_or_offset % 256) == 0,
                    "%s: workspace offsets must be non-negative multiples of 256", who);
    return KXC_HIP_OK;
}

inline void* Resolve(const kxc_hip_plan* p, kxc_hip_buf b, void** args) {
    if (b.kind == KXC_HIP_BUF_ARG) return args[b.index_or_offset];
    if (b.kind == KXC_HIP_BUF_WORKSPACE) return static_cast<char*>(p->workspace) + b.index_or_offset;
    if (b.kind == KXC_HIP_BUF_ARG_OFFSET)
        return static_cast<char*>(args[b.index_or_offset >> 48]) + (b.index_or_offset & ((int64_t{1} << 48) - 1));
    return nullptr;
}

int32_t Begin(kxc_hip_plan* p, const char* who) {
    KXC_HIP_REQUIRE(p != nullptr, "%s: plan is NULL", who);
    KXC_HIP_REQUIRE(!p->finalized, "%s: plan is already finalized", who);
    return KXC_HIP_OK;
}

}  // namespace

#define KXC_PLAN_BEGIN(who) if (int32_t _rc = Begin(plan, who)) return _rc
#define KXC_PLAN_BUF(b, optional, who) if (int32_t _rc = CheckBuf(plan, b, optional, who)) return _rc

extern "C" {

int32_t kxc_hip_plan_create(int32_t device_id, int32_t num_packed_args, kxc_hip_plan** out) {
    KXC_HIP_REQUIRE(out != nullptr, "kxc_hip_plan_create: out is NULL");
    KXC_HIP_REQUIRE(num_packed_args >= 0, "kxc_hip_plan_create: negative argument count");
    kxc_hip_plan* p = new kxc_hip_plan();
    p->device_id = device_id;
    p->num_args = num_packed_args;
    *out = p;
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_destroy(kxc_hip_plan* plan) {
    if (!plan) return KXC_HIP_OK;
    hipError_t e = hipSuccess;
    if (plan->workspace) e = hipFree(plan->workspace);
    for (Node& n : plan->nodes) {
        if (n.fork_event) (void)hipEventDestroy(n.fork_event);
        if (n.done_event) (void)hipEventDestroy(n.done_event);
    }
    if (plan->side_stream) (void)hipStreamDestroy(plan->side_stream);
    for (int32_t c = 0; c < kMaxChains; ++c) {
        if (plan->chain_streams[c]) (void)hipStreamDestroy(plan->chain_streams[c]);
        if (plan->chain_done[c]) (void)hipEventDestroy(plan->chain_done[c]);
    }
    if (plan->chain_fork) (void)hipEventDestroy(plan->chain_fork);
    if (plan->constants_ready) (void)hipEventDestroy(plan->constants_ready);
    if (plan->graph_exec) (void)hipGraphExecDestroy(plan->graph_exec);
    if (plan->graph) (void)hipGraphDestroy(plan->graph);
    delete plan;
    KXC_HIP_CALL(e, "plan workspace free");
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_conv2d(kxc_hip_plan* plan, const kxc_hip_conv2d_desc* desc, kxc_hip_buf x, kxc_hip_buf w,
                                kxc_hip_buf bias, kxc_hip_buf residual, kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_conv2d";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(desc != nullptr, "%s: desc is NULL", who);
    KXC_PLAN_BUF(x, false, who); KXC_PLAN_BUF(w, false, who); KXC_PLAN_BUF(y, false, who);
    KXC_PLAN_BUF(bias, !(desc->flags & KXC_HIP_CONV_BIAS), who);
    KXC_PLAN_BUF(residual, !(desc->flags & KXC_HIP_CONV_RESIDUAL), who);
    KXC_HIP_REQUIRE(!(desc->flags & KXC_HIP_CONV_HPOOL) || kxc_hip_conv2d_hpool_supported(desc),
                    "%s: no kernel with the pooling epilogue covers this shape", who);
    Node n{};
    n.kind = NodeKind::kConv2D;
    n.conv = *desc;
    n.bufs[0] = x; n.bufs[1] = w; n.bufs[2] = bias; n.bufs[3] = residual; n.bufs[4] = y;
    n.symbol = std::string("kxc_conv2d_nchw_f32.") + kxc_hip_conv2d_variant(desc);
    if (desc->flags & KXC_HIP_CONV_BIAS) n.symbol += "+bias";
    if (desc->flags & KXC_HIP_CONV_RESIDUAL) n.symbol += "+add";
    if (desc->flags & KXC_HIP_CONV_RELU) n.symbol += "+relu";
    if (desc->flags & KXC_HIP_CONV_HPOOL) n.symbol += "+maxpool3w";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_conv2d_winograd(kxc_hip_plan* plan, const kxc_hip_conv2d_desc* desc, kxc_hip_buf x, kxc_hip_buf w,
                                         kxc_hip_buf bias, kxc_hip_buf residual, kxc_hip_buf y, kxc_hip_buf u) {
    const char* who = "kxc_hip_plan_add_conv2d_winograd";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(desc != nullptr, "%s: desc is NULL", who);
    KXC_HIP_REQUIRE(kxc_hip_conv2d_winograd_supported(desc), "%s: not a 3x3 stride-1 convolution with c %% 4 == 0", who);
    KXC_HIP_REQUIRE(!(desc->flags & KXC_HIP_CONV_HPOOL), "%s: the pooling epilogue belongs to kxc_hip_plan_add_conv2d", who);
    KXC_HIP_REQUIRE(u.kind == KXC_HIP_BUF_WORKSPACE, "%s: the transformed weights live in the plan workspace", who);
    KXC_PLAN_BUF(u, false, who);
    if (int32_t rc = kxc_hip_plan_add_conv2d(plan, desc, x, w, bias, residual, y)) return rc;
    Node& n = plan->nodes.back();
    n.i32[0] = 1;
    n.bufs[5] = u;
    n.symbol = std::string("kxc_conv2d_nchw_f32.") + kxc_hip_conv2d_winograd_variant(desc);
    if (desc->flags & KXC_HIP_CONV_BIAS) n.symbol += "+bias";
    if (desc->flags & KXC_HIP_CONV_RESIDUAL) n.symbol += "+add";
    if (desc->flags & KXC_HIP_CONV_RELU) n.symbol += "+relu";
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_conv2d_pair(kxc_hip_plan* plan, const kxc_hip_conv2d_desc* desc, kxc_hip_buf x, kxc_hip_buf w,
                                     kxc_hip_buf bias, kxc_hip_buf residual, kxc_hip_buf y, kxc_hip_buf w2, kxc_hip_buf bias2,
                                     kxc_hip_buf y2) {
    const char* who = "kxc_hip_plan_add_conv2d_pair";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(desc != nullptr, "%s: desc is NULL", who);
    KXC_HIP_REQUIRE(kxc_hip_conv2d_pair_supported(desc), "%s: no kernel with a second output covers this shape", who);
    KXC_HIP_REQUIRE(!(desc->flags & KXC_HIP_CONV_HPOOL), "%s: the pooling epilogue belongs to kxc_hip_plan_add_conv2d", who);
    KXC_PLAN_BUF(w2, false, who); KXC_PLAN_BUF(bias2, true, who); KXC_PLAN_BUF(y2, false, who);
    if (int32_t rc = kxc_hip_plan_add_conv2d(plan, desc, x, w, bias, residual, y)) return rc;
    Node& n = plan->nodes.back();
    n.i32[0] = 2;                      // params = {w2, bias2, y2}
    n.params = {w2, bias2, y2};
    n.symbol = std::string("kxc_conv2d_nchw_f32.") + kxc_hip_conv2d_pair_variant(desc);
    if (desc->flags & KXC_HIP_CONV_BIAS) n.symbol += "+bias";
    if (desc->flags & KXC_HIP_CONV_RESIDUAL) n.symbol += "+add";
    if (desc->flags & KXC_HIP_CONV_RELU) n.symbol += "+relu";
    n.symbol += "|conv1x1";
    if (bias2.kind != KXC_HIP_BUF_NONE) n.symbol += "+bias";
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_invalidate_constants(kxc_hip_plan* plan) {
    KXC_HIP_REQUIRE(plan != nullptr, "kxc_hip_plan_invalidate_constants: plan is NULL");
    for (Node& n : plan->nodes) n.transformed_from = nullptr;
    for (PackJob& j : plan->packs) j.packed_from = nullptr;
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_freeze_constants(kxc_hip_plan* plan, int32_t frozen) {
    KXC_HIP_REQUIRE(plan != nullptr, "kxc_hip_plan_freeze_constants: plan is NULL");
    plan->constants_frozen = frozen != 0;
    for (Node& n : plan->nodes) n.transformed_from = nullptr;      // the next run transforms what it is given
    for (PackJob& j : plan->packs) j.packed_from = nullptr;
    if (plan->graph_exec) {       // a captured graph holds the other mode's launches
        (void)hipGraphExecDestroy(plan->graph_exec); plan->graph_exec = nullptr;
        if (plan->graph) { (void)hipGraphDestroy(plan->graph); plan->graph = nullptr; }
        plan->graph_args.clear();
        plan->graph_stream = nullptr;
    }
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_pool2d(kxc_hip_plan* plan, const kxc_hip_pool2d_desc* desc, kxc_hip_buf x, kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_pool2d";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(desc != nullptr, "%s: desc is NULL", who);
    KXC_PLAN_BUF(x, false, who); KXC_PLAN_BUF(y, false, who);
    Node n{};
    n.kind = NodeKind::kPool2D;
    n.pool = *desc;
    n.bufs[0] = x; n.bufs[1] = y;
    n.symbol = desc->is_avg ? "kxc_avg_pool2d_f32" : "kxc_max_pool2d_f32";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_global_avg_pool2d(kxc_hip_plan* plan, int64_t nn, int64_t c, int64_t h, int64_t w,
                                           kxc_hip_buf x, kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_global_avg_pool2d";
    KXC_PLAN_BEGIN(who);
    KXC_PLAN_BUF(x, false, who); KXC_PLAN_BUF(y, false, who);
    Node n{};
    n.kind = NodeKind::kGlobalAvgPool;
    n.dims[0] = nn; n.dims[1] = c; n.dims[2] = h; n.dims[3] = w;
    n.bufs[0] = x; n.bufs[1] = y;
    n.symbol = "kxc_global_avg_pool2d_f32";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_gemm(kxc_hip_plan* plan, int64_t m, int64_t nn, int64_t k, float alpha, float beta,
                              int32_t transB, int64_t c_len, kxc_hip_buf a, kxc_hip_buf b, kxc_hip_buf c, kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_gemm";
    KXC_PLAN_BEGIN(who);
    KXC_PLAN_BUF(a, false, who); KXC_PLAN_BUF(b, false, who); KXC_PLAN_BUF(c, true, who); KXC_PLAN_BUF(y, false, who);
    Node n{};
    n.kind = NodeKind::kGemm;
    n.dims[0] = m; n.dims[1] = nn; n.dims[2] = k; n.dims[3] = c_len;
    n.f[0] = alpha; n.f[1] = beta; n.i32[0] = transB;
    n.bufs[0] = a; n.bufs[1] = b; n.bufs[2] = c; n.bufs[3] = y;
    n.symbol = "kxc_gemm_f32";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_binary(kxc_hip_plan* plan, int32_t op, const int64_t* a_shape, int32_t a_ndim,
                                const int64_t* b_shape, int32_t b_ndim, int32_t relu, kxc_hip_buf a, kxc_hip_buf b,
                                kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_binary";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(op >= 0 && op <= 3 && a_ndim >= 0 && a_ndim <= 6 && b_ndim >= 0 && b_ndim <= 6, "%s: bad op or rank", who);
    KXC_HIP_REQUIRE((a_ndim == 0 || a_shape) && (b_ndim == 0 || b_shape), "%s: shape is NULL", who);
    KXC_PLAN_BUF(a, false, who); KXC_PLAN_BUF(b, false, who); KXC_PLAN_BUF(y, false, who);
    Node n{};
    n.kind = NodeKind::kBinary;
    n.i32[0] = op; n.i32[1] = a_ndim; n.i32[2] = b_ndim; n.i32[3] = relu;
    for (int i = 0; i < a_ndim; ++i) n.a_shape[i] = a_shape[i];
    for (int i = 0; i < b_ndim; ++i) n.b_shape[i] = b_shape[i];
    n.bufs[0] = a; n.bufs[1] = b; n.bufs[2] = y;
    static const char* names[4] = {"kxc_add_f32", "kxc_subtract_f32", "kxc_multiply_f32", "kxc_divide_f32"};
    n.symbol = names[op];
    if (relu) n.symbol += "+relu";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_relu(kxc_hip_plan* plan, int64_t count, kxc_hip_buf x, kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_relu";
    KXC_PLAN_BEGIN(who);
    KXC_PLAN_BUF(x, false, who); KXC_PLAN_BUF(y, false, who);
    Node n{};
    n.kind = NodeKind::kRelu;
    n.dims[0] = count;
    n.bufs[0] = x; n.bufs[1] = y;
    n.symbol = "kxc_relu_f32";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_copy(kxc_hip_plan* plan, int64_t nbytes, kxc_hip_buf x, kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_copy";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(nbytes >= 0, "%s: negative size", who);
    KXC_PLAN_BUF(x, false, who); KXC_PLAN_BUF(y, false, who);
    Node n{};
    n.kind = NodeKind::kCopy;
    n.dims[0] = nbytes;
    n.bufs[0] = x; n.bufs[1] = y;
    n.symbol = "kxc_copy";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_qconv2d(kxc_hip_plan* plan, const kxc_hip_qconv2d_desc* desc, kxc_hip_buf x, kxc_hip_buf w,
                                 kxc_hip_buf bias, kxc_hip_buf mult, kxc_hip_buf residual, kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_qconv2d";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(desc != nullptr, "%s: desc is NULL", who);
    KXC_PLAN_BUF(x, false, who); KXC_PLAN_BUF(w, false, who); KXC_PLAN_BUF(mult, false, who); KXC_PLAN_BUF(y, false, who);
    KXC_PLAN_BUF(bias, !(desc->flags & KXC_HIP_CONV_BIAS), who);
    KXC_PLAN_BUF(residual, !(desc->flags & KXC_HIP_CONV_RESIDUAL), who);
    Node n{};
    n.kind = NodeKind::kQConv2D;
    n.qconv = *desc;
    n.bufs[0] = x; n.bufs[1] = w; n.bufs[2] = bias; n.bufs[3] = mult; n.bufs[4] = residual; n.bufs[5] = y;
    n.symbol = "kxc_qconv2d_nchw_i8";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_quantize(kxc_hip_plan* plan, int64_t count, float scale, kxc_hip_buf x, kxc_hip_buf q) {
    const char* who = "kxc_hip_plan_add_quantize";
    KXC_PLAN_BEGIN(who);
    KXC_PLAN_BUF(x, false, who); KXC_PLAN_BUF(q, false, who);
    Node n{};
    n.kind = NodeKind::kQuantize;
    n.dims[0] = count; n.f[0] = scale;
    n.bufs[0] = x; n.bufs[1] = q;
    n.symbol = "kxc_quantize_f32_i8";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_maxpool2d_i8(kxc_hip_plan* plan, const kxc_hip_pool2d_desc* desc, kxc_hip_buf x, kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_maxpool2d_i8";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(desc != nullptr, "%s: desc is NULL", who);
    KXC_PLAN_BUF(x, false, who); KXC_PLAN_BUF(y, false, who);
    Node n{};
    n.kind = NodeKind::kMaxPoolI8;
    n.pool = *desc;
    n.bufs[0] = x; n.bufs[1] = y;
    n.symbol = "kxc_max_pool2d_i8";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_global_avg_pool2d_i8(kxc_hip_plan* plan, int64_t nn, int64_t c, int64_t h, int64_t w, float mult,
                                              kxc_hip_buf x, kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_global_avg_pool2d_i8";
    KXC_PLAN_BEGIN(who);
    KXC_PLAN_BUF(x, false, who); KXC_PLAN_BUF(y, false, who);
    Node n{};
    n.kind = NodeKind::kGlobalAvgPoolI8;
    n.dims[0] = nn; n.dims[1] = c; n.dims[2] = h; n.dims[3] = w; n.f[0] = mult;
    n.bufs[0] = x; n.bufs[1] = y;
    n.symbol = "kxc_global_avg_pool2d_i8";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_qdense(kxc_hip_plan* plan, int64_t m, int64_t nn, int64_t k, kxc_hip_buf a, kxc_hip_buf b,
                                kxc_hip_buf bias, kxc_hip_buf mult, kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_qdense";
    KXC_PLAN_BEGIN(who);
    KXC_PLAN_BUF(a, false, who); KXC_PLAN_BUF(b, false, who); KXC_PLAN_BUF(bias, true, who);
    KXC_PLAN_BUF(mult, false, who); KXC_PLAN_BUF(y, false, who);
    Node n{};
    n.kind = NodeKind::kQDense;
    n.dims[0] = m; n.dims[1] = nn; n.dims[2] = k;
    n.bufs[0] = a; n.bufs[1] = b; n.bufs[2] = bias; n.bufs[3] = mult; n.bufs[4] = y;
    n.symbol = "kxc_qdense_i8";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

// ---- the same int8 operators on the channel-blocked "c16" layout (qconv_c16_i8.hip); i32[0] = 1 marks them
int32_t kxc_hip_plan_add_qconv2d_c16(kxc_hip_plan* plan, const kxc_hip_qconv2d_desc* desc, kxc_hip_buf x,
                                     kxc_hip_buf w_packed, kxc_hip_buf bias, kxc_hip_buf mult, kxc_hip_buf residual,
                                     kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_qconv2d_c16";
    if (int32_t rc = kxc_hip_plan_add_qconv2d(plan, desc, x, w_packed, bias, mult, residual, y)) return rc;
    Node& n = plan->nodes.back();
    const char* variant = kxc_hip_qconv2d_c16_variant(desc);
    if (std::strcmp(variant, "none") == 0) {
        const std::string inner = LastError();
        plan->nodes.pop_back();
        return Fail(KXC_HIP_ERR_INVALID, "%s: %s", who, inner.c_str());
    }
    n.i32[0] = 1;
    n.symbol = std::string("kxc_qconv2d_c16_i8:") + variant;
    return KXC_HIP_OK;
}

// i32[0] = 3: the c16 convolution with a second output; params = {w2_packed, bias2, mult2, y2}
int32_t kxc_hip_plan_add_qconv2d_c16_pair(kxc_hip_plan* plan, const kxc_hip_qconv2d_desc* desc, kxc_hip_buf x,
                                          kxc_hip_buf w_packed, kxc_hip_buf bias, kxc_hip_buf mult, kxc_hip_buf residual,
                                          kxc_hip_buf y, kxc_hip_buf w2_packed, kxc_hip_buf bias2, kxc_hip_buf mult2,
                                          kxc_hip_buf y2) {
    const char* who = "kxc_hip_plan_add_qconv2d_c16_pair";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(desc != nullptr, "%s: desc is NULL", who);
    KXC_HIP_REQUIRE(kxc_hip_qconv2d_c16_pair_supported(desc), "%s: no kernel with a second output covers this shape", who);
    KXC_PLAN_BUF(w2_packed, false, who); KXC_PLAN_BUF(bias2, true, who); KXC_PLAN_BUF(mult2, false, who); KXC_PLAN_BUF(y2, false, who);
    if (int32_t rc = kxc_hip_plan_add_qconv2d_c16(plan, desc, x, w_packed, bias, mult, residual, y)) return rc;
    Node& n = plan->nodes.back();
    n.i32[0] = 3;
    n.params = {w2_packed, bias2, mult2, y2};
    n.symbol += "|qconv1x1";
    if (bias2.kind != KXC_HIP_BUF_NONE) n.symbol += "+bias";
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_qconv2d_c4(kxc_hip_plan* plan, const kxc_hip_qconv2d_desc* desc, kxc_hip_buf x_c4,
                                    kxc_hip_buf w_packed, kxc_hip_buf bias, kxc_hip_buf mult, kxc_hip_buf y_c16) {
    const char* who = "kxc_hip_plan_add_qconv2d_c4";
    KXC_HIP_REQUIRE(desc != nullptr, "%s: desc is NULL", who);
    KXC_HIP_REQUIRE(!(desc->flags & KXC_HIP_CONV_RESIDUAL), "%s: no residual operand on the first layer", who);
    size_t bytes = 0;
    if (int32_t rc = kxc_hip_qconv2d_c4_packed_bytes(desc, &bytes)) return rc;
    kxc_hip_buf none;
    none.kind = KXC_HIP_BUF_NONE; none.index_or_offset = 0;
    if (int32_t rc = kxc_hip_plan_add_qconv2d(plan, desc, x_c4, w_packed, bias, mult, none, y_c16)) return rc;
    Node& n = plan->nodes.back();
    n.i32[0] = 2;
    n.symbol = "kxc_qconv2d_c4_i8:qmfma_k7x7s2_c4";
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_qconv2d_c4_maxpool(kxc_hip_plan* plan, const kxc_hip_qconv2d_desc* desc, kxc_hip_buf x_c4,
                                            kxc_hip_buf w_packed, kxc_hip_buf bias, kxc_hip_buf mult, kxc_hip_buf y_c16) {
    const char* who = "kxc_hip_plan_add_qconv2d_c4_maxpool";
    KXC_HIP_REQUIRE(desc != nullptr, "%s: desc is NULL", who);
    KXC_HIP_REQUIRE(kxc_hip_qconv2d_c4_maxpool_supported(desc), "%s: the first-layer kernel with the pool does not cover this shape", who);
    if (int32_t rc = kxc_hip_plan_add_qconv2d_c4(plan, desc, x_c4, w_packed, bias, mult, y_c16)) return rc;
    Node& n = plan->nodes.back();
    n.i32[0] = 4;
    n.symbol = "kxc_qconv2d_c4_i8:qmfma_k7x7s2_c4+maxpool3x3s2";
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_quantize_c4(kxc_hip_plan* plan, int64_t nn, int64_t c, int64_t hw, float scale, kxc_hip_buf x,
                                     kxc_hip_buf q) {
    if (int32_t rc = kxc_hip_plan_add_quantize(plan, nn, scale, x, q)) return rc;
    Node& n = plan->nodes.back();
    n.dims[0] = nn; n.dims[1] = c; n.dims[2] = hw;
    n.i32[0] = 2;
    n.symbol = "kxc_quantize_f32_nchw_to_c4_i8";
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_quantize_c16(kxc_hip_plan* plan, int64_t nn, int64_t c, int64_t hw, float scale, kxc_hip_buf x,
                                      kxc_hip_buf q) {
    if (int32_t rc = kxc_hip_plan_add_quantize(plan, nn, scale, x, q)) return rc;
    Node& n = plan->nodes.back();
    n.dims[0] = nn; n.dims[1] = c; n.dims[2] = hw;
    n.i32[0] = 1;
    n.symbol = "kxc_quantize_f32_nchw_to_c16_i8";
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_maxpool2d_c16_i8(kxc_hip_plan* plan, const kxc_hip_pool2d_desc* desc, kxc_hip_buf x,
                                          kxc_hip_buf y) {
    if (int32_t rc = kxc_hip_plan_add_maxpool2d_i8(plan, desc, x, y)) return rc;
    Node& n = plan->nodes.back();
    n.i32[0] = 1;
    n.symbol = "kxc_max_pool2d_c16_i8";
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_global_avg_pool2d_c16_i8(kxc_hip_plan* plan, int64_t nn, int64_t c, int64_t h, int64_t w,
                                                  float mult, kxc_hip_buf x, kxc_hip_buf y) {
    if (int32_t rc = kxc_hip_plan_add_global_avg_pool2d_i8(plan, nn, c, h, w, mult, x, y)) return rc;
    Node& n = plan->nodes.back();
    n.i32[0] = 1;
    n.symbol = "kxc_global_avg_pool2d_c16_i8";
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_i8_layout(kxc_hip_plan* plan, int32_t to_c16, int64_t nn, int64_t c, int64_t hw, kxc_hip_buf x,
                                   kxc_hip_buf y) {
    const char* who = "kxc_hip_plan_add_i8_layout";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(nn >= 0 && c > 0 && hw >= 0, "%s: bad shape", who);
    KXC_PLAN_BUF(x, false, who); KXC_PLAN_BUF(y, false, who);
    Node n{};
    n.kind = NodeKind::kI8Layout;
    n.dims[0] = nn; n.dims[1] = c; n.dims[2] = hw;
    n.i32[0] = to_c16 ? 1 : 0;
    n.bufs[0] = x; n.bufs[1] = y;
    n.symbol = to_c16 ? "kxc_i8_nchw_to_c16" : "kxc_i8_c16_to_nchw";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_add_qconv_weight_pack(kxc_hip_plan* plan, int32_t kind, const kxc_hip_qconv2d_desc* desc,
                                           kxc_hip_buf w_oihw, kxc_hip_buf w_packed, int32_t every_run) {
    const char* who = "kxc_hip_plan_add_qconv_weight_pack";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(desc != nullptr, "%s: desc is NULL", who);
    KXC_HIP_REQUIRE(w_oihw.kind == KXC_HIP_BUF_ARG || w_oihw.kind == KXC_HIP_BUF_ARG_OFFSET,
                    "%s: the weights must be a packed argument (they are read before the first node runs)", who);
    KXC_HIP_REQUIRE(w_packed.kind == KXC_HIP_BUF_WORKSPACE, "%s: the packed weights live in the plan workspace", who);
    KXC_PLAN_BUF(w_oihw, false, who); KXC_PLAN_BUF(w_packed, false, who);
    PackJob j;
    j.kind = kind; j.desc = *desc; j.w = w_oihw; j.wp = w_packed; j.every_run = every_run ? 1 : 0;
    size_t bytes = 0;
    const QPackJob probe{kind, desc, nullptr, nullptr};
    if (int32_t rc = QPackedBytes(probe, &bytes)) return rc;
    plan->packs.push_back(j);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_num_weight_packs(const kxc_hip_plan* plan) { return plan ? static_cast<int32_t>(plan->packs.size()) : 0; }

int32_t kxc_hip_plan_add_module_kernel(kxc_hip_plan* plan, void* function, const char* symbol, const uint32_t grid[3],
                                       const uint32_t block[3], uint32_t shared_bytes, const kxc_hip_buf* params,
                                       int32_t num_params) {
    const char* who = "kxc_hip_plan_add_module_kernel";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(function && grid && block && num_params >= 0 && (num_params == 0 || params), "%s: NULL argument", who);
    KXC_HIP_REQUIRE(grid[0] > 0 && grid[1] > 0 && grid[2] > 0 && block[0] > 0 && block[1] > 0 && block[2] > 0,
                    "%s: empty grid or block", who);
    KXC_HIP_REQUIRE(static_cast<uint64_t>(block[0]) * block[1] * block[2] <= 1024, "%s: more than 1024 threads per block", who);
    Node n{};
    n.kind = NodeKind::kModuleKernel;
    n.function = function;
    for (int i = 0; i < 3; ++i) { n.grid[i] = grid[i]; n.block[i] = block[i]; }
    n.shared_bytes = shared_bytes;
    for (int i = 0; i < num_params; ++i) {
        KXC_PLAN_BUF(params[i], false, who);
        n.params.push_back(params[i]);
    }
    n.symbol = symbol ? symbol : "kxc_module_kernel";
    plan->nodes.push_back(n);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_finalize(kxc_hip_plan* plan, size_t workspace_bytes) {
    KXC_HIP_REQUIRE(plan != nullptr, "kxc_hip_plan_finalize: plan is NULL");
    KXC_HIP_REQUIRE(!plan->finalized, "kxc_hip_plan_finalize: plan is already finalized");
    // every workspace operand whose size the node's geometry fixes must end inside the workspace
    for (const Node& n : plan->nodes) {
        std::vector<std::pair<kxc_hip_buf, size_t>> extents;
        OperandExtents(n, &extents);
        for (const auto& e : extents) {
            if (e.first.kind != KXC_HIP_BUF_WORKSPACE) continue;
            const size_t off = static_cast<size_t>(e.first.index_or_offset);
            KXC_HIP_REQUIRE(off <= workspace_bytes && e.second <= workspace_bytes - off,
                            "kxc_hip_plan_finalize: node %s: an operand of %zu bytes at workspace offset %zu does not fit the "
                            "%zu-byte workspace", n.symbol.c_str(), e.second, off, workspace_bytes);
        }
    }
    for (const Node& n : plan->nodes) {
        auto check = [&](kxc_hip_buf b) {
            return !(b.kind == KXC_HIP_BUF_WORKSPACE && static_cast<size_t>(b.index_or_offset) >= workspace_bytes &&
                     workspace_bytes > 0) &&
                   !(b.kind == KXC_HIP_BUF_WORKSPACE && workspace_bytes == 0);
        };
        for (const kxc_hip_buf& b : n.bufs)
            KXC_HIP_REQUIRE(b.kind != KXC_HIP_BUF_WORKSPACE || check(b),
                            "kxc_hip_plan_finalize: node %s uses a workspace offset beyond %zu bytes", n.symbol.c_str(),
                            workspace_bytes);
        for (const kxc_hip_buf& b : n.params)
            KXC_HIP_REQUIRE(b.kind != KXC_HIP_BUF_WORKSPACE || check(b),
                            "kxc_hip_plan_finalize: node %s uses a workspace offset beyond %zu bytes", n.symbol.c_str(),
                            workspace_bytes);
    }
    for (const PackJob& j : plan->packs) {
        size_t bytes = 0;
        const QPackJob probe{j.kind, &j.desc, nullptr, nullptr};
        if (int32_t rc = QPackedBytes(probe, &bytes)) return rc;
        const size_t off = static_cast<size_t>(j.wp.index_or_offset);
        KXC_HIP_REQUIRE(off <= workspace_bytes && bytes <= workspace_bytes - off,
                        "kxc_hip_plan_finalize: packed weights of %zu bytes at workspace offset %zu do not fit the %zu-byte workspace",
                        bytes, off, workspace_bytes);
    }
    // the variants below are chosen for select_lanes equal launches side by side
    struct LanesScope {
        int32_t prev;
        explicit LanesScope(int32_t lanes) : prev(kxc_hip_set_select_lanes(lanes)) {}
        ~LanesScope() { kxc_hip_set_select_lanes(prev); }
    } lanes_scope(plan->select_lanes);
    // Resolve every convolution launch now: the runs only add the operand pointers and the stream.  The node's
    // symbol names the variant resolved here (the one chosen when the node was added may have been picked under
    // other environment switches).  (Before anything is allocated: a failure here leaves nothing behind.)
    for (Node& n : plan->nodes) {
        if (n.kind != NodeKind::kConv2D) continue;
        KXC_HIP_CALL(hipSetDevice(plan->device_id), "HIP SetDevice");
        {
            const std::string prefix = "kxc_conv2d_nchw_f32.";
            const char* variant = n.i32[0] == 1   ? kxc_hip_conv2d_winograd_variant(&n.conv)
                                  : n.i32[0] == 2 ? kxc_hip_conv2d_pair_variant(&n.conv)
                                                  : kxc_hip_conv2d_variant(&n.conv);
            const size_t end = n.symbol.find_first_of("+|", prefix.size());
            if (n.symbol.compare(0, prefix.size(), prefix) == 0)
                n.symbol = prefix + variant + (end == std::string::npos ? std::string() : n.symbol.substr(end));
        }
        if (n.i32[0] == 1) {
            kxc_hip::PreparedWinograd* p = nullptr;
            if (int32_t rc = kxc_hip::PrepareWinograd(&n.conv, &p)) return rc;
            n.prepared_wino.reset(p, kxc_hip::FreePreparedWinograd);
        } else {
            kxc_hip::PreparedConv* p = nullptr;
            if (int32_t rc = kxc_hip::PrepareConv2d(&n.conv, n.i32[0] == 2, &p)) return rc;
            n.prepared_conv.reset(p, kxc_hip::FreePreparedConv);
        }
    }
    // Streams, events and the workspace: what a failed call has created so far is kept by the plan and reused by a
    // second call (kxc_hip_plan_destroy releases it either way).
    for (Node& n : plan->nodes) {
        if (n.lane != 1) continue;
        if (!plan->side_stream) {
            KXC_HIP_CALL(hipSetDevice(plan->device_id), "HIP SetDevice");
            KXC_HIP_CALL(hipStreamCreateWithFlags(&plan->side_stream, hipStreamNonBlocking), "plan side stream");
        }
        if (!n.fork_event) KXC_HIP_CALL(hipEventCreateWithFlags(&n.fork_event, hipEventDisableTiming), "plan event");
        if (!n.done_event) KXC_HIP_CALL(hipEventCreateWithFlags(&n.done_event, hipEventDisableTiming), "plan event");
    }
    for (const Node& n : plan->nodes) plan->num_chains = std::max(plan->num_chains, n.chain);
    if (plan->num_chains > 0) {
        KXC_HIP_CALL(hipSetDevice(plan->device_id), "HIP SetDevice");
        if (!plan->chain_fork) KXC_HIP_CALL(hipEventCreateWithFlags(&plan->chain_fork, hipEventDisableTiming), "plan event");
        for (int32_t c = 0; c < plan->num_chains; ++c) {
            if (!plan->chain_streams[c])
                KXC_HIP_CALL(hipStreamCreateWithFlags(&plan->chain_streams[c], hipStreamNonBlocking), "plan chain stream");
            if (!plan->chain_done[c]) KXC_HIP_CALL(hipEventCreateWithFlags(&plan->chain_done[c], hipEventDisableTiming), "plan event");
        }
    }
    if (workspace_bytes > 0 && !plan->workspace) {
        KXC_HIP_CALL(hipSetDevice(plan->device_id), "HIP SetDevice");
        KXC_HIP_CALL(hipMalloc(&plan->workspace, workspace_bytes), "plan workspace allocation");
        NoteDeviceAllocation();
    }
    plan->workspace_bytes = workspace_bytes;
    plan->finalized = true;
    return KXC_HIP_OK;
}

}  // extern "C"

namespace {

int32_t CheckRunArgs(kxc_hip_plan* plan, void** args, const char* who) {
    KXC_HIP_REQUIRE(plan != nullptr, "%s: plan is NULL", who);
    KXC_HIP_REQUIRE(plan->finalized, "%s: plan is not finalized", who);
    KXC_HIP_REQUIRE(plan->num_args == 0 || args != nullptr, "%s: packed_args is NULL", who);
    for (int i = 0; i < plan->num_args; ++i)
        KXC_HIP_REQUIRE(args[i] != nullptr, "%s: packed argument %d is NULL", who, i);
    return KXC_HIP_OK;
}

// The filter transforms of the plan's Winograd nodes and the weight packs of its int8 convolutions, each kind in one
// launch on `stream`: every one (only_changed: those whose weight pointer differs from the one last prepared, and the
// packs marked every_run).  *launched tells whether anything ran.  What was prepared is recorded only after its
// launch has been enqueued without error, so a failed run is repeated by the next one.
int32_t TransformConstants(kxc_hip_plan* plan, void** args, hipStream_t stream, bool only_changed, bool* launched) {
    std::vector<WinoWeightJob> jobs;
    std::vector<std::pair<Node*, const void*>> touched;
    for (Node& n : plan->nodes) {
        if (n.kind != NodeKind::kConv2D || n.i32[0] != 1) continue;
        const void* w = Resolve(plan, n.bufs[1], args);
        if (only_changed && n.transformed_from == w) continue;
        touched.emplace_back(&n, w);
        // (nodes of different chains that share a transformed-weight buffer: one transform)
        float* const u = static_cast<float*>(Resolve(plan, n.bufs[5], args));
        bool have = false;
        for (const WinoWeightJob& j : jobs) have = have || (j.u == u && j.w == w);
        if (!have) jobs.push_back({&n.conv, static_cast<const float*>(w), u});
    }
    std::vector<QPackJob> packs;
    std::vector<std::pair<PackJob*, const void*>> packed;
    for (PackJob& j : plan->packs) {
        const void* w = Resolve(plan, j.w, args);
        if (only_changed && !j.every_run && j.packed_from == w) continue;
        packed.emplace_back(&j, w);
        int8_t* const wp = static_cast<int8_t*>(Resolve(plan, j.wp, args));
        bool have = false;
        for (const QPackJob& q : packs) have = have || (q.wp == wp && q.w == w && q.kind == j.kind);
        if (!have) packs.push_back({j.kind, &j.desc, static_cast<const int8_t*>(w), wp});
    }
    *launched = !jobs.empty() || !packs.empty();
    if (!jobs.empty()) {
        if (int32_t rc = LaunchWinogradWeightTransforms(jobs.data(), static_cast<int32_t>(jobs.size()), stream)) return rc;
        for (auto& t : touched) t.first->transformed_from = t.second;
    }
    if (!packs.empty()) {
        if (int32_t rc = LaunchQWeightPacks(packs.data(), static_cast<int32_t>(packs.size()), stream)) return rc;
        for (auto& t : packed) t.first->packed_from = t.second;
    }
    return KXC_HIP_OK;
}

// Frozen constants: transform what has not been seen yet (outside any stream capture), and order a run on another
// stream after the transforms.
int32_t EnsureFrozenConstants(kxc_hip_plan* plan, void** args, hipStream_t stream) {
    bool launched = false;
    if (int32_t rc = TransformConstants(plan, args, stream, true, &launched)) return rc;
    if (launched) {
        if (!plan->constants_ready)
            KXC_HIP_CALL(hipEventCreateWithFlags(&plan->constants_ready, hipEventDisableTiming), "plan event");
        KXC_HIP_CALL(hipEventRecord(plan->constants_ready, stream), "hipEventRecord");
        plan->constants_recorded = true;
        plan->constants_stream = stream;
    } else if (plan->constants_recorded && plan->constants_stream != stream) {
        KXC_HIP_CALL(hipStreamWaitEvent(stream, plan->constants_ready, 0), "hipStreamWaitEvent");
    }
    return KXC_HIP_OK;
}

// Enqueues one node on stream s.
int32_t RunNode(kxc_hip_plan* plan, Node& n, void** args, void* s) {
    {
        int32_t rc = KXC_HIP_OK;
        auto B = [&](int i) { return Resolve(plan, n.bufs[i], args); };
        switch (n.kind) {
            case NodeKind::kConv2D:
                // (launches resolved at finalize; s is never NULL here)
                if (n.i32[0] == 1) {
                    // (the transformed weights in B(5) were written by TransformConstants at the start of the run)
                    rc = kxc_hip::LaunchPreparedWinograd(n.prepared_wino.get(), static_cast<const float*>(B(0)),
                                                         static_cast<const float*>(B(5)), static_cast<const float*>(B(2)),
                                                         static_cast<const float*>(B(3)), static_cast<float*>(B(4)),
                                                         kxc_hip::ResolveStream(s));
                    break;
                }
                {
                    const bool pair = n.i32[0] == 2;
                    rc = kxc_hip::LaunchPreparedConv2d(
                        n.prepared_conv.get(), static_cast<const float*>(B(0)), static_cast<const float*>(B(1)),
                        static_cast<const float*>(B(2)), static_cast<const float*>(B(3)), static_cast<float*>(B(4)),
                        pair ? static_cast<const float*>(Resolve(plan, n.params[0], args)) : nullptr,
                        pair ? static_cast<const float*>(Resolve(plan, n.params[1], args)) : nullptr,
                        pair ? static_cast<float*>(Resolve(plan, n.params[2], args)) : nullptr, kxc_hip::ResolveStream(s));
                }
                break;
            case NodeKind::kPool2D:
                rc = kxc_hip_pool2d_f32(&n.pool, static_cast<const float*>(B(0)), static_cast<float*>(B(1)), s);
                break;
            case NodeKind::kGlobalAvgPool:
                rc = kxc_hip_global_avg_pool2d_f32(static_cast<const float*>(B(0)), static_cast<float*>(B(1)), n.dims[0],
                                                   n.dims[1], n.dims[2], n.dims[3], s);
                break;
            case NodeKind::kGemm:
                rc = kxc_hip_gemm_f32(static_cast<const float*>(B(0)), static_cast<const float*>(B(1)),
                                      static_cast<const float*>(B(2)), static_cast<float*>(B(3)), n.dims[0], n.dims[1],
                                      n.dims[2], n.f[0], n.f[1], n.i32[0], n.dims[3], s);
                break;
            case NodeKind::kBinary:
                rc = kxc_hip_broadcast_binary_f32(n.i32[0], static_cast<const float*>(B(0)), n.a_shape, n.i32[1],
                                                  static_cast<const float*>(B(1)), n.b_shape, n.i32[2],
                                                  static_cast<float*>(B(2)), n.i32[3], s);
                break;
            case NodeKind::kRelu:
                rc = kxc_hip_relu_f32(static_cast<const float*>(B(0)), static_cast<float*>(B(1)), n.dims[0], s);
                break;
            case NodeKind::kCopy: {
                hipError_t e = hipMemcpyAsync(B(1), B(0), static_cast<size_t>(n.dims[0]), hipMemcpyDeviceToDevice,
                                              reinterpret_cast<hipStream_t>(s));
                if (e != hipSuccess) rc = Fail(KXC_HIP_ERR_RUNTIME, "plan copy failed: %s", hipGetErrorString(e));
                break;
            }
            case NodeKind::kQConv2D:
                if (n.i32[0] == 4) {
                    rc = kxc_hip_qconv2d_c4_maxpool_i8(&n.qconv, static_cast<const int8_t*>(B(0)), static_cast<const int8_t*>(B(1)),
                                                       static_cast<const int32_t*>(B(2)), static_cast<const float*>(B(3)),
                                                       static_cast<int8_t*>(B(5)), s);
                    break;
                }
                if (n.i32[0] == 2) {
                    rc = kxc_hip_qconv2d_c4_i8(&n.qconv, static_cast<const int8_t*>(B(0)), static_cast<const int8_t*>(B(1)),
                                               static_cast<const int32_t*>(B(2)), static_cast<const float*>(B(3)),
                                               static_cast<int8_t*>(B(5)), s);
                    break;
                }
                if (n.i32[0] == 3) {
                    rc = kxc_hip_qconv2d_c16_pair_i8(&n.qconv, static_cast<const int8_t*>(B(0)), static_cast<const int8_t*>(B(1)),
                                                     static_cast<const int32_t*>(B(2)), static_cast<const float*>(B(3)),
                                                     static_cast<const int8_t*>(B(4)), static_cast<int8_t*>(B(5)),
                                                     static_cast<const int8_t*>(Resolve(plan, n.params[0], args)),
                                                     static_cast<const int32_t*>(Resolve(plan, n.params[1], args)),
                                                     static_cast<const float*>(Resolve(plan, n.params[2], args)),
                                                     static_cast<int8_t*>(Resolve(plan, n.params[3], args)), s);
                    break;
                }
                if (n.i32[0] == 1) {
                    rc = kxc_hip_qconv2d_c16_i8(&n.qconv, static_cast<const int8_t*>(B(0)), static_cast<const int8_t*>(B(1)),
                                                static_cast<const int32_t*>(B(2)), static_cast<const float*>(B(3)),
                                                static_cast<const int8_t*>(B(4)), static_cast<int8_t*>(B(5)), s);
                    break;
                }
                rc = kxc_hip_qconv2d_nchw_i8(&n.qconv, static_cast<const int8_t*>(B(0)), static_cast<const int8_t*>(B(1)),
                                             static_cast<const int32_t*>(B(2)), static_cast<const float*>(B(3)),
                                             static_cast<const int8_t*>(B(4)), static_cast<int8_t*>(B(5)), s);
                break;
            case NodeKind::kQuantize:
                if (n.i32[0] == 2) {
                    rc = kxc_hip_quantize_f32_nchw_to_c4_i8(static_cast<const float*>(B(0)), static_cast<int8_t*>(B(1)),
                                                            n.dims[0], n.dims[1], n.dims[2], n.f[0], s);
                    break;
                }
                if (n.i32[0] == 1) {
                    rc = kxc_hip_quantize_f32_nchw_to_c16_i8(static_cast<const float*>(B(0)), static_cast<int8_t*>(B(1)),
                                                             n.dims[0], n.dims[1], n.dims[2], n.f[0], s);
                    break;
                }
                rc = kxc_hip_quantize_f32_i8(static_cast<const float*>(B(0)), static_cast<int8_t*>(B(1)), n.dims[0], n.f[0], s);
                break;
            case NodeKind::kMaxPoolI8:
                if (n.i32[0] == 1) {
                    rc = kxc_hip_maxpool2d_c16_i8(&n.pool, static_cast<const int8_t*>(B(0)), static_cast<int8_t*>(B(1)), s);
                    break;
                }
                rc = kxc_hip_maxpool2d_i8(&n.pool, static_cast<const int8_t*>(B(0)), static_cast<int8_t*>(B(1)), s);
                break;
            case NodeKind::kGlobalAvgPoolI8:
                if (n.i32[0] == 1) {
                    rc = kxc_hip_global_avg_pool2d_c16_i8(static_cast<const int8_t*>(B(0)), static_cast<int8_t*>(B(1)),
                                                          n.dims[0], n.dims[1], n.dims[2], n.dims[3], n.f[0], s);
                    break;
                }
                rc = kxc_hip_global_avg_pool2d_i8(static_cast<const int8_t*>(B(0)), static_cast<int8_t*>(B(1)), n.dims[0],
                                                  n.dims[1], n.dims[2], n.dims[3], n.f[0], s);
                break;
            case NodeKind::kQDense:
                rc = kxc_hip_qdense_i8(static_cast<const int8_t*>(B(0)), static_cast<const int8_t*>(B(1)),
                                       static_cast<const int32_t*>(B(2)), static_cast<const float*>(B(3)),
                                       static_cast<float*>(B(4)), n.dims[0], n.dims[1], n.dims[2], s);
                break;
            case NodeKind::kI8Layout:
                rc = n.i32[0] ? kxc_hip_i8_nchw_to_c16(static_cast<const int8_t*>(B(0)), static_cast<int8_t*>(B(1)), n.dims[0],
                                                       n.dims[1], n.dims[2], s)
                              : kxc_hip_i8_c16_to_nchw(static_cast<const int8_t*>(B(0)), static_cast<int8_t*>(B(1)), n.dims[0],
                                                       n.dims[1], n.dims[2], s);
                break;
            case NodeKind::kModuleKernel: {
                // every parameter is a device pointer; hipModuleLaunchKernel wants the address of each
                std::vector<void*> values(n.params.size());
                std::vector<void*> addrs(n.params.size());
                for (size_t i = 0; i < n.params.size(); ++i) {
                    values[i] = Resolve(plan, n.params[i], args);
                    addrs[i] = &values[i];
                }
                rc = kxc_hip_module_launch(n.function, n.grid, n.block, n.shared_bytes, s, addrs.data());
                break;
            }
        }
        if (rc != KXC_HIP_OK) {
            const std::string inner = LastError();
            return Fail(rc, "plan node %s: %s", n.symbol.c_str(), inner.c_str());
        }
    }
    return KXC_HIP_OK;
}

}  // namespace

extern "C" {

}  // extern "C"

namespace {

// Enqueues every node: main lane on `main_stream`, side-lane nodes on the plan's side stream between a fork and a
// join event (also the pattern stream capture records as parallel graph branches).
int32_t EnqueueAll(kxc_hip_plan* plan, void** args, hipStream_t main_stream) {
    void* s = static_cast<void*>(main_stream);
    if (!plan->constants_frozen) {
        bool launched = false;
        if (int32_t rc = TransformConstants(plan, args, main_stream, false, &launched)) return rc;
    }
    // chains: everything enqueued on the main stream so far happens before their first node
    if (plan->num_chains > 0) {
        KXC_HIP_CALL(hipEventRecord(plan->chain_fork, main_stream), "hipEventRecord");
        for (int32_t c = 0; c < plan->num_chains; ++c)
            KXC_HIP_CALL(hipStreamWaitEvent(plan->chain_streams[c], plan->chain_fork, 0), "hipStreamWaitEvent");
    }
    std::vector<Node*> unjoined;      // side-lane nodes the main lane has not waited for yet
    for (Node& n : plan->nodes) {
        if (n.chain > 0) {
            if (int32_t rc = RunNode(plan, n, args, plan->chain_streams[n.chain - 1])) return rc;
            continue;
        }
        if (n.lane == 1 && plan->side_stream) {
            // everything enqueued so far on the main lane happens before the side node; the side node then runs
            // concurrently with the main-lane nodes that follow, until a node marked `join`
            KXC_HIP_CALL(hipEventRecord(n.fork_event, main_stream), "hipEventRecord");
            KXC_HIP_CALL(hipStreamWaitEvent(plan->side_stream, n.fork_event, 0), "hipStreamWaitEvent");
            if (int32_t rc = RunNode(plan, n, args, plan->side_stream)) return rc;
            KXC_HIP_CALL(hipEventRecord(n.done_event, plan->side_stream), "hipEventRecord");
            unjoined.push_back(&n);
            continue;
        }
        if (n.join) {
            for (Node* side : unjoined) KXC_HIP_CALL(hipStreamWaitEvent(main_stream, side->done_event, 0), "hipStreamWaitEvent");
            unjoined.clear();
        }
        if (int32_t rc = RunNode(plan, n, args, s)) return rc;
    }
    for (Node* side : unjoined) KXC_HIP_CALL(hipStreamWaitEvent(main_stream, side->done_event, 0), "hipStreamWaitEvent");
    // ... and whatever follows on the main stream happens after their last
    for (int32_t c = 0; c < plan->num_chains; ++c) {
        KXC_HIP_CALL(hipEventRecord(plan->chain_done[c], plan->chain_streams[c]), "hipEventRecord");
        KXC_HIP_CALL(hipStreamWaitEvent(main_stream, plan->chain_done[c], 0), "hipStreamWaitEvent");
    }
    return KXC_HIP_OK;
}

void DropGraph(kxc_hip_plan* plan) {
    if (plan->graph_exec) (void)hipGraphExecDestroy(plan->graph_exec);
    if (plan->graph) (void)hipGraphDestroy(plan->graph);
    plan->graph_exec = nullptr;
    plan->graph = nullptr;
    plan->graph_args.clear();
    plan->graph_stream = nullptr;
}

}  // namespace

extern "C" {

int32_t kxc_hip_plan_run(kxc_hip_plan* plan, void** args, void* stream) {
    if (int32_t rc = CheckRunArgs(plan, args, "kxc_hip_plan_run")) return rc;
    hipStream_t main_stream = reinterpret_cast<hipStream_t>(stream ? stream : static_cast<void*>(CurrentStream()));
    if (plan->constants_frozen)
        if (int32_t rc = EnsureFrozenConstants(plan, args, main_stream)) return rc;
    // Graph replay needs a real stream (the null stream cannot be captured) and one eager run before the
    // capture, so that everything that allocates lazily (split-reduction scratch, function attributes) exists.
    // The captured kernels hold the addresses of that stream's scratch buffers, so a run on another stream
    // captures again.
    if (!plan->graph_enabled || main_stream == nullptr) return EnqueueAll(plan, args, main_stream);
    const std::vector<void*> now(args, args + plan->num_args);
    if (plan->graph_exec && now == plan->graph_args && plan->graph_stream == main_stream) {
        KXC_HIP_CALL(hipGraphLaunch(plan->graph_exec, main_stream), "hipGraphLaunch");
        return KXC_HIP_OK;
    }
    if (plan->eager_runs < 1 || plan->eager_stream != main_stream) {
        plan->eager_runs = 1;
        plan->eager_stream = main_stream;
        return EnqueueAll(plan, args, main_stream);
    }
    DropGraph(plan);
    KXC_HIP_CALL(hipStreamBeginCapture(main_stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
    const int32_t rc = EnqueueAll(plan, args, main_stream);
    hipGraph_t graph = nullptr;
    const hipError_t end = hipStreamEndCapture(main_stream, &graph);
    if (rc != KXC_HIP_OK) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc;
    }
    if (end != hipSuccess || graph == nullptr)
        return Fail(KXC_HIP_ERR_RUNTIME, "kxc_hip_plan_run: stream capture failed: %s", hipGetErrorString(end));
    plan->graph = graph;
    const hipError_t inst = hipGraphInstantiate(&plan->graph_exec, plan->graph, nullptr, nullptr, 0);
    if (inst != hipSuccess) {
        DropGraph(plan);
        return Fail(KXC_HIP_ERR_RUNTIME, "kxc_hip_plan_run: hipGraphInstantiate failed: %s", hipGetErrorString(inst));
    }
    plan->graph_args = now;
    plan->graph_stream = main_stream;
    KXC_HIP_CALL(hipGraphLaunch(plan->graph_exec, main_stream), "hipGraphLaunch");     // the capture itself ran nothing
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_enable_graph(kxc_hip_plan* plan, int32_t enable) {
    KXC_HIP_REQUIRE(plan != nullptr, "kxc_hip_plan_enable_graph: plan is NULL");
    plan->graph_enabled = enable != 0;
    if (!plan->graph_enabled) DropGraph(plan);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_set_concurrency(kxc_hip_plan* plan, int32_t node, int32_t lane, int32_t join) {
    const char* who = "kxc_hip_plan_set_concurrency";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(node >= 0 && node < static_cast<int32_t>(plan->nodes.size()), "%s: node %d out of range", who, node);
    KXC_HIP_REQUIRE((lane == 0 || lane == 1) && (join == 0 || join == 1) && !(lane == 1 && join == 1),
                    "%s: lane must be 0 or 1, join 0 or 1, and a side-lane node cannot join", who);
    plan->nodes[node].lane = lane;
    plan->nodes[node].join = join;
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_set_chain(kxc_hip_plan* plan, int32_t node, int32_t chain) {
    const char* who = "kxc_hip_plan_set_chain";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(node >= 0 && node < static_cast<int32_t>(plan->nodes.size()), "%s: node %d out of range", who, node);
    KXC_HIP_REQUIRE(chain >= 0 && chain <= kMaxChains, "%s: chain must be in [0, %d]", who, kMaxChains);
    KXC_HIP_REQUIRE(chain == 0 || (plan->nodes[node].lane == 0 && plan->nodes[node].join == 0),
                    "%s: a node of a chain takes no part in the side lane", who);
    plan->nodes[node].chain = chain;
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_interleave_chains(kxc_hip_plan* plan, int32_t* new_index, int32_t capacity) {
    const char* who = "kxc_hip_plan_interleave_chains";
    KXC_PLAN_BEGIN(who);
    const int32_t n = static_cast<int32_t>(plan->nodes.size());
    KXC_HIP_REQUIRE(new_index == nullptr || capacity >= n, "%s: room for %d indices, %d nodes", who, capacity, n);
    // round k takes the k-th node of the main lane, then the k-th node of every chain: each stream keeps its order
    std::vector<std::vector<int32_t>> by_chain(kMaxChains + 1);
    for (int32_t i = 0; i < n; ++i) by_chain[plan->nodes[i].chain].push_back(i);
    std::vector<int32_t> order;
    for (size_t k = 0; static_cast<int32_t>(order.size()) < n; ++k)
        for (const auto& c : by_chain)
            if (k < c.size()) order.push_back(c[k]);
    std::vector<Node> moved;
    moved.reserve(plan->nodes.size());
    for (int32_t pos = 0; pos < n; ++pos) {
        moved.push_back(std::move(plan->nodes[order[pos]]));
        if (new_index) new_index[order[pos]] = pos;
    }
    plan->nodes.swap(moved);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_set_select_lanes(kxc_hip_plan* plan, int32_t lanes) {
    const char* who = "kxc_hip_plan_set_select_lanes";
    KXC_PLAN_BEGIN(who);
    KXC_HIP_REQUIRE(lanes >= 1 && lanes <= 16, "%s: lanes must be in [1, 16]", who);
    plan->select_lanes = lanes;
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_run_profiled(kxc_hip_plan* plan, void** args, void* stream, kxc_hip_launch_record* records,
                                  int32_t capacity, int32_t* count) {
    const char* who = "kxc_hip_plan_run_profiled";
    if (int32_t rc = CheckRunArgs(plan, args, who)) return rc;
    KXC_HIP_REQUIRE(count != nullptr && (capacity == 0 || records != nullptr), "%s: NULL output", who);
    const int32_t nodes = static_cast<int32_t>(plan->nodes.size());
    *count = nodes;
    KXC_HIP_REQUIRE(capacity >= nodes, "%s: %d records needed, room for %d", who, nodes, capacity);
    void* s = stream ? stream : static_cast<void*>(CurrentStream());
    hipStream_t hs = reinterpret_cast<hipStream_t>(s);
    ActivitySuppress no_activity_records;      // this run times its launches itself
    // one event before every node and one after the last: node i ran between events i and i+1
    std::vector<hipEvent_t> ev(static_cast<size_t>(nodes) + 1, nullptr);
    int32_t rc = KXC_HIP_OK;
    {
        bool launched = false;
        rc = plan->constants_frozen ? EnsureFrozenConstants(plan, args, hs) : TransformConstants(plan, args, hs, false, &launched);
        if (rc != KXC_HIP_OK) return rc;
    }
    for (auto& e : ev)
        if (hipEventCreate(&e) != hipSuccess) { rc = Fail(KXC_HIP_ERR_RUNTIME, "%s: hipEventCreate failed", who); break; }
    for (int32_t i = 0; rc == KXC_HIP_OK && i < nodes; ++i) {
        Node& n = plan->nodes[i];
        if (hipEventRecord(ev[i], hs) != hipSuccess) { rc = Fail(KXC_HIP_ERR_RUNTIME, "%s: hipEventRecord failed", who); break; }
        LastLaunch() = LaunchNote();
        rc = RunNode(plan, n, args, s);
        if (rc != KXC_HIP_OK) break;
        kxc_hip_launch_record& r = records[i];
        std::memset(&r, 0, sizeof(r));
        std::snprintf(r.kernel_symbol, sizeof(r.kernel_symbol), "%s", n.symbol.c_str());
        r.kind = n.kind == NodeKind::kCopy ? KXC_HIP_RECORD_MEMCPY : KXC_HIP_RECORD_KERNEL;
        const LaunchNote& note = LastLaunch();
        for (int k = 0; k < 3; ++k) { r.grid[k] = note.grid[k]; r.block[k] = note.block[k]; }
        r.dynamic_shared_memory = note.dynamic_lds;
        if (n.kind == NodeKind::kCopy) r.bytes = n.dims[0];
    }
    if (rc == KXC_HIP_OK && hipEventRecord(ev[nodes], hs) != hipSuccess)
        rc = Fail(KXC_HIP_ERR_RUNTIME, "%s: hipEventRecord failed", who);
    if (rc == KXC_HIP_OK && hipEventSynchronize(ev[nodes]) != hipSuccess)
        rc = Fail(KXC_HIP_ERR_RUNTIME, "%s: hipEventSynchronize failed", who);
    for (int32_t i = 0; rc == KXC_HIP_OK && i < nodes; ++i) {
        float start_ms = 0.0f, dur_ms = 0.0f;
        if (hipEventElapsedTime(&start_ms, ev[0], ev[i]) != hipSuccess ||
            hipEventElapsedTime(&dur_ms, ev[i], ev[i + 1]) != hipSuccess) {
            rc = Fail(KXC_HIP_ERR_RUNTIME, "%s: hipEventElapsedTime failed", who);
            break;
        }
        records[i].start_ns = static_cast<int64_t>(static_cast<double>(start_ms) * 1e6);
        records[i].duration_ns = static_cast<int64_t>(static_cast<double>(dur_ms) * 1e6);
    }
    for (auto& e : ev)
        if (e) (void)hipEventDestroy(e);
    return rc;
}

// ---- serialisation: one text line per node, every field as a number (floats as hex floats, exact)
int32_t kxc_hip_plan_serialize(const kxc_hip_plan* plan, char* buffer, size_t capacity, size_t* needed) {
    KXC_HIP_REQUIRE(plan != nullptr && needed != nullptr, "kxc_hip_plan_serialize: NULL argument");
    KXC_HIP_REQUIRE(plan->finalized, "kxc_hip_plan_serialize: plan is not finalized");
    std::string out;
    char tmp[96];
    auto I = [&](long long v) { std::snprintf(tmp, sizeof(tmp), " %lld", v); out += tmp; };
    auto F = [&](float v) { std::snprintf(tmp, sizeof(tmp), " %a", static_cast<double>(v)); out += tmp; };
    // (version 2 added the plan's select_lanes and every node's chain, version 3 the weight packs)
    out += "kxc_hip_plan 3";
    I(plan->num_args); I(static_cast<long long>(plan->workspace_bytes)); I(static_cast<long long>(plan->nodes.size()));
    I(plan->select_lanes);
    I(static_cast<long long>(plan->packs.size()));
    out += "\n";
    for (const Node& n : plan->nodes) {
        KXC_HIP_REQUIRE(n.symbol.find_first_of(" \n\t") == std::string::npos,
                        "kxc_hip_plan_serialize: kernel symbol '%s' contains white space", n.symbol.c_str());
        out += "node";
        I(static_cast<int>(n.kind));
        out += " " + n.symbol;
        for (const kxc_hip_buf& b : n.bufs) { I(b.kind); I(b.index_or_offset); }
        const kxc_hip_conv2d_desc& c = n.conv;
        for (long long v : {(long long)c.n, (long long)c.c, (long long)c.h, (long long)c.w, (long long)c.o, (long long)c.kh,
                            (long long)c.kw, (long long)c.stride_h, (long long)c.stride_w, (long long)c.pad_h, (long long)c.pad_w,
                            (long long)c.dil_h, (long long)c.dil_w, (long long)c.flags}) I(v);
        const kxc_hip_qconv2d_desc& q = n.qconv;
        for (long long v : {(long long)q.n, (long long)q.c, (long long)q.h, (long long)q.w, (long long)q.o, (long long)q.kh,
                            (long long)q.kw, (long long)q.stride_h, (long long)q.stride_w, (long long)q.pad_h, (long long)q.pad_w,
                            (long long)q.flags}) I(v);
        F(q.res_mult);
        const kxc_hip_pool2d_desc& pd = n.pool;
        for (long long v : {(long long)pd.n, (long long)pd.c, (long long)pd.h, (long long)pd.w, (long long)pd.kh, (long long)pd.kw,
                            (long long)pd.stride_h, (long long)pd.stride_w, (long long)pd.pad_top, (long long)pd.pad_left,
                            (long long)pd.pad_bottom, (long long)pd.pad_right, (long long)pd.ceil_mode, (long long)pd.is_avg}) I(v);
        for (int64_t v : n.dims) I(v);
        for (float v : n.f) F(v);
        for (int32_t v : n.i32) I(v);
        for (int64_t v : n.a_shape) I(v);
        for (int64_t v : n.b_shape) I(v);
        for (uint32_t v : n.grid) I(v);
        for (uint32_t v : n.block) I(v);
        I(n.shared_bytes);
        I(n.lane); I(n.join); I(n.chain);
        I(static_cast<long long>(n.params.size()));
        for (const kxc_hip_buf& b : n.params) { I(b.kind); I(b.index_or_offset); }
        out += "\n";
    }
    for (const PackJob& j : plan->packs) {
        out += "pack";
        I(j.kind); I(j.every_run);
        I(j.w.kind); I(j.w.index_or_offset); I(j.wp.kind); I(j.wp.index_or_offset);
        const kxc_hip_qconv2d_desc& q = j.desc;
        for (long long v : {(long long)q.n, (long long)q.c, (long long)q.h, (long long)q.w, (long long)q.o, (long long)q.kh,
                            (long long)q.kw, (long long)q.stride_h, (long long)q.stride_w, (long long)q.pad_h, (long long)q.pad_w,
                            (long long)q.flags}) I(v);
        F(q.res_mult);
        out += "\n";
    }
    *needed = out.size() + 1;
    if (buffer == nullptr || capacity == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(capacity >= *needed, "kxc_hip_plan_serialize: %zu bytes needed, room for %zu", *needed, capacity);
    std::memcpy(buffer, out.c_str(), *needed);
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_deserialize(const char* text, int32_t device_id, kxc_hip_module* const* modules, int32_t num_modules,
                                 kxc_hip_plan** out_plan) {
    const char* who = "kxc_hip_plan_deserialize";
    KXC_HIP_REQUIRE(text != nullptr && out_plan != nullptr, "%s: NULL argument", who);
    std::istringstream in{std::string(text)};
    std::string magic;
    long long version = 0, num_args = 0, workspace = 0, count = 0;
    long long select_lanes = 1, num_packs = 0;
    in >> magic >> version >> num_args >> workspace >> count;
    if (in && version >= 2) in >> select_lanes;
    if (in && version >= 3) in >> num_packs;
    KXC_HIP_REQUIRE(in && magic == "kxc_hip_plan" && version >= 1 && version <= 3, "%s: not a version-1, -2 or -3 plan", who);
    KXC_HIP_REQUIRE(num_packs >= 0 && num_packs < (1 << 20), "%s: implausible header", who);
    KXC_HIP_REQUIRE(select_lanes >= 1 && select_lanes <= 16, "%s: implausible header", who);
    KXC_HIP_REQUIRE(num_args >= 0 && num_args < (1 << 20) && workspace >= 0 && count >= 0 && count < (1 << 24),
                    "%s: implausible header", who);
    kxc_hip_plan* plan = nullptr;
    if (int32_t rc = kxc_hip_plan_create(device_id, static_cast<int32_t>(num_args), &plan)) return rc;
    plan->select_lanes = static_cast<int32_t>(select_lanes);
    auto fail = [&](const char* what) {
        kxc_hip_plan_destroy(plan);
        return Fail(KXC_HIP_ERR_INVALID, "%s: %s", who, what);
    };
    for (long long k = 0; k < count; ++k) {
        std::string tag;
        long long kind = -1;
        Node n{};
        in >> tag >> kind >> n.symbol;
        if (!in || tag != "node" || kind < 0 || kind > static_cast<long long>(kLastNodeKind)) return fail("bad node line");
        n.kind = static_cast<NodeKind>(kind);
        long long v = 0;
        auto I = [&]() { in >> v; return v; };
        auto F = [&]() { std::string t; in >> t; return static_cast<float>(std::strtod(t.c_str(), nullptr)); };
        for (kxc_hip_buf& b : n.bufs) { b.kind = static_cast<int32_t>(I()); b.index_or_offset = I(); }
        kxc_hip_conv2d_desc& c = n.conv;
        c.n = I(); c.c = I(); c.h = I(); c.w = I(); c.o = I(); c.kh = I(); c.kw = I(); c.stride_h = I(); c.stride_w = I();
        c.pad_h = I(); c.pad_w = I(); c.dil_h = I(); c.dil_w = I(); c.flags = static_cast<uint32_t>(I());
        kxc_hip_qconv2d_desc& q = n.qconv;
        q.n = I(); q.c = I(); q.h = I(); q.w = I(); q.o = I(); q.kh = I(); q.kw = I(); q.stride_h = I(); q.stride_w = I();
        q.pad_h = I(); q.pad_w = I(); q.flags = static_cast<uint32_t>(I()); q.res_mult = F();
        kxc_hip_pool2d_desc& pd = n.pool;
        pd.n = I(); pd.c = I(); pd.h = I(); pd.w = I(); pd.kh = I(); pd.kw = I(); pd.stride_h = I(); pd.stride_w = I();
        pd.pad_top = I(); pd.pad_left = I(); pd.pad_bottom = I(); pd.pad_right = I(); pd.ceil_mode = I(); pd.is_avg = I();
        for (int64_t& d : n.dims) d = I();
        for (float& f : n.f) f = F();
        for (int32_t& i : n.i32) i = static_cast<int32_t>(I());
        for (int64_t& d : n.a_shape) d = I();
        for (int64_t& d : n.b_shape) d = I();
        for (uint32_t& g : n.grid) g = static_cast<uint32_t>(I());
        for (uint32_t& b : n.block) b = static_cast<uint32_t>(I());
        n.shared_bytes = static_cast<uint32_t>(I());
        n.lane = static_cast<int32_t>(I()); n.join = static_cast<int32_t>(I());
        if (version >= 2) n.chain = static_cast<int32_t>(I());
        if (n.lane < 0 || n.lane > 1 || n.join < 0 || n.join > 1 || n.chain < 0 || n.chain > kMaxChains ||
            (n.chain > 0 && (n.lane || n.join)))
            return fail("bad concurrency flags");
        const long long np = I();
        if (!in || np < 0 || np > 4096) return fail("bad parameter count");
        for (long long i = 0; i < np; ++i) {
            kxc_hip_buf b;
            b.kind = static_cast<int32_t>(I()); b.index_or_offset = I();
            n.params.push_back(b);
        }
        if (!in) return fail("truncated node line");
        auto buf_ok = [&](const kxc_hip_buf& b) {
            if (b.kind == KXC_HIP_BUF_ARG) return b.index_or_offset >= 0 && b.index_or_offset < num_args;
            if (b.kind == KXC_HIP_BUF_WORKSPACE) return b.index_or_offset >= 0 && b.index_or_offset < workspace;
            if (b.kind == KXC_HIP_BUF_ARG_OFFSET)
                return b.index_or_offset >= 0 && (b.index_or_offset >> 48) < num_args && (b.index_or_offset & 15) == 0;
            return b.kind == KXC_HIP_BUF_NONE;
        };
        for (const kxc_hip_buf& b : n.bufs) if (!buf_ok(b)) return fail("buffer operand out of range");
        for (const kxc_hip_buf& b : n.params) if (!buf_ok(b)) return fail("kernel parameter out of range");
        if (n.kind == NodeKind::kConv2D && (n.conv.flags & KXC_HIP_CONV_HPOOL) &&
            (n.i32[0] != 0 || !kxc_hip_conv2d_hpool_supported(&n.conv)))
            return fail("bad convolution node with the pooling epilogue");
        if (n.kind == NodeKind::kConv2D && n.i32[0] == 1 &&
            (!kxc_hip_conv2d_winograd_supported(&n.conv) || n.bufs[5].kind != KXC_HIP_BUF_WORKSPACE))
            return fail("bad Winograd convolution node");
        if (n.kind == NodeKind::kConv2D && n.i32[0] == 2 &&
            (!kxc_hip_conv2d_pair_supported(&n.conv) || n.params.size() != 3 || n.params[0].kind == KXC_HIP_BUF_NONE ||
             n.params[2].kind == KXC_HIP_BUF_NONE))
            return fail("bad convolution-pair node");
        if (n.kind == NodeKind::kQConv2D && (n.i32[0] < 0 || n.i32[0] > 4 || (n.i32[0] == 4 && !kxc_hip_qconv2d_c4_maxpool_supported(&n.qconv))))
            return fail("bad int8 convolution node");
        if (n.kind == NodeKind::kQConv2D && n.i32[0] == 3 &&
            (!kxc_hip_qconv2d_c16_pair_supported(&n.qconv) || n.params.size() != 4 || n.params[0].kind == KXC_HIP_BUF_NONE ||
             n.params[2].kind == KXC_HIP_BUF_NONE || n.params[3].kind == KXC_HIP_BUF_NONE))
            return fail("bad int8 convolution-pair node");
        if (n.kind == NodeKind::kModuleKernel) {
            // generated kernels are found by name in the modules the caller compiled from the saved source
            for (int32_t m = 0; m < num_modules && !n.function; ++m) {
                void* fn = nullptr;
                if (modules && modules[m] && kxc_hip_module_get_function(modules[m], n.symbol.c_str(), &fn) == KXC_HIP_OK) n.function = fn;
            }
            if (!n.function) return fail(("generated kernel not found in the given modules: " + n.symbol).c_str());
            if (static_cast<uint64_t>(n.block[0]) * n.block[1] * n.block[2] > 1024 || n.grid[0] == 0 || n.block[0] == 0)
                return fail("bad launch geometry");
        }
        plan->nodes.push_back(n);
    }
    for (long long k = 0; k < num_packs; ++k) {
        std::string tag;
        PackJob j;
        long long v = 0;
        auto I = [&]() { in >> v; return v; };
        in >> tag;
        if (!in || tag != "pack") return fail("bad pack line");
        j.kind = static_cast<int32_t>(I()); j.every_run = static_cast<int32_t>(I());
        j.w.kind = static_cast<int32_t>(I()); j.w.index_or_offset = I();
        j.wp.kind = static_cast<int32_t>(I()); j.wp.index_or_offset = I();
        kxc_hip_qconv2d_desc& q = j.desc;
        q.n = I(); q.c = I(); q.h = I(); q.w = I(); q.o = I(); q.kh = I(); q.kw = I(); q.stride_h = I(); q.stride_w = I();
        q.pad_h = I(); q.pad_w = I(); q.flags = static_cast<uint32_t>(I());
        std::string t;
        in >> t;
        q.res_mult = static_cast<float>(std::strtod(t.c_str(), nullptr));
        if (!in) return fail("truncated pack line");
        const bool w_ok = (j.w.kind == KXC_HIP_BUF_ARG && j.w.index_or_offset >= 0 && j.w.index_or_offset < num_args) ||
                          (j.w.kind == KXC_HIP_BUF_ARG_OFFSET && j.w.index_or_offset >= 0 && (j.w.index_or_offset >> 48) < num_args &&
                           (j.w.index_or_offset & 15) == 0);
        if (!w_ok || j.wp.kind != KXC_HIP_BUF_WORKSPACE || j.wp.index_or_offset < 0 || j.wp.index_or_offset >= workspace ||
            j.wp.index_or_offset % 256 != 0)
            return fail("pack operand out of range");
        size_t bytes = 0;
        const QPackJob probe{j.kind, &j.desc, nullptr, nullptr};
        if (QPackedBytes(probe, &bytes) != KXC_HIP_OK) return fail("bad pack descriptor");
        plan->packs.push_back(j);
    }
    if (int32_t rc = kxc_hip_plan_finalize(plan, static_cast<size_t>(workspace))) {
        kxc_hip_plan_destroy(plan);
        return rc;
    }
    *out_plan = plan;
    return KXC_HIP_OK;
}

int32_t kxc_hip_plan_num_nodes(const kxc_hip_plan* plan) { return plan ? static_cast<int32_t>(plan->nodes.size()) : 0; }

const char* kxc_hip_plan_node_symbol(const kxc_hip_plan* plan, int32_t i) {
    if (!plan || i < 0 || i >= static_cast<int32_t>(plan->nodes.size())) return "";
    return plan->nodes[i].symbol.c_str();
}

void* kxc_hip_plan_workspace(const kxc_hip_plan* plan) { return plan ? plan->workspace : nullptr; }

}  // extern "C"
