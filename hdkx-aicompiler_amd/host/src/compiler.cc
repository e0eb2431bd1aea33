// compiler.cc -- Compiler::Compile and CompiledModule (see compiler.h).
#include "kxc/compiler.h"
#include "kxc/runtime_session.h"
#include "kxc/profiling.h"
#include "json_reader.h"

#include <dlfcn.h>
#include <unistd.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <sstream>
#include <unordered_map>
#include <unordered_set>

#include "kxc_hip.h"

namespace kxc {
namespace api {

using relay::OpNode;

constexpr const char* kKernelEntrySymbol = "kxc_kernel_main";   // src/api/compiler.cc:30

CompileConfig CompileConfig::AOT(Target target, int opt_level) {
    auto n = std::make_shared<CompileConfigNode>();
    n->mode = CompileMode::kAOT;
    n->opt_level = opt_level;
    n->target = target;
    return CompileConfig(n);
}
CompileConfig CompileConfig::JIT(Target target) {
    auto n = std::make_shared<CompileConfigNode>();
    n->mode = CompileMode::kJIT;
    n->opt_level = 1;
    n->target = target;
    n->enable_hot_swap = false;
    return CompileConfig(n);
}
CompileConfig CompileConfig::Adaptive(Target target, std::vector<std::vector<int64_t>> suggested_shapes) {
    auto n = std::make_shared<CompileConfigNode>();
    n->mode = CompileMode::kAdaptive;
    n->opt_level = 2;
    n->target = target;
    n->suggested_input_shapes = std::move(suggested_shapes);
    return CompileConfig(n);
}

class CompiledModuleImpl {
public:
    CompileConfig config;
    tir::PrimFunc prim_func;
    std::string source;
    Array<runtime::NDArray> constants;
    int64_t input_count = 0, constant_count = 0;
    std::vector<KernelExecInfo> execs;
    std::string status = "not compiled";
    int num_values = 0;
    std::vector<int> input_value_ids, constant_value_ids;
    int output_value = -1;
    // The compiled function (include/api/compiler.h:96-105 keeps a codegen::CompiledKernel the same way): owns the
    // generated library of the host back end, or the launch plan and run-time compiled modules of the hip back end.
    codegen::CompiledKernel kernel;
    // hip back end: the plan the kernel owns (alias), and what a dry build (no GPU) keeps instead
    kxc_hip_plan* plan = nullptr;
    std::vector<kxc_hip_module*> modules;        // moved into the kernel node once the plan is loaded
    std::vector<std::string> module_sources;     // one per generated module (dry builds keep the sources only)
    size_t workspace_bytes = 0;
    bool ready = false;
    std::shared_ptr<profiling::ProfileContext> profile_context;      // from config->profile_options, when enabled

    // Hands the plan and the modules to a kernel node (callable = the plan was finalized on a GPU).
    void AdoptHipKernel(bool callable) {
        auto node = std::make_shared<codegen::CompiledKernelNode>();
        node->kernel_name = "kxc_kernel_main";
        node->backend = codegen::CodeGenBackend::kHIP;
        node->jit_resource = plan;
        node->func_ptr = callable ? static_cast<void*>(plan) : nullptr;
        for (auto* m : modules) node->hip_modules.push_back(m);
        modules.clear();
        node->device_id = config->target->device.device_id();
        node->sync_after_run = config->sync_after_run;
        if (prim_func.defined())
            for (const auto& v : prim_func->params) {
                auto it = prim_func->buffer_map.find(v.get());
                if (it != prim_func->buffer_map.end()) node->param_buffers.push_back(it->second);
            }
        kernel = codegen::CompiledKernel(node);
    }
    ~CompiledModuleImpl() {
        // (before a kernel node adopted them)
        if (!kernel.defined()) {
            if (plan) kxc_hip_plan_destroy(plan);
            for (auto* m : modules) kxc_hip_module_free(m);
        }
    }
};

namespace {

// ------------------------------------------------------------------ host back end
void CompileHost(const Function& typed, const CompileConfig& config, CompiledModuleImpl* m) {
    relay::LoweredFunc lowered = relay::LowerToTIRDetailed(typed);
    m->prim_func = tir::RunTIRPassPipeline(lowered.func, {"fold_constant", "simplify_expr"});
    m->constants = lowered.constants;
    m->input_count = m->prim_func->int_attrs.at("kxc.input_count");
    m->constant_count = m->prim_func->int_attrs.at("kxc.constant_count");
    codegen::CodeGenC cg;
    m->source = cg.Generate(m->prim_func, kKernelEntrySymbol);
    static std::atomic<int> counter{0};
    const char* tmp = std::getenv("TMPDIR");
    const std::string base = std::string(tmp && *tmp ? tmp : "/tmp") + "/kxc_jit_" + std::to_string(getpid()) + "_" +
                             std::to_string(counter.fetch_add(1));
    const std::string c_path = base + ".c";
    const std::string so_path = base + ".so";
    {
        std::ofstream out(c_path);
        out << m->source;
    }
    const int level = config->opt_level < 0 ? 0 : config->opt_level > 3 ? 3 : config->opt_level;
    // strict fp32: no contraction, no fast-math -- results do not depend on the optimisation level
    const std::string cmd = "cc -std=gnu11 -O" + std::to_string(level) +
                            " -fno-fast-math -ffp-contract=off -shared -fPIC -w -o " + so_path + " " + c_path + " -lm 2>&1";
    FILE* pipe = popen(cmd.c_str(), "r");
    if (!pipe) throw std::runtime_error("host compiler could not be started");
    std::string log;
    char buf[512];
    while (fgets(buf, sizeof(buf), pipe)) log += buf;
    const int rc = pclose(pipe);
    std::remove(c_path.c_str());
    if (rc != 0) throw std::runtime_error("host compilation of the generated C failed:\n" + log);
    auto node = std::make_shared<codegen::CompiledKernelNode>();
    node->kernel_name = kKernelEntrySymbol;
    node->backend = codegen::CodeGenBackend::kC;
    node->so_path = so_path;
    node->lib_handle = dlopen(so_path.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (!node->lib_handle) throw std::runtime_error(std::string("dlopen failed: ") + dlerror());
    node->func_ptr = dlsym(node->lib_handle, kKernelEntrySymbol);
    if (!node->func_ptr) throw std::runtime_error("generated library lacks kxc_kernel_main");
    for (const auto& v : m->prim_func->params) {
        auto it = m->prim_func->buffer_map.find(v.get());
        if (it != m->prim_func->buffer_map.end()) node->param_buffers.push_back(it->second);
    }
    m->kernel = codegen::CompiledKernel(node);
    KernelExecInfo e;
    e.op_name = "main";
    e.kernel_symbol = kKernelEntrySymbol;
    m->execs.push_back(e);
    m->ready = true;
    m->status = "ready (host C back end)";
}

// ------------------------------------------------------------------ hip back end
struct Arena {
    std::vector<std::pair<int64_t, int64_t>> free_list;   // offset, size
    int64_t top = 0;
    std::pair<int64_t, int64_t> Alloc(int64_t nbytes) {
        const int64_t size = (std::max<int64_t>(nbytes, 1) + 255) / 256 * 256;
        for (size_t i = 0; i < free_list.size(); ++i) {
            if (free_list[i].second >= size) {
                const int64_t off = free_list[i].first;
                if (free_list[i].second == size) free_list.erase(free_list.begin() + i);
                else { free_list[i].first += size; free_list[i].second -= size; }
                return {off, size};
            }
        }
        const int64_t off = top;
        top += size;
        return {off, size};
    }
    void Release(std::pair<int64_t, int64_t> blk) {
        free_list.push_back(blk);
        std::sort(free_list.begin(), free_list.end());
        std::vector<std::pair<int64_t, int64_t>> merged;
        for (auto& b : free_list) {
            if (!merged.empty() && merged.back().first + merged.back().second == b.first) merged.back().second += b.second;
            else merged.push_back(b);
        }
        free_list.swap(merged);
    }
};

struct Group {
    const CallNode* head = nullptr;     // the operator that is launched
    const CallNode* tail = nullptr;     // the last call folded into it (its value is the group's output)
    const RelayExprNode* residual = nullptr;
    bool fused_relu = false;
    const CallNode* pool = nullptr;     // a pooling call behind it that the head's launches produce as well (then the tail)
};

template <typename T>
const T* OpAttr(const OpNode* op, const char* key) {
    auto it = op->attrs.find(key);
    return it == op->attrs.end() ? nullptr : std::any_cast<T>(&it->second);
}
bool OpFlag(const OpNode* op, const char* key) {
    const bool* b = OpAttr<bool>(op, key);
    return b && *b;
}
const TensorTypeNode* TT(const Type& t) { return t.As<TensorTypeNode>(); }
int64_t TypeBytes(const Type& t) { return Product(TT(t)->shape) * tir::DTypeFromString(TT(t)->dtype).bytes(); }

class HipBuilder {
public:
    // lanes > 1: `f` is one share of the batch (relay::SplitBatch) and is emitted `lanes` times into the one plan,
    // share k as chain k of the plan, on the k-th part of parameter 0 and of the result
    HipBuilder(const Function& f, const CompileConfig& cfg, CompiledModuleImpl* m, bool dry, int lanes = 1)
        : f_(f), cfg_(cfg), m_(m), dry_(dry), lanes_(lanes) {}

    void Build() {
        Number();
        FormGroups();
        AssignLayouts();
        FusePoolsByLayout();
        if (kxc_hip_plan_create(cfg_->target->device.device_id(), static_cast<int32_t>(num_args_), &m_->plan))
            throw std::runtime_error(std::string("plan creation failed: ") + kxc_hip_last_error());
        // variants are chosen for `lanes` equal launches side by side: by the queries made while the plan is built
        // (this thread) and by the plan when it is finalized
        struct LanesScope {
            int32_t prev;
            explicit LanesScope(int32_t lanes) : prev(kxc_hip_set_select_lanes(lanes)) {}
            ~LanesScope() { kxc_hip_set_select_lanes(prev); }
        } lanes_scope(lanes_);
        if (lanes_ > 1) {
            if (kxc_hip_plan_set_select_lanes(m_->plan, lanes_)) throw std::runtime_error(std::string("plan_set_select_lanes failed: ") + kxc_hip_last_error());
            in_share_bytes_ = TypeBytes(f_->params[0].checked_type());
            out_share_bytes_ = TypeBytes(f_->body.checked_type());
        }
        for (lane_ = 0; lane_ < lanes_; ++lane_) {
            // a share's activations live in workspace regions of its own (the shares run at the same time)
            arena_.free_list.clear();
            slot_.clear();
            alias_.clear();
            persistent_cursor_ = 0;
            const int32_t first_node = kxc_hip_plan_num_nodes(m_->plan);
            const size_t first_exec = m_->execs.size();
            Emit();
            if (lane_ == 0) continue;
            for (int32_t node = first_node; node < kxc_hip_plan_num_nodes(m_->plan); ++node)
                if (kxc_hip_plan_set_chain(m_->plan, node, lane_))
                    throw std::runtime_error(std::string("plan_set_chain failed: ") + kxc_hip_last_error());
            for (size_t e = first_exec; e < m_->execs.size(); ++e) m_->execs[e].kernel_symbol += " @share" + std::to_string(lane_);
        }
        if (lanes_ > 1 && !(std::getenv("KXC_HIP_INTERLEAVE") && std::getenv("KXC_HIP_INTERLEAVE")[0] == '0')) {
            // the shares' launches alternate in the plan, so that a run feeds every stream at the same pace
            std::vector<int32_t> new_index(static_cast<size_t>(kxc_hip_plan_num_nodes(m_->plan)));
            if (kxc_hip_plan_interleave_chains(m_->plan, new_index.data(), static_cast<int32_t>(new_index.size())))
                throw std::runtime_error(std::string("plan_interleave_chains failed: ") + kxc_hip_last_error());
            if (new_index.size() == m_->execs.size()) {
                std::vector<KernelExecInfo> moved(m_->execs.size());
                for (size_t i = 0; i < new_index.size(); ++i) moved[static_cast<size_t>(new_index[i])] = m_->execs[i];
                m_->execs.swap(moved);
            }
        }
        m_->workspace_bytes = static_cast<size_t>(arena_.top);
        if (!dry_) {
            if (kxc_hip_plan_finalize(m_->plan, m_->workspace_bytes))
                throw std::runtime_error(std::string("plan finalize failed: ") + kxc_hip_last_error());
            if (cfg_->hip_constants_frozen) kxc_hip_plan_freeze_constants(m_->plan, 1);
            m_->AdoptHipKernel(true);
            m_->ready = true;
            m_->status = "ready (hip back end, " + std::to_string(m_->execs.size()) + " launches)";
        } else {
            m_->AdoptHipKernel(false);
            m_->status = "compiled without loading (no GPU): " + std::to_string(m_->execs.size()) + " launches";
        }
    }

private:
    // ---- value numbering: one id per Relay expression; DFS in argument order (the lowering's order)
    void Number() {
        for (const auto& p : f_->params) {
            value_id_[p.get()] = next_value_++;
            m_->input_value_ids.push_back(value_id_[p.get()]);
            arg_index_[p.get()] = static_cast<int>(arg_index_.size());
        }
        num_inputs_ = static_cast<int>(f_->params.size());
        Visit(f_->body);
        num_args_ = num_inputs_ + static_cast<int>(constants_.size()) + 1;
        for (size_t k = 0; k < constants_.size(); ++k) arg_index_[constants_[k]] = num_inputs_ + static_cast<int>(k);
        m_->num_values = next_value_;
        m_->output_value = value_id_.at(f_->body.get());
    }
    void Visit(const Expr& e) {
        if (value_id_.count(e.get())) return;
        if (const auto* c = e.As<ConstantNode>()) {
            value_id_[e.get()] = next_value_++;
            m_->constant_value_ids.push_back(value_id_[e.get()]);
            constants_.push_back(e.get());
            m_->constants.push_back(c->data);
            return;
        }
        const auto* call = e.As<CallNode>();
        if (!call) throw std::runtime_error("hip back end: unsupported Relay node (free variable or non-call expression)");
        for (const auto& a : call->args) {
            Visit(a);
            consumers_[a.get()].push_back(call);
        }
        value_id_[e.get()] = next_value_++;
        topo_.push_back(call);
        expr_of_[call] = e;
    }

    const CallNode* SoleConsumer(const RelayExprNode* e) const {
        auto it = consumers_.find(e);
        if (it == consumers_.end() || it->second.size() != 1 || e == f_->body.get()) return nullptr;
        return it->second[0];
    }
    static bool IsOp(const CallNode* c, const char* name) {
        const auto* op = c->op.As<OpNode>();
        return op && op->name == name;
    }
    static bool IsF32(const Type& t) { return TT(t) && TT(t)->dtype == "float32"; }

    // ---- fusion: conv(+bias) -> [add(conv_out, skip)] -> [relu];  binary -> [relu]
    void FormGroups() {
        std::unordered_set<const CallNode*> absorbed;
        for (const CallNode* c : topo_) {
            if (absorbed.count(c)) continue;
            const auto* op = c->op.As<OpNode>();
            Group g;
            g.head = g.tail = c;
            const bool dispatchable = cfg_->hip_use_handwritten && OpAttr<relay::FHIPDispatch>(op, "FHIPDispatch") &&
                                      IsF32(c->checked_type_);
            if (cfg_->hip_fuse && dispatchable) {
                if (OpFlag(op, "THIPFusable")) {
                    const CallNode* n = SoleConsumer(g.tail);
                    if (n && !absorbed.count(n) && IsOp(n, "add") && n->args.size() == 2 && n->args[0].get() != n->args[1].get()) {
                        const RelayExprNode* other = n->args[0].get() == g.tail ? n->args[1].get() : n->args[0].get();
                        if (TT(other->checked_type_)->shape == TT(c->checked_type_)->shape && IsF32(other->checked_type_)) {
                            g.residual = other;
                            g.tail = n;
                            absorbed.insert(n);
                        }
                    }
                    n = SoleConsumer(g.tail);
                    if (n && !absorbed.count(n) && IsOp(n, "nn_relu")) { g.fused_relu = true; g.tail = n; absorbed.insert(n); }
                    // ... -> pooling, when the operator can take part of the window in its own launch
                    n = SoleConsumer(g.tail);
                    const auto* pool_query = OpAttr<relay::FHIPPoolQuery>(op, "FHIPPoolQuery");
                    const char* pool_env = std::getenv("KXC_HIP_FUSE_POOL");            // "0" switches it off
                    if (n && pool_query && !absorbed.count(n) && g.tail != f_->body.get() && !(pool_env && pool_env[0] == '0') &&
                        (IsOp(n, "nn_max_pool2d") || IsOp(n, "nn_avg_pool2d")) && IsF32(n->checked_type_)) {
                        Array<Type> types;
                        for (const auto& a : c->args) types.push_back(a.checked_type());
                        if ((*pool_query)(c->attrs, types, g.fused_relu, g.residual != nullptr, n->op.As<OpNode>()->name, n->attrs)) {
                            g.pool = n;
                            g.tail = n;
                            absorbed.insert(n);
                        }
                    }
                } else if (OpFlag(op, "THIPFusableRelu") && TT(c->checked_type_)->shape.size() <= 6) {
                    const CallNode* n = SoleConsumer(g.tail);
                    if (n && !absorbed.count(n) && IsOp(n, "nn_relu")) { g.fused_relu = true; g.tail = n; absorbed.insert(n); }
                }
            }
            group_of_tail_[g.tail] = groups_.size();
            groups_.push_back(g);
        }
    }

    // ---- layouts of int8 activations between launches (relay::HIPLayout).  Every call whose operator has an
    // "FHIPLayoutQuery" says, in topological order, which layouts its kernel takes and writes given the layouts its
    // inputs exist in; a value whose producer writes any layout ("THIPLayoutFollowsConsumers": qnn_quantize) takes
    // the layout its consumers agree on (a first pass collects their wishes, a second one runs with the decision).
    // Edges whose ends disagree get a converter when the call is emitted.
    void AssignLayouts() {
        if (!cfg_->hip_use_handwritten) return;
        std::unordered_map<const RelayExprNode*, int> decided;       // follows-consumers values, after pass 0
        for (int pass = 0; pass < 2; ++pass) {
            layout_.clear();
            choice_.clear();
            std::unordered_map<const RelayExprNode*, std::vector<int>> wishes;
            for (const CallNode* c : topo_) {
                const auto* op = c->op.As<OpNode>();
                const auto* query = OpAttr<relay::FHIPDispatch>(op, "FHIPDispatch") ? OpAttr<relay::FHIPLayoutQuery>(op, "FHIPLayoutQuery") : nullptr;
                relay::HIPLayoutChoice choice;
                choice.inputs.assign(c->args.size(), relay::kHIPLayoutPlain);
                if (query) {
                    Array<Type> types;
                    std::vector<int> offered;
                    std::vector<bool> is_arg;
                    for (const auto& a : c->args) {
                        types.push_back(a.checked_type());
                        auto it = layout_.find(a.get());
                        offered.push_back(it == layout_.end() ? relay::kHIPLayoutPlain : it->second);
                        is_arg.push_back(arg_index_.count(a.get()) > 0);
                    }
                    choice = (*query)(c->attrs, types, c->checked_type_, offered, is_arg);
                    if (choice.inputs.size() != c->args.size()) choice.inputs.assign(c->args.size(), relay::kHIPLayoutPlain);
                }
                for (size_t i = 0; i < c->args.size(); ++i) {
                    auto it = layout_.find(c->args[i].get());
                    if (it != layout_.end() && it->second == relay::kHIPLayoutAny) wishes[c->args[i].get()].push_back(choice.inputs[i]);
                }
                choice_[c] = choice;
                if (OpFlag(op, "THIPLayoutFollowsConsumers") && OpAttr<relay::FHIPDispatch>(op, "FHIPDispatch")) {
                    auto d = decided.find(c);
                    layout_[c] = pass == 0 || d == decided.end() ? static_cast<int>(relay::kHIPLayoutAny) : d->second;
                } else {
                    layout_[c] = choice.output;
                }
            }
            if (pass == 0) {
                bool any = false;
                for (const auto& kv : layout_) {
                    if (kv.second != relay::kHIPLayoutAny) continue;
                    any = true;
                    int agreed = relay::kHIPLayoutPlain;
                    const auto w = wishes.find(kv.first);
                    if (w != wishes.end() && !w->second.empty() && kv.first != f_->body.get()) {
                        agreed = w->second[0];
                        for (int l : w->second) if (l != agreed) agreed = relay::kHIPLayoutPlain;
                    }
                    decided[kv.first] = agreed;
                }
                if (!any) break;       // no value's layout was left open: the first pass is final
            }
        }
        for (auto& kv : layout_) if (kv.second == relay::kHIPLayoutAny) kv.second = relay::kHIPLayoutPlain;
    }
    // Pool fusion that depends on the layouts just assigned (the fp32 one is decided in FormGroups): a call of an
    // operator with an "FHIPPoolQuery" that stands alone, whose only reader is a pooling call that stands alone, and
    // whose kernel was given a layout other than plain for its first input -- the int8 first layer on its 4-channel
    // input.  The pooling call's group dissolves into the convolution's.
    void FusePoolsByLayout() {
        if (!cfg_->hip_fuse || !cfg_->hip_use_handwritten) return;
        const char* pool_env = std::getenv("KXC_HIP_FUSE_POOL");            // "0" switches it off
        if (pool_env && pool_env[0] == '0') return;
        for (size_t gi = 0; gi < groups_.size(); ++gi) {
            Group& g = groups_[gi];
            if (g.head != g.tail || g.pool || g.residual || g.fused_relu || g.head == f_->body.get()) continue;
            const auto* op = g.head->op.As<OpNode>();
            const auto* query = OpAttr<relay::FHIPPoolQuery>(op, "FHIPPoolQuery");
            auto ch = choice_.find(g.head);
            if (!query || IsF32(g.head->checked_type_) || ch == choice_.end() || ch->second.inputs.empty() ||
                ch->second.inputs[0] == relay::kHIPLayoutPlain)
                continue;
            const CallNode* n = SoleConsumer(g.head);
            if (!n || !(IsOp(n, "nn_max_pool2d") || IsOp(n, "nn_avg_pool2d"))) continue;
            auto pg = group_of_tail_.find(n);
            if (pg == group_of_tail_.end() || groups_[pg->second].head != n) continue;        // the pool is not on its own
            auto pch = choice_.find(n);
            if (pch == choice_.end() || pch->second.inputs.empty() || pch->second.inputs[0] != ch->second.output || LayoutOf(n) != ch->second.output)
                continue;
            Array<Type> types;
            for (const auto& a : g.head->args) types.push_back(a.checked_type());
            if (!(*query)(g.head->attrs, types, false, false, n->op.As<OpNode>()->name, n->attrs)) continue;
            group_of_tail_.erase(g.head);
            group_of_tail_[n] = gi;          // (the pooling call's own group is no longer reachable and is never emitted)
            g.pool = n;
            g.tail = n;
        }
    }
    int LayoutOf(const RelayExprNode* e) const {
        auto it = layout_.find(Resolve(e));
        return it == layout_.end() ? static_cast<int>(relay::kHIPLayoutPlain) : it->second;
    }
    int64_t ValueBytes(const RelayExprNode* e) const { return relay::HIPLayoutBytes(e->checked_type_, LayoutOf(e)); }
    // One converter launch between the plain and the channel-blocked layout of an int8 value.
    void EmitLayoutConvert(const RelayExprNode* value, int from, int to, relay::HIPBuffer src, relay::HIPBuffer dst) {
        const auto* t = TT(value->checked_type_);
        const bool ok = t && t->dtype == "int8" && t->shape.size() == 4 &&
                        ((from == relay::kHIPLayoutPlain && to == relay::kHIPLayoutC16) || (from == relay::kHIPLayoutC16 && to == relay::kHIPLayoutPlain));
        if (!ok) throw std::runtime_error("hip back end: no converter between activation layouts " + std::to_string(from) + " and " + std::to_string(to));
        if (kxc_hip_plan_add_i8_layout(m_->plan, to == relay::kHIPLayoutC16 ? 1 : 0, t->shape[0], t->shape[1], t->shape[2] * t->shape[3],
                                       {src.kind, src.index_or_offset}, {dst.kind, dst.index_or_offset}))
            throw std::runtime_error(std::string("plan layout converter failed: ") + kxc_hip_last_error());
        KernelExecInfo info;
        info.op_name = "layout_convert";
        info.kernel_symbol = to == relay::kHIPLayoutC16 ? "kxc_i8_nchw_to_c16" : "kxc_i8_c16_to_nchw";
        info.input_values.push_back(value_id_.at(value));
        info.output_values.push_back(value_id_.at(value));
        m_->execs.push_back(info);
    }

    // ---- buffers
    relay::HIPBuffer BufferOf(const RelayExprNode* e) {
        e = Resolve(e);
        auto a = arg_index_.find(e);
        if (a != arg_index_.end()) {
            if (lanes_ > 1 && e == f_->params[0].get())
                return {KXC_HIP_BUF_ARG_OFFSET, KXC_HIP_ARG_OFFSET(a->second, lane_ * in_share_bytes_)};
            return {KXC_HIP_BUF_ARG, a->second};
        }
        auto s = slot_.find(e);
        if (s == slot_.end()) {
            const auto* c = dynamic_cast<const CallNode*>(e);
            const auto* op = c ? c->op.As<OpNode>() : nullptr;
            throw std::runtime_error("hip back end: value " + std::to_string(value_id_.count(e) ? value_id_.at(e) : -1) +
                                     " (" + (op ? op->name : std::string("?")) + ") used before it is produced");
        }
        return {KXC_HIP_BUF_WORKSPACE, s->second.first};
    }
    const RelayExprNode* Resolve(const RelayExprNode* e) const {
        auto it = alias_.find(e);
        while (it != alias_.end()) { e = it->second; it = alias_.find(e); }
        return e;
    }

    void Emit() {
        // emission order = topo order of the group tails
        std::vector<size_t> order;
        for (const CallNode* c : topo_) {
            auto it = group_of_tail_.find(c);
            if (it != group_of_tail_.end()) order.push_back(it->second);
        }
        // Pairs: a call B whose launch can ride on an earlier call A of the same operator on the same input (the
        // operator's FHIPPairQuery decides: a block's 1x1 downsample on its first convolution).  B's group leaves
        // the emission order; A's launch writes both values.  B's other inputs must exist before A runs (function
        // parameters or constants), and B is unfused and comes after A, so nothing between them reads B's value.
        std::vector<int> carries(groups_.size(), -1);
        const char* pair_env = std::getenv("KXC_HIP_PAIR");                     // "0" switches pairing off
        if (cfg_->hip_fuse && cfg_->hip_use_handwritten && cfg_->hip_pair_convolutions && !(pair_env && pair_env[0] == '0')) {
            std::vector<bool> merged(groups_.size(), false);
            for (size_t sb = 1; sb < order.size(); ++sb) {
                const Group& gb = groups_[order[sb]];
                const auto* opb = gb.head->op.As<OpNode>();
                const auto* query = OpAttr<relay::FHIPPairQuery>(opb, "FHIPPairQuery");
                if (!query || gb.head != gb.tail || gb.residual || gb.fused_relu) continue;
                if (gb.tail == f_->body.get() || !OpAttr<relay::FHIPDispatch>(opb, "FHIPDispatch")) continue;
                bool inputs_ready = true;
                for (size_t i = 1; i < gb.head->args.size(); ++i)
                    inputs_ready = inputs_ready && arg_index_.count(Resolve(gb.head->args[i].get())) > 0;
                if (!inputs_ready) continue;
                Array<Type> b_types;
                for (const auto& a : gb.head->args) b_types.push_back(a.checked_type());
                for (size_t sa = 0; sa < sb; ++sa) {
                    const size_t ia = order[sa];
                    const Group& ga = groups_[ia];
                    if (merged[ia] || carries[ia] >= 0 || ga.pool || ga.head->op.get() != gb.head->op.get()) continue;
                    if (ga.tail == f_->body.get() || TT(ga.head->checked_type_)->dtype != TT(gb.head->checked_type_)->dtype) continue;
                    if (Resolve(ga.head->args[0].get()) != Resolve(gb.head->args[0].get())) continue;
                    // both launches must read the shared input and write their results in the same layouts
                    if (LayoutOf(ga.tail) != LayoutOf(gb.tail) || choice_.at(ga.head).inputs[0] != choice_.at(gb.head).inputs[0]) continue;
                    if (TT(ga.tail->checked_type_)->shape != TT(gb.tail->checked_type_)->shape) continue;
                    Array<Type> a_types;
                    std::vector<bool> a_const;
                    for (const auto& a : ga.head->args) {
                        a_types.push_back(a.checked_type());
                        a_const.push_back(dynamic_cast<const ConstantNode*>(Resolve(a.get())) != nullptr);
                    }
                    const char* wino_env = std::getenv("KXC_HIP_WINOGRAD");
                    if (!cfg_->hip_winograd || (wino_env && wino_env[0] == '0')) a_const.assign(a_const.size(), false);
                    if (!(*query)(ga.head->attrs, a_types, a_const, gb.head->attrs, b_types)) continue;
                    carries[ia] = static_cast<int>(order[sb]);
                    merged[order[sb]] = true;
                    break;
                }
            }
            std::vector<size_t> kept;
            for (size_t g : order)
                if (!merged[g]) kept.push_back(g);
            order.swap(kept);
        }
        // Independent branches: a hand-written convolution whose value is only the residual operand of a later
        // fused convolution (a block's 1x1 downsample) and that does not depend on the group emitted just before
        // it moves in front of that group and runs on the plan's side lane, concurrently with it; the consumer
        // joins.  side_of[g] = group that joins, or -1.
        std::vector<int> side_join(groups_.size(), -1);
        std::vector<bool> joins(groups_.size(), false);
        const char* conc_env = std::getenv("KXC_HIP_CONCURRENT_BRANCHES");     // "0" switches the side lane off
        // (the shares of a batch already overlap: no side lane inside a share)
        if (cfg_->hip_fuse && cfg_->hip_use_handwritten && cfg_->hip_concurrent_branches && !dry_ && lanes_ == 1 &&
            !(conc_env && conc_env[0] == '0')) {
            for (size_t step = 1; step < order.size(); ++step) {
                const Group& g = groups_[order[step]];
                const Group& prev = groups_[order[step - 1]];
                if (!IsOp(g.head, "nn_conv2d") || !IsOp(prev.head, "nn_conv2d") || g.residual || !IsF32(g.head->checked_type_)) continue;
                if (side_join[order[step - 1]] >= 0 || joins[order[step - 1]]) continue;
                bool depends = false;
                for (const auto& a : g.head->args) depends = depends || Resolve(a.get()) == prev.tail;
                if (depends) continue;
                int consumer = -1;
                for (size_t later = step + 1; later < order.size() && consumer < 0; ++later)
                    if (groups_[order[later]].residual == g.tail) consumer = static_cast<int>(order[later]);
                const CallNode* sole = SoleConsumer(g.tail);
                if (consumer < 0 || !sole || !IsOp(sole, "add")) continue;
                // The fork and the join cost about 15 us of idle stream time between them, so a short branch is
                // cheaper in line.  Measured on ResNet-18: the side lane gains 1-1.5 % at batch 64-128 and loses
                // 1-7 % at batch 1-32; branches of 3 Mi output elements and more are the ones that gained.
                int64_t branch_elems = 1;
                for (int64_t d : TT(g.tail->checked_type_)->shape) branch_elems *= d;
                int64_t min_elems = 3 << 20;
                if (const char* e = std::getenv("KXC_HIP_CONCURRENT_MIN_ELEMS")) min_elems = std::atoll(e);
                if (branch_elems < min_elems) continue;
                side_join[order[step]] = consumer;
                joins[consumer] = true;
                std::swap(order[step - 1], order[step]);
            }
        }
        // last reader of every (resolved) value, in emission steps; alias ops are transparent
        std::unordered_map<const RelayExprNode*, int> last_use;
        std::vector<bool> is_alias(groups_.size(), false);
        for (size_t step = 0; step < order.size(); ++step) {
            const Group& g = groups_[order[step]];
            const auto* op = g.head->op.As<OpNode>();
            if (OpFlag(op, "THIPAlias") && g.tail != f_->body.get() && g.head == g.tail &&
                LayoutOf(g.head->args[0].get()) == relay::kHIPLayoutPlain) {
                is_alias[order[step]] = true;
                alias_[g.head] = g.head->args[0].get();
            }
        }
        for (size_t step = 0; step < order.size(); ++step) {
            const Group& g = groups_[order[step]];
            if (is_alias[order[step]]) continue;
            for (const auto& a : g.head->args) last_use[Resolve(a.get())] = static_cast<int>(step);
            if (g.residual) last_use[Resolve(g.residual)] = static_cast<int>(step);
            if (carries[order[step]] >= 0)
                for (const auto& a : groups_[carries[order[step]]].head->args) last_use[Resolve(a.get())] = static_cast<int>(step);
        }
        last_use[Resolve(f_->body.get())] = static_cast<int>(order.size());
        // a side-lane launch may still be reading its operands until the join has been enqueued
        for (size_t step = 0; step < order.size(); ++step) {
            if (side_join[order[step]] < 0) continue;
            int join_step = static_cast<int>(step);
            for (size_t later = step + 1; later < order.size(); ++later)
                if (static_cast<int>(order[later]) == side_join[order[step]]) join_step = static_cast<int>(later);
            for (const auto& a : groups_[order[step]].head->args) {
                int& lu = last_use[Resolve(a.get())];
                if (lu < join_step) lu = join_step;
            }
        }

        for (size_t step = 0; step < order.size(); ++step) {
            const Group& g = groups_[order[step]];
            if (is_alias[order[step]]) continue;
            const auto* op = g.head->op.As<OpNode>();
            // output buffer (a result that is not produced in the function's own layout goes through a slot and a converter)
            relay::HIPBuffer out, final_out;
            std::vector<std::pair<int64_t, int64_t>> temps;        // slots that live for this step only
            const int out_layout = LayoutOf(g.tail);
            const bool convert_result = g.tail == f_->body.get() && out_layout != relay::kHIPLayoutPlain;
            if (g.tail == f_->body.get()) {
                out = {KXC_HIP_BUF_ARG, num_args_ - 1};
                if (lanes_ > 1) out = {KXC_HIP_BUF_ARG_OFFSET, KXC_HIP_ARG_OFFSET(num_args_ - 1, lane_ * out_share_bytes_)};
                if (convert_result) {
                    final_out = out;
                    temps.push_back(arena_.Alloc(ValueBytes(g.tail)));
                    out = {KXC_HIP_BUF_WORKSPACE, temps.back().first};
                }
            } else {
                slot_[g.tail] = arena_.Alloc(ValueBytes(g.tail));
                out = {KXC_HIP_BUF_WORKSPACE, slot_[g.tail].first};
            }
            relay::HIPDispatchContext ctx;
            ctx.attrs = g.head->attrs;
            const relay::HIPLayoutChoice* choice = nullptr;
            {
                auto ch = choice_.find(g.head);
                if (ch != choice_.end()) choice = &ch->second;
            }
            for (size_t i = 0; i < g.head->args.size(); ++i) {
                const auto& a = g.head->args[i];
                ctx.input_types.push_back(a.checked_type());
                const int have = LayoutOf(a.get()), want = choice ? choice->inputs[i] : static_cast<int>(relay::kHIPLayoutPlain);
                ctx.input_layouts.push_back(want);
                if (have == want) {
                    ctx.inputs.push_back(BufferOf(a.get()));
                } else {
                    temps.push_back(arena_.Alloc(relay::HIPLayoutBytes(a.checked_type(), want)));
                    const relay::HIPBuffer converted{KXC_HIP_BUF_WORKSPACE, temps.back().first};
                    EmitLayoutConvert(a.get(), have, want, BufferOf(a.get()), converted);
                    ctx.inputs.push_back(converted);
                }
            }
            ctx.output_layout = out_layout;
            for (const auto& a : g.head->args) {
                ctx.input_constant.push_back(dynamic_cast<const ConstantNode*>(Resolve(a.get())) != nullptr);
                ctx.input_argument.push_back(arg_index_.count(Resolve(a.get())) > 0);
            }
            const char* wino_env = std::getenv("KXC_HIP_WINOGRAD");                 // "0" switches Winograd off
            ctx.winograd_allowed = cfg_->hip_winograd && !(wino_env && wino_env[0] == '0');
            ctx.alloc_persistent = [this](int64_t bytes) {
                // (the shares of a batch ask in the same order and share what the first one got: transformed or
                // packed weights do not depend on the batch)
                if (lane_ > 0 && persistent_cursor_ < persistent_.size()) return persistent_[persistent_cursor_++];
                // above everything handed out so far and never released: no activation of an earlier or later
                // step ever shares the region, so what the first run wrote there is still valid in the next
                const int64_t off = arena_.top;
                arena_.top += (std::max<int64_t>(bytes, 1) + 255) / 256 * 256;
                persistent_.push_back(relay::HIPBuffer{KXC_HIP_BUF_WORKSPACE, off});
                return persistent_.back();
            };
            const Group* carried = carries[order[step]] >= 0 ? &groups_[carries[order[step]]] : nullptr;
            if (carried) {
                slot_[carried->tail] = arena_.Alloc(ValueBytes(carried->tail));
                ctx.has_pair = true;
                ctx.pair_attrs = carried->head->attrs;
                for (size_t i = 0; i < carried->head->args.size(); ++i) {
                    const auto& a = carried->head->args[i];
                    ctx.pair_input_types.push_back(a.checked_type());
                    // (input 0 is the first call's; the others are packed arguments, which are always plain)
                    ctx.pair_inputs.push_back(i == 0 ? ctx.inputs[0] : BufferOf(a.get()));
                }
                ctx.pair_output = {KXC_HIP_BUF_WORKSPACE, slot_[carried->tail].first};
                ctx.pair_output_layout = LayoutOf(carried->tail);
            }
            if (g.pool) {
                ctx.has_pool = true;
                ctx.pool_op = g.pool->op.As<OpNode>()->name;
                ctx.pool_attrs = g.pool->attrs;
                ctx.alloc_temp = [this, &temps](int64_t bytes) {
                    temps.push_back(arena_.Alloc(bytes));
                    return relay::HIPBuffer{KXC_HIP_BUF_WORKSPACE, temps.back().first};
                };
            }
            ctx.out_type = g.tail->checked_type_;
            ctx.output = out;
            ctx.fused_relu = g.fused_relu;
            ctx.has_residual = g.residual != nullptr;
            if (g.residual) ctx.residual = BufferOf(g.residual);

            KernelExecInfo info;
            info.op_name = op->name;
            for (const auto& a : g.head->args) info.input_values.push_back(value_id_.at(a.get()));
            if (g.residual) info.input_values.push_back(value_id_.at(g.residual));
            info.output_values.push_back(value_id_.at(g.tail));
            if (carried) {
                for (size_t i = 1; i < carried->head->args.size(); ++i) info.input_values.push_back(value_id_.at(carried->head->args[i].get()));
                info.output_values.push_back(value_id_.at(carried->tail));
            }

            std::string symbol;
            const int32_t first_node = kxc_hip_plan_num_nodes(m_->plan);
            const auto* dispatch = cfg_->hip_use_handwritten ? OpAttr<relay::FHIPDispatch>(op, "FHIPDispatch") : nullptr;
            if (OpFlag(op, "THIPAlias")) {
                // a view that is the function's result: materialise it with a copy
                if (kxc_hip_plan_add_copy(m_->plan, TypeBytes(g.tail->checked_type_), {ctx.inputs[0].kind, ctx.inputs[0].index_or_offset},
                                          {out.kind, out.index_or_offset}))
                    throw std::runtime_error(std::string("plan copy failed: ") + kxc_hip_last_error());
                symbol = "kxc_copy";
            } else if (dispatch) {
                symbol = (*dispatch)(ctx, m_->plan);
            }
            if (!symbol.empty()) {
                info.kernel_symbol = symbol;
                m_->execs.push_back(info);
                const int32_t added = kxc_hip_plan_num_nodes(m_->plan) - first_node;
                if (g.pool) {
                    // the launches behind the first one finish the pooling call
                    for (int32_t k = 1; k < added; ++k) {
                        KernelExecInfo more;
                        more.op_name = ctx.pool_op;
                        more.kernel_symbol = kxc_hip_plan_node_symbol(m_->plan, first_node + k);
                        more.input_values.push_back(value_id_.at(g.tail));
                        more.output_values.push_back(value_id_.at(g.tail));
                        m_->execs.push_back(more);
                    }
                }
                const bool side = side_join[order[step]] >= 0 && added == 1;
                if ((side || joins[order[step]]) && added >= 1 &&
                    kxc_hip_plan_set_concurrency(m_->plan, first_node, side ? 1 : 0, joins[order[step]] ? 1 : 0))
                    throw std::runtime_error(std::string("plan_set_concurrency failed: ") + kxc_hip_last_error());
            } else {
                if (g.fused_relu || g.residual || carried || g.pool) throw std::runtime_error("hip back end: operator declined a fused launch: " + op->name);
                for (int l : ctx.input_layouts)
                    if (l != relay::kHIPLayoutPlain) throw std::runtime_error("hip back end: operator declined the layout it asked for: " + op->name);
                if (out_layout != relay::kHIPLayoutPlain) throw std::runtime_error("hip back end: operator declined the layout it asked for: " + op->name);
                EmitGenerated(g, ctx, info, static_cast<int>(step));
            }
            if (convert_result) EmitLayoutConvert(g.tail, out_layout, relay::kHIPLayoutPlain, out, final_out);
            for (auto& t : temps) arena_.Release(t);
            // release everything whose last reader has now been enqueued
            for (auto it = slot_.begin(); it != slot_.end();) {
                auto lu = last_use.find(it->first);
                if (lu == last_use.end() || lu->second <= static_cast<int>(step)) {
                    if (lu == last_use.end() && it->first == g.tail) { ++it; continue; }   // produced now, unread: keep until end
                    arena_.Release(it->second);
                    it = slot_.erase(it);
                } else {
                    ++it;
                }
            }
        }
    }

    // ---- operators without a hand-written kernel: FRelayToTE -> TIR -> CodeGenHIP -> hipRTC
    void EmitGenerated(const Group& g, const relay::HIPDispatchContext& ctx, const KernelExecInfo& info, int step) {
        Array<Var> params;
        Array<Expr> args;
        for (size_t i = 0; i < g.head->args.size(); ++i) {
            Var v("in" + std::to_string(i), g.head->args[i].checked_type());
            params.push_back(v);
            args.push_back(v);
        }
        Function mini(params, Call(g.head->op, args, g.head->attrs));
        relay::LoweredFunc lowered = relay::LowerToTIRDetailed(relay::InferTypePass(mini));
        tir::PrimFunc pf = tir::RunTIRPassPipeline(lowered.func, {"fold_constant", "simplify_expr"});
        codegen::CodeGenHIP cg;
        codegen::HIPModuleSource src = cg.Generate(pf, "kxc_g" + std::to_string(step));
        if (!compiled_.count(src.source)) m_->source += src.source;
        // buffers: mini-function parameters map to the group's operands, intermediates to scratch slots
        std::unordered_map<const tir::ExprNode*, relay::HIPBuffer> buf;
        for (size_t i = 0; i < g.head->args.size(); ++i) buf[pf->params[i].get()] = ctx.inputs[i];
        buf[pf->params.back().get()] = ctx.output;
        std::vector<std::pair<int64_t, int64_t>> scratch;
        for (const auto& im : lowered.intermediates) {
            scratch.push_back(arena_.Alloc(im.elements * im.dtype.bytes()));
            buf[im.var] = {KXC_HIP_BUF_WORKSPACE, scratch.back().first};
        }
        kxc_hip_module* module = nullptr;
        std::vector<char> log(16384, 0);
        // (the shares of a batch generate the same source for the same step: compiled once)
        auto cached = compiled_.find(src.source);
        if (cached != compiled_.end()) {
            module = cached->second;
        } else {
            m_->module_sources.push_back(src.source);
            if (dry_) {
                size_t size = 0;
                if (kxc_hip_module_compile_only(src.source.c_str(), "kxc_generated.hip", &size, log.data(), log.size()))
                    throw std::runtime_error(std::string("generated HIP source does not compile: ") + kxc_hip_last_error());
            } else {
                if (kxc_hip_module_compile(src.source.c_str(), "kxc_generated.hip", &module, log.data(), log.size()))
                    throw std::runtime_error(std::string("generated HIP source does not compile: ") + kxc_hip_last_error());
                m_->modules.push_back(module);
            }
            compiled_[src.source] = module;
        }
        for (const auto& k : src.kernels) {
            KernelExecInfo e = info;
            e.kernel_symbol = k.symbol + " [generated:" + k.schedule + "]";
            m_->execs.push_back(e);
            if (dry_) continue;
            void* fn = nullptr;
            if (kxc_hip_module_get_function(module, k.symbol.c_str(), &fn))
                throw std::runtime_error(std::string("generated kernel not found: ") + kxc_hip_last_error());
            std::vector<kxc_hip_buf> params_buf;
            for (const tir::ExprNode* b : k.buffers) {
                auto it = buf.find(b);
                if (it == buf.end()) throw std::runtime_error("generated kernel uses an unmapped buffer");
                params_buf.push_back({it->second.kind, it->second.index_or_offset});
            }
            if (kxc_hip_plan_add_module_kernel(m_->plan, fn, k.symbol.c_str(), k.grid, k.block, k.shared_bytes, params_buf.data(),
                                               static_cast<int32_t>(params_buf.size())))
                throw std::runtime_error(std::string("plan_add_module_kernel failed: ") + kxc_hip_last_error());
        }
        for (auto& s : scratch) arena_.Release(s);
    }

    const Function& f_;
    const CompileConfig& cfg_;
    CompiledModuleImpl* m_;
    bool dry_;
    int lanes_ = 1, lane_ = 0;
    int64_t in_share_bytes_ = 0, out_share_bytes_ = 0;
    std::vector<relay::HIPBuffer> persistent_;
    size_t persistent_cursor_ = 0;
    std::unordered_map<std::string, kxc_hip_module*> compiled_;
    int next_value_ = 0, num_inputs_ = 0, num_args_ = 0;
    std::unordered_map<const RelayExprNode*, int> value_id_, arg_index_;
    std::vector<const RelayExprNode*> constants_;
    std::unordered_map<const RelayExprNode*, std::vector<const CallNode*>> consumers_;
    std::vector<const CallNode*> topo_;
    std::unordered_map<const CallNode*, Expr> expr_of_;
    std::vector<Group> groups_;
    std::unordered_map<const CallNode*, size_t> group_of_tail_;
    std::unordered_map<const RelayExprNode*, const RelayExprNode*> alias_;
    std::unordered_map<const RelayExprNode*, int> layout_;                       // how each value lies in memory (HIPLayout)
    std::unordered_map<const CallNode*, relay::HIPLayoutChoice> choice_;         // what each call's kernel takes and writes
    std::unordered_map<const RelayExprNode*, std::pair<int64_t, int64_t>> slot_;
    Arena arena_;
};

}  // namespace

namespace {
bool HasQuantisedCalls(const Expr& body) {
    std::unordered_set<const RelayExprNode*> seen;
    std::vector<const RelayExprNode*> stack{body.get()};
    while (!stack.empty()) {
        const RelayExprNode* e = stack.back();
        stack.pop_back();
        if (!e || !seen.insert(e).second) continue;
        const auto* call = dynamic_cast<const CallNode*>(e);
        if (!call) continue;
        const auto* op = call->op.As<OpNode>();
        if (op && op->name.compare(0, 4, "qnn_") == 0) return true;
        for (const auto& a : call->args) stack.push_back(a.get());
    }
    return false;
}

// The caller's active context, else one made from the configuration's profile_options when those are enabled
// (src/api/compiler.cc:32-40).
std::shared_ptr<profiling::ProfileContext> MaybeCreateProfileContext(const CompileConfig& config) {
    if (profiling::CurrentContext()) return profiling::CurrentContext();
    if (!config.defined() || !config->profile_options.enabled) return nullptr;
    return profiling::ProfileContext::Create(config->profile_options);
}
}  // namespace

CompiledModule Compiler::Compile(Function func, CompileConfig config) {
    if (!config.defined() || !config->target.defined()) throw std::runtime_error("Compiler::Compile: config has no target");
    std::shared_ptr<profiling::ProfileContext> own_context;
    std::unique_ptr<profiling::ActivationScope> own_activation;
    if (!profiling::CurrentContext()) {
        own_context = MaybeCreateProfileContext(config);
        if (own_context) own_activation = std::make_unique<profiling::ActivationScope>(own_context, own_context->NextRunId("compile"));
    }
    struct FlushOnExit {
        std::shared_ptr<profiling::ProfileContext> ctx;
        ~FlushOnExit() { if (ctx) ctx->Flush(); }
    } flush{own_context};
    if (config->mode == CompileMode::kAdaptive) {
        // the session compiles (ahead-of-time mode) on demand; every suggested shape is warmed up now, each as the
        // shape of a single input (src/api/compiler.cc:64-80)
        CompiledModule adaptive;
        adaptive.session_ = std::make_shared<runtime::RuntimeSession>(func, config, profiling::CurrentContext());
        for (const auto& shape : config->suggested_input_shapes) adaptive.session_->WarmUp({shape});
        adaptive.session_profile_ = own_context;
        return adaptive;
    }
    auto impl = std::make_shared<CompiledModuleImpl>();
    impl->config = config;
    impl->profile_context = own_context;
    profiling::EventSpec cspec;
    cspec.component = "compiler";
    cspec.event_type = "compile";
    cspec.device = config->target->kind;
    profiling::ScopedSpan compile_span = profiling::CurrentSpan(cspec);
    Function typed;
    {
        profiling::EventSpec e;
        e.component = "relay.transform";
        e.event_type = "pass";
        e.pass_name = "InferType";
        profiling::ScopedSpan span = profiling::CurrentSpan(e);
        typed = relay::InferTypePass(func);
    }
    if (config->target->kind == "hip") {
        // the whole-function TIR is kept for inspection (GetPrimFunc) and fixes the parameter order
        relay::LoweredFunc whole = relay::LowerToTIRDetailed(typed);
        impl->prim_func = tir::RunTIRPassPipeline(whole.func, {"fold_constant", "simplify_expr"});
        impl->input_count = impl->prim_func->int_attrs.at("kxc.input_count");
        impl->constant_count = impl->prim_func->int_attrs.at("kxc.constant_count");
        const bool dry = config->target->attrs.exists == 0;
        {
            profiling::EventSpec e;
            e.component = "backend.hip";
            e.event_type = "build_plan";
            e.device = "hip:" + std::to_string(config->target->device.device_id());
            profiling::ScopedSpan span = profiling::CurrentSpan(e);
            // shares of the batch side by side (CompileConfigNode::hip_batch_lanes; KXC_HIP_BATCH_LANES overrides)
            int want = config->hip_batch_lanes;
            if (const char* e = std::getenv("KXC_HIP_BATCH_LANES")) want = std::atoi(e);
            if (want < 0 || want > 8) throw std::runtime_error("hip_batch_lanes must be in [0, 8]");
            Function share;
            int lanes = 1;
            if (want != 1 && config->hip_use_handwritten && !typed->params.empty()) {
                const auto* t0 = typed->params[0].checked_type().As<TensorTypeNode>();
                const int64_t batch = t0 && !t0->shape.empty() ? t0->shape[0] : 0;
                // (measured on ResNet-18: the fp32 network gains from two shares from batch 64 on, the quantised one,
                // whose launches are 7-15 us each, from batch 128 on)
                const int ask = want == 0 ? (batch >= (HasQuantisedCalls(typed->body) ? 128 : 64) ? 2 : 1) : want;
                if (ask > 1) {
                    share = relay::SplitBatch(typed, ask);
                    if (share.defined() && (TypeBytes(share->params[0].checked_type()) % 16 != 0 || TypeBytes(share->body.checked_type()) % 16 != 0))
                        share = Function();       // a share of an argument must start on a 16-byte boundary
                    if (share.defined()) lanes = ask;
                    else if (want > 1)
                        throw std::runtime_error("hip_batch_lanes = " + std::to_string(want) + ": the graph cannot be split along the batch of parameter 0");
                }
            }
            HipBuilder builder(lanes > 1 ? share : typed, config, impl.get(), dry, lanes);
            builder.Build();
            span.AddMetric("batch_lanes", static_cast<double>(lanes));
            span.AddMetric("launches", static_cast<double>(impl->execs.size()));
            span.AddMetric("workspace_bytes", static_cast<double>(impl->workspace_bytes));
        }
        if (static_cast<int64_t>(impl->constants.size()) != impl->constant_count)
            throw std::runtime_error("hip back end: constant order disagrees with the lowering");
    } else {
        profiling::EventSpec e;
        e.component = "codegen";
        e.event_type = "host_c_compile";
        profiling::ScopedSpan span = profiling::CurrentSpan(e);
        CompileHost(typed, config, impl.get());
    }
    CompiledModule module(impl);
    if (auto ctx = profiling::CurrentContext()) {
        if (ctx->options().enabled && ctx->options().record_execution_plan_details && config->target->kind == "hip")
            ctx->WriteArtifact("execution_plan.json", module.ExecutionPlanJSON());
        if (profiling::ShouldCaptureIR(ctx, true, false) && !impl->source.empty())
            ctx->WriteArtifact(config->target->kind == "hip" ? "generated_kernels.hip" : "kernel_main.c", impl->source);
    }
    return module;
}

void CompiledModule::Run(const std::vector<void*>& packed_args, const std::vector<std::vector<int64_t>>& input_shapes) {
    if (session_) { session_->Run(packed_args, input_shapes); return; }
    Run(packed_args);
}
void CompiledModule::WarmUp(const std::vector<std::vector<int64_t>>& input_shapes) {
    if (session_) session_->WarmUp(input_shapes);
}
void CompiledModule::WaitAll() {
    if (session_) session_->WaitAll();
}

void CompiledModule::Run(const std::vector<void*>& packed_args) {
    if (session_) throw std::runtime_error("Adaptive mode requires Run(args, input_shapes). Use the overload with input_shapes.");
    if (!impl_ || !impl_->ready) throw std::runtime_error("CompiledModule::Run: module is not ready: " + GetStatus());
    const size_t expect = static_cast<size_t>(impl_->input_count + impl_->constant_count + 1);
    if (packed_args.size() != expect)
        throw std::runtime_error("CompiledModule::Run: expected " + std::to_string(expect) + " packed arguments, got " +
                                 std::to_string(packed_args.size()));
    // a module compiled with profile_options carries its own context (src/api/compiler.cc:149-168)
    std::unique_ptr<profiling::ActivationScope> activation;
    if (impl_->profile_context && !profiling::CurrentContext())
        activation = std::make_unique<profiling::ActivationScope>(impl_->profile_context, impl_->profile_context->NextRunId("execute"));
    struct FlushOnExit {
        std::shared_ptr<profiling::ProfileContext> ctx;
        ~FlushOnExit() { if (ctx) ctx->Flush(); }
    } flush{activation ? impl_->profile_context : nullptr};
    // (src/api/compiler.cc:158-163: one "compiled_module_run" span per call, carrying the kernel's name)
    profiling::EventSpec mspec;
    mspec.component = "runtime";
    mspec.event_type = "compiled_module_run";
    mspec.kernel_symbol = impl_->kernel->kernel_name;
    profiling::ScopedSpan module_span = profiling::CurrentSpan(mspec);
    if (impl_->kernel->backend != codegen::CodeGenBackend::kHIP) {
        impl_->kernel(packed_args);
        return;
    }
    auto ctx = profiling::CurrentContext();
    if (ctx && ctx->options().enabled && ctx->options().enable_gpu_activity && ctx->gpu_activity_mode() != 2) {
        // One "runtime" span for the call, one "backend.hip" event per launch from the plan's HIP events.
        // (With rocprofiler-sdk as the source every dispatch is recorded by the profiler and the plan runs as usual.)
        profiling::EventSpec rspec;
        rspec.component = "runtime";
        rspec.event_type = "kernel_run";
        rspec.kernel_symbol = "kxc_kernel_main";
        const std::string device = "hip:" + std::to_string(impl_->config->target->device.device_id());
        rspec.device = device;
        profiling::ScopedSpan run_span(ctx, rspec);
        std::vector<kxc_hip_launch_record> records(impl_->execs.size() + 8);
        int32_t count = 0;
        const std::int64_t t0 = ctx->NowNs();
        if (kxc_hip_plan_run_profiled(impl_->plan, const_cast<void**>(packed_args.data()), nullptr, records.data(),
                                      static_cast<int32_t>(records.size()), &count)) {
            run_span.SetStatus("error");
            throw std::runtime_error(std::string("Kernel kxc_kernel_main failed: ") + kxc_hip_last_error());
        }
        for (int32_t i = 0; i < count; ++i) {
            const kxc_hip_launch_record& r = records[i];
            profiling::EventSpec e;
            e.component = "backend.hip";
            e.event_type = r.kind == KXC_HIP_RECORD_MEMCPY ? "hip_memcpy" : "hip_kernel";
            e.device = device;
            e.kernel_symbol = r.kernel_symbol;
            if (static_cast<size_t>(i) < impl_->execs.size()) e.op_name = impl_->execs[i].op_name;
            e.fields["backend.hip.launch_index"] = std::to_string(i);
            e.fields["backend.hip.timing_source"] = "hip_events";
            e.metrics["grid_x"] = r.grid[0]; e.metrics["grid_y"] = r.grid[1]; e.metrics["grid_z"] = r.grid[2];
            e.metrics["block_x"] = r.block[0]; e.metrics["block_y"] = r.block[1]; e.metrics["block_z"] = r.block[2];
            e.metrics["dynamic_shared_memory"] = r.dynamic_shared_memory;
            if (r.kind == KXC_HIP_RECORD_MEMCPY) e.metrics["bytes"] = static_cast<double>(r.bytes);
            ctx->RecordCompletedSpan(e, profiling::CurrentRunId(), ctx->NextSpanId(), run_span.span_id(), t0 + r.start_ns,
                                     t0 + r.start_ns + r.duration_ns);
        }
        run_span.AddMetric("launches", count);
        return;     // the profiled run has already waited for the last launch
    }
    impl_->kernel(packed_args);
}

bool CompiledModule::IsReady() const { return session_ || (impl_ && impl_->ready && impl_->kernel.IsReady()); }
const codegen::CompiledKernel& CompiledModule::GetKernel() const {
    if (!impl_) throw std::runtime_error("GetKernel: empty module");
    return impl_->kernel;
}
std::string CompiledModule::GetProfileBundlePath() const {
    if (session_) return session_profile_ ? session_profile_->bundle_dir() : "";
    return impl_ && impl_->profile_context ? impl_->profile_context->bundle_dir() : "";
}
std::string CompiledModule::GetStatus() const { return session_ ? session_->GetStatus() : impl_ ? impl_->status : "empty"; }
const tir::PrimFunc& CompiledModule::GetPrimFunc() const { return impl_->prim_func; }
const std::string& CompiledModule::GetSource() const { return impl_->source; }
void CompiledModule::SaveCSource(const std::string& path) const {
    std::ofstream out(path);
    if (!out) throw std::runtime_error("SaveCSource: cannot open " + path);
    out << impl_->source;
}
const Array<runtime::NDArray>& CompiledModule::GetConstants() const { return impl_->constants; }
int64_t CompiledModule::input_count() const { return impl_->input_count; }
int64_t CompiledModule::constant_count() const { return impl_->constant_count; }
const std::vector<KernelExecInfo>& CompiledModule::GetKernelExecs() const { return impl_->execs; }
size_t CompiledModule::workspace_bytes() const { return impl_->workspace_bytes; }
void CompiledModule::EnableGraphReplay(bool enable) {
    if (!impl_ || !impl_->plan) throw std::runtime_error("EnableGraphReplay: not a loaded hip module");
    if (kxc_hip_plan_enable_graph(impl_->plan, enable ? 1 : 0)) throw std::runtime_error(std::string("EnableGraphReplay: ") + kxc_hip_last_error());
}

std::vector<int64_t> CompiledModule::RunTimed(const std::vector<void*>& packed_args) {
    if (!impl_ || !impl_->plan || !impl_->ready) throw std::runtime_error("RunTimed: not a loaded hip module");
    const size_t expect = static_cast<size_t>(impl_->input_count + impl_->constant_count + 1);
    if (packed_args.size() != expect) throw std::runtime_error("RunTimed: expected " + std::to_string(expect) + " packed arguments");
    std::vector<kxc_hip_launch_record> records(static_cast<size_t>(kxc_hip_plan_num_nodes(impl_->plan)) + 1);
    int32_t count = 0;
    if (kxc_hip_plan_run_profiled(impl_->plan, const_cast<void**>(packed_args.data()), nullptr, records.data(),
                                  static_cast<int32_t>(records.size()), &count))
        throw std::runtime_error(std::string("RunTimed: ") + kxc_hip_last_error());
    std::vector<int64_t> out;
    for (int32_t i = 0; i < count; ++i) out.push_back(records[i].duration_ns);
    return out;
}

void CompiledModule::FreezeConstants(bool frozen) {
    if (!impl_ || !impl_->plan) throw std::runtime_error("FreezeConstants: not a loaded hip module");
    if (kxc_hip_plan_freeze_constants(impl_->plan, frozen ? 1 : 0)) throw std::runtime_error(std::string("FreezeConstants: ") + kxc_hip_last_error());
}
void CompiledModule::InvalidateConstants() {
    if (!impl_ || !impl_->plan) throw std::runtime_error("InvalidateConstants: not a loaded hip module");
    if (kxc_hip_plan_invalidate_constants(impl_->plan)) throw std::runtime_error(std::string("InvalidateConstants: ") + kxc_hip_last_error());
}

std::string CompiledModule::ExecutionPlanJSON() const {
    std::ostringstream os;
    os << "{\"schema_version\":1,\"num_values\":" << impl_->num_values << ",\"output_value\":" << impl_->output_value
       << ",\"input_value_ids\":[";
    for (size_t i = 0; i < impl_->input_value_ids.size(); ++i) os << (i ? "," : "") << impl_->input_value_ids[i];
    os << "],\"constant_value_ids\":[";
    for (size_t i = 0; i < impl_->constant_value_ids.size(); ++i) os << (i ? "," : "") << impl_->constant_value_ids[i];
    os << "],\"nodes\":[";
    for (size_t i = 0; i < impl_->execs.size(); ++i) {
        const auto& e = impl_->execs[i];
        os << (i ? "," : "") << "{\"kind\":\"kernel\",\"input_values\":[";
        for (size_t k = 0; k < e.input_values.size(); ++k) os << (k ? "," : "") << e.input_values[k];
        os << "],\"output_values\":[";
        for (size_t k = 0; k < e.output_values.size(); ++k) os << (k ? "," : "") << e.output_values[k];
        os << "],\"worker_set\":[0],\"op_name\":\"" << json::Escape(e.op_name) << "\",\"kernel_symbol\":\""
           << json::Escape(e.kernel_symbol) << "\"}";
    }
    os << "]";
    // Beyond the reference's schema (src/base/execution_plan.cc:674-877 keeps value ids and kernel symbols):
    // what is needed to run the function again without compiling it -- see Compiler::LoadExecutionPlan.
    os << ",\"kxc_hip\":{\"target_kind\":\"" << json::Escape(impl_->config->target->kind) << "\",\"input_count\":"
       << impl_->input_count << ",\"constant_count\":" << impl_->constant_count << ",\"workspace_bytes\":"
       << impl_->workspace_bytes << ",\"generated_modules\":[";
    for (size_t i = 0; i < impl_->module_sources.size(); ++i)
        os << (i ? "," : "") << "\"" << json::Escape(impl_->module_sources[i]) << "\"";
    os << "]";
    if (impl_->plan && impl_->ready) {     // a build without a GPU records launches but cannot run them
        size_t needed = 0;
        if (kxc_hip_plan_serialize(impl_->plan, nullptr, 0, &needed))
            throw std::runtime_error(std::string("ExecutionPlanJSON: ") + kxc_hip_last_error());
        std::string text(needed, '\0');
        if (kxc_hip_plan_serialize(impl_->plan, &text[0], text.size(), &needed))
            throw std::runtime_error(std::string("ExecutionPlanJSON: ") + kxc_hip_last_error());
        text.resize(needed - 1);
        os << ",\"launch_plan\":\"" << json::Escape(text) << "\"";
    }
    os << "}}";
    return os.str();
}

CompiledModule Compiler::LoadExecutionPlan(const std::string& plan_json, CompileConfig config) {
    if (!config.defined() || !config->target.defined() || config->target->kind != "hip")
        throw std::runtime_error("LoadExecutionPlan: a hip target is required");
    if (config->target->attrs.exists == 0) throw std::runtime_error("LoadExecutionPlan: no GPU to load the plan on");
    profiling::EventSpec spec;
    spec.component = "compiler";
    spec.event_type = "load_execution_plan";
    profiling::ScopedSpan span = profiling::CurrentSpan(spec);
    const json::Value root = json::Reader(plan_json).Parse();
    if (root.at("schema_version").integer != 1) throw std::runtime_error("LoadExecutionPlan: unsupported schema_version");
    const json::Value& hip = root.at("kxc_hip");
    if (hip.at("target_kind").string != "hip" || !hip.has("launch_plan"))
        throw std::runtime_error("LoadExecutionPlan: the plan carries no launch description for the hip target");
    auto impl = std::make_shared<CompiledModuleImpl>();
    impl->config = config;
    impl->input_count = hip.at("input_count").integer;
    impl->constant_count = hip.at("constant_count").integer;
    impl->num_values = static_cast<int>(root.at("num_values").integer);
    impl->output_value = static_cast<int>(root.at("output_value").integer);
    for (const auto& v : root.at("input_value_ids").array) impl->input_value_ids.push_back(static_cast<int>(v.integer));
    for (const auto& v : root.at("constant_value_ids").array) impl->constant_value_ids.push_back(static_cast<int>(v.integer));
    for (const auto& n : root.at("nodes").array) {
        if (n.at("kind").string != "kernel") throw std::runtime_error("LoadExecutionPlan: only kernel nodes can be replayed");
        KernelExecInfo e;
        e.op_name = n.at("op_name").string;
        e.kernel_symbol = n.at("kernel_symbol").string;
        for (const auto& v : n.at("input_values").array) e.input_values.push_back(static_cast<int>(v.integer));
        for (const auto& v : n.at("output_values").array) e.output_values.push_back(static_cast<int>(v.integer));
        impl->execs.push_back(e);
    }
    std::vector<char> log(16384, 0);
    for (const auto& m : hip.at("generated_modules").array) {
        kxc_hip_module* module = nullptr;
        if (kxc_hip_module_compile(m.string.c_str(), "kxc_generated.hip", &module, log.data(), log.size()))
            throw std::runtime_error(std::string("LoadExecutionPlan: saved kernel source does not compile: ") + kxc_hip_last_error());
        impl->modules.push_back(module);
        impl->module_sources.push_back(m.string);
        impl->source += m.string;
    }
    if (kxc_hip_plan_deserialize(hip.at("launch_plan").string.c_str(), config->target->device.device_id(), impl->modules.data(),
                                 static_cast<int32_t>(impl->modules.size()), &impl->plan))
        throw std::runtime_error(std::string("LoadExecutionPlan: ") + kxc_hip_last_error());
    if (kxc_hip_plan_num_nodes(impl->plan) != static_cast<int32_t>(impl->execs.size()))
        throw std::runtime_error("LoadExecutionPlan: node list and launch plan disagree");
    impl->workspace_bytes = static_cast<size_t>(hip.at("workspace_bytes").integer);
    if (config->hip_constants_frozen) kxc_hip_plan_freeze_constants(impl->plan, 1);
    impl->AdoptHipKernel(true);
    impl->ready = true;
    impl->status = "loaded from an execution plan";
    return CompiledModule(impl);
}

}  // namespace api
}  // namespace kxc
