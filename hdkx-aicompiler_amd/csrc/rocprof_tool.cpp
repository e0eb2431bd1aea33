// rocprof_tool.cpp -- libkxc_hip_rocprof.so: GPU activity records from rocprofiler-sdk's buffered tracing, the
// tool-library counterpart of the reference's CUPTI activity adapter (src/base/profiling.cc:250-695: CUPTI is
// loaded lazily, activity kinds RUNTIME / MEMCPY / MEMSET / KERNEL are enabled, a buffer-completed callback converts
// records into backend events).  Unlike the records libkxc_hip.so takes at its own call sites (activity.hip), these
// cover every HIP call of the process: copies and kernels enqueued by the application or another library appear as
// well.
//
// The library exports rocprofiler_configure, so it registers like any rocprofiler-sdk tool: listed in
// ROCP_TOOL_LIBRARIES, or -- what libkxc_hip.so does for kxc_hip_activity_enable(2) -- loaded with dlopen and
// registered with rocprofiler_force_configure BEFORE the process makes its first HIP call (the HIP runtime hands its
// dispatch table to registered tools while it initialises; later is too late and kxc_rocprof_prepare says so).
// One context with three buffered services (kernel dispatch, memory copy, HIP runtime API with arguments) feeds one
// buffer; a copy or fill call and the device work it caused are joined into one memcpy / memset record; a
// code-object callback (in a second context that always runs) keeps kernel names.  The tracing context only runs
// between kxc_rocprof_start and kxc_rocprof_stop.
// Host code only: no kernels, no device memory.
#include <rocprofiler-sdk/registration.h>
#include <rocprofiler-sdk/rocprofiler.h>

#include <cxxabi.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "kxc_hip.h"

namespace {

struct Tool {
    std::mutex mu;
    rocprofiler_context_id_t ctx{0};          // the three buffered services; runs between start and stop
    rocprofiler_context_id_t names_ctx{0};    // the code-object callback; runs from registration on
    rocprofiler_buffer_id_t buffer{0};
    bool configured = false;        // our initialize callback ran and every service was accepted
    bool running = false;
    std::string status = "not registered";
    std::unordered_map<uint64_t, std::string> kernel_names;      // kernel_id -> name
    std::unordered_map<uint64_t, int32_t> agent_index;           // agent handle -> logical GPU index
    std::vector<kxc_hip_activity_record> done;
    uint64_t dropped = 0;
};
// Nobody may ever drain: beyond these counts new records are dropped (and counted) instead of kept.
constexpr size_t kMaxRecords = 1u << 20;
constexpr size_t kMaxOpenTransfers = 1u << 16;

Tool& T() {
    static Tool* t = new Tool();     // never destroyed: callbacks may arrive during process exit
    return *t;
}

int64_t SteadyNs() {
    return std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// rocprofiler timestamps -> the steady clock the other activity records use
int64_t ClockOffsetNs() {
    rocprofiler_timestamp_t ts = 0;
    if (rocprofiler_get_timestamp(&ts) != ROCPROFILER_STATUS_SUCCESS) return 0;
    return SteadyNs() - static_cast<int64_t>(ts);
}

void CodeObjectCallback(rocprofiler_callback_tracing_record_t record, rocprofiler_user_data_t*, void*) {
    if (record.kind != ROCPROFILER_CALLBACK_TRACING_CODE_OBJECT ||
        record.operation != ROCPROFILER_CODE_OBJECT_DEVICE_KERNEL_SYMBOL_REGISTER || record.phase != ROCPROFILER_CALLBACK_PHASE_LOAD)
        return;
    const auto* sym = static_cast<const rocprofiler_callback_tracing_code_object_kernel_symbol_register_data_t*>(record.payload);
    if (!sym || !sym->kernel_name) return;
    // symbol names carry the kernel descriptor's suffix and C++ mangling; the bundle's kernel_symbol has neither
    std::string name = sym->kernel_name;
    if (name.size() > 3 && name.compare(name.size() - 3, 3, ".kd") == 0) name.resize(name.size() - 3);
    int status = 0;
    if (char* plain = abi::__cxa_demangle(name.c_str(), nullptr, nullptr, &status)) {
        if (status == 0) name = plain;
        std::free(plain);
    }
    std::lock_guard<std::mutex> lock(T().mu);
    T().kernel_names[sym->kernel_id] = name;
}

void Name(kxc_hip_activity_record* r, const char* s) { std::snprintf(r->name, sizeof(r->name), "%s", s ? s : ""); }

// What a copy or fill call asked for, kept until the device work it enqueued reports back under the same
// correlation id (a blit kernel of the runtime or an SDMA copy), so that the bundle shows ONE memcpy / memset
// activity with the call's byte count and direction and the device's times, as CUPTI's records do.
struct Transfer {
    bool fill = false;
    int64_t bytes = 0;
    int32_t copy_kind = 3, value = 0;
    uint64_t stream = 0, thread_id = 0;
    int64_t api_start_ns = 0, api_end_ns = 0;
    char api[40] = {0};
};

int32_t CopyKind(hipMemcpyKind k) {
    switch (k) {
        case hipMemcpyHostToDevice: return 0;
        case hipMemcpyDeviceToHost: return 1;
        case hipMemcpyDeviceToDevice: return 2;
        case hipMemcpyHostToHost: return 3;
        default: return 4;       // hipMemcpyDefault: the runtime decides from the pointers
    }
}

// Fills `t` when the call is one of the copy / fill entry points whose arguments say how many bytes move.
bool TransferOf(const rocprofiler_buffer_tracing_hip_api_ext_record_t& p, Transfer* t) {
    const auto& a = p.args;
    switch (p.operation) {
        case ROCPROFILER_HIP_RUNTIME_API_ID_hipMemcpy:
            t->bytes = static_cast<int64_t>(a.hipMemcpy.sizeBytes); t->copy_kind = CopyKind(a.hipMemcpy.kind); return true;
        case ROCPROFILER_HIP_RUNTIME_API_ID_hipMemcpyAsync:
            t->bytes = static_cast<int64_t>(a.hipMemcpyAsync.sizeBytes); t->copy_kind = CopyKind(a.hipMemcpyAsync.kind);
            t->stream = reinterpret_cast<uint64_t>(a.hipMemcpyAsync.stream); return true;
        case ROCPROFILER_HIP_RUNTIME_API_ID_hipMemcpyWithStream:
            t->bytes = static_cast<int64_t>(a.hipMemcpyWithStream.sizeBytes); t->copy_kind = CopyKind(a.hipMemcpyWithStream.kind);
            t->stream = reinterpret_cast<uint64_t>(a.hipMemcpyWithStream.stream); return true;
        case ROCPROFILER_HIP_RUNTIME_API_ID_hipMemcpyHtoD:
            t->bytes = static_cast<int64_t>(a.hipMemcpyHtoD.sizeBytes); t->copy_kind = 0; return true;
        case ROCPROFILER_HIP_RUNTIME_API_ID_hipMemcpyDtoH:
            t->bytes = static_cast<int64_t>(a.hipMemcpyDtoH.sizeBytes); t->copy_kind = 1; return true;
        case ROCPROFILER_HIP_RUNTIME_API_ID_hipMemcpyDtoD:
            t->bytes = static_cast<int64_t>(a.hipMemcpyDtoD.sizeBytes); t->copy_kind = 2; return true;
        case ROCPROFILER_HIP_RUNTIME_API_ID_hipMemset:
            t->fill = true; t->bytes = static_cast<int64_t>(a.hipMemset.sizeBytes); t->value = a.hipMemset.value; return true;
        case ROCPROFILER_HIP_RUNTIME_API_ID_hipMemsetAsync:
            t->fill = true; t->bytes = static_cast<int64_t>(a.hipMemsetAsync.sizeBytes); t->value = a.hipMemsetAsync.value;
            t->stream = reinterpret_cast<uint64_t>(a.hipMemsetAsync.stream); return true;
        default: return false;
    }
}

std::unordered_map<uint64_t, Transfer>& Transfers() {      // by correlation id; guarded by T().mu
    static auto* m = new std::unordered_map<uint64_t, Transfer>();
    return *m;
}

void TransferRecord(const Transfer& x, uint64_t correlation, kxc_hip_activity_record* r) {
    std::memset(r, 0, sizeof(*r));
    r->kind = x.fill ? KXC_HIP_ACTIVITY_MEMSET : KXC_HIP_ACTIVITY_MEMCPY;
    Name(r, x.api);
    r->bytes = x.bytes; r->value = x.value; r->copy_kind = x.copy_kind;
    r->stream = x.stream; r->thread_id = x.thread_id; r->correlation_id = correlation;
    r->start_ns = x.api_start_ns; r->end_ns = x.api_end_ns;        // replaced by the device's times when there are any
}

// Copies and fills whose call returned at least `min_age_ns` ago and for which no device work has reported: the
// runtime moved the bytes itself (small pageable copies); they are recorded with the call's times.  (mu held)
void EmitSettledTransfers(int64_t now_ns, int64_t min_age_ns) {
    auto& m = Transfers();
    for (auto it = m.begin(); it != m.end();) {
        if (now_ns - it->second.api_end_ns >= min_age_ns) {
            kxc_hip_activity_record r;
            TransferRecord(it->second, it->first, &r);
            T().done.push_back(r);
            it = m.erase(it);
        } else {
            ++it;
        }
    }
}

void BufferCallback(rocprofiler_context_id_t, rocprofiler_buffer_id_t, rocprofiler_record_header_t** headers, size_t count,
                    void*, uint64_t drop_count) {
    const int64_t offset = ClockOffsetNs();
    Tool& t = T();
    std::lock_guard<std::mutex> lock(t.mu);
    t.dropped += drop_count;
    auto agent_of = [&](uint64_t handle) {
        auto a = t.agent_index.find(handle);
        return a != t.agent_index.end() ? a->second : 0;
    };
    // the calls first: a device record of the same batch then finds what its call asked for
    for (size_t i = 0; i < count; ++i) {
        const rocprofiler_record_header_t* h = headers[i];
        if (!h || h->category != ROCPROFILER_BUFFER_CATEGORY_TRACING || !h->payload || h->kind != ROCPROFILER_BUFFER_TRACING_HIP_RUNTIME_API_EXT) continue;
        const auto* p = static_cast<const rocprofiler_buffer_tracing_hip_api_ext_record_t*>(h->payload);
        kxc_hip_activity_record r;
        std::memset(&r, 0, sizeof(r));
        r.kind = KXC_HIP_ACTIVITY_RUNTIME_API;
        const char* name = nullptr;
        uint64_t len = 0;
        if (rocprofiler_query_buffer_tracing_kind_operation_name(p->kind, p->operation, &name, &len) != ROCPROFILER_STATUS_SUCCESS || !name) name = "?";
        Name(&r, name);
        r.start_ns = static_cast<int64_t>(p->start_timestamp) + offset;
        r.end_ns = static_cast<int64_t>(p->end_timestamp) + offset;
        r.correlation_id = p->correlation_id.internal;
        r.thread_id = p->thread_id;
        r.return_value = static_cast<int32_t>(p->retval.hipError_t_retval);
        if (t.done.size() < kMaxRecords) t.done.push_back(r);
        else ++t.dropped;
        Transfer x;
        if (r.return_value == 0 && Transfers().size() < kMaxOpenTransfers && TransferOf(*p, &x) && x.bytes > 0) {
            x.thread_id = p->thread_id; x.api_start_ns = r.start_ns; x.api_end_ns = r.end_ns;
            std::snprintf(x.api, sizeof(x.api), "%s", name);
            Transfers()[r.correlation_id] = x;
        }
    }
    for (size_t i = 0; i < count; ++i) {
        const rocprofiler_record_header_t* h = headers[i];
        if (!h || h->category != ROCPROFILER_BUFFER_CATEGORY_TRACING || !h->payload) continue;
        kxc_hip_activity_record r;
        std::memset(&r, 0, sizeof(r));
        if (h->kind == ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH) {
            const auto* d = static_cast<const rocprofiler_buffer_tracing_kernel_dispatch_record_t*>(h->payload);
            const int64_t start = static_cast<int64_t>(d->start_timestamp) + offset, end = static_cast<int64_t>(d->end_timestamp) + offset;
            auto x = Transfers().find(d->correlation_id.internal);
            if (x != Transfers().end()) {
                // the runtime's own copy / fill kernel: the activity is the transfer, not a kernel of the application
                TransferRecord(x->second, x->first, &r);
                Transfers().erase(x);
                r.stream = r.stream ? r.stream : d->dispatch_info.queue_id.handle;
            } else {
                r.kind = KXC_HIP_ACTIVITY_KERNEL;
                auto it = t.kernel_names.find(d->dispatch_info.kernel_id);
                Name(&r, it != t.kernel_names.end() ? it->second.c_str() : "?");
                // HSA grid sizes count work-items; the bundle's grid_* are workgroups, as CUDA's and HIP's are
                const rocprofiler_dim3_t& g = d->dispatch_info.grid_size;
                const rocprofiler_dim3_t& w = d->dispatch_info.workgroup_size;
                r.block[0] = w.x; r.block[1] = w.y; r.block[2] = w.z;
                r.grid[0] = w.x ? g.x / w.x : g.x; r.grid[1] = w.y ? g.y / w.y : g.y; r.grid[2] = w.z ? g.z / w.z : g.z;
                r.dynamic_shared_memory = d->dispatch_info.group_segment_size;     // static + dynamic LDS of the dispatch
                r.correlation_id = d->correlation_id.internal;
                r.thread_id = d->thread_id;
                r.stream = d->dispatch_info.queue_id.handle;
            }
            r.start_ns = start; r.end_ns = end;
            r.timed_on_gpu = 1;
            r.device_id = agent_of(d->dispatch_info.agent_id.handle);
        } else if (h->kind == ROCPROFILER_BUFFER_TRACING_MEMORY_COPY) {
            const auto* c = static_cast<const rocprofiler_buffer_tracing_memory_copy_record_t*>(h->payload);
            auto x = Transfers().find(c->correlation_id.internal);
            if (x != Transfers().end()) {
                TransferRecord(x->second, x->first, &r);
                Transfers().erase(x);
            } else {
                r.kind = KXC_HIP_ACTIVITY_MEMCPY;
                Name(&r, "memory_copy");
                r.correlation_id = c->correlation_id.internal;
                r.thread_id = c->thread_id;
            }
            r.bytes = static_cast<int64_t>(c->bytes);
            switch (c->operation) {
                case ROCPROFILER_MEMORY_COPY_HOST_TO_DEVICE: r.copy_kind = 0; break;
                case ROCPROFILER_MEMORY_COPY_DEVICE_TO_HOST: r.copy_kind = 1; break;
                case ROCPROFILER_MEMORY_COPY_DEVICE_TO_DEVICE: r.copy_kind = 2; break;
                default: r.copy_kind = 3; break;
            }
            r.start_ns = static_cast<int64_t>(c->start_timestamp) + offset;
            r.end_ns = static_cast<int64_t>(c->end_timestamp) + offset;
            r.timed_on_gpu = 1;
            r.device_id = agent_of(c->operation == ROCPROFILER_MEMORY_COPY_DEVICE_TO_HOST ? c->src_agent_id.handle : c->dst_agent_id.handle);
        } else {
            continue;
        }
        if (t.done.size() < kMaxRecords) t.done.push_back(r);
        else ++t.dropped;
    }
}

rocprofiler_status_t AgentCallback(rocprofiler_agent_version_t version, const void** agents, size_t count, void*) {
    if (version != ROCPROFILER_AGENT_INFO_VERSION_0) return ROCPROFILER_STATUS_SUCCESS;
    std::lock_guard<std::mutex> lock(T().mu);
    for (size_t i = 0; i < count; ++i) {
        const auto* a = static_cast<const rocprofiler_agent_v0_t*>(agents[i]);
        if (a->type == ROCPROFILER_AGENT_TYPE_GPU) T().agent_index[a->id.handle] = a->logical_node_type_id;
    }
    return ROCPROFILER_STATUS_SUCCESS;
}

#define KXC_TOOL_TRY(call, what)                                                                        \
    do {                                                                                                \
        const rocprofiler_status_t st_ = (call);                                                        \
        if (st_ != ROCPROFILER_STATUS_SUCCESS) {                                                        \
            T().status = std::string(what) + ": " + rocprofiler_get_status_string(st_);                 \
            return -1;                                                                                  \
        }                                                                                               \
    } while (0)

int ToolInit(rocprofiler_client_finalize_t, void*) {
    Tool& t = T();
    (void)rocprofiler_query_available_agents(ROCPROFILER_AGENT_INFO_VERSION_0, AgentCallback, sizeof(rocprofiler_agent_v0_t), nullptr);
    // Kernel names come with the code objects, which HIP loads when a module's first kernel is launched -- possibly
    // long before anybody asks for activity records.  The callback therefore has a context of its own that runs from
    // now on (it is invoked once per kernel symbol and costs nothing afterwards).
    KXC_TOOL_TRY(rocprofiler_create_context(&t.names_ctx), "create_context");
    KXC_TOOL_TRY(rocprofiler_configure_callback_tracing_service(t.names_ctx, ROCPROFILER_CALLBACK_TRACING_CODE_OBJECT, nullptr, 0,
                                                                CodeObjectCallback, nullptr),
                 "code object tracing");
    KXC_TOOL_TRY(rocprofiler_start_context(t.names_ctx), "start_context (kernel names)");
    KXC_TOOL_TRY(rocprofiler_create_context(&t.ctx), "create_context");
    // 4 MiB, delivered when seven eighths full or flushed; records are never overwritten
    constexpr size_t kBytes = 4u << 20;
    KXC_TOOL_TRY(rocprofiler_create_buffer(t.ctx, kBytes, kBytes - kBytes / 8, ROCPROFILER_BUFFER_POLICY_LOSSLESS, BufferCallback,
                                           nullptr, &t.buffer),
                 "create_buffer");
    KXC_TOOL_TRY(rocprofiler_configure_buffer_tracing_service(t.ctx, ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH, nullptr, 0, t.buffer),
                 "kernel dispatch tracing");
    KXC_TOOL_TRY(rocprofiler_configure_buffer_tracing_service(t.ctx, ROCPROFILER_BUFFER_TRACING_MEMORY_COPY, nullptr, 0, t.buffer),
                 "memory copy tracing");
    KXC_TOOL_TRY(rocprofiler_configure_buffer_tracing_service(t.ctx, ROCPROFILER_BUFFER_TRACING_HIP_RUNTIME_API_EXT, nullptr, 0, t.buffer),
                 "HIP runtime API tracing");
    rocprofiler_callback_thread_t thread{};
    KXC_TOOL_TRY(rocprofiler_create_callback_thread(&thread), "create_callback_thread");
    KXC_TOOL_TRY(rocprofiler_assign_callback_thread(t.buffer, thread), "assign_callback_thread");
    int valid = 0;
    KXC_TOOL_TRY(rocprofiler_context_is_valid(t.ctx, &valid), "context_is_valid");
    if (!valid) { t.status = "context is not valid"; return -1; }
    t.configured = true;
    t.status = "registered";
    return 0;
}

void ToolFini(void*) {
    Tool& t = T();
    if (t.configured) (void)rocprofiler_flush_buffer(t.buffer);
    t.running = false;
    t.configured = false;
    t.status = "finalized";
}

}  // namespace

extern "C" {

rocprofiler_tool_configure_result_t* rocprofiler_configure(uint32_t, const char*, uint32_t, rocprofiler_client_id_t* client_id) {
    if (client_id) client_id->name = "kxc_hip_activity";
    static rocprofiler_tool_configure_result_t result{sizeof(rocprofiler_tool_configure_result_t), &ToolInit, &ToolFini, nullptr};
    return &result;
}

// Registers the tool if the process has not configured rocprofiler-sdk yet.  0: the context exists.  Otherwise the
// reason is in kxc_rocprof_status() -- typically that HIP was initialised before this call.
int32_t kxc_rocprof_prepare(void) {
    Tool& t = T();
    if (t.configured) return 0;
    int initialised = 0;
    (void)rocprofiler_is_initialized(&initialised);
    if (initialised == 0) {
        const rocprofiler_status_t st = rocprofiler_force_configure(&rocprofiler_configure);
        if (st != ROCPROFILER_STATUS_SUCCESS && !t.configured)
            t.status = std::string("rocprofiler_force_configure: ") + rocprofiler_get_status_string(st);
    } else if (!t.configured && t.status == "not registered") {
        t.status = "rocprofiler-sdk was configured before this tool was loaded (a HIP call came first): request the "
                   "tool before the first HIP call, or list this library in ROCP_TOOL_LIBRARIES";
    }
    return t.configured ? 0 : 1;
}

const char* kxc_rocprof_status(void) { return T().status.c_str(); }

int32_t kxc_rocprof_start(void) {
    Tool& t = T();
    if (!t.configured) return 1;
    if (t.running) return 0;
    const rocprofiler_status_t st = rocprofiler_start_context(t.ctx);
    if (st != ROCPROFILER_STATUS_SUCCESS) { t.status = std::string("start_context: ") + rocprofiler_get_status_string(st); return 1; }
    t.running = true;
    return 0;
}

int32_t kxc_rocprof_stop(void) {
    Tool& t = T();
    if (!t.configured || !t.running) return 0;
    (void)rocprofiler_stop_context(t.ctx);
    t.running = false;
    return 0;
}

// Flushes the buffer and hands over the records delivered so far (capacity 0: only counts them).
int32_t kxc_rocprof_drain(kxc_hip_activity_record* records, int32_t capacity, int32_t* count) {
    Tool& t = T();
    if (!count || (capacity > 0 && !records)) return 1;
    if (t.configured) {
        const rocprofiler_status_t st = rocprofiler_flush_buffer(t.buffer);
        if (st != ROCPROFILER_STATUS_SUCCESS && st != ROCPROFILER_STATUS_ERROR_BUFFER_BUSY)
            t.status = std::string("flush_buffer: ") + rocprofiler_get_status_string(st);
    }
    std::lock_guard<std::mutex> lock(t.mu);
    EmitSettledTransfers(SteadyNs(), 50000000);      // calls that returned 50 ms ago and never reached the device
    const int32_t n = static_cast<int32_t>(t.done.size());
    *count = n;
    if (capacity == 0) return 0;
    if (capacity < n) return 1;
    for (int32_t i = 0; i < n; ++i) records[i] = t.done[static_cast<size_t>(i)];
    t.done.clear();
    return 0;
}

uint64_t kxc_rocprof_dropped(void) { return T().dropped; }

}  // extern "C"
