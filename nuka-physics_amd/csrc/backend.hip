// PHI-shaped HIP backend: buffer types and buffers, the backend with its stream, eager dispatch through an op
// table, plans as captured HIP graphs, events, and the device / registry-entry tables.
// Counterpart of src/phi/backend_cuda/{cuda_backend.cu, cuda_buffer.cu, device.cu, ops/registry.cu}.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>

#include "backend.h"
#include "nk_ops.h"

namespace nkh {

const char* OpName(NkOp op) {
    static const char* const names[] = {
#define X(name) #name,
        NKH_OP_CATALOG(X)
#undef X
    };
    return op < NkOp::Count ? names[static_cast<uint16_t>(op)] : "?";
}

namespace {

// ops/registry.cu:28 SetCudaOp: a null slot is Status::Unsupported
OpFn g_ops[static_cast<size_t>(NkOp::Count)] = {};
std::once_flag g_ops_once;

void RegisterOps() {
    auto set = [](NkOp op, OpFn fn) { g_ops[static_cast<size_t>(op)] = fn; };
    set(NkOp::ApplyDrives, &OpApplyDrives);
    set(NkOp::ArticulationDynamics, &OpArticulationDynamics);
    set(NkOp::IntegrateVelocity, &OpIntegrateVelocity);
    set(NkOp::FkWorldPoses, &OpFkWorldPoses);
    set(NkOp::IntegratePosition, &OpIntegratePosition);
    set(NkOp::BuildAabbs, &OpBuildAabbs);
    set(NkOp::LbvhBuild, &OpLbvhBuild);
    set(NkOp::LbvhQueryPairs, &OpLbvhQueryPairs);
    set(NkOp::NarrowphasePrimitives, &OpNarrowphasePrimitives);
    set(NkOp::AssembleRows, &OpAssembleRows);
    set(NkOp::SyncLinkBodyPose, &OpSyncLinkBodyPose);
    set(NkOp::NarrowphaseHeightfield, &OpNarrowphaseHeightfield);
    set(NkOp::ContactWarmStart, &OpContactWarmStart);
    set(NkOp::SnapshotStepVelocity, &OpSnapshotStepVelocity);
    set(NkOp::FkLinkVelocities, &OpFkLinkVelocities);
    set(NkOp::BlockDescentSolve, &OpBlockDescentSolve);
    set(NkOp::ReadoutDrives, &OpReadoutDrives);
    set(NkOp::ReadoutContactWrench, &OpReadoutContactWrench);
    set(NkOp::AccumulateStep, &OpAccumulateStep);
    set(NkOp::ReferenceWeights, &OpReferenceWeights);
    set(NkOp::ArticulationDamping, &OpArticulationDamping);
}

void Fail(nuka_phi_execution_error* error, Status status, uint16_t op, int native, const char* message) {
    if (error == nullptr) return;
    error->status = static_cast<uint8_t>(status);
    error->failed_op = op;
    error->native_code = native;
    std::snprintf(error->message, sizeof(error->message), "%s", message);
}

// ---- buffers (cuda_buffer.cu) ---------------------------------------------------------------------------
struct BufferType { const nuka_phi_buffer_type_i* iface; bool host; hipStream_t* stream; int device; };
struct Buffer { const nuka_phi_buffer_i* iface; void* base; size_t bytes; bool host; hipStream_t* stream; };

const char* BtName(nuka_phi_buffer_type* t) { return reinterpret_cast<BufferType*>(t)->host ? "HIP_Host" : "HIP"; }
size_t BtAlignment(nuka_phi_buffer_type*) { return 256u; }
int BtIsHost(nuka_phi_buffer_type* t) { return reinterpret_cast<BufferType*>(t)->host ? 1 : 0; }

void BufFree(nuka_phi_buffer* b) {
    auto* buffer = reinterpret_cast<Buffer*>(b);
    if (buffer == nullptr) return;
    if (buffer->base != nullptr) { if (buffer->host) (void)hipHostFree(buffer->base); else (void)hipFree(buffer->base); }
    delete buffer;
}
void* BufBase(nuka_phi_buffer* b) { return reinterpret_cast<Buffer*>(b)->base; }
bool InRange(const Buffer* b, size_t off, size_t n) { return off <= b->bytes && n <= b->bytes - off; }
uint8_t BufUpload(nuka_phi_buffer* b, const void* src, size_t off, size_t n) {
    auto* buffer = reinterpret_cast<Buffer*>(b);
    if (!InRange(buffer, off, n) || (src == nullptr && n > 0u)) return uint8_t(Status::InvalidArgument);
    if (n == 0u) return uint8_t(Status::Ok);
    const hipError_t e = hipMemcpyAsync(static_cast<char*>(buffer->base) + off, src, n, hipMemcpyHostToDevice, *buffer->stream);
    return uint8_t(e == hipSuccess && hipStreamSynchronize(*buffer->stream) == hipSuccess ? Status::Ok : Status::Failed);
}
uint8_t BufDownload(nuka_phi_buffer* b, void* dst, size_t off, size_t n) {
    auto* buffer = reinterpret_cast<Buffer*>(b);
    if (!InRange(buffer, off, n) || (dst == nullptr && n > 0u)) return uint8_t(Status::InvalidArgument);
    if (n == 0u) return uint8_t(Status::Ok);
    const hipError_t e = hipMemcpyAsync(dst, static_cast<char*>(buffer->base) + off, n, hipMemcpyDeviceToHost, *buffer->stream);
    return uint8_t(e == hipSuccess && hipStreamSynchronize(*buffer->stream) == hipSuccess ? Status::Ok : Status::Failed);
}
uint8_t BufMemset(nuka_phi_buffer* b, uint8_t v, size_t off, size_t n) {
    auto* buffer = reinterpret_cast<Buffer*>(b);
    if (!InRange(buffer, off, n)) return uint8_t(Status::InvalidArgument);
    if (n == 0u) return uint8_t(Status::Ok);
    return uint8_t(hipMemsetAsync(static_cast<char*>(buffer->base) + off, v, n, *buffer->stream) == hipSuccess ? Status::Ok : Status::Failed);
}
uint8_t BufCopyFrom(nuka_phi_buffer* dst, nuka_phi_buffer* src, size_t doff, size_t soff, size_t n) {
    auto* d = reinterpret_cast<Buffer*>(dst);
    auto* s = reinterpret_cast<Buffer*>(src);
    if (!InRange(d, doff, n) || !InRange(s, soff, n)) return uint8_t(Status::InvalidArgument);
    if (n == 0u) return uint8_t(Status::Ok);
    return uint8_t(hipMemcpyAsync(static_cast<char*>(d->base) + doff, static_cast<char*>(s->base) + soff, n, hipMemcpyDeviceToDevice,
                                  *d->stream) == hipSuccess ? Status::Ok : Status::Failed);
}
const nuka_phi_buffer_i kBufferI = {BufFree, BufBase, BufUpload, BufDownload, BufMemset, BufCopyFrom};

nuka_phi_buffer* BtAlloc(nuka_phi_buffer_type* t, size_t bytes, uint8_t* status) {
    auto* type = reinterpret_cast<BufferType*>(t);
    auto set = [&](Status s) { if (status != nullptr) *status = uint8_t(s); };
    auto* buffer = new (std::nothrow) Buffer{&kBufferI, nullptr, bytes, type->host, type->stream};
    if (buffer == nullptr) { set(Status::OutOfMemory); return nullptr; }
    if (bytes > 0u) {
        if (hipSetDevice(type->device) != hipSuccess) { (void)hipGetLastError(); delete buffer; set(Status::Failed); return nullptr; }
        const size_t padded = (bytes + 255u) & ~size_t{255u};
        const hipError_t e = type->host ? hipHostMalloc(&buffer->base, padded, hipHostMallocDefault) : hipMalloc(&buffer->base, padded);
        if (e != hipSuccess) { (void)hipGetLastError(); delete buffer; set(Status::OutOfMemory); return nullptr; }
    }
    set(Status::Ok);
    return reinterpret_cast<nuka_phi_buffer*>(buffer);
}
const nuka_phi_buffer_type_i kBufferTypeI = {BtName, BtAlloc, BtAlignment, BtIsHost};

// ---- backend (cuda_backend.cu) --------------------------------------------------------------------------
struct Plan { hipGraph_t graph; hipGraphExec_t exec; size_t nodes; int n_calls; };
struct Event { hipEvent_t event; };

struct Backend {
    const nuka_phi_backend_i* iface;
    int device;
    hipStream_t stream;
    bool owns_stream;
    BufferType device_type, host_type;
};

const char* BeName(nuka_phi_backend*) { return "HIP"; }
void BeFree(nuka_phi_backend* b) {
    auto* be = reinterpret_cast<Backend*>(b);
    if (be == nullptr) return;
    (void)hipStreamSynchronize(be->stream);
    if (be->owns_stream) (void)hipStreamDestroy(be->stream);
    delete be;
}

Status DispatchOn(Backend* be, const ModelView& m, const DataView& d, const nuka_phi_op_call& call) {
    if (call.op >= static_cast<uint16_t>(NkOp::Count)) return Status::InvalidArgument;
    const OpFn fn = g_ops[call.op];
    if (fn == nullptr) return Status::Unsupported;
    return fn(m, d, call.params, be->stream);
}

// IntegratePosition, FkWorldPoses, FkLinkVelocities and, if it follows, SyncLinkBodyPose at the head of `calls` as one
// launch: the number of calls served, 0 when the head is something else or the merged kernel does not serve these
// parameters (Unsupported: the ops then run one by one).  Any other failure of the merged launch is the plan's
// failure and comes back through `status`, never as a quiet fall back that would dispatch the ops a second time.
int MergeStepTail(Backend* be, const ModelView& m, const DataView& d, const nuka_phi_op_call* calls, int n, Status* failure) {
    if (n < 3 || calls[0].op != uint16_t(NkOp::IntegratePosition) || calls[1].op != uint16_t(NkOp::FkWorldPoses) ||
        calls[2].op != uint16_t(NkOp::FkLinkVelocities)) return 0;
    const bool bodies = n >= 4 && calls[3].op == uint16_t(NkOp::SyncLinkBodyPose);
    const Status status = OpStepTail(m, d, static_cast<const IntegratePositionParams*>(calls[0].params),
                                     static_cast<const FkWorldPosesParams*>(calls[1].params),
                                     static_cast<const FkLinkVelocitiesParams*>(calls[2].params),
                                     bodies ? static_cast<const SyncLinkBodyPoseParams*>(calls[3].params) : nullptr, be->stream);
    if (status != Status::Ok && status != Status::Unsupported) *failure = status;
    return status == Status::Ok ? (bodies ? 4 : 3) : 0;
}

// SyncLinkBodyPose, BuildAabbs, LbvhBuild, LbvhQueryPairs, NarrowphasePrimitives at the head of `calls` as one launch
int MergeCollisionHead(Backend* be, const ModelView& m, const DataView& d, const nuka_phi_op_call* calls, int n, Status* failure) {
    if (n < 5 || calls[0].op != uint16_t(NkOp::SyncLinkBodyPose) || calls[1].op != uint16_t(NkOp::BuildAabbs) ||
        calls[2].op != uint16_t(NkOp::LbvhBuild) || calls[3].op != uint16_t(NkOp::LbvhQueryPairs) ||
        calls[4].op != uint16_t(NkOp::NarrowphasePrimitives) || calls[2].params == nullptr) return 0;
    const Status status = OpCollisionHead(m, d, static_cast<const SyncLinkBodyPoseParams*>(calls[0].params),
                                          static_cast<const BuildAabbsParams*>(calls[1].params),
                                          static_cast<const LbvhQueryPairsParams*>(calls[3].params),
                                          static_cast<const NarrowphasePrimitivesParams*>(calls[4].params), be->stream);
    if (status != Status::Ok && status != Status::Unsupported) *failure = status;
    return status == Status::Ok ? 5 : 0;
}

uint8_t BeDispatch(nuka_phi_backend* b, const nuka_phi_model_view* m, const nuka_phi_data_view* d, const nuka_phi_op_call* call) {
    if (b == nullptr || m == nullptr || d == nullptr || call == nullptr) return uint8_t(Status::InvalidArgument);
    return uint8_t(DispatchOn(reinterpret_cast<Backend*>(b), *reinterpret_cast<const ModelView*>(m),
                              *reinterpret_cast<const DataView*>(d), *call));
}

uint8_t BeSynchronize(nuka_phi_backend* b, nuka_phi_execution_error* error) {
    auto* be = reinterpret_cast<Backend*>(b);
    const hipError_t e = hipStreamSynchronize(be->stream);
    if (e != hipSuccess) {
        Fail(error, Status::Failed, uint16_t(NkOp::Count), int(e), hipGetErrorString(e));
        return uint8_t(Status::Failed);
    }
    return uint8_t(Status::Ok);
}

// A plan is the op list captured once into a HIP graph on the backend's stream (cuda_backend.cu:245-361).  Ops
// launch kernels only - no memsets or allocations - so the captured graph holds kernel nodes alone.
nuka_phi_plan* BePlanCreate(nuka_phi_backend* b, const nuka_phi_model_view* m, const nuka_phi_data_view* d,
                            const nuka_phi_op_call* calls, int n_calls, nuka_phi_execution_error* error) {
    auto* be = reinterpret_cast<Backend*>(b);
    if (m == nullptr || d == nullptr || calls == nullptr || n_calls <= 0) {
        Fail(error, Status::InvalidArgument, uint16_t(NkOp::Count), 0, "plan_create: empty op list");
        return nullptr;
    }
    for (int i = 0; i < n_calls; ++i)
        if (calls[i].op >= uint16_t(NkOp::Count) || g_ops[calls[i].op] == nullptr) {
            Fail(error, Status::Unsupported, calls[i].op, 0, "plan_create: op not supported by the HIP backend");
            return nullptr;
        }
    hipError_t e = hipStreamBeginCapture(be->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) { Fail(error, Status::Failed, uint16_t(NkOp::Count), int(e), hipGetErrorString(e)); return nullptr; }
    Status status = Status::Ok;
    uint16_t failed = uint16_t(NkOp::Count);
    const ModelView& model = *reinterpret_cast<const ModelView*>(m);
    const DataView& data = *reinterpret_cast<const DataView*>(d);
    for (int i = 0; i < n_calls && status == Status::Ok; ++i) {
        // The ops after the solve, and those between the dynamics and the row assembly, each take about a launch's time:
        // where the list holds them in a row, one kernel runs them (StepTailKernel, CollisionHeadKernel); where it cannot,
        // they go one by one as dispatched.
        int merged = MergeStepTail(be, model, data, calls + i, n_calls - i, &status);
        if (merged == 0 && status == Status::Ok) merged = MergeCollisionHead(be, model, data, calls + i, n_calls - i, &status);
        if (status != Status::Ok) { failed = calls[i].op; break; }
        if (merged > 0) { i += merged - 1; continue; }
        status = DispatchOn(be, model, data, calls[i]);
        if (status != Status::Ok) failed = calls[i].op;
    }
    hipGraph_t graph = nullptr;
    e = hipStreamEndCapture(be->stream, &graph);
    if (status != Status::Ok || e != hipSuccess || graph == nullptr) {
        if (graph != nullptr) (void)hipGraphDestroy(graph);
        (void)hipGetLastError();
        Fail(error, status != Status::Ok ? status : Status::Failed, failed, int(e), "plan_create: capture failed");
        return nullptr;
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        Fail(error, Status::Failed, uint16_t(NkOp::Count), int(e), hipGetErrorString(e));
        return nullptr;
    }
    size_t nodes = 0u;
    (void)hipGraphGetNodes(graph, nullptr, &nodes);
    return reinterpret_cast<nuka_phi_plan*>(new Plan{graph, exec, nodes, n_calls});
}

uint8_t BePlanExecute(nuka_phi_backend* b, nuka_phi_plan* p, nuka_phi_execution_error* error) {
    auto* be = reinterpret_cast<Backend*>(b);
    auto* plan = reinterpret_cast<Plan*>(p);
    if (plan == nullptr) return uint8_t(Status::InvalidArgument);
    const hipError_t e = hipGraphLaunch(plan->exec, be->stream);
    if (e != hipSuccess) { Fail(error, Status::Failed, uint16_t(NkOp::Count), int(e), hipGetErrorString(e)); return uint8_t(Status::Failed); }
    return uint8_t(Status::Ok);
}

uint8_t BePlanExecuteRepeated(nuka_phi_backend* b, nuka_phi_plan* p, uint32_t count, uint32_t* submitted,
                              nuka_phi_execution_error* error) {
    if (submitted == nullptr) return uint8_t(Status::InvalidArgument);
    *submitted = 0u;
    for (; *submitted < count; ++*submitted) {
        const uint8_t status = BePlanExecute(b, p, error);
        if (status != uint8_t(Status::Ok)) return status;
    }
    return uint8_t(Status::Ok);
}

void BePlanFree(nuka_phi_backend*, nuka_phi_plan* p) {
    auto* plan = reinterpret_cast<Plan*>(p);
    if (plan == nullptr) return;
    (void)hipGraphExecDestroy(plan->exec);
    (void)hipGraphDestroy(plan->graph);
    delete plan;
}

nuka_phi_event* BeEventNew(nuka_phi_backend*) {
    auto* ev = new (std::nothrow) Event{nullptr};
    if (ev == nullptr || hipEventCreate(&ev->event) != hipSuccess) { delete ev; return nullptr; }
    return reinterpret_cast<nuka_phi_event*>(ev);
}
void BeEventRecord(nuka_phi_backend* b, nuka_phi_event* e) {
    if (e != nullptr) (void)hipEventRecord(reinterpret_cast<Event*>(e)->event, reinterpret_cast<Backend*>(b)->stream);
}
void BeEventWait(nuka_phi_backend*, nuka_phi_event* e) { if (e != nullptr) (void)hipEventSynchronize(reinterpret_cast<Event*>(e)->event); }
void BeEventFree(nuka_phi_backend*, nuka_phi_event* e) {
    auto* ev = reinterpret_cast<Event*>(e);
    if (ev == nullptr) return;
    (void)hipEventDestroy(ev->event);
    delete ev;
}
float BeEventElapsedMs(nuka_phi_backend*, nuka_phi_event* a, nuka_phi_event* b) {
    float ms = 0.0f;
    if (a == nullptr || b == nullptr ||
        hipEventElapsedTime(&ms, reinterpret_cast<Event*>(a)->event, reinterpret_cast<Event*>(b)->event) != hipSuccess) return -1.0f;
    return ms;
}
nuka_phi_resource_info BeResourceInfo(nuka_phi_backend* b) {
    nuka_phi_resource_info info{};
    size_t free_b = 0u, total_b = 0u;
    if (hipMemGetInfo(&free_b, &total_b) == hipSuccess) { info.free_bytes = free_b; info.total_bytes = total_b; }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, reinterpret_cast<Backend*>(b)->device) == hipSuccess) {
        info.compute_units = uint32_t(prop.multiProcessorCount);
        info.threads_per_unit = uint32_t(prop.maxThreadsPerMultiProcessor);
    }
    return info;
}
nuka_phi_plan_metrics BePlanMetrics(nuka_phi_backend*, nuka_phi_plan* p) {
    nuka_phi_plan_metrics metrics{};
    if (p != nullptr) { metrics.nodes = reinterpret_cast<Plan*>(p)->nodes; metrics.kernels = metrics.nodes; metrics.capture_lanes = 1u; }
    return metrics;
}

const nuka_phi_backend_i kBackendI = {BeName, BeFree, BeDispatch, BeSynchronize, BePlanCreate, BePlanExecute, BePlanFree,
                                      BeEventNew, BeEventRecord, BeEventWait, BeEventFree, BeEventElapsedMs, BeResourceInfo,
                                      BePlanMetrics, BePlanExecuteRepeated};

// ---- device and registry entry (device.cu, cuda_backend.cu:714) -----------------------------------------
struct Device { const nuka_phi_device_i* iface; int index; char name[256]; BufferType device_type, host_type; };
hipStream_t g_default_stream = nullptr;   // device-level buffer types move bytes on the default stream
struct RegistryEntry { const nuka_phi_registry_entry_i* iface; Device devices[16]; size_t count; };

const char* DevName(nuka_phi_device* d) { return reinterpret_cast<Device*>(d)->name; }
void DevMemory(nuka_phi_device* d, size_t* free_b, size_t* total_b) {
    size_t f = 0u, t = 0u;
    if (hipSetDevice(reinterpret_cast<Device*>(d)->index) != hipSuccess || hipMemGetInfo(&f, &t) != hipSuccess) { f = 0u; t = 0u; (void)hipGetLastError(); }
    if (free_b != nullptr) *free_b = f;
    if (total_b != nullptr) *total_b = t;
}
nuka_phi_backend* DevInitBackend(nuka_phi_device* d, const char*) {
    return reinterpret_cast<nuka_phi_backend*>(CreateBackend(reinterpret_cast<Device*>(d)->index, nullptr));
}
nuka_phi_buffer_type* DevBufferType(nuka_phi_device* d) { return reinterpret_cast<nuka_phi_buffer_type*>(&reinterpret_cast<Device*>(d)->device_type); }
nuka_phi_buffer_type* DevHostBufferType(nuka_phi_device* d) { return reinterpret_cast<nuka_phi_buffer_type*>(&reinterpret_cast<Device*>(d)->host_type); }
bool DevSupportsOp(nuka_phi_device*, uint16_t op) {
    std::call_once(g_ops_once, RegisterOps);
    return op < uint16_t(NkOp::Count) && g_ops[op] != nullptr ? 1 : 0;
}
const nuka_phi_device_i kDeviceI = {DevName, DevMemory, DevInitBackend, DevBufferType, DevHostBufferType, DevSupportsOp};

const char* RegName(nuka_phi_registry_entry*) { return "HIP"; }
size_t RegDeviceCount(nuka_phi_registry_entry* r) { return reinterpret_cast<RegistryEntry*>(r)->count; }
nuka_phi_device* RegGetDevice(nuka_phi_registry_entry* r, size_t i) {
    auto* entry = reinterpret_cast<RegistryEntry*>(r);
    return i < entry->count ? reinterpret_cast<nuka_phi_device*>(&entry->devices[i]) : nullptr;
}
void* RegGetProcAddress(nuka_phi_registry_entry*, const char* name) {
    if (name == nullptr) return nullptr;
    if (std::strcmp(name, "nuka_hip_op_name") == 0) return reinterpret_cast<void*>(&nuka_hip_op_name);
    if (std::strcmp(name, "nuka_hip_op_from_name") == 0) return reinterpret_cast<void*>(&nuka_hip_op_from_name);
    // the views by field name
    if (std::strcmp(name, "nuka_hip_view_field_count") == 0) return reinterpret_cast<void*>(&nuka_hip_view_field_count);
    if (std::strcmp(name, "nuka_hip_view_field") == 0) return reinterpret_cast<void*>(&nuka_hip_view_field);
    if (std::strcmp(name, "nuka_hip_model_view_bytes") == 0) return reinterpret_cast<void*>(&nuka_hip_model_view_bytes);
    if (std::strcmp(name, "nuka_hip_data_view_bytes") == 0) return reinterpret_cast<void*>(&nuka_hip_data_view_bytes);
    if (std::strcmp(name, "nuka_hip_bind_views") == 0) return reinterpret_cast<void*>(&nuka_hip_bind_views);
    if (std::strcmp(name, "nuka_hip_model_view_set_count") == 0) return reinterpret_cast<void*>(&nuka_hip_model_view_set_count);
    return nullptr;
}
const nuka_phi_registry_entry_i kRegistryI = {RegName, RegDeviceCount, RegGetDevice, RegGetProcAddress};

}  // namespace

void* CreateBackend(int device, void* borrowed_stream) {
    std::call_once(g_ops_once, RegisterOps);
    if (hipSetDevice(device) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    auto* be = new (std::nothrow) Backend{};
    if (be == nullptr) return nullptr;
    be->iface = &kBackendI;
    be->device = device;
    if (borrowed_stream != nullptr) { be->stream = static_cast<hipStream_t>(borrowed_stream); be->owns_stream = false; }
    else {
        if (hipStreamCreateWithFlags(&be->stream, hipStreamNonBlocking) != hipSuccess) { (void)hipGetLastError(); delete be; return nullptr; }
        be->owns_stream = true;
    }
    InitArticulationKernels();
    InitSolverKernels();
    InitContactKernels();
    be->device_type = BufferType{&kBufferTypeI, false, &be->stream, device};
    be->host_type = BufferType{&kBufferTypeI, true, &be->stream, device};
    return be;
}

hipStream_t BackendStream(void* backend) { return static_cast<Backend*>(backend)->stream; }
nuka_phi_buffer_type* BackendDeviceBufferType(void* backend) { return reinterpret_cast<nuka_phi_buffer_type*>(&static_cast<Backend*>(backend)->device_type); }
nuka_phi_buffer_type* BackendHostBufferType(void* backend) { return reinterpret_cast<nuka_phi_buffer_type*>(&static_cast<Backend*>(backend)->host_type); }
bool BackendSupportsOp(NkOp op) {
    std::call_once(g_ops_once, RegisterOps);
    return op < NkOp::Count && g_ops[static_cast<size_t>(op)] != nullptr;
}

}  // namespace nkh

extern "C" {

nuka_phi_registry_entry* nuka_hip_register_backend_entry(void) {
    static nkh::RegistryEntry entry{};
    static std::once_flag once;
    std::call_once(once, [] {
        entry.iface = &nkh::kRegistryI;
        int count = 0;
        if (hipGetDeviceCount(&count) != hipSuccess) { (void)hipGetLastError(); count = 0; }
        entry.count = size_t(count < 16 ? count : 16);
        for (size_t i = 0u; i < entry.count; ++i) {
            entry.devices[i].iface = &nkh::kDeviceI;
            entry.devices[i].index = int(i);
            entry.devices[i].device_type = nkh::BufferType{&nkh::kBufferTypeI, false, &nkh::g_default_stream, int(i)};
            entry.devices[i].host_type = nkh::BufferType{&nkh::kBufferTypeI, true, &nkh::g_default_stream, int(i)};
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, int(i)) == hipSuccess) std::snprintf(entry.devices[i].name, sizeof(entry.devices[i].name), "%s", prop.name);
            else std::snprintf(entry.devices[i].name, sizeof(entry.devices[i].name), "HIP device %zu", i);
        }
    });
    return reinterpret_cast<nuka_phi_registry_entry*>(&entry);
}

uint16_t nuka_hip_op_count(void) { return uint16_t(nkh::NkOp::Count); }
const char* nuka_hip_op_name(uint16_t op) { return nkh::OpName(static_cast<nkh::NkOp>(op)); }
int nuka_hip_op_from_name(const char* name) {
    if (name == nullptr) return -1;
    for (uint16_t op = 0u; op < uint16_t(nkh::NkOp::Count); ++op)
        if (std::strcmp(name, nkh::OpName(static_cast<nkh::NkOp>(op))) == 0) return int(op);
    return -1;
}

}  // extern "C"
