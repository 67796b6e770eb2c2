// Host side of the gfx950 backend: the object behind the C ABI in include/infr_hip.h.
//
// Mirrors the reference's `Backend` contract (crates/infr-core/src/backend.rs:630-1088):
// buffers are opaque device allocations, a plan is a validated copy of the graph plus its
// internal scratch, execute() resolves the caller's bindings and walks the op list in
// order, launching kernels on one HIP stream.  Nothing here computes on the CPU: when no
// gfx950 device is present, creation fails.
#include <hip/hip_runtime.h>

#include <atomic>
#include <climits>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <new>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/infr_hip.h"
#include "../../include/infr_hip_probe.h"
#include "kernels.h"

namespace {

thread_local std::string g_last_error;

infr_status fail(infr_status st, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return st;
}

// No exception crosses the C ABI: every entry point that can allocate host memory or touch a container is a
// function-try-block whose handler lands here (called inside a catch clause; rethrows to classify).
infr_status guard_fail(const char* what) noexcept {
    try {
        try {
            throw;
        } catch (const std::bad_alloc&) {
            return fail(INFR_ERR_BACKEND, "%s: out of host memory", what);
        } catch (const std::exception& e) {
            return fail(INFR_ERR_BACKEND, "%s: %s", what, e.what());
        } catch (...) {
            return fail(INFR_ERR_BACKEND, "%s: unknown exception", what);
        }
    } catch (...) {
        return INFR_ERR_BACKEND;   // not even the message could be stored
    }
}

#define HIP_TRY(expr)                                                                                        \
    do {                                                                                                     \
        hipError_t e_ = (expr);                                                                              \
        if (e_ != hipSuccess) return fail(INFR_ERR_BACKEND, "hip: %s failed: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

// Scratch of infr_hip_moe_ffn_static, the entry point that allocates nothing: routing results and the activation rows
// between the two expert stages live in this file-scope device array.  Every GPU holds its own copy at its own
// address until the process ends; host code never passes the array's name to a kernel (the name is only a host-side
// stand-in): infr_hip_create asks for the current device's address once and all uses go through that pointer.
static __device__ __align__(256) unsigned char scratch[INFR_HIP_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
// Calls into the allocating part of the runtime made by this library (device and host memory, events), process-wide:
// what the test of the entry point that allocates nothing reads before and after its calls.
std::atomic<uint64_t> g_alloc_calls{0};
void* g_scratch_ptr[kMaxDevices] = {};   // per device ordinal, filled by infr_hip_create with that device current

constexpr uint64_t kBackendMagic = 0x494e465242454e44ull;  // "INFRBEND"
constexpr uint64_t kBufferMagic = 0x494e465242554646ull;   // "INFRBUFF"
constexpr uint64_t kPlanMagic = 0x494e4652504c414eull;     // "INFRPLAN"
// Token rows from which Op::MoeFfn buckets tokens by expert and runs grouped GEMMs on the matrix
// cores (f16 operands, f32 accumulation) instead of one GEMV pass per token row.
constexpr uint32_t kBatchedMinRows = 32;
// Token rows from which a decode batch is bucketed by expert so that each selected expert's rows are
// read from HBM once (same f32-accurate inner product as the per-token kernels).
constexpr uint32_t kBucketedMinRows = 16;
// ... and only when the expected number of distinct experts of the batch is below this share of its pairs.
constexpr double kBucketedMaxDistinctRatio = 0.62;
// Token rows from which a dense Op::Linear runs as one bucket of the grouped GEMMs.
constexpr uint32_t kLinearBatchedMinRows = 128;

bool geometry(int dtype, int* elems, int* bytes) {
    switch (dtype) {
        case INFR_F32: case INFR_I32: case INFR_U32: *elems = 1; *bytes = 4; return true;
        case INFR_F16: case INFR_BF16: *elems = 1; *bytes = 2; return true;
        case INFR_Q4_0: *elems = 32; *bytes = 18; return true;
        case INFR_Q4_1: *elems = 32; *bytes = 20; return true;
        case INFR_Q5_0: *elems = 32; *bytes = 22; return true;
        case INFR_Q5_1: *elems = 32; *bytes = 24; return true;
        case INFR_Q8_0: *elems = 32; *bytes = 34; return true;
        case INFR_Q2K: *elems = 256; *bytes = 84; return true;
        case INFR_Q3K: *elems = 256; *bytes = 110; return true;
        case INFR_Q4K: *elems = 256; *bytes = 144; return true;
        case INFR_Q5K: *elems = 256; *bytes = 176; return true;
        case INFR_Q6K: *elems = 256; *bytes = 210; return true;
        case INFR_IQ4_NL: *elems = 32; *bytes = 18; return true;
        case INFR_IQ4_XS: *elems = 256; *bytes = 136; return true;
        case INFR_TQ1_0: *elems = 256; *bytes = 54; return true;
        case INFR_TQ2_0: *elems = 256; *bytes = 66; return true;
        case INFR_Q2_0: *elems = 64; *bytes = 18; return true;
        case INFR_MXFP4: *elems = 32; *bytes = 17; return true;
        case INFR_NVFP4: *elems = 64; *bytes = 36; return true;
        case INFR_IQ1_S: *elems = 256; *bytes = 50; return true;
        case INFR_IQ1_M: *elems = 256; *bytes = 56; return true;
        case INFR_IQ2_XXS: *elems = 256; *bytes = 66; return true;
        case INFR_IQ2_XS: *elems = 256; *bytes = 74; return true;
        case INFR_IQ2_S: *elems = 256; *bytes = 82; return true;
        case INFR_IQ3_XXS: *elems = 256; *bytes = 98; return true;
        case INFR_IQ3_S: *elems = 256; *bytes = 110; return true;
        default: return false;
    }
}

const char* dtype_name(int dt) {
    static const char* names[] = {"F32", "F16", "Bf16", "I32", "U32", "Q4_0", "Q4_1", "Q5_0", "Q5_1", "Q8_0",
                                  "Q2K", "Q3K", "Q4K", "Q5K", "Q6K", "Iq1S", "Iq1M", "Iq2Xxs", "Iq2Xs", "Iq2S", "Iq3Xxs",
                                  "Iq3S", "Iq4Nl", "Iq4Xs", "Tq1_0", "Tq2_0", "I2S", "Q2_0", "Mxfp4", "Nvfp4"};
    if (dt >= 0 && dt < (int)(sizeof names / sizeof names[0])) return names[dt];
    return "dtype?";
}

struct ProfSlot {
    uint64_t launches = 0;
    double total_ms = 0, min_ms = 1e30, max_ms = 0;
};

}  // namespace

struct infr_hip_buffer {
    uint64_t magic = kBufferMagic;
    infr_hip_backend* be = nullptr;
    void* dptr = nullptr;
    size_t len = 0;  // logical length the caller asked for (>= 4)
    size_t cap = 0;  // allocated bytes
    int usage = 0;
};

struct MoeScratch {
    float* logits = nullptr;  // [rows, n_expert]
    float* probs = nullptr;   // [rows, n_expert]
    int32_t* ids = nullptr;   // [rows, n_used]
    float* weights = nullptr; // [rows, n_used]
    float* h = nullptr;       // [rows, n_used, nff] (bucket order on the batched path); shared by all ops of a plan
    int rows = 0;
    // batched path (bucketing + grouped GEMMs); the large buffers are shared by all ops of a plan
    bool batched = false;    // >= kBatchedMinRows: grouped GEMMs on the matrix cores
    bool bucketed = false;   // kBucketedMinRows .. : f32-accurate GEMV per (expert, bucket), weights read once per expert
    bool units_batch = false;   // with bucketed: batches of banks in the other affine formats, unit kernels over the buckets
    bool units_mfma = false;    // with batched: the grouped GEMMs decode through the 32-element units (any affine format)
    int32_t* live_ids = nullptr;  // [pairs] ids with the pairs an expert-parallel band dropped set to -1
    int32_t* offsets = nullptr;   // [n_expert + 1]
    int32_t* pair_src = nullptr;  // [rows * n_used]
    int32_t* slot_pair = nullptr; // [rows * n_used]
    _Float16* xh = nullptr;       // [rows, ne]
    float* xs = nullptr;          // [rows]
    _Float16* hh = nullptr;       // [rows * n_used, nff]
    float* hs = nullptr;          // [rows * n_used]
    float* y = nullptr;           // [rows * n_used, ne]
    int single_launch = 0;        // one token row as one launch: 1 = stages in order (k_layer.hip), 2 = guessed selection (k_layer_stream.hip)
};

struct infr_hip_plan {
    uint64_t magic = kPlanMagic;
    infr_hip_backend* be = nullptr;
    std::vector<infr_tensor_decl> tensors;
    std::vector<infr_op> ops;
    std::vector<uint64_t> numel;       // per tensor
    std::vector<size_t> internal_off;  // per tensor: offset into arena (Internal only)
    void* arena = nullptr;             // Internal tensors + per-op scratch
    size_t arena_bytes = 0;
    std::vector<MoeScratch> moe;       // per op (valid for MoeFfn ops)
    // Op::Linear with a batch of rows on the matrix cores: the rows are one bucket of the grouped GEMM.
    struct LinearBatch {
        int mode = 0;                  // 0: GEMV kernels; 1: grouped_mfma6 (Q4_K/Q6_K/Q8_0); 2: unit-decoder GEMM
        size_t offsets_off = 0;        // arena offset of the bucket table {0, m}
    };
    std::vector<LinearBatch> lin;      // per op (valid for Linear ops)
    _Float16* lin_xh = nullptr;        // shared by all ops of a plan: f16 rows, then their scales
    char* layer_ws = nullptr;          // workspace of the in-order single-launch MoeFfn kernel, shared by all ops of the plan
    char* stream_ws = nullptr;         // the same for the kernel that guesses the selection (its records are tagged differently)
    int last_moe_op = -1;
    // Launch fusion of the dense SwiGLU FFN the reference emits beside the routed experts
    // (crates/infr-llama/src/runner.rs:8116-8174: Linear gate, Linear up, GatedAct, Linear down, Add).
    // fuse[i]: what op i does at execute time.
    enum Fuse : uint8_t { kPlain = 0, kSkip, kGateUpAct, kLinearAdd, kMoeShared };
    struct FuseOp {
        Fuse kind = kPlain;
        uint32_t a = 0, b = 0;   // kGateUpAct: index of the up Linear and of the GatedAct; kLinearAdd: index of the Add;
                                 // kMoeShared: index of the always-on expert's first Linear and of its down Linear
        uint32_t gated = 0;      // kMoeShared: 1 + index of the Op::MoeSharedExpertAdd that closes the pattern (0: a plain Op::Add)
        uint32_t norm = 0;       // MoeFfn: 1 + index of the Op::RmsNorm its logits kernel applies to the token row
        uint32_t res = 0;        // MoeFfn: 1 + index of the following Op::Add folded into the combine
    };
    std::vector<FuseOp> fuse;
    std::vector<FuseOp> fuse_head;     // kMoeShared: the records of the ops it absorbed, as they were before
    int32_t* zero_ids = nullptr;       // [max rows of a fused gate/up] expert id 0 for every row
    std::vector<size_t> copy_tmp;      // per op: arena offset of the staging window of an aliasing Copy, else 0
    ~infr_hip_plan() {
        magic = 0;
        if (arena) (void)hipFree(arena);   // the caller has made the plan's device current and drained its stream
    }
};

struct infr_hip_backend {
    uint64_t magic = kBackendMagic;
    int device = 0;
    hipStream_t stream = nullptr;
    hipDeviceProp_t prop{};
    infr_hip_config cfg{};
    std::mutex mu;  // serialises stream submission and profiling state
    std::atomic<int> prof_on{0};
    std::atomic<bool> probe_grouped_loads_only{false};   // measurement: see infr_hip_probe_grouped_loads_only
    std::map<std::string, ProfSlot> prof;
    struct Pending { std::string name; hipEvent_t a, b; };
    std::vector<Pending> pending;
    std::vector<hipEvent_t> event_pool;
    void* static_scratch = nullptr;   // this device's copy of the file-scope scratch array (infr_hip_moe_ffn_static)
    // Single-launch Op::MoeFfn (k_layer.hip): a word in pinned host memory the kernel raises when one of its bounded
    // waits runs out; read after every stream synchronisation.  Once raised the backend keeps to the three-launch path.
    uint32_t* fault_host = nullptr;
    uint32_t* fault_dev = nullptr;
    std::atomic<int> single_launch_off{0};   // MoeFfn ops that still take three launches after a single-launch kernel gave up
    std::atomic<int> single_launch_faults{0};   // launches that gave up so far
    std::atomic<int> inorder_off{0};         // the in-order single-launch kernel stays off after it gave up (its sequence word did not advance)
    // The object outlives infr_hip_destroy while buffers or plans still point at it (the reference's buffers keep their
    // device alive the same way): destroy drains and closes the stream and drops the creator's reference, the last
    // buffer / plan freed afterwards deletes the object.
    std::atomic<int> refs{1};
    std::atomic<int> closed{0};
};

namespace {

bool ok_backend(const infr_hip_backend* be) { return be && be->magic == kBackendMagic && !be->closed.load(); }
void release_backend(infr_hip_backend* be) {
    if (be && be->magic == kBackendMagic && be->refs.fetch_sub(1) == 1) {
        be->magic = 0;
        delete be;
    }
}
bool ok_buffer(const infr_hip_buffer* b) { return b && b->magic == kBufferMagic; }
bool ok_plan(const infr_hip_plan* p) { return p && p->magic == kPlanMagic; }

// After a stream synchronisation: did a single-launch MoeFfn kernel give up a bounded wait?  The results of that
// execute are not valid; the error is reported once and the next kSingleLaunchPause MoeFfn ops take three launches
// (whatever shared the device has that long to finish) before the single-launch kernel is tried again.
constexpr int kSingleLaunchPause = 256;
infr_status check_fault(infr_hip_backend* be) {
    if (!be->fault_host || !*(volatile uint32_t*)be->fault_host) return INFR_OK;
    *(volatile uint32_t*)be->fault_host = 0;
    // a device on which the hand-overs keep failing (partitioned, or workgroups dealt to the XCDs in another way) must
    // not pay a timed-out launch and an error every few hundred ops: the third time is for good
    const int faults = be->single_launch_faults.fetch_add(1) + 1;
    be->single_launch_off.store(faults >= 3 ? INT_MAX : kSingleLaunchPause);
    be->inorder_off.store(1);
    return fail(INFR_ERR_BACKEND,
                "MoeFfn: the single-launch kernel timed out waiting for a peer workgroup (is the device shared or partitioned?); "
                "the results since the last synchronisation are invalid: run those executes again (the next %d MoeFfn ops take the three-launch path)",
                kSingleLaunchPause);
}

// Times one kernel launch when profiling is on: the events ride on the kernel's own dispatch
// (begin / end of execution), see INFR_LAUNCH.
struct Timed {
    infr_hip_backend* be;
    const char* name;
    infr::LaunchTiming lt{nullptr, nullptr};
    Timed(infr_hip_backend* be_, const char* n) : be(be_), name(n) {   // be_ == nullptr: never timed (no event is created)
        if (!be || !be->prof_on.load(std::memory_order_relaxed)) return;
        auto get = [&]() {
            hipEvent_t e = nullptr;
            if (!be->event_pool.empty()) { e = be->event_pool.back(); be->event_pool.pop_back(); }
            else { g_alloc_calls++; if (hipEventCreate(&e) != hipSuccess) e = nullptr; }
            return e;
        };
        lt.start = get();
        lt.stop = get();
        if (lt.start && lt.stop) infr::tl_launch_timing = &lt;
    }
    ~Timed() {
        if (infr::tl_launch_timing != &lt) return;
        infr::tl_launch_timing = nullptr;
        be->pending.push_back({name, lt.start, lt.stop});
    }
};

void drain_prof(infr_hip_backend* be) {
    for (auto& p : be->pending) {
        float ms = 0;
        if (hipEventSynchronize(p.b) == hipSuccess && hipEventElapsedTime(&ms, p.a, p.b) == hipSuccess) {
            ProfSlot& s = be->prof[p.name];
            s.launches++;
            s.total_ms += ms;
            if (ms < s.min_ms) s.min_ms = ms;
            if (ms > s.max_ms) s.max_ms = ms;
        }
        be->event_pool.push_back(p.a);
        be->event_pool.push_back(p.b);
    }
    be->pending.clear();
}

// Single-launch kernel with a guessed selection: is every router logit computed once for the whole grid (and handed
// over across the XCDs), or by every group of 32 workgroups for itself (eight reads of the router)?
int moe_logits_once(const infr_hip_backend* be, const infr_op_moe_ffn& m) {
    if (be->cfg.single_launch_logits == 1) return 1;
    if (be->cfg.single_launch_logits == 2) return 0;
    (void)m;
    return 1;   // measured equal or faster on every shape the kernel takes, and the router is read once
}

// The per-token path of Op::MoeFfn (1 to 31 token rows; the bucketed path takes batches of 16 or more whose pairs fall on few distinct experts) once logits are in rp.logits and gp / rp are filled in:
// routing (inside the gate/up kernel where that is cheaper than a launch), gate/up with the gated activation,
// down with the rank-ordered combine.  timed == false: no profiling events (nothing is created or allocated).
void moe_per_token(infr_hip_backend* be, hipStream_t s, infr::MoeGemvParams& gp, const infr::RouteParams& rp, int rows,
                   uint32_t n_expert_total, bool timed) {
    infr_hip_backend* tb = timed ? be : nullptr;
    // Every block of the gate/up kernel routes its own token row: two of its waves do, while the others turn the row
    // into fixed-point cells, which measured 1 to 3 % faster than a launch of the routing kernel at every batch of the
    // per-token path.  The unit-format kernel routes on its only four waves and keeps the older rule.
    const bool fast_gu = infr::moe_gate_up_routes_inline(gp);
    const bool units = !fast_gu && !gp.sh_gate && infr::moe_gate_up_units_supported(gp);
    gp.route_inline = (fast_gu || (units && infr::moe_gate_up_units_routes_inline(gp) &&
                                   (rows == 1 || (uint64_t)rows * n_expert_total <= 512))) ? 1 : 0;
    if (!gp.route_inline) {
        Timed t(tb, "route_topk");
        infr::launch_route(s, rp);
    }
    {
        Timed t(tb, gp.sh_gate ? "moe_route_gate_up_shared" : units ? (gp.route_inline ? "moe_route_gate_up_units" : "moe_gate_up_units")
                    : gp.route_inline ? "moe_route_gate_up" : "moe_gate_up");
        infr::launch_moe_gate_up(s, gp);
    }
    gp.x = nullptr;
    if (!gp.sh_down && !infr::moe_down_is_fast(gp) && infr::moe_down_units_supported(gp)) {
        // a down bank without an integer-dot kernel: the unit kernel over all slots of a row with the
        // rank-ordered weighted sum at its end, or per-pair rows and the sum as a launch of its own
        // (one or two token rows: from four rows on the per-pair grid spreads better; C2 shape, MXFP4:
        // 1 row 11.2 -> 6.9 us, 4 rows 22.6 -> 23.6, 8 rows 36.6 -> 45.4)
        if (rows <= 2 && infr::moe_down_combine_units_supported(gp)) {
            Timed t(tb, "moe_down_combine_units");
            infr::launch_moe_down_combine_units(s, gp);
            return;
        }
        {
            Timed t(tb, "moe_down_units");
            infr::launch_moe_down_units(s, gp);
        }
        Timed t(tb, "moe_unbucket_combine");
        infr::launch_unbucket_combine(s, gp.y, nullptr, gp.weights, rows, gp.ne, gp.n_used, gp.weight_before, gp.dst, 1,
                                      nullptr, gp.addend, gp.skip_zero_w);
        return;
    }
    Timed t(tb, gp.sh_down ? "moe_down_combine_shared" : "moe_down_combine");
    infr::launch_moe_down_combine(s, gp);
}

// Every tensor id an op names (INFR_NO_TENSOR for absent options), for the walk that checks the bindings of a whole
// plan before its first launch.
int op_tensors(const infr_op& op, uint32_t (&ids)[12], const char** role) {
    int n = 0;
    switch (op.kind) {
        case INFR_OP_MOE_FFN: {
            const infr_op_moe_ffn& m = op.u.moe_ffn;
            *role = "MoeFfn";
            ids[n++] = m.x; ids[n++] = m.router_x; ids[n++] = m.router; ids[n++] = m.gate_exps;
            if (!m.fused_gate_up) ids[n++] = m.up_exps;
            ids[n++] = m.down_exps; ids[n++] = m.dst; ids[n++] = m.down_scale; ids[n++] = m.exp_probs_b; ids[n++] = m.expert_ids;
            break;
        }
        case INFR_OP_LINEAR: *role = "Linear"; ids[n++] = op.u.linear.x; ids[n++] = op.u.linear.weight; ids[n++] = op.u.linear.dst; break;
        case INFR_OP_GATED_ACT: *role = "GatedAct"; ids[n++] = op.u.gated_act.gate; ids[n++] = op.u.gated_act.up; ids[n++] = op.u.gated_act.dst; break;
        case INFR_OP_ADD: *role = "Add"; ids[n++] = op.u.add.a; ids[n++] = op.u.add.b; ids[n++] = op.u.add.dst; break;
        case INFR_OP_MOE_SHARED_EXPERT_ADD: {
            const infr_op_moe_shared_expert_add& a = op.u.moe_shared_expert_add;
            *role = "MoeSharedExpertAdd";
            ids[n++] = a.moe; ids[n++] = a.shexp; ids[n++] = a.gate; ids[n++] = a.dst;
            break;
        }
        case INFR_OP_COPY:
        case INFR_OP_COPY_STRIDED: *role = "Copy"; ids[n++] = op.u.copy.src; ids[n++] = op.u.copy.dst; break;
        case INFR_OP_RMS_NORM:
        case INFR_OP_RMS_NORM_ADD: *role = "RmsNorm"; ids[n++] = op.u.rms_norm.x; ids[n++] = op.u.rms_norm.weight; ids[n++] = op.u.rms_norm.dst; break;
        default: *role = "op"; break;
    }
    return n;
}

size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

// ============================================================================ lifecycle
extern "C" const char* infr_hip_last_error(void) { return g_last_error.c_str(); }

extern "C" infr_status infr_hip_create(int device_ordinal, const infr_hip_config* cfg, infr_hip_backend** out) try {
    if (!out) return fail(INFR_ERR_INVALID, "infr_hip_create: out is null");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0)
        return fail(INFR_ERR_BACKEND, "hip backend: no HIP device visible (%s); this backend has no CPU fallback",
                    e == hipSuccess ? "device count 0" : hipGetErrorString(e));
    if (device_ordinal < 0 || device_ordinal >= n)
        return fail(INFR_ERR_INVALID, "hip backend: device ordinal %d out of range (0..%d)", device_ordinal, n - 1);
    HIP_TRY(hipSetDevice(device_ordinal));
    auto* be = new infr_hip_backend();
    be->device = device_ordinal;
    if (cfg) be->cfg = *cfg;
    e = hipGetDeviceProperties(&be->prop, device_ordinal);
    if (e != hipSuccess) {
        delete be;
        return fail(INFR_ERR_BACKEND, "hip: hipGetDeviceProperties failed: %s", hipGetErrorString(e));
    }
    if (strncmp(be->prop.gcnArchName, "gfx950", 6) != 0) {
        std::string arch = be->prop.gcnArchName;
        delete be;
        return fail(INFR_ERR_UNSUPPORTED, "hip backend: kernels are built for gfx950 only, device %d is %s",
                    device_ordinal, arch.c_str());
    }
    e = hipStreamCreateWithFlags(&be->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete be;
        return fail(INFR_ERR_BACKEND, "hip: hipStreamCreate failed: %s", hipGetErrorString(e));
    }
    if (device_ordinal < kMaxDevices) {
        // this device's address of the static scratch array, once per device, with the device current
        std::lock_guard<std::mutex> lk(g_scratch_mu);
        if (!g_scratch_ptr[device_ordinal]) {
            void* ptr = nullptr;
            e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !ptr) {
                (void)hipStreamDestroy(be->stream);
                delete be;
                return fail(INFR_ERR_BACKEND, "hip: hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
            }
            g_scratch_ptr[device_ordinal] = ptr;
        }
        be->static_scratch = g_scratch_ptr[device_ordinal];
    }
    {
        void* host = nullptr;
        void* dev = nullptr;
        g_alloc_calls++;
        e = hipHostMalloc(&host, 64, hipHostMallocMapped);
        if (e == hipSuccess) {
            memset(host, 0, 64);
            e = hipHostGetDevicePointer(&dev, host, 0);
        }
        if (e != hipSuccess) {
            if (host) (void)hipHostFree(host);
            (void)hipStreamDestroy(be->stream);
            delete be;
            return fail(INFR_ERR_BACKEND, "hip: pinned fault word: %s", hipGetErrorString(e));
        }
        be->fault_host = (uint32_t*)host;
        be->fault_dev = (uint32_t*)dev;
    }
    *out = be;
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_create"); }

extern "C" void infr_hip_destroy(infr_hip_backend* be) try {
    if (!ok_backend(be)) return;
    {
        std::lock_guard<std::mutex> lk(be->mu);
        (void)hipSetDevice(be->device);
        (void)hipStreamSynchronize(be->stream);
        for (auto& p : be->pending) { (void)hipEventDestroy(p.a); (void)hipEventDestroy(p.b); }
        for (auto e : be->event_pool) (void)hipEventDestroy(e);
        be->pending.clear();
        be->event_pool.clear();
        (void)hipStreamDestroy(be->stream);
        be->stream = nullptr;
        if (be->fault_host) (void)hipHostFree(be->fault_host);
        be->fault_host = be->fault_dev = nullptr;
        be->closed.store(1);   // every later call on this handle is refused; buffers and plans can still be freed
    }
    release_backend(be);
} catch (...) {
}

extern "C" const char* infr_hip_name(const infr_hip_backend* be) { return ok_backend(be) ? "hip-gfx950" : ""; }

extern "C" infr_status infr_hip_capabilities_get(const infr_hip_backend* be, infr_hip_capabilities* out) try {
    if (!ok_backend(be) || !out) return fail(INFR_ERR_INVALID, "capabilities: bad handle");
    memset(out, 0, sizeof *out);
    // some driver stacks report an empty marketing name; the architecture string is always there
    snprintf(out->name, sizeof out->name, "hip-gfx950 (%s)", be->prop.name[0] ? be->prop.name : be->prop.gcnArchName);
    out->f16 = 1; out->bf16 = 1; out->i8 = 1; out->i8_dot = 1;
    out->subgroup_min = 64; out->subgroup_max = 64;
    out->integrated = 0;
    out->compute_units = (uint32_t)be->prop.multiProcessorCount;
    out->buffer_device_address = 1;
    out->max_shared_memory_bytes = (uint32_t)be->prop.sharedMemPerBlock;
    out->unified_memory = 0;
    out->decode_replay = 0;
    out->combined_gu = 0;
    out->graph_input_inplace = 1;
    out->device_memory_bytes = (uint64_t)be->prop.totalGlobalMem;
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_capabilities_get"); }

// ============================================================================ memory
static infr_status alloc_impl(infr_hip_backend* be, size_t bytes, int32_t usage, bool zero, infr_hip_buffer** out) {
    if (!ok_backend(be) || !out) return fail(INFR_ERR_INVALID, "alloc: bad handle");
    *out = nullptr;
    if (usage < INFR_USAGE_WEIGHTS || usage > INFR_USAGE_HOST_WEIGHTS)
        return fail(INFR_ERR_INVALID, "alloc: unknown buffer usage %d", usage);
    size_t len = bytes < 4 ? 4 : bytes;  // reference: vec![0u8; bytes.max(4)]
    size_t cap = round_up(len + 16, 256);  // 16 bytes of slack: kernels that fetch weight rows in 16-byte chunks may run past the last row's end
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    void* p = nullptr;
    g_alloc_calls++;
    hipError_t e = hipMalloc(&p, cap);
    if (e != hipSuccess)
        return fail(INFR_ERR_BACKEND, "alloc: hipMalloc(%zu) failed: %s", cap, hipGetErrorString(e));
    if (zero) infr::launch_fill_zero(be->stream, p, cap);
    infr_hip_buffer* b = new (std::nothrow) infr_hip_buffer();
    if (!b) {
        (void)hipFree(p);
        return fail(INFR_ERR_BACKEND, "alloc: out of host memory");
    }
    b->be = be; b->dptr = p; b->len = len; b->cap = cap; b->usage = usage;
    be->refs.fetch_add(1);   // the buffer keeps its backend alive
    *out = b;
    return INFR_OK;
}

extern "C" infr_status infr_hip_alloc(infr_hip_backend* be, size_t bytes, int32_t usage, infr_hip_buffer** out) try {
    return alloc_impl(be, bytes, usage, true, out);
} catch (...) { return guard_fail("infr_hip_alloc"); }
extern "C" infr_status infr_hip_alloc_uninit(infr_hip_backend* be, size_t bytes, int32_t usage, infr_hip_buffer** out) try {
    return alloc_impl(be, bytes, usage, false, out);
} catch (...) { return guard_fail("infr_hip_alloc_uninit"); }
extern "C" size_t infr_hip_buffer_len(const infr_hip_buffer* buf) { return ok_buffer(buf) ? buf->len : 0; }
extern "C" uint64_t infr_hip_buffer_device_addr(const infr_hip_buffer* buf) {
    return ok_buffer(buf) ? (uint64_t)(uintptr_t)buf->dptr : 0;
}
extern "C" void infr_hip_buffer_free(infr_hip_buffer* buf) try {
    if (!ok_buffer(buf)) return;
    infr_hip_backend* be = buf->be;   // alive: the buffer holds a reference
    {
        std::lock_guard<std::mutex> lk(be->mu);
        (void)hipSetDevice(be->device);
        if (!be->closed.load()) (void)hipStreamSynchronize(be->stream);  // work that still reads it must drain first
        (void)hipFree(buf->dptr);
    }
    buf->magic = 0;
    delete buf;
    release_backend(be);
} catch (...) {
}

static infr_status check_owned(infr_hip_backend* be, const infr_hip_buffer* b, const char* what) {
    if (!ok_backend(be)) return fail(INFR_ERR_INVALID, "%s: backend handle is not a hip backend", what);
    if (!ok_buffer(b)) return fail(INFR_ERR_INVALID, "%s: buffer is not a hip buffer", what);
    if (b->be != be) return fail(INFR_ERR_INVALID, "%s: buffer belongs to another backend instance", what);
    return INFR_OK;
}

extern "C" infr_status infr_hip_upload_range(infr_hip_backend* be, infr_hip_buffer* dst, size_t offset,
                                             const void* src, size_t n) try {
    if (infr_status st = check_owned(be, dst, "upload")) return st;
    if (n && !src) return fail(INFR_ERR_INVALID, "upload: src is null");
    if (offset > dst->len || n > dst->len - offset)
        return fail(INFR_ERR_BACKEND, "upload: byte range %zu..%zu exceeds buffer size %zu", offset, offset + n, dst->len);
    if (n == 0) return INFR_OK;
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    HIP_TRY(hipMemcpyAsync((char*)dst->dptr + offset, src, n, hipMemcpyHostToDevice, be->stream));
    HIP_TRY(hipStreamSynchronize(be->stream));  // src may be freed by the caller on return
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_upload_range"); }
extern "C" infr_status infr_hip_upload(infr_hip_backend* be, infr_hip_buffer* dst, const void* src, size_t n) try {
    return infr_hip_upload_range(be, dst, 0, src, n);
} catch (...) { return guard_fail("infr_hip_upload"); }
extern "C" infr_status infr_hip_download_range(infr_hip_backend* be, const infr_hip_buffer* src, size_t offset,
                                               void* dst, size_t n) try {
    if (infr_status st = check_owned(be, src, "download")) return st;
    if (n && !dst) return fail(INFR_ERR_INVALID, "download: dst is null");
    if (offset > src->len || n > src->len - offset)
        return fail(INFR_ERR_BACKEND, "download_range: byte range %zu..%zu exceeds committed buffer size %zu", offset,
                    offset + n, src->len);
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    if (n) HIP_TRY(hipMemcpyAsync(dst, (const char*)src->dptr + offset, n, hipMemcpyDeviceToHost, be->stream));
    HIP_TRY(hipStreamSynchronize(be->stream));
    return check_fault(be);
} catch (...) { return guard_fail("infr_hip_download_range"); }
extern "C" infr_status infr_hip_download(infr_hip_backend* be, const infr_hip_buffer* src, void* dst, size_t n) try {
    return infr_hip_download_range(be, src, 0, dst, n);
} catch (...) { return guard_fail("infr_hip_download"); }
extern "C" infr_status infr_hip_copy_buffer(infr_hip_backend* be, const infr_hip_buffer* src, infr_hip_buffer* dst,
                                            size_t n) try {
    if (infr_status st = check_owned(be, src, "copy_buffer")) return st;
    if (infr_status st = check_owned(be, dst, "copy_buffer")) return st;
    if (n > src->len || n > dst->len)
        return fail(INFR_ERR_BACKEND, "copy_buffer: %zu bytes exceed src (%zu) or dst (%zu)", n, src->len, dst->len);
    if (n == 0) return INFR_OK;
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    HIP_TRY(hipMemcpyAsync(dst->dptr, src->dptr, n, hipMemcpyDeviceToDevice, be->stream));
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_copy_buffer"); }

extern "C" infr_status infr_hip_sync(infr_hip_backend* be) try {
    if (!ok_backend(be)) return fail(INFR_ERR_INVALID, "sync: bad handle");
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    HIP_TRY(hipStreamSynchronize(be->stream));
    HIP_TRY(hipGetLastError());
    return check_fault(be);
} catch (...) { return guard_fail("infr_hip_sync"); }

// ---- shared with sibling translation units of this library (not part of the public ABI)
extern "C" infr_status infr_hip_internal_fail(infr_status st, const char* msg) try { return fail(st, "%s", msg); } catch (...) { return guard_fail("infr_hip_internal_fail"); }

// Validates [byte_offset, byte_offset+bytes) of buf, makes the device current and returns the
// device pointer and the backend's stream WITH the submission lock held; the caller enqueues
// its work and then calls infr_hip_internal_unlock.  On error the lock is not held.
extern "C" infr_status infr_hip_internal_buffer_span(infr_hip_backend* be, infr_hip_buffer* buf, size_t byte_offset,
                                                     size_t bytes, void** dptr, hipStream_t* stream) try {
    if (infr_status st = check_owned(be, buf, "buffer_span")) return st;
    if (byte_offset > buf->len || bytes > buf->len - byte_offset)
        return fail(INFR_ERR_BACKEND, "byte range %zu..%zu exceeds buffer size %zu", byte_offset, byte_offset + bytes,
                    buf->len);
    be->mu.lock();
    hipError_t e = hipSetDevice(be->device);
    if (e != hipSuccess) {
        be->mu.unlock();
        return fail(INFR_ERR_BACKEND, "hip: hipSetDevice failed: %s", hipGetErrorString(e));
    }
    *dptr = (char*)buf->dptr + byte_offset;
    *stream = be->stream;
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_internal_buffer_span"); }
extern "C" void infr_hip_internal_unlock(infr_hip_backend* be) { be->mu.unlock(); }

// ============================================================================ compile
namespace {

struct Check {
    const infr_hip_plan& p;
    std::string err;
    infr_status st = INFR_OK;
    bool tensor(uint32_t id, const char* role, bool optional = false) {
        if (id == INFR_NO_TENSOR && optional) return true;
        if (id >= p.tensors.size()) {
            set(INFR_ERR_INVALID, std::string(role) + ": tensor id out of range");
            return false;
        }
        return true;
    }
    void set(infr_status s, const std::string& m) {
        if (st == INFR_OK) { st = s; err = m; }
    }
    int dt(uint32_t id) const { return p.tensors[id].dtype; }
    uint64_t n(uint32_t id) const { return p.numel[id]; }
    int kind(uint32_t id) const { return p.tensors[id].kind; }
    void want_f32(uint32_t id, const char* role) {
        if (dt(id) != INFR_F32) set(INFR_ERR_UNSUPPORTED, std::string(role) + " must be F32, got " + dtype_name(dt(id)));
    }
    void want_numel(uint32_t id, uint64_t expect, const char* role) {
        if (n(id) != expect)
            set(INFR_ERR_INVALID, std::string(role) + ": declared " + std::to_string(n(id)) + " elements, op needs " +
                                      std::to_string(expect));
    }
    void want_weight_dtype(uint32_t id, uint64_t in_f, const char* role) {
        int be = 0, bb = 0;
        if (!geometry(dt(id), &be, &bb) || dt(id) == INFR_I32 || dt(id) == INFR_U32) {
            set(INFR_ERR_UNSUPPORTED, std::string(role) + ": weight dtype " + dtype_name(dt(id)) +
                                          " has no decode on this backend (decoded: F32/F16/Bf16, Q4_0 Q4_1 Q5_0 Q5_1 Q8_0, Q2K..Q6K, "
                                          "IQ4_NL IQ4_XS MXFP4 NVFP4 TQ1_0 TQ2_0 Q2_0 and the grid i-quants)");
            return;
        }
        if (in_f % (uint64_t)be != 0)
            set(INFR_ERR_INVALID, std::string(role) + ": row length " + std::to_string(in_f) +
                                      " is not a whole number of " + dtype_name(dt(id)) + " blocks");
    }
    void want_writable(uint32_t id, const char* role) {
        if (kind(id) == INFR_KIND_WEIGHT) set(INFR_ERR_INVALID, std::string(role) + ": destination is a Weight");
    }
};

size_t tensor_bytes(const infr_tensor_decl& t, uint64_t numel) {
    int be = 1, bb = 4;
    if (!geometry(t.dtype, &be, &bb)) return 0;
    return (size_t)((numel + (uint64_t)be - 1) / (uint64_t)be) * (size_t)bb;
}

}  // namespace

extern "C" infr_status infr_hip_compile(infr_hip_backend* be, const infr_graph* g, infr_hip_plan** out) try {
    if (!ok_backend(be) || !g || !out) return fail(INFR_ERR_INVALID, "compile: bad handle");
    *out = nullptr;
    if ((g->n_tensors && !g->tensors) || (g->n_ops && !g->ops)) return fail(INFR_ERR_INVALID, "compile: null arrays");
    std::unique_ptr<infr_hip_plan> holder(new infr_hip_plan());   // freed on every early return and on an exception
    infr_hip_plan* plan = holder.get();
    plan->be = be;
    plan->tensors.assign(g->tensors, g->tensors + g->n_tensors);
    plan->ops.assign(g->ops, g->ops + g->n_ops);
    plan->numel.resize(g->n_tensors);
    plan->internal_off.assign(g->n_tensors, (size_t)-1);
    plan->moe.resize(g->n_ops);
    plan->lin.resize(g->n_ops);
    auto bail = [&](infr_status st, const std::string& m) {
        holder.reset();
        return fail(st, "%s", m.c_str());
    };
    size_t arena = 0;
    for (uint32_t i = 0; i < g->n_tensors; i++) {
        const infr_tensor_decl& t = plan->tensors[i];
        if (t.rank > 4) return bail(INFR_ERR_INVALID, "compile: tensor rank > 4");
        if (t.kind < INFR_KIND_INPUT || t.kind > INFR_KIND_OUTPUT) return bail(INFR_ERR_INVALID, "compile: bad tensor kind");
        uint64_t n = 1;
        for (uint32_t d = 0; d < t.rank; d++) n *= t.shape[d];
        plan->numel[i] = n;
        if (t.kind == INFR_KIND_INTERNAL) {
            if (t.dtype != INFR_F32) return bail(INFR_ERR_UNSUPPORTED, "compile: Internal tensors must be F32");
            plan->internal_off[i] = arena;
            arena += round_up((size_t)n * 4 + 4, 256);
        }
    }
    Check c{*plan};
    std::vector<size_t> moe_off(g->n_ops, 0);
    plan->copy_tmp.assign(g->n_ops, 0);
    size_t shared_need = 0;
    for (uint32_t oi = 0; oi < g->n_ops && c.st == INFR_OK; oi++) {
        const infr_op& op = plan->ops[oi];
        switch (op.kind) {
            case INFR_OP_MOE_FFN: {
                const infr_op_moe_ffn& m = op.u.moe_ffn;
                bool ok = c.tensor(m.x, "MoeFfn.x") && c.tensor(m.router_x, "MoeFfn.router_x") &&
                          c.tensor(m.router, "MoeFfn.router") && c.tensor(m.gate_exps, "MoeFfn.gate_exps") &&
                          c.tensor(m.down_exps, "MoeFfn.down_exps") && c.tensor(m.dst, "MoeFfn.dst") &&
                          c.tensor(m.down_scale, "MoeFfn.down_scale", true) &&
                          c.tensor(m.exp_probs_b, "MoeFfn.exp_probs_b", true) &&
                          c.tensor(m.expert_ids, "MoeFfn.expert_ids", true) &&
                          (m.fused_gate_up || c.tensor(m.up_exps, "MoeFfn.up_exps"));
                if (!ok) break;
                if (!m.ne || !m.n_expert || !m.n_used || !m.n_ff_exp || m.n_used > m.n_expert) {
                    c.set(INFR_ERR_INVALID, "MoeFfn: ne/n_expert/n_used/n_ff_exp must be positive and n_used <= n_expert");
                    break;
                }
                if (m.n_expert > 2048 || m.n_used > 64) { c.set(INFR_ERR_UNSUPPORTED, "MoeFfn: n_expert > 2048 or n_used > 64"); break; }
                // expert-parallel band (graph.rs:1307-1319): global routing, the expert tensors hold only the
                // shard [ep_base, ep_base + ep_n_local)
                if (m.has_ep_band && (m.ep_n_local == 0 || (uint64_t)m.ep_base + m.ep_n_local > m.n_expert)) {
                    c.set(INFR_ERR_INVALID, "MoeFfn: ep_band is not a non-empty range inside [0, n_expert)");
                    break;
                }
                const uint64_t n_local = m.has_ep_band ? m.ep_n_local : m.n_expert;
                // Same refusals as the reference (crates/infr-cpu/src/lib.rs:3613-3629).
                if (m.has_swiglu_clamp && (m.act == INFR_ACT_SIGMOID || m.weight_before)) {
                    c.set(INFR_ERR_INVALID, "MoeFfn: swiglu_clamp is defined for the gated SiLU/GELU forms with "
                                            "output-side weighting only");
                    break;
                }
                if (m.expert_ids != INFR_NO_TENSOR && (m.exp_probs_b != INFR_NO_TENSOR || m.n_expert_groups > 1)) {
                    c.set(INFR_ERR_INVALID, "MoeFfn: expert_ids (hash routing) supplies the selection, so exp_probs_b "
                                            "and group routing must be absent");
                    break;
                }
                if (m.act < INFR_ACT_SILU || m.act > INFR_ACT_SIGMOID || m.gating < INFR_GATING_SOFTMAX ||
                    m.gating > INFR_GATING_SQRT_SOFTPLUS) {
                    c.set(INFR_ERR_INVALID, "MoeFfn: unknown activation or gating");
                    break;
                }
                if (m.n_expert_groups > 1 && m.n_expert % m.n_expert_groups != 0) {
                    c.set(INFR_ERR_INVALID, "MoeFfn: n_expert is not a multiple of n_expert_groups");
                    break;
                }
                c.want_f32(m.x, "MoeFfn.x");
                c.want_f32(m.router_x, "MoeFfn.router_x");
                c.want_f32(m.dst, "MoeFfn.dst");
                c.want_writable(m.dst, "MoeFfn.dst");
                if (c.n(m.x) % m.ne != 0) { c.set(INFR_ERR_INVALID, "MoeFfn.x: element count is not a multiple of ne"); break; }
                uint64_t rows = c.n(m.x) / m.ne;  // reference: rows = xs.len() / ne (lib.rs:3644)
                c.want_numel(m.router_x, rows * m.ne, "MoeFfn.router_x");
                c.want_numel(m.dst, rows * m.ne, "MoeFfn.dst");
                c.want_numel(m.router, (uint64_t)m.n_expert * m.ne, "MoeFfn.router");
                uint64_t gu_rows = m.fused_gate_up ? 2ull * m.n_ff_exp : m.n_ff_exp;
                c.want_numel(m.gate_exps, n_local * gu_rows * m.ne, "MoeFfn.gate_exps");
                if (!m.fused_gate_up) c.want_numel(m.up_exps, n_local * m.n_ff_exp * m.ne, "MoeFfn.up_exps");
                c.want_numel(m.down_exps, n_local * m.ne * m.n_ff_exp, "MoeFfn.down_exps");
                c.want_weight_dtype(m.router, m.ne, "MoeFfn.router");
                c.want_weight_dtype(m.gate_exps, m.ne, "MoeFfn.gate_exps");
                if (!m.fused_gate_up) c.want_weight_dtype(m.up_exps, m.ne, "MoeFfn.up_exps");
                c.want_weight_dtype(m.down_exps, m.n_ff_exp, "MoeFfn.down_exps");
                if (m.down_scale != INFR_NO_TENSOR) { c.want_f32(m.down_scale, "MoeFfn.down_scale"); c.want_numel(m.down_scale, n_local, "MoeFfn.down_scale"); }
                if (m.exp_probs_b != INFR_NO_TENSOR) { c.want_f32(m.exp_probs_b, "MoeFfn.exp_probs_b"); c.want_numel(m.exp_probs_b, m.n_expert, "MoeFfn.exp_probs_b"); }
                if (m.expert_ids != INFR_NO_TENSOR) {
                    if (c.dt(m.expert_ids) != INFR_I32) c.set(INFR_ERR_UNSUPPORTED, "MoeFfn.expert_ids must be I32");
                    if (c.n(m.expert_ids) < rows * m.n_used) c.set(INFR_ERR_INVALID, "MoeFfn.expert_ids holds fewer than rows*n_used slots");
                }
                if (rows > 0x7fffffffull / (m.n_used * (uint64_t)m.n_ff_exp + 1)) { c.set(INFR_ERR_UNSUPPORTED, "MoeFfn: rows too large"); break; }
                // per-op scratch: logits, probs, ids, weights (+ bucketing tables); h and the batched
                // path's staging buffers live in one region shared by every op of the plan
                moe_off[oi] = arena;
                arena += round_up((size_t)rows * m.n_expert * 4 + 4, 256) * 2;
                arena += round_up((size_t)rows * m.n_used * 4 + 4, 256) * 2;
                const size_t pairs = (size_t)rows * m.n_used;
                size_t shared = round_up((pairs + rows) * m.n_ff_exp * 4 + 4, 256);   // one more slot per row: see kMoeShared
                const uint32_t min_rows = be->cfg.moe_batched_min_rows ? be->cfg.moe_batched_min_rows : kBatchedMinRows;
                bool batched = rows >= min_rows && m.n_used <= 64 && !m.fused_gate_up &&
                               c.dt(m.gate_exps) == c.dt(m.up_exps) &&
                               infr::grouped_supported(c.dt(m.gate_exps), (int)m.ne) &&
                               infr::grouped_supported(c.dt(m.down_exps), (int)m.n_ff_exp);
                // a bank in one of the other affine formats: the same path with the unit-decoder GEMM for all three
                // ... unless the batch selects each expert one and a half times or less: then no bucket fills a corner
                // of a 128-token tile, and the per-pair unit GEMV, which streams an expert's rows at full width, is
                // faster (2880 x 2880 MXFP4 banks, 128 experts, top-4: 32 rows 0.66 ms, 64 rows 1.04 ms, against the
                // 1.2 ms that one tile pass over every expert costs)
                const bool sparse_batch = 2 * pairs <= 3 * (size_t)n_local && be->cfg.moe_batched_min_rows == 0;
                const bool units_mfma = !batched && rows >= min_rows && m.n_used <= 64 && !sparse_batch &&
                                        (m.fused_gate_up || c.dt(m.gate_exps) == c.dt(m.up_exps)) &&
                                        infr::grouped_units_supported(c.dt(m.gate_exps), (int)m.ne) &&
                                        infr::grouped_units_supported(c.dt(m.down_exps), (int)m.n_ff_exp);
                if (units_mfma) batched = true;
                plan->moe[oi].units_mfma = units_mfma;
                if (batched) {
                    arena += round_up(((size_t)m.n_expert + 2) * 4, 256) + 3 * round_up(pairs * 4 + 4, 256);
                    shared += round_up((size_t)rows * m.ne * 2, 256) + round_up((size_t)rows * 4, 256) +
                              round_up(pairs * m.n_ff_exp * 2, 256) + round_up(pairs * 4, 256) +
                              round_up(pairs * m.ne * 4, 256);
                }
                bool bucketed = false;
                // Bucketing pays when the batch's pairs fall on few enough distinct experts: with uniform routing
                // E * (1 - (1 - K/E)^rows) of them are expected, and the bucketed kernels move a byte about 0.6 times as
                // fast as the per-token kernels do (128 experts, top-8, 16 rows: 3.2 against 4.9 TB/s), so they win below
                // that ratio of distinct experts to pairs (128 experts, top-8: from 18 rows on; 256 experts, top-8: not
                // before the matrix-core path takes over; measured on both sides of the threshold).
                const double expect_distinct = (double)m.n_expert * (1.0 - std::pow(1.0 - (double)m.n_used / (double)m.n_expert, (double)rows));
                const bool few_distinct = expect_distinct < kBucketedMaxDistinctRatio * (double)rows * (double)m.n_used;
                if (!batched && rows >= kBucketedMinRows && few_distinct && m.n_used <= 64) {
                    infr::MoeGemvParams probe{};
                    probe.gate_dt = c.dt(m.gate_exps);
                    probe.up_dt = m.fused_gate_up ? probe.gate_dt : c.dt(m.up_exps);
                    probe.down_dt = c.dt(m.down_exps);
                    probe.fused_gate_up = (int)m.fused_gate_up;
                    probe.ne = (int)m.ne;
                    probe.nff = (int)m.n_ff_exp;
                    bucketed = infr::moe_bucketed_supported(probe);
                }
                // banks without a matrix-core decoder: from the batched threshold on, the unit kernels walk the
                // expert buckets (weights fetched once per chunk of tokens)
                const bool units_batch = !batched && !bucketed && rows >= min_rows && m.n_used <= 64 && !sparse_batch &&
                                         infr::moe_units_batch_supported(c.dt(m.gate_exps),
                                                                         m.fused_gate_up ? c.dt(m.gate_exps) : c.dt(m.up_exps),
                                                                         c.dt(m.down_exps), (int)m.ne, (int)m.n_ff_exp);
                if (units_batch) bucketed = true;
                plan->moe[oi].units_batch = units_batch;
                if (bucketed) {
                    arena += round_up(((size_t)m.n_expert + 2) * 4, 256) + 3 * round_up(pairs * 4 + 4, 256);
                    shared += round_up(pairs * m.ne * 4, 256);
                }
                if (!batched && !bucketed) shared += round_up(pairs * m.ne * 4, 256);   // per-pair down results of the unit kernels
                if (shared > shared_need) shared_need = shared;
                if (!batched && !bucketed && rows * m.n_used > 65535) {
                    // the per-token kernels put the token rows (the generic ones rows * n_used) on the grid's y axis
                    c.set(INFR_ERR_UNSUPPORTED, "MoeFfn: " + std::to_string(rows) + " token rows on expert banks without a "
                          "batched kernel (" + dtype_name(c.dt(m.gate_exps)) + " / " + dtype_name(c.dt(m.down_exps)) +
                          ") exceed the per-token path's grid (rows * n_used <= 65535)");
                    break;
                }
                {
                    // the logits kernel's staging must fit the LDS: refused here, not in the middle of execute
                    int re = 1, rb = 4;
                    geometry(c.dt(m.router), &re, &rb);
                    if (!infr::router_logits_fits(c.dt(m.router), (size_t)(m.ne / re) * rb, (int)m.ne, (int)rows)) {
                        c.set(INFR_ERR_UNSUPPORTED, "MoeFfn: ne=" + std::to_string(m.ne) + " does not fit the router kernel's LDS budget");
                        break;
                    }
                }
                plan->moe[oi].rows = (int)rows;
                plan->moe[oi].batched = batched;
                plan->moe[oi].bucketed = bucketed;
                break;
            }
            case INFR_OP_LINEAR: {
                const infr_op_linear& l = op.u.linear;
                if (!(c.tensor(l.x, "Linear.x") && c.tensor(l.weight, "Linear.weight") && c.tensor(l.dst, "Linear.dst"))) break;
                if (!l.in_f || !l.out_f) { c.set(INFR_ERR_INVALID, "Linear: in_f/out_f must be positive"); break; }
                c.want_f32(l.x, "Linear.x");
                c.want_f32(l.dst, "Linear.dst");
                c.want_writable(l.dst, "Linear.dst");
                c.want_numel(l.x, (uint64_t)l.m * l.in_f, "Linear.x");
                c.want_numel(l.dst, (uint64_t)l.m * l.out_f, "Linear.dst");
                c.want_weight_dtype(l.weight, l.in_f, "Linear.weight");
                if (c.n(l.weight) % l.in_f != 0 || l.w_off % l.in_f != 0 ||
                    (uint64_t)l.w_off / l.in_f + l.out_f > c.n(l.weight) / l.in_f)
                    c.set(INFR_ERR_INVALID, "Linear: w_off/out_f select rows outside the weight tensor");
                if (c.st == INFR_OK) {
                    // a batch of rows (prefill): f16 operands on the matrix cores, as Op::MoeFfn does from the same row count
                    // (one bucket means ceil(m / 128) x ceil(out_f / 256) tiles in all: below about a tile of rows the
                    // GEMV kernels, which spread over the output rows, are faster)
                    const uint32_t min_rows = be->cfg.moe_batched_min_rows ? be->cfg.moe_batched_min_rows : kLinearBatchedMinRows;
                    const int dt = c.dt(l.weight);
                    int mode = 0;
                    if (l.m >= min_rows && l.m <= (1u << 24)) {
                        if (infr::grouped_supported(dt, (int)l.in_f)) mode = 1;
                        else if (infr::grouped_units_supported(dt, (int)l.in_f)) mode = 2;
                    }
                    plan->lin[oi].mode = mode;
                    if (mode) {
                        plan->lin[oi].offsets_off = arena;
                        arena += 256;
                        const size_t shared = round_up((size_t)l.m * l.in_f * 2, 256) + round_up((size_t)l.m * 4, 256);
                        if (shared > shared_need) shared_need = shared;
                    }
                }
                break;
            }
            case INFR_OP_GATED_ACT: {
                const infr_op_gated_act& a = op.u.gated_act;
                if (!(c.tensor(a.gate, "GatedAct.gate") && c.tensor(a.up, "GatedAct.up") && c.tensor(a.dst, "GatedAct.dst"))) break;
                c.want_f32(a.gate, "GatedAct.gate");
                c.want_f32(a.up, "GatedAct.up");
                c.want_f32(a.dst, "GatedAct.dst");
                c.want_writable(a.dst, "GatedAct.dst");
                c.want_numel(a.dst, (uint64_t)a.rows * a.nff, "GatedAct.dst");
                if (a.has_swiglu_clamp && a.act == INFR_ACT_SIGMOID)
                    c.set(INFR_ERR_INVALID, "GatedAct: swiglu_clamp is defined for the gated SiLU/GELU forms only");
                if (a.act < INFR_ACT_SILU || a.act > INFR_ACT_SIGMOID) c.set(INFR_ERR_INVALID, "GatedAct: unknown activation");
                {
                    // highest element each operand is read at must exist
                    uint64_t rows = a.rows, nff = a.nff;
                    if (rows && nff) {
                        uint64_t umax = (a.up_stride == 0 ? (rows - 1) * nff : (rows - 1) * (uint64_t)a.up_stride) + a.up_off + nff;
                        uint64_t gmax;
                        if (a.gate_block_width > 0) {
                            uint64_t headw = a.gate_block_width / 2;
                            if (headw == 0) { c.set(INFR_ERR_INVALID, "GatedAct: gate_block_width < 2"); break; }
                            uint64_t head = (nff - 1) / headw, off = (nff - 1) % headw;
                            gmax = (rows - 1) * (uint64_t)a.gate_stride + head * a.gate_block_width + headw + off + 1;
                        } else {
                            gmax = (a.gate_stride > 0 ? (rows - 1) * (uint64_t)a.gate_stride : (rows - 1) * nff) + nff;
                        }
                        if (umax > c.n(a.up)) c.set(INFR_ERR_INVALID, "GatedAct.up: strides read past the tensor");
                        if (gmax > c.n(a.gate)) c.set(INFR_ERR_INVALID, "GatedAct.gate: strides read past the tensor");
                    }
                }
                break;
            }
            case INFR_OP_ADD: {
                const infr_op_add& a = op.u.add;
                if (!(c.tensor(a.a, "Add.a") && c.tensor(a.b, "Add.b") && c.tensor(a.dst, "Add.dst"))) break;
                c.want_f32(a.a, "Add.a"); c.want_f32(a.b, "Add.b"); c.want_f32(a.dst, "Add.dst");
                c.want_writable(a.dst, "Add.dst");
                if (c.n(a.a) < a.n || c.n(a.b) < a.n || c.n(a.dst) < a.n) c.set(INFR_ERR_INVALID, "Add: n exceeds an operand");
                break;
            }
            case INFR_OP_MOE_SHARED_EXPERT_ADD: {
                const infr_op_moe_shared_expert_add& a = op.u.moe_shared_expert_add;
                if (!(c.tensor(a.moe, "MoeSharedExpertAdd.moe") && c.tensor(a.shexp, "MoeSharedExpertAdd.shexp") &&
                      c.tensor(a.gate, "MoeSharedExpertAdd.gate") && c.tensor(a.dst, "MoeSharedExpertAdd.dst"))) break;
                c.want_f32(a.moe, "MoeSharedExpertAdd.moe"); c.want_f32(a.shexp, "MoeSharedExpertAdd.shexp");
                c.want_f32(a.gate, "MoeSharedExpertAdd.gate"); c.want_f32(a.dst, "MoeSharedExpertAdd.dst");
                c.want_writable(a.dst, "MoeSharedExpertAdd.dst");
                uint64_t tot = (uint64_t)a.rows * a.n;
                if (c.n(a.moe) < tot || c.n(a.shexp) < tot || c.n(a.dst) < tot || c.n(a.gate) < a.rows)
                    c.set(INFR_ERR_INVALID, "MoeSharedExpertAdd: rows*n exceeds an operand");
                break;
            }
            case INFR_OP_RMS_NORM:
            case INFR_OP_RMS_NORM_ADD: {
                const infr_op_rms_norm& nr = op.u.rms_norm;
                if (!(c.tensor(nr.x, "RmsNorm.x") && c.tensor(nr.weight, "RmsNorm.weight") && c.tensor(nr.dst, "RmsNorm.dst"))) break;
                c.want_f32(nr.x, "RmsNorm.x"); c.want_f32(nr.weight, "RmsNorm.weight"); c.want_f32(nr.dst, "RmsNorm.dst");
                c.want_writable(nr.dst, "RmsNorm.dst");
                if (!nr.dim) { c.set(INFR_ERR_INVALID, "RmsNorm: dim must be positive"); break; }
                const uint64_t tot = (uint64_t)nr.rows * nr.dim;
                if (c.n(nr.x) < tot || c.n(nr.dst) < tot || c.n(nr.weight) < nr.dim)
                    c.set(INFR_ERR_INVALID, "RmsNorm: rows*dim exceeds an operand");
                if (nr.rows > 0x7fffffffu / nr.dim) c.set(INFR_ERR_UNSUPPORTED, "RmsNorm: more than 2^31 elements");
                break;
            }
            case INFR_OP_COPY:
            case INFR_OP_COPY_STRIDED: {
                const infr_op_copy& cp = op.u.copy;
                if (!(c.tensor(cp.src, "Copy.src") && c.tensor(cp.dst, "Copy.dst"))) break;
                c.want_writable(cp.dst, "Copy.dst");
                const int dt = c.dt(cp.src);
                if (dt != c.dt(cp.dst)) { c.set(INFR_ERR_INVALID, "Copy: src and dst differ in dtype"); break; }
                if (!(dt == INFR_F32 || dt == INFR_I32 || dt == INFR_U32 || dt == INFR_F16 || dt == INFR_BF16)) {
                    c.set(INFR_ERR_UNSUPPORTED, "Copy: only F32/I32/U32/F16/BF16 tensors");
                    break;
                }
                const uint64_t rows = op.kind == INFR_OP_COPY ? 1 : cp.rows;
                if (rows && cp.n) {
                    const uint64_t s_end = cp.src_off + (rows - 1) * (uint64_t)cp.src_stride + cp.n;
                    const uint64_t d_end = cp.dst_off + (rows - 1) * (uint64_t)cp.dst_stride + cp.n;
                    if (s_end > c.n(cp.src) || d_end > c.n(cp.dst)) { c.set(INFR_ERR_INVALID, "Copy: window outside a tensor"); break; }
                    if (rows > 65535) { c.set(INFR_ERR_UNSUPPORTED, "Copy: more than 65535 rows"); break; }
                    if (cp.src == cp.dst) {
                        // the source window is staged first (the CPU backend clones it, lib.rs:3540-3545)
                        plan->copy_tmp[oi] = arena;
                        arena += round_up(rows * cp.n * 4, 256);
                    }
                }
                break;
            }
            default:
                c.set(INFR_ERR_UNSUPPORTED, "compile: op kind " + std::to_string(op.kind) +
                                                " is not on the routed-expert FFN path this backend implements");
        }
        if (c.st != INFR_OK) c.err = "op " + std::to_string(oi) + ": " + c.err;
    }
    if (c.st != INFR_OK) return bail(c.st, c.err);
    const size_t shared_off = arena;
    arena += shared_need;

    // ---- launch fusion: Linear + Linear + GatedAct on one input -> one gate/up kernel; Linear + Add
    // -> one kernel.  A temporary may disappear only if it is an Internal tensor written once and read
    // once.  The fused kernels run the same inner products and the same rounding sequence, so the
    // results are the bits the separate ops give.
    plan->fuse.assign(g->n_ops, infr_hip_plan::FuseOp{});
    plan->fuse_head = plan->fuse;
    size_t zero_rows = 0;
    if (!be->cfg.disable_op_fusion) {
        std::vector<int> reads(plan->tensors.size(), 0), writes(plan->tensors.size(), 0);
        auto rd = [&](uint32_t t) { if (t != INFR_NO_TENSOR && t < reads.size()) reads[t]++; };
        auto wr = [&](uint32_t t) { if (t != INFR_NO_TENSOR && t < writes.size()) writes[t]++; };
        for (uint32_t oi = 0; oi < g->n_ops; oi++) {
            const infr_op& op = plan->ops[oi];
            switch (op.kind) {
                case INFR_OP_MOE_FFN: {
                    const infr_op_moe_ffn& m = op.u.moe_ffn;
                    rd(m.x); rd(m.router_x); rd(m.router); rd(m.gate_exps); rd(m.up_exps); rd(m.down_exps);
                    rd(m.down_scale); rd(m.exp_probs_b); rd(m.expert_ids); wr(m.dst);
                    break;
                }
                case INFR_OP_LINEAR: rd(op.u.linear.x); rd(op.u.linear.weight); wr(op.u.linear.dst); break;
                case INFR_OP_GATED_ACT: rd(op.u.gated_act.gate); rd(op.u.gated_act.up); wr(op.u.gated_act.dst); break;
                case INFR_OP_ADD: rd(op.u.add.a); rd(op.u.add.b); wr(op.u.add.dst); break;
                case INFR_OP_MOE_SHARED_EXPERT_ADD: {
                    const infr_op_moe_shared_expert_add& a = op.u.moe_shared_expert_add;
                    rd(a.moe); rd(a.shexp); rd(a.gate); wr(a.dst);
                    break;
                }
                case INFR_OP_COPY:
                case INFR_OP_COPY_STRIDED: rd(op.u.copy.src); rd(op.u.copy.dst); wr(op.u.copy.dst); break;   // a partial write keeps the rest
                case INFR_OP_RMS_NORM: rd(op.u.rms_norm.x); rd(op.u.rms_norm.weight); wr(op.u.rms_norm.dst); break;
                case INFR_OP_RMS_NORM_ADD:
                    rd(op.u.rms_norm.x); rd(op.u.rms_norm.weight); rd(op.u.rms_norm.dst); wr(op.u.rms_norm.dst);
                    break;
                default: break;
            }
        }
        auto temp = [&](uint32_t t) {
            return plan->tensors[t].kind == INFR_KIND_INTERNAL && reads[t] == 1 && writes[t] == 1;
        };
        for (uint32_t oi = 0; oi + 1 < g->n_ops; oi++) {
            if (plan->fuse[oi].kind != infr_hip_plan::kPlain || plan->ops[oi].kind != INFR_OP_LINEAR) continue;
            const infr_op_linear& l1 = plan->ops[oi].u.linear;
            if (l1.m == 0) continue;
            if (plan->lin[oi].mode) continue;   // a batch on the matrix cores: the epilogues there take no second operand
            // Linear, Linear, GatedAct
            if (oi + 2 < g->n_ops && plan->ops[oi + 1].kind == INFR_OP_LINEAR && plan->ops[oi + 2].kind == INFR_OP_GATED_ACT) {
                const infr_op_linear& l2 = plan->ops[oi + 1].u.linear;
                const infr_op_gated_act& ga = plan->ops[oi + 2].u.gated_act;
                const bool gate_first = ga.gate == l1.dst && ga.up == l2.dst, up_first = ga.gate == l2.dst && ga.up == l1.dst;
                infr::MoeGemvParams probe{};
                probe.gate_dt = probe.up_dt = c.dt(l1.weight);
                probe.ne = (int)l1.in_f;
                probe.n_used = 1;
                if ((gate_first || up_first) && l1.x == l2.x && l1.m == l2.m && l1.in_f == l2.in_f && l1.out_f == l2.out_f &&
                    l1.w_off == 0 && l2.w_off == 0 && l1.dst != l2.dst && c.dt(l1.weight) == c.dt(l2.weight) &&
                    temp(l1.dst) && temp(l2.dst) && ga.rows == l1.m && ga.nff == l1.out_f && ga.up_off == 0 &&
                    ga.gate_block_width == 0 && (ga.up_stride == 0 || ga.up_stride == ga.nff) &&
                    (ga.gate_stride == 0 || ga.gate_stride == ga.nff) && ga.dst != l1.x &&
                    infr::moe_gate_up_routes_inline(probe)) {
                    plan->fuse[oi].kind = infr_hip_plan::kGateUpAct;
                    plan->fuse[oi].a = gate_first ? oi + 1 : oi;       // the up Linear
                    plan->fuse[oi].b = oi + 2;
                    plan->fuse[oi + 1].kind = plan->fuse[oi + 2].kind = infr_hip_plan::kSkip;
                    if (l1.m > zero_rows) zero_rows = l1.m;
                    continue;
                }
            }
            // Linear, Add
            if (plan->ops[oi + 1].kind == INFR_OP_ADD && plan->fuse[oi + 1].kind == infr_hip_plan::kPlain) {
                const infr_op_add& ad = plan->ops[oi + 1].u.add;
                const bool is_b = ad.b == l1.dst && ad.a != l1.dst, is_a = ad.a == l1.dst && ad.b != l1.dst;
                if ((is_a || is_b) && temp(l1.dst) && (uint64_t)ad.n == (uint64_t)l1.m * l1.out_f && ad.dst != l1.x) {
                    plan->fuse[oi].kind = infr_hip_plan::kLinearAdd;
                    plan->fuse[oi].a = oi + 1;
                    plan->fuse[oi + 1].kind = infr_hip_plan::kSkip;
                }
            }
        }
        // MoeFfn followed by an always-on ("shared") expert on the same rows whose result is added to
        // the routed sum: on the per-token path the expert runs as one more slot of the two routed
        // kernels.  The slot's inner products are the ones the fused Linear kernels run, its weight is
        // exactly 1 and it is combined last, which is the Add's rounding: the bits do not change.
        plan->fuse_head = plan->fuse;
        for (uint32_t oi = 0; oi + 5 < g->n_ops; oi++) {
            if (plan->ops[oi].kind != INFR_OP_MOE_FFN) continue;
            // the gated form (crates/infr-llama/src/seam/runner.rs:8104-8163): the gate-logit Linear (out_f = 1) comes
            // first and Op::MoeSharedExpertAdd closes the pattern; that Linear stays a launch of its own
            const bool gated = oi + 6 < g->n_ops && plan->ops[oi + 1].kind == INFR_OP_LINEAR &&
                               plan->ops[oi + 1].u.linear.out_f == 1 && plan->fuse[oi + 1].kind == infr_hip_plan::kPlain &&
                               plan->ops[oi + 6].kind == INFR_OP_MOE_SHARED_EXPERT_ADD;
            const uint32_t b0 = gated ? oi + 2 : oi + 1;   // first op of the dense FFN
            if (plan->fuse[b0].kind != infr_hip_plan::kGateUpAct) continue;
            if (gated ? plan->fuse[b0 + 3].kind != infr_hip_plan::kPlain || plan->ops[b0 + 3].kind != INFR_OP_LINEAR
                      : plan->fuse[b0 + 3].kind != infr_hip_plan::kLinearAdd)
                continue;
            const infr_op_moe_ffn& m = plan->ops[oi].u.moe_ffn;
            const MoeScratch& sc = plan->moe[oi];
            const infr_hip_plan::FuseOp fg = plan->fuse[b0];
            const infr_op_linear& lu = plan->ops[fg.a].u.linear;
            const infr_op_linear& lg = plan->ops[fg.a == b0 ? b0 + 1 : b0].u.linear;
            const infr_op_gated_act& ga = plan->ops[b0 + 2].u.gated_act;
            const infr_op_linear& ld = plan->ops[b0 + 3].u.linear;
            uint32_t other;
            if (gated) {
                const infr_op_moe_shared_expert_add& sa = plan->ops[oi + 6].u.moe_shared_expert_add;
                const infr_op_linear& lq = plan->ops[oi + 1].u.linear;
                if (sa.shexp != ld.dst || !temp(ld.dst) || sa.gate != lq.dst || !temp(lq.dst) || (int)sa.rows != sc.rows ||
                    sa.n != m.ne || lq.x != m.x || (int)lq.m != sc.rows || lq.in_f != m.ne)
                    continue;
                other = sa.moe;
            } else {
                const infr_op_add& ad = plan->ops[b0 + 4].u.add;
                other = ad.a == ld.dst ? ad.b : ad.a;
            }
            // the per-token kernels only: every row's blocks read the always-on expert's rows
            // again, from the L2 after the first
            if (sc.batched || sc.bucketed || m.fused_gate_up) continue;
            if (lg.x != m.x || (int)lg.m != sc.rows || lg.in_f != m.ne || lg.out_f != m.n_ff_exp) continue;
            if (ld.x != ga.dst || !temp(ga.dst) || ld.in_f != m.n_ff_exp || ld.out_f != m.ne || ld.w_off != 0) continue;
            if (other != m.dst || !temp(m.dst)) continue;
            if (c.dt(lg.weight) != c.dt(m.gate_exps) || c.dt(lu.weight) != c.dt(m.up_exps) ||
                c.dt(ld.weight) != c.dt(m.down_exps))
                continue;
            if (ga.act != m.act || ga.has_swiglu_clamp != m.has_swiglu_clamp ||
                (ga.has_swiglu_clamp && ga.swiglu_clamp != m.swiglu_clamp))
                continue;
            infr::MoeGemvParams probe{};
            probe.gate_dt = c.dt(m.gate_exps); probe.up_dt = c.dt(m.up_exps); probe.down_dt = c.dt(m.down_exps);
            probe.ne = (int)m.ne; probe.nff = (int)m.n_ff_exp; probe.n_used = (int)m.n_used; probe.n_expert = (int)m.n_expert;
            probe.rows = sc.rows;
            probe.route.n_expert = (int)m.n_expert; probe.route.n_used = (int)m.n_used;
            probe.route.n_groups = (int)m.n_expert_groups; probe.route.n_groups_used = (int)m.n_expert_groups_used;
            probe.sh_gate = probe.sh_up = probe.sh_down = (const uint8_t*)plan;   // any non-null value: shape checks only
            if (m.n_used >= 63 || !infr::moe_gate_up_routes_inline(probe) || !infr::moe_down_is_fast(probe)) continue;
            plan->fuse[oi].kind = infr_hip_plan::kMoeShared;
            plan->fuse[oi].a = b0;
            plan->fuse[oi].b = b0 + 3;
            plan->fuse[oi].gated = gated ? oi + 7 : 0;
            // (the gate-logit Linear of the gated form is launched by the fused op, ahead of the kernel that reads it)
            for (uint32_t k = oi + 1; k <= b0 + 4; k++) plan->fuse[k].kind = infr_hip_plan::kSkip;
        }
        // MoeFfn -> Add (the residual; the reference's moe_add rewrite, crates/infr-core/src/fusion.rs:20-24):
        // every combine kernel ends with "other operand + finished sum", the Add's own rounding.
        // RmsNorm -> MoeFfn on one token row (fusion.rs:15-19 with moe_ok): the logits kernel normalises the
        // raw row while staging it and stores the normalised row, which the expert kernels then read.
        for (uint32_t oi = 0; oi < g->n_ops; oi++) {
            if (plan->ops[oi].kind != INFR_OP_MOE_FFN) continue;
            const infr_hip_plan::Fuse kind = plan->fuse[oi].kind;
            if (kind != infr_hip_plan::kPlain && kind != infr_hip_plan::kMoeShared) continue;
            const infr_op_moe_ffn& m = plan->ops[oi].u.moe_ffn;
            const MoeScratch& sc = plan->moe[oi];
            const uint32_t close = plan->fuse[oi].b + 1;   // kMoeShared: the Add / MoeSharedExpertAdd that ends the pattern
            const uint32_t nx = kind == infr_hip_plan::kMoeShared ? close + 1 : oi + 1;
            const uint32_t sum_t = kind != infr_hip_plan::kMoeShared ? m.dst
                                   : plan->fuse[oi].gated ? plan->ops[close].u.moe_shared_expert_add.dst
                                                          : plan->ops[close].u.add.dst;
            if (nx < g->n_ops && plan->ops[nx].kind == INFR_OP_ADD && plan->fuse[nx].kind == infr_hip_plan::kPlain && sc.rows > 0) {
                const infr_op_add& ad = plan->ops[nx].u.add;
                const bool one_side = (ad.a == sum_t) != (ad.b == sum_t);
                if (one_side && temp(sum_t) && (uint64_t)ad.n == (uint64_t)sc.rows * m.ne) {
                    plan->fuse[oi].res = nx + 1;
                    plan->fuse[nx].kind = infr_hip_plan::kSkip;
                }
            }
            if (oi > 0 && plan->ops[oi - 1].kind == INFR_OP_RMS_NORM && plan->fuse[oi - 1].kind == infr_hip_plan::kPlain) {
                const infr_op_rms_norm& nr = plan->ops[oi - 1].u.rms_norm;
                int re = 1, rb = 4;
                geometry(c.dt(m.router), &re, &rb);
                if (nr.rows == 1 && sc.rows == 1 && !sc.batched && !sc.bucketed && nr.dim == m.ne && nr.dst == m.router_x &&
                    nr.x != nr.dst && infr::router_logits_can_norm(c.dt(m.router), (size_t)(m.ne / re) * rb, (int)m.ne, 1)) {
                    plan->fuse[oi].norm = oi;   // 1 + (oi - 1)
                    plan->fuse[oi - 1].kind = infr_hip_plan::kSkip;
                }
            }
        }
    }
    // One token row through a MoeFfn: the whole op (with an always-on expert folded in, if there is one) as one launch
    // when the shape fits one of the two single-launch kernels.  An RmsNorm folded into the logits kernel is unfolded
    // again: it costs one small launch, the single launch saves two large ones.
    size_t layer_ws = 0, stream_ws = 0;
    if (!be->cfg.disable_single_launch_moe && be->prop.multiProcessorCount >= 256) {
        for (uint32_t oi = 0; oi < g->n_ops; oi++) {
            if (plan->ops[oi].kind != INFR_OP_MOE_FFN) continue;
            const infr_hip_plan::Fuse kind = plan->fuse[oi].kind;
            if (kind != infr_hip_plan::kPlain && kind != infr_hip_plan::kMoeShared) continue;
            const infr_op_moe_ffn& m = plan->ops[oi].u.moe_ffn;
            MoeScratch& sc = plan->moe[oi];
            if ((sc.rows != 1 && sc.rows != 2 && sc.rows != 4 && sc.rows != 8) || sc.batched || sc.bucketed || c.dt(m.router) != INFR_F32) continue;
            infr::MoeLayerParams probe{};
            probe.g.rows = sc.rows; probe.g.ne = (int)m.ne; probe.g.nff = (int)m.n_ff_exp; probe.g.n_used = (int)m.n_used;
            probe.g.n_expert = (int)(m.has_ep_band ? m.ep_n_local : m.n_expert);
            probe.g.gate_dt = c.dt(m.gate_exps);
            probe.g.up_dt = m.fused_gate_up ? probe.g.gate_dt : c.dt(m.up_exps);
            probe.g.down_dt = c.dt(m.down_exps);
            probe.g.n_cu = be->prop.multiProcessorCount;
            probe.g.weight_before = (int)m.weight_before;
            probe.g.skip_zero_w = (int)m.has_ep_band;
            probe.g.route.n_expert = (int)m.n_expert; probe.g.route.n_used = (int)m.n_used;
            probe.g.route.n_groups = (int)m.n_expert_groups; probe.g.route.n_groups_used = (int)m.n_expert_groups_used;
            probe.g.route.gating = m.gating;
            probe.g.route.exp_probs_b = m.exp_probs_b == INFR_NO_TENSOR ? nullptr : (const float*)plan;   // non-null: given
            probe.g.route.expert_ids = m.expert_ids == INFR_NO_TENSOR ? nullptr : (const int32_t*)plan;
            probe.g.route.ep_n = m.has_ep_band ? (int)m.ep_n_local : 0;
            probe.router_row_floats = m.ne;
            probe.logits_once = moe_logits_once(be, m);
            if (kind == infr_hip_plan::kMoeShared) probe.g.sh_gate = probe.g.sh_up = probe.g.sh_down = (const uint8_t*)plan;
            if (!be->cfg.disable_single_launch_guess && infr::moe_layer_stream_supported(probe)) {
                sc.single_launch = 2;
                stream_ws = std::max(stream_ws, infr::moe_layer_stream_workspace_bytes((int)m.ne, (int)m.n_ff_exp, (int)m.n_expert, sc.rows));
            } else if (kind == infr_hip_plan::kPlain && infr::moe_layer_fused_supported(probe)) {
                sc.single_launch = 1;
                layer_ws = std::max(layer_ws, infr::moe_layer_workspace_bytes((int)m.ne, (int)m.n_ff_exp, (int)m.n_expert));
            } else {
                continue;
            }
            // An RmsNorm folded into the logits kernel stays folded for the streaming kernel, which normalises the row
            // itself (and for the three launches it falls back to); the in-order kernel has no such fold, and the gated
            // always-on expert's gate-logit launch reads the normalised row before the layer's launch: both take the norm
            // as an op of its own.
            bool keep_norm = false;
            if (plan->fuse[oi].norm && sc.single_launch == 2 && !plan->fuse[oi].gated) {
                const infr_op_rms_norm& nr = plan->ops[plan->fuse[oi].norm - 1].u.rms_norm;
                probe.norm_w = (const float*)plan;   // non-null: asked for
                keep_norm = sc.rows == 1 && m.x == nr.dst && infr::moe_layer_stream_supported(probe);
            }
            if (plan->fuse[oi].norm && !keep_norm) {
                plan->fuse[plan->fuse[oi].norm - 1].kind = infr_hip_plan::kPlain;
                plan->fuse[oi].norm = 0;
            }
        }
    }
    const size_t stream_ws_off = arena;
    arena += round_up(stream_ws, 256);
    const size_t layer_ws_off = arena;
    arena += round_up(layer_ws, 256);
    const size_t zero_off = arena;
    arena += round_up(zero_rows * 4 + 4, 256);

    std::lock_guard<std::mutex> lk(be->mu);
    hipError_t e = hipSetDevice(be->device);
    if (e == hipSuccess && arena) { g_alloc_calls++; e = hipMalloc(&plan->arena, arena); }
    if (e != hipSuccess) return bail(INFR_ERR_BACKEND, std::string("compile: scratch hipMalloc failed: ") + hipGetErrorString(e));
    plan->arena_bytes = arena;
    for (uint32_t oi = 0; oi < g->n_ops; oi++) {
        if (plan->ops[oi].kind != INFR_OP_MOE_FFN) continue;
        const infr_op_moe_ffn& m = plan->ops[oi].u.moe_ffn;
        MoeScratch& s = plan->moe[oi];
        char* p = (char*)plan->arena + moe_off[oi];
        size_t rows = (size_t)s.rows;
        s.logits = (float*)p; p += round_up(rows * m.n_expert * 4 + 4, 256);
        s.probs = (float*)p;  p += round_up(rows * m.n_expert * 4 + 4, 256);
        s.ids = (int32_t*)p;  p += round_up(rows * m.n_used * 4 + 4, 256);
        s.weights = (float*)p; p += round_up(rows * m.n_used * 4 + 4, 256);
        const size_t pairs = rows * m.n_used;
        if (s.batched || s.bucketed) {
            s.offsets = (int32_t*)p;   p += round_up(((size_t)m.n_expert + 2) * 4, 256);
            s.pair_src = (int32_t*)p;  p += round_up(pairs * 4 + 4, 256);
            s.slot_pair = (int32_t*)p; p += round_up(pairs * 4 + 4, 256);
            s.live_ids = (int32_t*)p;
        }
        p = (char*)plan->arena + shared_off;
        s.h = (float*)p; p += round_up((pairs + rows) * m.n_ff_exp * 4 + 4, 256);
        if (s.batched) {
            s.xh = (_Float16*)p; p += round_up(rows * m.ne * 2, 256);
            s.xs = (float*)p;    p += round_up(rows * 4, 256);
            s.hh = (_Float16*)p; p += round_up(pairs * m.n_ff_exp * 2, 256);
            s.hs = (float*)p;    p += round_up(pairs * 4, 256);
            s.y = (float*)p;
        } else {
            s.y = (float*)p;
        }
    }
    plan->layer_ws = layer_ws ? (char*)plan->arena + layer_ws_off : nullptr;
    plan->stream_ws = stream_ws ? (char*)plan->arena + stream_ws_off : nullptr;
    plan->zero_ids = (int32_t*)((char*)plan->arena + zero_off);   // stays zero: the arena is zero-filled and nothing writes here
    if (plan->arena) infr::launch_fill_zero(be->stream, plan->arena, arena);
    for (uint32_t oi = 0; oi < g->n_ops; oi++) {
        if (plan->ops[oi].kind != INFR_OP_LINEAR || !plan->lin[oi].mode) continue;
        const infr_op_linear& l = plan->ops[oi].u.linear;
        plan->lin_xh = (_Float16*)((char*)plan->arena + shared_off);
        const int32_t table[2] = {0, (int32_t)l.m};
        e = hipMemcpyAsync((char*)plan->arena + plan->lin[oi].offsets_off, table, sizeof table, hipMemcpyHostToDevice, be->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(be->stream);   // `table` is on this stack frame
        if (e != hipSuccess)
            return bail(INFR_ERR_BACKEND, std::string("compile: bucket table upload failed: ") + hipGetErrorString(e));
    }
    be->refs.fetch_add(1);   // the plan keeps its backend alive
    *out = holder.release();
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_compile"); }

extern "C" void infr_hip_plan_free(infr_hip_plan* plan) try {
    if (!ok_plan(plan)) return;
    infr_hip_backend* be = plan->be;   // alive: the plan holds a reference
    {
        std::lock_guard<std::mutex> lk(be->mu);
        (void)hipSetDevice(be->device);
        if (!be->closed.load()) (void)hipStreamSynchronize(be->stream);
        delete plan;   // frees the arena
    }
    release_backend(be);
} catch (...) {
}

// ============================================================================ execute
extern "C" infr_status infr_hip_execute(infr_hip_backend* be, infr_hip_plan* plan, const infr_binding* bindings,
                                        uint32_t n_bindings) try {
    if (!ok_backend(be)) return fail(INFR_ERR_INVALID, "execute: backend handle is not a hip backend");
    if (!ok_plan(plan) || plan->be != be) return fail(INFR_ERR_BACKEND, "hip backend: incompatible plan");
    if (n_bindings && !bindings) return fail(INFR_ERR_INVALID, "execute: bindings is null");
    const size_t nt = plan->tensors.size();
    std::vector<const infr_hip_buffer*> bound(nt, nullptr);
    for (uint32_t i = 0; i < n_bindings; i++) {
        if (bindings[i].tensor >= nt) return fail(INFR_ERR_INVALID, "execute: binding for tensor %u, graph has %zu", bindings[i].tensor, nt);
        if (infr_status st = check_owned(be, bindings[i].buffer, "execute")) return st;
        bound[bindings[i].tensor] = bindings[i].buffer;  // re-binding an id overwrites (backend.rs:582-590)
    }
    // Resolve every tensor the ops touch to a device pointer, checking extents.
    std::vector<void*> ptr(nt, nullptr);
    for (size_t i = 0; i < nt; i++) {
        const infr_tensor_decl& t = plan->tensors[i];
        if (t.kind == INFR_KIND_INTERNAL) {
            ptr[i] = (char*)plan->arena + plan->internal_off[i];
        } else if (bound[i]) {
            size_t need = tensor_bytes(t, plan->numel[i]);
            if (bound[i]->len < need)
                return fail(INFR_ERR_BACKEND, "execute: tensor %zu needs %zu bytes, bound buffer holds %zu", i, need, bound[i]->len);
            ptr[i] = bound[i]->dptr;
        }
    }
    auto need = [&](uint32_t id, const char* role) -> bool {
        if (id == INFR_NO_TENSOR) return true;
        if (!ptr[id]) {
            const char* k = plan->tensors[id].kind == INFR_KIND_WEIGHT ? "Weight" : plan->tensors[id].kind == INFR_KIND_INPUT ? "Input" : "Output";
            fail(INFR_ERR_BACKEND, "hip backend: unbound %s (%s, tensor %u)", k, role, id);
            return false;
        }
        return true;
    };
    // every tensor of every op is resolved before the first launch: a plan either runs whole or not at all
    for (size_t oi = 0; oi < plan->ops.size(); oi++) {
        uint32_t ids[12];
        const char* role = "op";
        const int n_ids = op_tensors(plan->ops[oi], ids, &role);
        for (int k = 0; k < n_ids; k++)
            if (!need(ids[k], role)) return INFR_ERR_BACKEND;
    }
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    hipStream_t s = be->stream;
    const int n_cu = be->prop.multiProcessorCount;
    for (size_t oi = 0; oi < plan->ops.size(); oi++) {
        const infr_op& op = plan->ops[oi];
        const infr_hip_plan::FuseOp fz = plan->fuse[oi];
        if (fz.kind == infr_hip_plan::kSkip) continue;
        if (fz.kind == infr_hip_plan::kGateUpAct) {
            const infr_op_linear& lu = plan->ops[fz.a].u.linear;                       // up
            const infr_op_linear& lg = plan->ops[fz.a == oi ? oi + 1 : oi].u.linear;   // gate
            const infr_op_gated_act& ga = plan->ops[fz.b].u.gated_act;
            if (!(need(lg.x, "Linear.x") && need(lg.weight, "Linear.weight") && need(lu.weight, "Linear.weight") &&
                  need(ga.dst, "GatedAct.dst")))
                return INFR_ERR_BACKEND;
            infr::MoeGemvParams gp{};
            gp.x = (const float*)ptr[lg.x];
            gp.ids = plan->zero_ids;
            gp.weights = (const float*)plan->zero_ids;   // never used: weight_before is off
            gp.gate = (const uint8_t*)ptr[lg.weight];
            gp.up = (const uint8_t*)ptr[lu.weight];
            gp.gate_dt = gp.up_dt = plan->tensors[lg.weight].dtype;
            gp.rows = (int)lg.m; gp.ne = (int)lg.in_f; gp.nff = (int)lg.out_f; gp.n_used = 1; gp.n_expert = 1;
            gp.act = ga.act; gp.has_clamp = (int)ga.has_swiglu_clamp; gp.clamp = ga.swiglu_clamp;
            gp.h = (float*)ptr[ga.dst]; gp.n_cu = n_cu;
            Timed t(be, "linear_gate_up_act");
            if (gp.rows >= 2 && infr::bucketed_rows_supported(gp.gate_dt, gp.ne)) {
                // several rows: one bucket of the bucketed kernel, two rows share each weight row
                gp.h = (float*)ptr[ga.dst];
                infr::launch_moe_gate_up_bucketed(s, gp);
            } else {
                infr::launch_moe_gate_up(s, gp);
            }
            continue;
        }
        if (fz.kind == infr_hip_plan::kLinearAdd) {
            const infr_op_linear& l = op.u.linear;
            const infr_op_add& ad = plan->ops[fz.a].u.add;
            const uint32_t other = ad.a == l.dst ? ad.b : ad.a;
            if (!(need(l.x, "Linear.x") && need(l.weight, "Linear.weight") && need(other, "Add.a") && need(ad.dst, "Add.dst")))
                return INFR_ERR_BACKEND;
            int we = 1, wb = 4;
            geometry(plan->tensors[l.weight].dtype, &we, &wb);
            size_t row_bytes = (size_t)(l.in_f / we) * wb;
            const uint8_t* w = (const uint8_t*)ptr[l.weight] + (size_t)(l.w_off / l.in_f) * row_bytes;
            Timed t(be, "linear_add");
            infr::launch_linear(s, (const float*)ptr[l.x], w, plan->tensors[l.weight].dtype, row_bytes, (int)l.m, (int)l.in_f,
                                (int)l.out_f, (float*)ptr[ad.dst], n_cu, (const float*)ptr[other]);
            continue;
        }
        switch (op.kind) {
            case INFR_OP_MOE_FFN: {
                const infr_op_moe_ffn& m = op.u.moe_ffn;
                if (!(need(m.x, "MoeFfn.x") && need(m.router_x, "MoeFfn.router_x") && need(m.router, "MoeFfn.router") &&
                      need(m.gate_exps, "MoeFfn.gate_exps") && (m.fused_gate_up || need(m.up_exps, "MoeFfn.up_exps")) &&
                      need(m.down_exps, "MoeFfn.down_exps") && need(m.dst, "MoeFfn.dst") &&
                      need(m.down_scale, "MoeFfn.down_scale") && need(m.exp_probs_b, "MoeFfn.exp_probs_b") &&
                      need(m.expert_ids, "MoeFfn.expert_ids")))
                    return INFR_ERR_BACKEND;
                MoeScratch& sc = plan->moe[oi];
                const int rows = sc.rows;
                plan->last_moe_op = (int)oi;
                if (rows == 0) break;
                int re = 1, rb = 4;
                geometry(plan->tensors[m.router].dtype, &re, &rb);
                size_t router_row_bytes = (size_t)(m.ne / re) * rb;
                infr::RouteParams rp{};
                rp.logits = sc.logits; rp.n_expert = (int)m.n_expert; rp.n_used = (int)m.n_used; rp.rows = rows;
                rp.gating = m.gating; rp.norm_w = (int)m.norm_w; rp.scale = m.scale;
                rp.exp_probs_b = m.exp_probs_b == INFR_NO_TENSOR ? nullptr : (const float*)ptr[m.exp_probs_b];
                rp.n_groups = (int)m.n_expert_groups; rp.n_groups_used = (int)m.n_expert_groups_used;
                rp.expert_ids = m.expert_ids == INFR_NO_TENSOR ? nullptr : (const int32_t*)ptr[m.expert_ids];
                rp.ep_lo = m.has_ep_band ? (int)m.ep_base : 0;
                rp.ep_n = m.has_ep_band ? (int)m.ep_n_local : 0;
                const uint32_t n_local = m.has_ep_band ? m.ep_n_local : m.n_expert;   // experts the weight tensors hold
                rp.ids = sc.ids; rp.weights = sc.weights; rp.probs = sc.probs;
                infr::MoeGemvParams gp{};
                gp.ids = sc.ids; gp.weights = sc.weights;
                gp.gate_dt = plan->tensors[m.gate_exps].dtype;
                gp.down_dt = plan->tensors[m.down_exps].dtype;
                size_t gbytes = tensor_bytes(plan->tensors[m.gate_exps], plan->numel[m.gate_exps]);
                size_t dbytes = tensor_bytes(plan->tensors[m.down_exps], plan->numel[m.down_exps]);
                gp.gate = (const uint8_t*)ptr[m.gate_exps];
                gp.gate_stride = gbytes / n_local;  // reference: gst = gb.len() / n_expert (lib.rs:3666)
                if (m.fused_gate_up) {
                    // gate rows first, up rows second inside each expert slice
                    gp.up = gp.gate + gp.gate_stride / 2;
                    gp.up_stride = gp.gate_stride;
                    gp.up_dt = gp.gate_dt;
                } else {
                    size_t ubytes = tensor_bytes(plan->tensors[m.up_exps], plan->numel[m.up_exps]);
                    gp.up = (const uint8_t*)ptr[m.up_exps];
                    gp.up_stride = ubytes / n_local;
                    gp.up_dt = plan->tensors[m.up_exps].dtype;
                }
                gp.down = (const uint8_t*)ptr[m.down_exps];
                gp.down_stride = dbytes / n_local;
                gp.down_scale = m.down_scale == INFR_NO_TENSOR ? nullptr : (const float*)ptr[m.down_scale];
                gp.rows = rows; gp.ne = (int)m.ne; gp.nff = (int)m.n_ff_exp; gp.n_used = (int)m.n_used; gp.n_expert = (int)n_local;
                gp.act = m.act; gp.has_clamp = (int)m.has_swiglu_clamp; gp.clamp = m.swiglu_clamp;
                gp.weight_before = (int)m.weight_before; gp.fused_gate_up = (int)m.fused_gate_up;
                gp.skip_zero_w = (int)m.has_ep_band;
                gp.h = sc.h; gp.dst = (float*)ptr[m.dst]; gp.n_cu = n_cu;
                gp.x = (const float*)ptr[m.x];
                if (fz.res) {
                    const infr_op_add& ad = plan->ops[fz.res - 1].u.add;
                    const uint32_t sum_t = fz.kind != infr_hip_plan::kMoeShared ? m.dst
                                           : fz.gated ? plan->ops[fz.b + 1].u.moe_shared_expert_add.dst
                                                      : plan->ops[fz.b + 1].u.add.dst;
                    const uint32_t other = ad.a == sum_t ? ad.b : ad.a;
                    if (!(need(other, "Add.a") && need(ad.dst, "Add.dst"))) return INFR_ERR_BACKEND;
                    gp.addend = (const float*)ptr[other];
                    gp.dst = (float*)ptr[ad.dst];
                }
                if (fz.kind == infr_hip_plan::kMoeShared && !sc.batched && !sc.bucketed) {
                    const infr_hip_plan::FuseOp fg = plan->fuse_head[fz.a];
                    const infr_op_linear& lu = plan->ops[fg.a].u.linear;
                    const infr_op_linear& lg = plan->ops[fg.a == fz.a ? fz.a + 1 : fz.a].u.linear;
                    const infr_op_linear& ld = plan->ops[fz.b].u.linear;
                    const uint32_t sum_dst = fz.gated ? plan->ops[fz.b + 1].u.moe_shared_expert_add.dst : plan->ops[fz.b + 1].u.add.dst;
                    if (!(need(lg.weight, "Linear.weight") && need(lu.weight, "Linear.weight") &&
                          need(ld.weight, "Linear.weight") && (fz.res || need(sum_dst, "Add.dst"))))
                        return INFR_ERR_BACKEND;
                    gp.sh_gate = (const uint8_t*)ptr[lg.weight];
                    gp.sh_up = (const uint8_t*)ptr[lu.weight];
                    gp.sh_down = (const uint8_t*)ptr[ld.weight];
                    if (!fz.res) gp.dst = (float*)ptr[sum_dst];
                    if (fz.gated) {
                        // the row's gate logit (a Linear with one output row) is launched ahead of the kernel that weighs
                        // with it, but behind whatever produces the row it reads (an RmsNorm folded into the logits kernel)
                        const infr_op_linear& lq = plan->ops[oi + 1].u.linear;
                        if (!(need(lq.x, "Linear.x") && need(lq.weight, "Linear.weight") && need(lq.dst, "Linear.dst")))
                            return INFR_ERR_BACKEND;
                        gp.sh_logit = (const float*)ptr[lq.dst];
                    }
                }
                auto launch_gate_logit = [&]() {
                    if (!gp.sh_logit) return;
                    const infr_op_linear& lq = plan->ops[oi + 1].u.linear;
                    int we = 1, wb = 4;
                    geometry(plan->tensors[lq.weight].dtype, &we, &wb);
                    const size_t rb = (size_t)(lq.in_f / we) * wb;
                    Timed t(be, "linear");
                    infr::launch_linear(s, (const float*)ptr[lq.x], (const uint8_t*)ptr[lq.weight] + (size_t)(lq.w_off / lq.in_f) * rb,
                                        plan->tensors[lq.weight].dtype, rb, (int)lq.m, (int)lq.in_f, (int)lq.out_f,
                                        (float*)ptr[lq.dst], n_cu);
                };
                bool single = sc.single_launch != 0;
                if (single && sc.single_launch == 1 && be->inorder_off.load(std::memory_order_relaxed)) single = false;
                if (single) {
                    const int off = be->single_launch_off.load(std::memory_order_relaxed);
                    if (off > 0) {
                        if (off != INT_MAX) be->single_launch_off.fetch_sub(1, std::memory_order_relaxed);
                        single = false;
                    }
                }
                if (single) {
                    infr::MoeLayerParams lp{};
                    lp.g = gp;
                    lp.g.route = rp;
                    lp.router = (const float*)ptr[m.router];
                    lp.router_row_floats = router_row_bytes / 4;
                    lp.router_x = (const float*)ptr[m.router_x];
                    lp.logits_out = sc.logits;
                    lp.fault = be->fault_dev;
                    lp.spin_limit = be->cfg.single_launch_spin_limit ? (int)be->cfg.single_launch_spin_limit - 1 : 1 << 15;
                    if (sc.single_launch == 2 && plan->stream_ws) {
                        char* ws = plan->stream_ws;
                        lp.cnt = (uint32_t*)ws;
                        lp.xa = (uint64_t*)(ws + 1024);
                        const size_t nr = (size_t)rows;   // every region holds one part per token row
                        lp.xl = lp.xa + nr * 8 * m.n_expert;
                        lp.xh = lp.xl + nr * 8 * m.n_expert;
                        lp.xs = lp.xh + nr * 8 * m.n_ff_exp;
                        lp.ypart = lp.xs + nr * m.n_ff_exp;
                        lp.late = be->fault_dev + 1;
                        lp.logits_once = moe_logits_once(be, m);
                        lp.guess_skew = (int)std::min<uint32_t>(be->cfg.single_launch_guess_skew, 8u);
                        bool norm_ok = true;
                        if (fz.norm) {   // the token row's RmsNorm, folded: the kernel normalises the raw row
                            const infr_op_rms_norm& nr = plan->ops[fz.norm - 1].u.rms_norm;
                            if (!(need(nr.x, "RmsNorm.x") && need(nr.weight, "RmsNorm.weight") && need(nr.dst, "RmsNorm.dst")))
                                return INFR_ERR_BACKEND;
                            lp.norm_x = (const float*)ptr[nr.x];
                            lp.norm_w = (const float*)ptr[nr.weight];
                            lp.norm_out = (float*)ptr[nr.dst];
                            lp.norm_eps = nr.eps;
                            lp.norm_for_x = m.x == nr.dst ? 1 : 0;
                            norm_ok = nr.x != nr.dst && m.x == nr.dst && rows == 1 && (((uintptr_t)lp.norm_x | (uintptr_t)lp.norm_w | (uintptr_t)lp.norm_out) & 15) == 0;
                        }
                        if (norm_ok && infr::moe_layer_stream_supported(lp) &&
                            (((uintptr_t)lp.router | (uintptr_t)lp.router_x | (uintptr_t)gp.x) & 15) == 0 && (lp.router_row_floats & 3) == 0) {
                            launch_gate_logit();   // (a gated always-on expert keeps its norm as an op: the row this reads is there)
                            Timed t(be, gp.sh_gate ? "moe_layer_shared" : "moe_layer");
                            if (infr::launch_moe_layer_stream(s, lp)) break;
                            return fail(INFR_ERR_BACKEND, "MoeFfn: the single-launch kernel refused a shape it had accepted");
                        }
                    } else if (sc.single_launch == 1 && plan->layer_ws) {
                        char* ws = plan->layer_ws;
                        lp.seq = (uint32_t*)ws;
                        lp.cnt = (uint32_t*)(ws + 16);
                        lp.xl = (uint64_t*)(ws + 256);
                        lp.xh = lp.xl + (size_t)8 * m.n_expert;
                        lp.ypart = lp.xh + (size_t)8 * m.n_ff_exp;
                        // asked first, so that no timing events are queued for a launch that does not happen
                        if ((((uintptr_t)lp.router | (uintptr_t)lp.router_x | (uintptr_t)gp.x) & 15) == 0 && (lp.router_row_floats & 3) == 0) {
                            Timed t(be, "moe_layer_inorder");
                            if (infr::launch_moe_layer_fused(s, lp)) break;
                            return fail(INFR_ERR_BACKEND, "MoeFfn: the single-launch kernel refused a shape it had accepted");
                        }
                    }
                }
                bool normed = false;
                if (fz.norm) {
                    const infr_op_rms_norm& nr = plan->ops[fz.norm - 1].u.rms_norm;
                    if (!(need(nr.x, "RmsNorm.x") && need(nr.weight, "RmsNorm.weight") && need(nr.dst, "RmsNorm.dst")))
                        return INFR_ERR_BACKEND;
                    infr::RouterNorm rn;
                    rn.weight = (const float*)ptr[nr.weight]; rn.eps = nr.eps; rn.xn_out = (float*)ptr[nr.dst];
                    {
                        Timed t(be, "rms_norm_router_logits");
                        normed = infr::launch_router_logits(s, (const uint8_t*)ptr[m.router], plan->tensors[m.router].dtype,
                                                            router_row_bytes, (const float*)ptr[nr.x], (int)m.ne,
                                                            (int)m.n_expert, rows, sc.logits, &rn);
                    }
                    if (!normed) {   // operands the fold cannot take (alignment): the op on its own
                        Timed t(be, "rms_norm");
                        infr::launch_rms_norm(s, (const float*)ptr[nr.x], rn.weight, rn.xn_out, 1, (int)nr.dim, nr.eps, 0);
                    }
                }
                if (!normed) {
                    Timed t(be, "router_logits");
                    if (!infr::launch_router_logits(s, (const uint8_t*)ptr[m.router], plan->tensors[m.router].dtype,
                                                    router_row_bytes, (const float*)ptr[m.router_x], (int)m.ne,
                                                    (int)m.n_expert, rows, sc.logits))
                        return fail(INFR_ERR_UNSUPPORTED, "MoeFfn: ne=%u does not fit the router kernel's LDS budget", m.ne);
                }
                if (sc.batched) {
                    const int pairs = rows * (int)m.n_used;
                    // the unit-decoder GEMM reads activations in natural k order, which is Q8_0's
                    const int a_dt_gu = sc.units_mfma ? INFR_Q8_0 : gp.gate_dt, a_dt_dn = sc.units_mfma ? INFR_Q8_0 : gp.down_dt;
                    {   // routing, and in the same launch the token rows as f16 for the gate/up GEMM
                        Timed t(be, "route_topk");
                        infr::launch_route_rows_to_f16(s, rp, a_dt_gu, gp.x, (int)m.ne, sc.xh, sc.xs);
                    }
                    {
                        Timed t(be, "moe_bucket");
                        const int32_t* bucket_ids = sc.ids;
                        if (m.has_ep_band) {   // pairs of foreign experts (weight 0) are not bucketed at all
                            infr::launch_mask_dropped_pairs(s, sc.ids, sc.weights, pairs, sc.live_ids);
                            bucket_ids = sc.live_ids;
                        }
                        infr::launch_bucket(s, bucket_ids, pairs, (int)n_local, sc.offsets, sc.pair_src, sc.slot_pair);
                    }
                    infr::GroupedParams q{};
                    q.loads_only = be->probe_grouped_loads_only.load() ? 1 : 0;
                    q.a = sc.xh; q.a_scale = sc.xs; q.offsets = sc.offsets; q.pair_src = sc.pair_src;
                    q.w0 = gp.gate; q.w0_stride = gp.gate_stride; q.w1 = gp.up; q.w1_stride = gp.up_stride;
                    q.route_w = sc.weights; q.down_scale = nullptr; q.out = sc.h;
                    q.K = (int)m.ne; q.N = (int)m.n_ff_exp; q.n_expert = (int)n_local; q.n_used = (int)m.n_used;
                    q.n_pairs = pairs; q.act = m.act; q.has_clamp = (int)m.has_swiglu_clamp; q.clamp = m.swiglu_clamp;
                    q.weight_before = (int)m.weight_before;
                    {
                        Timed t(be, sc.units_mfma ? "moe_grouped_units_gate_up" : "moe_grouped_gate_up");
                        if (sc.units_mfma) infr::launch_grouped_units_gate_up(s, gp.gate_dt, q);
                        else infr::launch_grouped_gate_up(s, gp.gate_dt, q);
                    }
                    {
                        Timed t(be, "rows_to_f16");
                        infr::launch_rows_to_f16(s, a_dt_dn, sc.h, pairs, (int)m.n_ff_exp, sc.hh, sc.hs);
                    }
                    q.a = sc.hh; q.a_scale = sc.hs; q.w0 = gp.down; q.w0_stride = gp.down_stride; q.w1 = nullptr; q.w1_stride = 0;
                    q.down_scale = gp.down_scale; q.out = sc.y; q.K = (int)m.n_ff_exp; q.N = (int)m.ne;
                    q.out_f16 = 1;   // y is written and read once: f16 halves that traffic, hs restores the scale
                    {
                        Timed t(be, sc.units_mfma ? "moe_grouped_units_down" : "moe_grouped_down");
                        if (sc.units_mfma) infr::launch_grouped_units_down(s, gp.down_dt, q);
                        else infr::launch_grouped_down(s, gp.down_dt, q);
                    }
                    {
                        Timed t(be, "moe_unbucket_combine");
                        infr::launch_unbucket_combine(s, sc.y, sc.slot_pair, sc.weights, rows, (int)m.ne, (int)m.n_used,
                                                      (int)m.weight_before, gp.dst, 0, sc.hs, gp.addend);
                    }
                    break;
                }
                if (sc.bucketed) {
                    const int pairs = rows * (int)m.n_used;
                    {
                        Timed t(be, "route_topk");
                        infr::launch_route(s, rp);
                    }
                    {
                        Timed t(be, "moe_bucket");
                        const int32_t* bucket_ids = sc.ids;
                        if (m.has_ep_band) {   // pairs of foreign experts (weight 0) are not bucketed at all
                            infr::launch_mask_dropped_pairs(s, sc.ids, sc.weights, pairs, sc.live_ids);
                            bucket_ids = sc.live_ids;
                        }
                        infr::launch_bucket(s, bucket_ids, pairs, (int)n_local, sc.offsets, sc.pair_src, sc.slot_pair);
                    }
                    gp.bk_offsets = sc.offsets; gp.bk_pair_src = sc.pair_src; gp.y = sc.y;
                    gp.max_bucket = m.expert_ids == INFR_NO_TENSOR ? rows : pairs;   // given ids may repeat an expert in a row
                    if (sc.units_batch) {
                        if ((((uintptr_t)gp.x | (uintptr_t)gp.h | (uintptr_t)gp.y) & 15) != 0)
                            return fail(INFR_ERR_BACKEND, "MoeFfn: activation rows must be 16-byte aligned");
                        {
                            Timed t(be, "moe_gate_up_units_bucketed");
                            infr::launch_moe_gate_up_units_bucketed(s, gp);
                        }
                        {
                            Timed t(be, "moe_down_units_bucketed");
                            infr::launch_moe_down_units_bucketed(s, gp);
                        }
                        Timed t(be, "moe_unbucket_combine");
                        infr::launch_unbucket_combine(s, sc.y, sc.slot_pair, sc.weights, rows, (int)m.ne, (int)m.n_used,
                                                      (int)m.weight_before, gp.dst, 0, nullptr, gp.addend);
                        break;
                    }
                    {
                        Timed t(be, "moe_gate_up_bucketed");
                        infr::launch_moe_gate_up_bucketed(s, gp);
                    }
                    gp.x = sc.h;
                    if (infr::moe_down_is_fast(gp)) {
                        // h is in flat (row, rank) order, which is what the per-token down kernel reads: it
                        // streams each pair's expert rows and combines in its epilogue, measured faster
                        // than the bucketed down kernel + combine up to the batched threshold
                        gp.x = nullptr;
                        Timed t(be, "moe_down_combine");
                        infr::launch_moe_down_combine(s, gp);
                        break;
                    }
                    {
                        Timed t(be, "moe_down_bucketed");
                        infr::MoeGemvParams gd = gp;
                        gd.addend = nullptr;   // the kernel writes per-pair rows; the addend joins the combined sum
                        infr::launch_moe_down_bucketed(s, gd);
                    }
                    {
                        Timed t(be, "moe_unbucket_combine");
                        infr::launch_unbucket_combine(s, sc.y, sc.slot_pair, sc.weights, rows, (int)m.ne, (int)m.n_used,
                                                      (int)m.weight_before, gp.dst, 1, nullptr, gp.addend);
                    }
                    break;
                }
                gp.route = rp;
                gp.y = sc.y;
                launch_gate_logit();
                moe_per_token(be, s, gp, rp, rows, m.n_expert, true);
                break;
            }
            case INFR_OP_LINEAR: {
                const infr_op_linear& l = op.u.linear;
                if (!(need(l.x, "Linear.x") && need(l.weight, "Linear.weight") && need(l.dst, "Linear.dst"))) return INFR_ERR_BACKEND;
                if (l.m == 0) break;
                int we = 1, wb = 4;
                geometry(plan->tensors[l.weight].dtype, &we, &wb);
                size_t row_bytes = (size_t)(l.in_f / we) * wb;
                const uint8_t* w = (const uint8_t*)ptr[l.weight] + (size_t)(l.w_off / l.in_f) * row_bytes;
                if (plan->lin[oi].mode) {
                    const int dt = plan->tensors[l.weight].dtype, mode = plan->lin[oi].mode;
                    _Float16* xh = plan->lin_xh;
                    float* xs = (float*)((char*)xh + round_up((size_t)l.m * l.in_f * 2, 256));
                    {
                        Timed t(be, "rows_to_f16");
                        // the unit-decoder GEMM reads activations in natural k order, which is Q8_0's
                        infr::launch_rows_to_f16(s, mode == 2 ? INFR_Q8_0 : dt, (const float*)ptr[l.x], (int)l.m, (int)l.in_f, xh, xs);
                    }
                    infr::GroupedParams q{};
                    q.loads_only = be->probe_grouped_loads_only.load() ? 1 : 0;
                    q.a = xh; q.a_scale = xs;
                    q.offsets = (const int32_t*)((const char*)plan->arena + plan->lin[oi].offsets_off);
                    q.w0 = w; q.w0_stride = 0;
                    q.out = (float*)ptr[l.dst];
                    q.K = (int)l.in_f; q.N = (int)l.out_f; q.n_expert = 1; q.n_used = 1; q.n_pairs = (int)l.m;
                    Timed t(be, mode == 2 ? "linear_grouped_units" : "linear_grouped");
                    if (mode == 2) infr::launch_grouped_units_down(s, dt, q);
                    else infr::launch_grouped_down(s, dt, q);
                    break;
                }
                Timed t(be, "linear");
                infr::launch_linear(s, (const float*)ptr[l.x], w, plan->tensors[l.weight].dtype, row_bytes, (int)l.m,
                                    (int)l.in_f, (int)l.out_f, (float*)ptr[l.dst], n_cu);
                break;
            }
            case INFR_OP_GATED_ACT: {
                const infr_op_gated_act& a = op.u.gated_act;
                if (!(need(a.gate, "GatedAct.gate") && need(a.up, "GatedAct.up") && need(a.dst, "GatedAct.dst"))) return INFR_ERR_BACKEND;
                Timed t(be, "gated_act");
                infr::launch_gated_act(s, (const float*)ptr[a.gate], (const float*)ptr[a.up], (float*)ptr[a.dst], (int)a.rows,
                                       (int)a.nff, a.act, (int)a.up_off, (int)a.up_stride, (int)a.gate_stride,
                                       (int)a.gate_block_width, (int)a.has_swiglu_clamp, a.swiglu_clamp);
                break;
            }
            case INFR_OP_ADD: {
                const infr_op_add& a = op.u.add;
                if (!(need(a.a, "Add.a") && need(a.b, "Add.b") && need(a.dst, "Add.dst"))) return INFR_ERR_BACKEND;
                Timed t(be, "add");
                infr::launch_add(s, (const float*)ptr[a.a], (const float*)ptr[a.b], (float*)ptr[a.dst], a.n);
                break;
            }
            case INFR_OP_MOE_SHARED_EXPERT_ADD: {
                const infr_op_moe_shared_expert_add& a = op.u.moe_shared_expert_add;
                if (!(need(a.moe, "MoeSharedExpertAdd.moe") && need(a.shexp, "MoeSharedExpertAdd.shexp") &&
                      need(a.gate, "MoeSharedExpertAdd.gate") && need(a.dst, "MoeSharedExpertAdd.dst")))
                    return INFR_ERR_BACKEND;
                Timed t(be, "moe_shared_expert_add");
                infr::launch_moe_shared_expert_add(s, (const float*)ptr[a.moe], (const float*)ptr[a.shexp],
                                                   (const float*)ptr[a.gate], (float*)ptr[a.dst], (int)a.rows, (int)a.n);
                break;
            }
            case INFR_OP_RMS_NORM:
            case INFR_OP_RMS_NORM_ADD: {
                const infr_op_rms_norm& nr = op.u.rms_norm;
                if (!(need(nr.x, "RmsNorm.x") && need(nr.weight, "RmsNorm.weight") && need(nr.dst, "RmsNorm.dst")))
                    return INFR_ERR_BACKEND;
                Timed t(be, "rms_norm");
                infr::launch_rms_norm(s, (const float*)ptr[nr.x], (const float*)ptr[nr.weight], (float*)ptr[nr.dst],
                                      (int)nr.rows, (int)nr.dim, nr.eps, op.kind == INFR_OP_RMS_NORM_ADD);
                break;
            }
            case INFR_OP_COPY:
            case INFR_OP_COPY_STRIDED: {
                const infr_op_copy& cp = op.u.copy;
                if (!(need(cp.src, "Copy.src") && need(cp.dst, "Copy.dst"))) return INFR_ERR_BACKEND;
                const uint32_t rows = op.kind == INFR_OP_COPY ? 1 : cp.rows;
                const int dt = plan->tensors[cp.src].dtype;
                const int eb = (dt == INFR_F16 || dt == INFR_BF16) ? 2 : 4;
                const char* src = (const char*)ptr[cp.src] + (size_t)cp.src_off * eb;
                char* dst = (char*)ptr[cp.dst] + (size_t)cp.dst_off * eb;
                Timed t(be, "copy");
                if (cp.src == cp.dst && rows && cp.n) {
                    char* tmp = (char*)plan->arena + plan->copy_tmp[oi];
                    infr::launch_copy_rows(s, src, tmp, rows, cp.n, cp.src_stride, cp.n, eb);
                    infr::launch_copy_rows(s, tmp, dst, rows, cp.n, cp.n, cp.dst_stride, eb);
                } else {
                    infr::launch_copy_rows(s, src, dst, rows, cp.n, cp.src_stride, cp.dst_stride, eb);
                }
                break;
            }
            default:
                return fail(INFR_ERR_UNSUPPORTED, "execute: op kind %d", op.kind);
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(INFR_ERR_BACKEND, "execute: kernel launch failed: %s", hipGetErrorString(e));
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_execute"); }

// ============================================================================ entry point without allocation
extern "C" infr_status infr_hip_moe_ffn_static(infr_hip_backend* be, const infr_hip_moe_ffn_static_args* a) try {
    if (!ok_backend(be) || !a) return fail(INFR_ERR_INVALID, "moe_ffn_static: bad handle");
    if (!be->static_scratch) return fail(INFR_ERR_BACKEND, "moe_ffn_static: device %d has no static scratch", be->device);
    const infr_hip_buffer* bufs[6] = {a->x, a->router, a->gate_exps, a->up_exps, a->down_exps, a->dst};
    static const char* const names[6] = {"x", "router", "gate_exps", "up_exps", "down_exps", "dst"};
    for (int i = 0; i < 6; i++) {
        if (!ok_buffer(bufs[i])) return fail(INFR_ERR_INVALID, "moe_ffn_static: %s is not a buffer", names[i]);
        if (bufs[i]->be != be) return fail(INFR_ERR_INVALID, "moe_ffn_static: %s belongs to another backend", names[i]);
    }
    if (a->rows == 0) return INFR_OK;
    if (a->ne == 0 || a->n_expert == 0 || a->n_used == 0 || a->n_ff_exp == 0 || a->n_used > a->n_expert)
        return fail(INFR_ERR_INVALID, "moe_ffn_static: ne/n_expert/n_used/n_ff_exp must be positive and n_used <= n_expert");
    if (a->rows >= kBucketedMinRows || a->n_expert > 2048 || a->n_used > 64)
        return fail(INFR_ERR_UNSUPPORTED, "moe_ffn_static: %u token rows / %u experts / top-%u: the entry point takes 1..%u rows, "
                    "up to 2048 experts, top-64", a->rows, a->n_expert, a->n_used, kBucketedMinRows - 1);
    // scratch layout: logits, probs [rows, n_expert]; ids, weights [rows, n_used]; h [rows, n_used, n_ff_exp]; y [rows, n_used, ne]
    const size_t pairs = (size_t)a->rows * a->n_used;
    const size_t sz_l = round_up((size_t)a->rows * a->n_expert * 4, 256), sz_p = round_up(pairs * 4, 256);
    const size_t sz_h = round_up(pairs * a->n_ff_exp * 4, 256), sz_y = round_up(pairs * a->ne * 4, 256);
    const size_t need = 2 * sz_l + 2 * sz_p + sz_h + sz_y;
    if (need > INFR_HIP_STATIC_SCRATCH_BYTES)
        return fail(INFR_ERR_UNSUPPORTED, "moe_ffn_static: these shapes need %zu bytes of scratch, the static scratch holds %u",
                    need, (unsigned)INFR_HIP_STATIC_SCRATCH_BYTES);
    // operand extents against the shapes
    const int dts[3] = {a->gate_dtype, a->up_dtype, a->down_dtype};
    const uint32_t kdims[3] = {a->ne, a->ne, a->n_ff_exp};
    size_t wbytes[3];
    for (int i = 0; i < 3; i++) {
        int el = 1, by = 4;
        if (!geometry(dts[i], &el, &by) || dts[i] == INFR_I32 || dts[i] == INFR_U32)
            return fail(INFR_ERR_UNSUPPORTED, "moe_ffn_static: %s has no decodable weight dtype (%d)", names[2 + i], dts[i]);
        if (kdims[i] % (uint32_t)el != 0)
            return fail(INFR_ERR_INVALID, "moe_ffn_static: %s rows of %u elements are not whole %s blocks", names[2 + i], kdims[i], dtype_name(dts[i]));
        wbytes[i] = (size_t)a->n_expert * a->n_ff_exp * a->ne / (size_t)el * (size_t)by;
        if (bufs[2 + i]->len < wbytes[i])
            return fail(INFR_ERR_INVALID, "moe_ffn_static: %s holds %zu bytes, the shapes need %zu", names[2 + i], bufs[2 + i]->len, wbytes[i]);
    }
    const size_t act_bytes = (size_t)a->rows * a->ne * 4, router_bytes = (size_t)a->n_expert * a->ne * 4;
    if (a->x->len < act_bytes || a->dst->len < act_bytes || a->router->len < router_bytes)
        return fail(INFR_ERR_INVALID, "moe_ffn_static: x / dst / router hold fewer bytes than [rows, ne] / [n_expert, ne] f32");
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    char* sp = static_cast<char*>(be->static_scratch);   // the device address, never the array's name
    float* logits = reinterpret_cast<float*>(sp);
    float* probs = reinterpret_cast<float*>(sp + sz_l);
    int32_t* ids = reinterpret_cast<int32_t*>(sp + 2 * sz_l);
    float* weights = reinterpret_cast<float*>(sp + 2 * sz_l + sz_p);
    float* h = reinterpret_cast<float*>(sp + 2 * sz_l + 2 * sz_p);
    float* y = reinterpret_cast<float*>(sp + 2 * sz_l + 2 * sz_p + sz_h);
    hipStream_t s = be->stream;
    const int rows = (int)a->rows;
    if (!infr::launch_router_logits(s, (const uint8_t*)a->router->dptr, INFR_F32, (size_t)a->ne * 4, (const float*)a->x->dptr,
                                    (int)a->ne, (int)a->n_expert, rows, logits))
        return fail(INFR_ERR_UNSUPPORTED, "moe_ffn_static: ne=%u does not fit the router kernel's LDS budget", a->ne);
    infr::RouteParams rp{};
    rp.logits = logits; rp.n_expert = (int)a->n_expert; rp.n_used = (int)a->n_used; rp.rows = rows;
    rp.gating = INFR_GATING_SOFTMAX; rp.norm_w = 1; rp.scale = 1.0f;
    rp.ids = ids; rp.weights = weights; rp.probs = probs;
    infr::MoeGemvParams gp{};
    gp.ids = ids; gp.weights = weights;
    gp.gate_dt = a->gate_dtype; gp.up_dt = a->up_dtype; gp.down_dt = a->down_dtype;
    gp.gate = (const uint8_t*)a->gate_exps->dptr; gp.gate_stride = wbytes[0] / a->n_expert;
    gp.up = (const uint8_t*)a->up_exps->dptr; gp.up_stride = wbytes[1] / a->n_expert;
    gp.down = (const uint8_t*)a->down_exps->dptr; gp.down_stride = wbytes[2] / a->n_expert;
    gp.rows = rows; gp.ne = (int)a->ne; gp.nff = (int)a->n_ff_exp; gp.n_used = (int)a->n_used; gp.n_expert = (int)a->n_expert;
    gp.act = INFR_ACT_SILU;
    gp.h = h; gp.y = y; gp.dst = (float*)a->dst->dptr; gp.x = (const float*)a->x->dptr;
    gp.n_cu = be->prop.multiProcessorCount;
    gp.route = rp;
    moe_per_token(be, s, gp, rp, rows, a->n_expert, false);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(INFR_ERR_BACKEND, "moe_ffn_static: kernel launch failed: %s", hipGetErrorString(e));
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_moe_ffn_static"); }

// ============================================================================ measurement aid
extern "C" infr_status infr_hip_probe_dependent_reads(infr_hip_backend* be, const infr_hip_buffer* pool,
                                                      const uint64_t* stage_bytes, uint32_t n_stages, uint32_t iters,
                                                      double* us_per_stage, double* us_per_chain) try {
    if (check_owned(be, pool, "probe") != INFR_OK) return INFR_ERR_INVALID;
    if (!stage_bytes || n_stages == 0 || n_stages > 16 || iters == 0 || iters > 100000)
        return fail(INFR_ERR_INVALID, "probe: 1..16 stages and 1..100000 iterations");
    for (uint32_t i = 0; i < n_stages; i++)
        if (stage_bytes[i] < 1024 || stage_bytes[i] * 4 > pool->len)
            return fail(INFR_ERR_INVALID, "probe: stage %u of %llu bytes needs 1 KB .. a quarter of the pool (%zu bytes)", i,
                        (unsigned long long)stage_bytes[i], pool->len);
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    uint32_t* ctl = nullptr;
    g_alloc_calls += 3;
    HIP_TRY(hipMalloc(&ctl, 256));
    hipEvent_t a = nullptr, b = nullptr;
    hipError_t e = hipEventCreate(&a);
    if (e == hipSuccess) e = hipEventCreate(&b);
    hipStream_t s = be->stream;
    const int n_cu = be->prop.multiProcessorCount;
    infr::launch_fill_zero(s, ctl, 256);
    uint32_t salt = 1;
    auto timed = [&](uint32_t first, uint32_t count, double* out) {
        for (uint32_t w = 0; w < 3 && e == hipSuccess; w++)   // warm-up
            for (uint32_t k = first; k < first + count; k++)
                infr::launch_probe_dependent_read(s, (const uint8_t*)pool->dptr, pool->len, stage_bytes[k], ctl, salt++, n_cu);
        if (e == hipSuccess) e = hipEventRecord(a, s);
        for (uint32_t it = 0; it < iters && e == hipSuccess; it++)
            for (uint32_t k = first; k < first + count; k++)
                infr::launch_probe_dependent_read(s, (const uint8_t*)pool->dptr, pool->len, stage_bytes[k], ctl, salt++, n_cu);
        if (e == hipSuccess) e = hipEventRecord(b, s);
        if (e == hipSuccess) e = hipEventSynchronize(b);
        float ms = 0.0f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, a, b);
        if (out) *out = (double)ms * 1e3 / iters;
    };
    for (uint32_t k = 0; k < n_stages; k++) timed(k, 1, us_per_stage ? us_per_stage + k : nullptr);
    timed(0, n_stages, us_per_chain);
    if (e == hipSuccess) e = hipGetLastError();
    if (a) (void)hipEventDestroy(a);
    if (b) (void)hipEventDestroy(b);
    (void)hipStreamSynchronize(s);
    (void)hipFree(ctl);
    if (e != hipSuccess) return fail(INFR_ERR_BACKEND, "probe: %s", hipGetErrorString(e));
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_probe_dependent_reads"); }

// ============================================================================ taps
extern "C" infr_status infr_hip_probe_late_experts(infr_hip_backend* be, uint64_t* out) try {
    if (!ok_backend(be) || !out) return fail(INFR_ERR_INVALID, "probe: bad handle");
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    HIP_TRY(hipStreamSynchronize(be->stream));
    *out = be->fault_host ? ((volatile uint32_t*)be->fault_host)[1] : 0;
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_probe_late_experts"); }

extern "C" infr_status infr_hip_probe_alloc_calls(uint64_t* out) try {
    if (!out) return fail(INFR_ERR_INVALID, "probe: out is null");
    *out = g_alloc_calls.load();
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_probe_alloc_calls"); }

extern "C" infr_status infr_hip_probe_grouped_loads_only(infr_hip_backend* be, int on) try {
    if (!ok_backend(be)) return fail(INFR_ERR_INVALID, "probe: bad handle");
    be->probe_grouped_loads_only.store(on != 0);
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_probe_grouped_loads_only"); }

extern "C" infr_status infr_hip_prof_enable(infr_hip_backend* be, int on) try {
    if (!ok_backend(be)) return fail(INFR_ERR_INVALID, "prof: bad handle");
    std::lock_guard<std::mutex> lk(be->mu);
    be->prof_on.store(on ? 1 : 0);
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_prof_enable"); }

extern "C" infr_status infr_hip_prof_read(infr_hip_backend* be, infr_hip_prof_entry* out, uint32_t cap, uint32_t* n_out) try {
    if (!ok_backend(be) || !n_out) return fail(INFR_ERR_INVALID, "prof: bad handle");
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    drain_prof(be);
    uint32_t n = 0;
    for (auto& kv : be->prof) {
        if (out && n < cap) {
            memset(&out[n], 0, sizeof out[n]);
            snprintf(out[n].kernel, sizeof out[n].kernel, "%s", kv.first.c_str());
            out[n].launches = kv.second.launches;
            out[n].total_ms = kv.second.total_ms;
            out[n].min_ms = kv.second.min_ms;
            out[n].max_ms = kv.second.max_ms;
        }
        n++;
    }
    *n_out = n;
    if (out) be->prof.clear();
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_prof_read"); }

extern "C" infr_status infr_hip_plan_moe_routing(infr_hip_backend* be, const infr_hip_plan* plan, uint32_t op_index,
                                                 int32_t* ids, float* weights, float* logits, float* probs) try {
    if (!ok_backend(be) || !ok_plan(plan) || plan->be != be) return fail(INFR_ERR_INVALID, "moe_routing: bad handle");
    if (op_index >= plan->ops.size() || plan->ops[op_index].kind != INFR_OP_MOE_FFN)
        return fail(INFR_ERR_INVALID, "moe_routing: op %u is not a MoeFfn", op_index);
    const infr_op_moe_ffn& m = plan->ops[op_index].u.moe_ffn;
    const MoeScratch& sc = plan->moe[op_index];
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    HIP_TRY(hipStreamSynchronize(be->stream));
    if (infr_status st = check_fault(be)) return st;
    size_t rows = (size_t)sc.rows;
    if (rows == 0) return INFR_OK;
    if (ids) HIP_TRY(hipMemcpy(ids, sc.ids, rows * m.n_used * 4, hipMemcpyDeviceToHost));
    if (weights) HIP_TRY(hipMemcpy(weights, sc.weights, rows * m.n_used * 4, hipMemcpyDeviceToHost));
    if (logits) HIP_TRY(hipMemcpy(logits, sc.logits, rows * m.n_expert * 4, hipMemcpyDeviceToHost));
    if (probs) HIP_TRY(hipMemcpy(probs, sc.probs, rows * m.n_expert * 4, hipMemcpyDeviceToHost));
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_plan_moe_routing"); }

extern "C" infr_status infr_hip_plan_moe_bucketing(infr_hip_backend* be, const infr_hip_plan* plan, uint32_t op_index,
                                                   int32_t* offsets, int32_t* pair_src, int32_t* slot_pair) try {
    if (!ok_backend(be) || !ok_plan(plan) || plan->be != be) return fail(INFR_ERR_INVALID, "moe_bucketing: bad handle");
    if (op_index >= plan->ops.size() || plan->ops[op_index].kind != INFR_OP_MOE_FFN)
        return fail(INFR_ERR_INVALID, "moe_bucketing: op %u is not a MoeFfn", op_index);
    const infr_op_moe_ffn& m = plan->ops[op_index].u.moe_ffn;
    const MoeScratch& sc = plan->moe[op_index];
    if (!sc.batched && !sc.bucketed)
        return fail(INFR_ERR_INVALID, "moe_bucketing: op %u runs the per-token path (%d rows), which does not bucket", op_index, sc.rows);
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    HIP_TRY(hipStreamSynchronize(be->stream));
    if (infr_status st = check_fault(be)) return st;
    const size_t pairs = (size_t)sc.rows * m.n_used;
    if (offsets) HIP_TRY(hipMemcpy(offsets, sc.offsets, ((size_t)m.n_expert + 1) * 4, hipMemcpyDeviceToHost));
    if (pair_src) HIP_TRY(hipMemcpy(pair_src, sc.pair_src, pairs * 4, hipMemcpyDeviceToHost));
    if (slot_pair) HIP_TRY(hipMemcpy(slot_pair, sc.slot_pair, pairs * 4, hipMemcpyDeviceToHost));
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_plan_moe_bucketing"); }

extern "C" infr_status infr_hip_dequant(infr_hip_backend* be, const infr_hip_buffer* src, int32_t dtype, uint64_t numel,
                                        infr_hip_buffer* dst) try {
    if (infr_status st = check_owned(be, src, "dequant")) return st;
    if (infr_status st = check_owned(be, dst, "dequant")) return st;
    int e = 1, b = 4;
    if (!geometry(dtype, &e, &b)) return fail(INFR_ERR_UNSUPPORTED, "dequant: dtype %s has no decode on this backend", dtype_name(dtype));
    if (numel % (uint64_t)e != 0) return fail(INFR_ERR_INVALID, "dequant: %llu elements is not a whole number of blocks", (unsigned long long)numel);
    size_t need_src = (size_t)(numel / (uint64_t)e) * (size_t)b;
    if (src->len < need_src) return fail(INFR_ERR_BACKEND, "dequant: source holds %zu bytes, %zu needed", src->len, need_src);
    if (dst->len < numel * 4) return fail(INFR_ERR_BACKEND, "dequant: destination holds %zu bytes, %llu needed", dst->len, (unsigned long long)numel * 4);
    std::lock_guard<std::mutex> lk(be->mu);
    HIP_TRY(hipSetDevice(be->device));
    Timed t(be, "dequant");
    infr::launch_dequant(be->stream, (const uint8_t*)src->dptr, dtype, numel, (float*)dst->dptr);
    return INFR_OK;
} catch (...) { return guard_fail("infr_hip_dequant"); }
