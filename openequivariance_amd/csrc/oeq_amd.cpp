// liboeq_amd.so: host runtime behind the C ABI declared in include/oeq_amd.h.
//
// Compiles HIP source with hiprtc, loads the code object once per device, and
// enqueues the generated kernels on the caller's stream. The only device-side
// object of this translation unit is the scratch array of the allocation-free
// entry point (oeq_conv_forward_static). The kernel argument lists used here are the contract the Python
// code generator (openequivariance_amd/codegen) emits against.
#include "oeq_amd.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

namespace {

thread_local std::string g_error;

int fail(int code, const char* fmt, ...) {
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

#define HIP_TRY(expr)                                                                  \
    do {                                                                               \
        hipError_t e_ = (expr);                                                        \
        if (e_ != hipSuccess)                                                          \
            return fail(OEQ_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_));   \
    } while (0)

constexpr int kMaxDevices = 16;

// A role is one kernel, or several launched back to back with the same arguments and the same
// launch shape (descriptors naming the same role, in order); `names` lists them.
struct RoleInfo {
    bool present = false;
    std::vector<std::string> names;
    unsigned block = 0;
    unsigned units_per_block = 1;
    unsigned max_blocks = 0;
    unsigned grid_multiple = 0;
};

struct DeviceSlot {
    std::vector<hipModule_t> modules;  // one per code object of the set, empty until first use on the device
    std::vector<hipFunction_t> fn[OEQ_ROLE_COUNT];
};

// A kernel set's code is one code object or a pack of several (the kernels of a large set compiled side by
// side, every kernel in exactly one of them): the 8 bytes "OEQPACK1", a uint64 count, that many uint64 byte
// sizes, then the code objects in that order, each starting on the next multiple of 64 bytes from the start
// of the pack.
constexpr char kPackMagic[8] = {'O', 'E', 'Q', 'P', 'A', 'C', 'K', '1'};
struct CodePart {
    size_t offset, size;
};

struct TimedLaunch {
    int role;
    hipEvent_t start, stop;
};

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Entries of the long-segment list that oeq_group_scan leaves behind a cursor array (the kernels in
// codegen/common.py use the same number).
constexpr int64_t OEQ_LONG_LIST = 126;

}  // namespace

struct oeq_kernels {
    std::vector<char> code;
    std::vector<CodePart> parts;  // the code objects within `code`
    oeq_problem_dims dims{};
    RoleInfo roles[OEQ_ROLE_COUNT];
    std::mutex mu;
    DeviceSlot slots[kMaxDevices];
    std::atomic<bool> timing{false};
    std::vector<TimedLaunch> timed;

    // Resolve the function for `role` on the current device (loading the code
    // object there on first use).
    int functions(int role, const std::vector<hipFunction_t>** out) {
        if (role < 0 || role >= OEQ_ROLE_COUNT || !roles[role].present)
            return fail(OEQ_ERR_INVALID, "kernel role %d is not part of this kernel set", role);
        int dev = 0;
        HIP_TRY(hipGetDevice(&dev));
        if (dev < 0 || dev >= kMaxDevices) return fail(OEQ_ERR_INVALID, "device index %d out of range", dev);
        std::lock_guard<std::mutex> lock(mu);
        DeviceSlot& s = slots[dev];
        if (s.modules.empty()) {
            auto unload = [&s]() {
                for (hipModule_t m : s.modules) (void)hipModuleUnload(m);
                s.modules.clear();
            };
            for (const CodePart& part : parts) {
                hipModule_t m = nullptr;
                hipError_t e = hipModuleLoadData(&m, code.data() + part.offset);
                if (e != hipSuccess) {
                    unload();
                    return fail(OEQ_ERR_HIP, "hipModuleLoadData failed: %s", hipGetErrorString(e));
                }
                s.modules.push_back(m);
            }
            for (int r = 0; r < OEQ_ROLE_COUNT; ++r) {
                if (!roles[r].present) continue;
                s.fn[r].clear();
                for (const std::string& name : roles[r].names) {
                    hipFunction_t f = nullptr;
                    hipError_t e = hipErrorNotFound;
                    for (size_t m = 0; m < s.modules.size() && e != hipSuccess; ++m)
                        e = hipModuleGetFunction(&f, s.modules[m], name.c_str());
                    if (e != hipSuccess) {
                        unload();
                        return fail(OEQ_ERR_HIP, "kernel '%s' not found in code object: %s", name.c_str(),
                                    hipGetErrorString(e));
                    }
                    s.fn[r].push_back(f);
                }
            }
            (void)hipGetLastError();  // lookups that missed in the first code objects of a pack are no error
        }
        *out = &s.fn[role];
        return OEQ_OK;
    }

    unsigned grid_for(int role, int64_t units) const {
        const RoleInfo& r = roles[role];
        int64_t blocks = (units + r.units_per_block - 1) / r.units_per_block;
        if (blocks < 1) blocks = 1;
        if (r.max_blocks && blocks > (int64_t)r.max_blocks) blocks = r.max_blocks;
        if (r.grid_multiple > 1) blocks = (blocks + r.grid_multiple - 1) / r.grid_multiple * r.grid_multiple;
        if (blocks > 0x7fffffffLL) blocks = 0x7fffffffLL;
        return (unsigned)blocks;
    }

    // Set by the allocation-free entry point for the duration of its call (on its thread): launches then
    // create no timing events.
    static thread_local bool no_events;
    // Set by the same entry point: long edge segments are not cut into chunks (their rows would need scratch
    // that the static buffer does not have).
    static thread_local bool no_hubs;

    bool loaded_on_current_device() {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return false;
        std::lock_guard<std::mutex> lock(mu);
        return !slots[dev].modules.empty();
    }

    int launch(int role, int64_t units, void** args, void* stream) {
        const std::vector<hipFunction_t>* fns = nullptr;
        int rc = functions(role, &fns);
        if (rc) return rc;
        unsigned grid = grid_for(role, units);
        if (no_events || !timing.load(std::memory_order_relaxed)) {
            for (hipFunction_t fn : *fns)
                HIP_TRY(hipModuleLaunchKernel(fn, grid, 1, 1, roles[role].block, 1, 1, 0, (hipStream_t)stream, args,
                                              nullptr));
            return OEQ_OK;
        }
        // profiling mode: bracket the role's kernels with events on their own stream
        TimedLaunch t{role, nullptr, nullptr};
        HIP_TRY(hipEventCreate(&t.start));
        HIP_TRY(hipEventCreate(&t.stop));
        HIP_TRY(hipEventRecord(t.start, (hipStream_t)stream));
        for (hipFunction_t fn : *fns)
            HIP_TRY(hipModuleLaunchKernel(fn, grid, 1, 1, roles[role].block, 1, 1, 0, (hipStream_t)stream, args,
                                          nullptr));
        HIP_TRY(hipEventRecord(t.stop, (hipStream_t)stream));
        std::lock_guard<std::mutex> lock(mu);
        timed.push_back(t);
        return OEQ_OK;
    }

    int fill_zero(void* p, size_t bytes, void* stream) {
        if (bytes == 0) return OEQ_OK;
        int64_t n = (int64_t)bytes;
        void* args[] = {&p, &n};
        return launch(OEQ_ROLE_FILL_ZERO, (n + 15) / 16, args, stream);
    }

    int segment_ptr(int64_t n_items, int64_t n_segments, const int64_t* keys, const int64_t* perm, int64_t* ptr,
                    void* stream) {
        void* args[] = {&n_items, &n_segments, &keys, &perm, &ptr};
        return launch(OEQ_ROLE_SEGMENT_PTR, n_items + 1, args, stream);
    }

    // Counting sort of the item indices 0..n_items-1 by key: ptr[0..n_segments] = segment starts,
    // perm = item indices grouped by key, ascending within a group (so the result depends on the key
    // list only); cursor (n_segments + 1 entries and the long-segment list, see ptr_bytes_of) and unordered
    // (n_items) are scratch.
    int group_by_key(int64_t n_items, int64_t n_segments, const int64_t* keys, int64_t* ptr, int64_t* cursor,
                     int64_t* unordered, int64_t* perm, void* stream) {
        int rc = fill_zero(ptr, (size_t)(n_segments + 1) * sizeof(int64_t), stream);
        if (rc) return rc;
        void* cargs[] = {&n_items, &keys, &ptr, &n_segments};
        rc = launch(OEQ_ROLE_GROUP_COUNT, n_items, cargs, stream);
        if (rc) return rc;
        int64_t n = n_segments + 1;
        void* sargs[] = {&n, &ptr, &cursor};
        rc = launch(OEQ_ROLE_GROUP_SCAN, 1, sargs, stream);
        if (rc) return rc;
        void* pargs[] = {&n_items, &keys, &cursor, &unordered, &n_segments};
        rc = launch(OEQ_ROLE_GROUP_SCATTER, n_items, pargs, stream);
        if (rc) return rc;
        // the scan left the segments longer than a wave should rank by itself behind the cursor entries
        const int64_t* long_list = cursor + n_segments + 1;
        void* oargs[] = {&n_segments, &ptr, &unordered, &perm, &long_list, &n_items};
        // one wave per segment, and at least one thread per 16 items so that few nodes with many items
        // still bring a grid wide enough for the long segments
        return launch(OEQ_ROLE_GROUP_ORDER, std::max(n_segments, n_items / 64), oargs, stream);
    }
};

thread_local bool oeq_kernels::no_events = false;
thread_local bool oeq_kernels::no_hubs = false;

// ---------------------------------------------------------------------------
// scratch memory of the allocation-free entry point
// ---------------------------------------------------------------------------

// One copy per GPU, held until the process ends. In host code the array's name is only a handle for
// hipGetSymbolAddress: the address kernels and fills work on is resolved once per device (with that device
// current) and kept in g_scratch_ptr.
#define OEQ_STATIC_SCRATCH_BYTES (32u << 20)
static __device__ __align__(256) unsigned char scratch[OEQ_STATIC_SCRATCH_BYTES];

namespace {
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mu;

int static_scratch(void** out) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(OEQ_ERR_INVALID, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(OEQ_ERR_HIP, "hipGetSymbolAddress returned a NULL address for the scratch array");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return OEQ_OK;
}
}  // namespace

extern "C" {

const char* oeq_last_error(void) { return g_error.c_str(); }
int oeq_abi_version(void) { return 6; }

int oeq_get_device_props(int device, oeq_device_props* out) {
    if (!out) return fail(OEQ_ERR_INVALID, "oeq_get_device_props: out is NULL");
    hipDeviceProp_t p;
    HIP_TRY(hipGetDeviceProperties(&p, device));
    std::memset(out, 0, sizeof(*out));
    std::snprintf(out->name, sizeof(out->name), "%s", p.name);
    std::string arch = p.gcnArchName;
    size_t colon = arch.find(':');
    if (colon != std::string::npos) arch.resize(colon);
    std::snprintf(out->arch, sizeof(out->arch), "%s", arch.c_str());
    out->wave_size = p.warpSize;
    out->compute_units = p.multiProcessorCount;
    out->lds_per_block = (int32_t)p.sharedMemPerBlock;
    out->max_threads_per_block = p.maxThreadsPerBlock;
    out->clock_khz = p.clockRate;
    out->l2_bytes = p.l2CacheSize;
    out->total_mem = (int64_t)p.totalGlobalMem;
    return OEQ_OK;
}

void oeq_free(void* p) { std::free(p); }

int oeq_jit_compile(const char* source, const char* arch, const char* const* options, int n_options, void** code,
                    size_t* code_size) {
    if (!source || !arch || !code || !code_size) return fail(OEQ_ERR_INVALID, "oeq_jit_compile: NULL argument");
    *code = nullptr;
    *code_size = 0;
    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, source, "oeq_kernels.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS) return fail(OEQ_ERR_COMPILE, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
    std::vector<std::string> opts;
    opts.push_back(std::string("--offload-arch=") + arch);
    for (int i = 0; i < n_options; ++i) opts.emplace_back(options[i]);
    std::vector<const char*> copts;
    for (auto& o : opts) copts.push_back(o.c_str());
    r = hiprtcCompileProgram(prog, (int)copts.size(), copts.data());
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, '\0');
        if (n) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        g_error = std::string("hiprtc compile failed (") + hiprtcGetErrorString(r) + "):\n" + log;
        return OEQ_ERR_COMPILE;
    }
    size_t n = 0;
    r = hiprtcGetCodeSize(prog, &n);
    if (r != HIPRTC_SUCCESS || n == 0) {
        hiprtcDestroyProgram(&prog);
        return fail(OEQ_ERR_COMPILE, "hiprtcGetCodeSize: %s", hiprtcGetErrorString(r));
    }
    void* buf = std::malloc(n);
    if (!buf) {
        hiprtcDestroyProgram(&prog);
        return fail(OEQ_ERR_NOMEM, "out of host memory for %zu-byte code object", n);
    }
    r = hiprtcGetCode(prog, (char*)buf);
    hiprtcDestroyProgram(&prog);
    if (r != HIPRTC_SUCCESS) {
        std::free(buf);
        return fail(OEQ_ERR_COMPILE, "hiprtcGetCode: %s", hiprtcGetErrorString(r));
    }
    *code = buf;
    *code_size = n;
    return OEQ_OK;
}

int oeq_kernels_create(const void* code, size_t code_size, const oeq_problem_dims* dims, const oeq_kernel_desc* descs,
                       int n_descs, oeq_kernels** out) {
    if (!code || !code_size || !dims || !descs || n_descs <= 0 || !out)
        return fail(OEQ_ERR_INVALID, "oeq_kernels_create: NULL or empty argument");
    if (dims->elem_size != 4 && dims->elem_size != 8)
        return fail(OEQ_ERR_INVALID, "oeq_kernels_create: elem_size must be 4 or 8, got %d", dims->elem_size);
    if (dims->L1_dim <= 0 || dims->L2_dim <= 0 || dims->L3_dim <= 0 || dims->weight_numel <= 0)
        return fail(OEQ_ERR_INVALID, "oeq_kernels_create: non-positive problem dimension");
    oeq_kernels* k = new (std::nothrow) oeq_kernels();
    if (!k) return fail(OEQ_ERR_NOMEM, "oeq_kernels_create: out of memory");
    k->code.assign((const char*)code, (const char*)code + code_size);
    if (code_size >= 16 && !memcmp(code, kPackMagic, 8)) {
        uint64_t count = 0;
        memcpy(&count, (const char*)code + 8, 8);
        bool ok = count >= 1 && count <= (code_size - 16) / 8;
        size_t at = ok ? 16 + 8 * (size_t)count : 0;
        for (uint64_t i = 0; ok && i < count; ++i) {
            uint64_t size = 0;
            memcpy(&size, (const char*)code + 16 + 8 * i, 8);
            at = align_up(at, 64);
            ok = size > 0 && at <= code_size && size <= code_size - at;
            if (ok) k->parts.push_back({at, (size_t)size});
            at += (size_t)size;
        }
        if (!ok) {
            delete k;
            return fail(OEQ_ERR_INVALID, "oeq_kernels_create: malformed code pack");
        }
    } else {
        k->parts.push_back({0, code_size});
    }
    k->dims = *dims;
    for (int i = 0; i < n_descs; ++i) {
        const oeq_kernel_desc& d = descs[i];
        if (d.role < 0 || d.role >= OEQ_ROLE_COUNT || !d.kernel_name || d.block_threads == 0 ||
            d.block_threads > 1024 || d.units_per_block == 0) {
            delete k;
            return fail(OEQ_ERR_INVALID, "oeq_kernels_create: bad kernel descriptor %d", i);
        }
        RoleInfo& r = k->roles[d.role];
        r.present = true;
        r.names.emplace_back(d.kernel_name);
        r.block = d.block_threads;
        r.units_per_block = d.units_per_block;
        r.max_blocks = d.max_blocks;
        r.grid_multiple = d.grid_multiple;
    }
    *out = k;
    return OEQ_OK;
}

void oeq_kernels_destroy(oeq_kernels* k) {
    if (!k) return;
    for (auto& t : k->timed) {  // timings nobody collected
        (void)hipEventDestroy(t.start);
        (void)hipEventDestroy(t.stop);
    }
    for (auto& s : k->slots)
        for (hipModule_t m : s.modules) (void)hipModuleUnload(m);
    delete k;
}

size_t oeq_segment_sum_workspace_bytes(const oeq_kernels* k, int64_t n_segments) {
    (void)k;
    return align_up((size_t)(n_segments + 1) * sizeof(int64_t), 256);
}

int oeq_segment_sum(oeq_kernels* k, int64_t n_segments, int64_t n_items, int64_t row_len, const void* src, void* dst,
                    const int64_t* keys, const int64_t* perm, void* workspace, size_t workspace_bytes, void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_segment_sum: NULL kernel set");
    if (n_segments < 0 || n_items < 0 || row_len <= 0) return fail(OEQ_ERR_INVALID, "oeq_segment_sum: bad size");
    if (n_segments == 0) return OEQ_OK;
    if (!dst) return fail(OEQ_ERR_INVALID, "oeq_segment_sum: NULL dst");
    if (n_items == 0) return k->fill_zero(dst, (size_t)n_segments * row_len * k->dims.elem_size, stream);
    if (!src || !keys) return fail(OEQ_ERR_INVALID, "oeq_segment_sum: NULL buffer");
    size_t need = oeq_segment_sum_workspace_bytes(k, n_segments);
    if (!workspace || workspace_bytes < need)
        return fail(OEQ_ERR_INVALID, "oeq_segment_sum: workspace too small (%zu < %zu bytes)", workspace_bytes, need);
    int64_t* ptr = (int64_t*)workspace;
    int rc = k->segment_ptr(n_items, n_segments, keys, perm, ptr, stream);
    if (rc) return rc;
    void* args[] = {&n_segments, &n_items, &row_len, &src, &dst, &perm, &ptr};
    return k->launch(OEQ_ROLE_SEGMENT_SUM, n_segments, args, stream);
}

size_t oeq_grouped_sum_workspace_bytes(const oeq_kernels* k, int64_t n_segments, int64_t n_items) {
    (void)k;
    // [ptr | cursor | perm | scratch perm]
    return 2 * align_up((size_t)(n_segments + 1 + 1 + OEQ_LONG_LIST) * sizeof(int64_t), 256) +
           2 * align_up((size_t)n_items * sizeof(int64_t), 256);
}

int oeq_grouped_sum(oeq_kernels* k, int64_t n_segments, int64_t n_items, int64_t row_len, const void* src, void* dst,
                    const int64_t* keys, void* workspace, size_t workspace_bytes, void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_grouped_sum: NULL kernel set");
    if (n_segments < 0 || n_items < 0 || row_len <= 0) return fail(OEQ_ERR_INVALID, "oeq_grouped_sum: bad size");
    if (n_segments == 0) return OEQ_OK;
    if (!dst) return fail(OEQ_ERR_INVALID, "oeq_grouped_sum: NULL dst");
    if (n_items == 0) return k->fill_zero(dst, (size_t)n_segments * row_len * k->dims.elem_size, stream);
    if (!src || !keys) return fail(OEQ_ERR_INVALID, "oeq_grouped_sum: NULL buffer");
    size_t need = oeq_grouped_sum_workspace_bytes(k, n_segments, n_items);
    if (!workspace || workspace_bytes < need)
        return fail(OEQ_ERR_INVALID, "oeq_grouped_sum: workspace too small (%zu < %zu bytes)", workspace_bytes, need);
    const size_t pb = align_up((size_t)(n_segments + 1 + 1 + OEQ_LONG_LIST) * sizeof(int64_t), 256);
    const size_t qb = align_up((size_t)n_items * sizeof(int64_t), 256);
    int64_t* ptr = (int64_t*)workspace;
    int64_t* cursor = (int64_t*)((char*)workspace + pb);
    int64_t* perm = (int64_t*)((char*)workspace + 2 * pb);
    int64_t* scratch = (int64_t*)((char*)workspace + 2 * pb + qb);
    int rc = k->group_by_key(n_items, n_segments, keys, ptr, cursor, scratch, perm, stream);
    if (rc) return rc;
    const int64_t* cperm = perm;
    void* args[] = {&n_segments, &n_items, &row_len, &src, &dst, &cperm, &ptr};
    return k->launch(OEQ_ROLE_SEGMENT_SUM, n_segments, args, stream);
}

int oeq_kernel_timing_enable(oeq_kernels* k, int enable) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_kernel_timing_enable: NULL kernel set");
    k->timing.store(enable != 0, std::memory_order_relaxed);
    return OEQ_OK;
}

int oeq_kernel_timing_collect(oeq_kernels* k, int role, double* total_ms, int64_t* launches) {
    if (!k || !total_ms || !launches) return fail(OEQ_ERR_INVALID, "oeq_kernel_timing_collect: NULL argument");
    std::vector<TimedLaunch> mine, rest;
    {
        std::lock_guard<std::mutex> lock(k->mu);
        for (auto& t : k->timed) (t.role == role ? mine : rest).push_back(t);
        k->timed.swap(rest);
    }
    double sum = 0.0;
    int rc = OEQ_OK;
    for (auto& t : mine) {
        float ms = 0.f;
        hipError_t e = hipEventSynchronize(t.stop);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, t.start, t.stop);
        if (e != hipSuccess) rc = fail(OEQ_ERR_HIP, "kernel timing failed: %s", hipGetErrorString(e));
        sum += ms;
        (void)hipEventDestroy(t.start);
        (void)hipEventDestroy(t.stop);
    }
    *total_ms = sum;
    *launches = (int64_t)mine.size();
    return rc;
}

// ---------------------------------------------------------------------------
// batched tensor product
// ---------------------------------------------------------------------------

int oeq_tp_forward(oeq_kernels* k, int64_t num_batch, const void* L1_in, const void* L2_in, const void* W, void* L3_out,
                   void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_tp_forward: NULL kernel set");
    if (num_batch < 0) return fail(OEQ_ERR_INVALID, "oeq_tp_forward: negative batch");
    if (num_batch == 0) return OEQ_OK;
    if (!L1_in || !L2_in || !W || !L3_out) return fail(OEQ_ERR_INVALID, "oeq_tp_forward: NULL buffer");
    void* args[] = {&num_batch, &L1_in, &L2_in, &W, &L3_out};
    return k->launch(OEQ_ROLE_TP_FORWARD, num_batch, args, stream);
}

size_t oeq_tp_backward_workspace_bytes(const oeq_kernels* k, int64_t num_batch) {
    if (!k || !k->dims.shared_weights || !k->roles[OEQ_ROLE_TP_BACKWARD].present) return 0;
    size_t rows = (size_t)k->grid_for(OEQ_ROLE_TP_BACKWARD, num_batch) * (size_t)k->dims.wpartial_per_block;
    return align_up(rows * (size_t)k->dims.weight_numel * (size_t)k->dims.elem_size, 256);
}

int oeq_tp_backward(oeq_kernels* k, int64_t num_batch, const void* L1_in, void* L1_grad, const void* L2_in,
                    void* L2_grad, const void* W, void* W_grad, const void* L3_grad, void* workspace,
                    size_t workspace_bytes, void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_tp_backward: NULL kernel set");
    if (num_batch < 0) return fail(OEQ_ERR_INVALID, "oeq_tp_backward: negative batch");
    const bool shared = k->dims.shared_weights != 0;
    if (num_batch == 0) {
        // per-row weights: every operand is empty; shared weights: the weight gradient is a sum over no rows
        if (!shared) return OEQ_OK;
        if (!W_grad) return fail(OEQ_ERR_INVALID, "oeq_tp_backward: NULL W_grad");
        return k->fill_zero(W_grad, (size_t)k->dims.weight_numel * k->dims.elem_size, stream);
    }
    if (!L1_in || !L1_grad || !L2_in || !L2_grad || !W || !W_grad || !L3_grad)
        return fail(OEQ_ERR_INVALID, "oeq_tp_backward: NULL buffer");
    size_t need = oeq_tp_backward_workspace_bytes(k, num_batch);
    if (need && (!workspace || workspace_bytes < need))
        return fail(OEQ_ERR_INVALID, "oeq_tp_backward: workspace too small (%zu < %zu bytes)", workspace_bytes, need);
    void* wpartial = need ? workspace : nullptr;
    void* args[] = {&num_batch, &L1_in, &L1_grad, &L2_in, &L2_grad, &W, &W_grad, &L3_grad, &wpartial};
    int rc = k->launch(OEQ_ROLE_TP_BACKWARD, num_batch, args, stream);
    if (rc || !shared) return rc;
    // Second pass: sum the per-block partial weight gradients in block order.
    int64_t n_partials = (int64_t)k->grid_for(OEQ_ROLE_TP_BACKWARD, num_batch) * k->dims.wpartial_per_block;
    int64_t wn = k->dims.weight_numel;
    void* rargs[] = {&n_partials, &wpartial, &W_grad, &wn};
    return k->launch(OEQ_ROLE_TP_BACKWARD_WREDUCE, wn, rargs, stream);
}

// ---------------------------------------------------------------------------
// fused graph convolution
// ---------------------------------------------------------------------------

// The generated kernels force every node and edge index into range with 32-bit arithmetic.
static int check_graph_size(const char* who, int64_t node_count, int64_t nnz) {
    if (node_count < 0 || nnz < 0) return fail(OEQ_ERR_INVALID, "%s: negative size", who);
    if (node_count > 0x7fffffffLL || nnz > 0x7fffffffLL)
        return fail(OEQ_ERR_INVALID, "%s: %lld nodes / %lld edges; at most 2^31 - 1 of each are supported", who,
                    (long long)node_count, (long long)nnz);
    return OEQ_OK;
}

// Shared weights, walk kernels: one partial weight-gradient row per wave group of the backward grid.
// A segment-pointer (or cursor) array: n + 1 entries, and behind them the list of long segments that
// oeq_group_scan leaves for oeq_group_order (a count and up to OEQ_LONG_LIST entries).
static size_t ptr_bytes_of(int64_t node_count) {
    return align_up((size_t)(node_count + 1 + 1 + OEQ_LONG_LIST) * sizeof(int64_t), 256);
}
static size_t perm_bytes_of(int64_t nnz) { return align_up((size_t)nnz * sizeof(int64_t), 256); }

static size_t conv_wpartial_bytes(const oeq_kernels* k, int64_t walk_positions, int role = OEQ_ROLE_CONV_BACKWARD) {
    if (!k->dims.shared_weights || !k->dims.wpartial_per_block || !k->roles[role].present) return 0;
    size_t rows = (size_t)k->grid_for(role, walk_positions) * (size_t)k->dims.wpartial_per_block;
    return align_up(rows * (size_t)k->dims.weight_numel * (size_t)k->dims.elem_size, 256);
}

// Long edge segments (a hub node) are walked in chunks of `hub_limit` edges: a node's own walk position takes
// the first chunk, every further chunk is an extra position listed in the index (hubptr / hubnode). 0 = whole
// segments (kernel sets without the table kernels, and the allocation-free entry point).
static int64_t hub_limit_of(const oeq_kernels* k) {
    if (oeq_kernels::no_hubs || k->dims.hub_limit <= 0) return 0;
    if (!k->roles[OEQ_ROLE_HUB_COUNT].present || !k->roles[OEQ_ROLE_HUB_FILL].present ||
        !k->roles[OEQ_ROLE_CONV_FIXUP_FORWARD].present)
        return 0;
    return k->dims.hub_limit;
}
// every extra position follows a full chunk of its node, so there are at most nnz / limit of them
static int64_t hub_capacity(const oeq_kernels* k, int64_t nnz) {
    const int64_t limit = hub_limit_of(k);
    return limit ? nnz / limit : 0;
}
// Walk positions that the kernel of `role` reserves for the extra chunks, at the front of its grid: the
// capacity rounded up to whole blocks and to the grid multiple of the role, so that the blocks behind them
// still divide evenly among the XCDs.
static int64_t hub_units(const oeq_kernels* k, int role, int64_t nnz) {
    const int64_t cap = hub_capacity(k, nnz);
    if (!cap || !k->roles[role].present) return 0;
    const int64_t g = std::max(1u, k->roles[role].units_per_block), m = std::max(1u, k->roles[role].grid_multiple);
    const int64_t blocks = ((cap + g - 1) / g + m - 1) / m * m;
    return blocks * g;
}
static size_t hub_rows_bytes(const oeq_kernels* k, int role, int64_t nnz) {
    return align_up((size_t)hub_units(k, role, nnz) * (size_t)k->dims.L3_dim * (size_t)k->dims.elem_size, 256);
}

// The index of an edge list: what the walk kernels derive from (rows, cols) alone. Receiver side: CSR
// pointers, in GROUPED mode the edge ids grouped by receiver, and the walk order of the nodes. Sender side
// (for the calls that reduce per-edge dX terms): CSR pointers over senders and, in GROUPED mode, the edge ids
// grouped by sender. Byte offsets into the index buffer (SIZE_MAX: piece not present); the pieces after
// `keep` are temporaries of the build.
struct IndexLayout {
    size_t rowptr = SIZE_MAX, colptr = SIZE_MAX, rperm = SIZE_MAX, sperm = SIZE_MAX, order = SIZE_MAX,
           hubptr = SIZE_MAX, hubnode = SIZE_MAX, shubptr = SIZE_MAX, shubnode = SIZE_MAX, hubcur = SIZE_MAX,
           keep = 0, cursor = SIZE_MAX, scratch = SIZE_MAX, key_a = SIZE_MAX, key_b = SIZE_MAX, optr = SIZE_MAX,
           ocursor = SIZE_MAX, oscratch = SIZE_MAX, total = 0;
};

static IndexLayout index_layout(const oeq_kernels* k, int64_t node_count, int64_t nnz, bool sender_side) {
    IndexLayout w;
    const size_t pb = ptr_bytes_of(node_count), qb = perm_bytes_of(nnz);
    const bool grouped = k->dims.deterministic == OEQ_CONV_GROUPED;
    const bool ordered = k->dims.order_hops > 0 && k->roles[OEQ_ROLE_ORDER_HOP].present;
    auto take = [&w](size_t bytes) { size_t at = w.total; w.total += bytes; return at; };
    w.rowptr = take(pb);
    if (sender_side) w.colptr = take(pb);
    if (grouped) w.rperm = take(qb);
    if (grouped && sender_side) w.sperm = take(qb);
    if (ordered) w.order = take(pb);
    const int64_t hub_cap = hub_capacity(k, nnz);
    if (hub_cap) {
        w.hubptr = take(pb);
        w.hubnode = take(align_up((size_t)hub_cap * sizeof(int64_t), 256));
        if (sender_side) {  // the same table over the senders' segments, for the ordered sum of the dX terms
            w.shubptr = take(pb);
            w.shubnode = take(align_up((size_t)hub_cap * sizeof(int64_t), 256));
        }
    }
    w.keep = w.total;
    if (hub_cap) w.hubcur = take(pb);
    if (grouped) {
        w.cursor = take(pb);
        w.scratch = take(qb);
    }
    if (ordered) {
        w.key_a = take(pb);
        w.key_b = take(pb);
        w.optr = take(pb);
        w.ocursor = take(pb);
        w.oscratch = take(pb);
    }
    return w;
}

// What a call needs besides operands and index: `terms` = the per-edge dX terms, `arrivals` = the per-sender
// arrival counters of OEQ_DX_ARRIVAL, `wpartial` = partial weight-gradient rows (shared weights).
struct ScratchLayout {
    size_t arrivals = SIZE_MAX, dx_tmp = SIZE_MAX, wpartial = SIZE_MAX, hub_rows = SIZE_MAX, shub_rows = SIZE_MAX,
           total = 0;
};

static ScratchLayout scratch_layout(const oeq_kernels* k, int64_t node_count, int64_t nnz, bool terms, bool arrivals,
                                    bool wpartial, int wpartial_role = OEQ_ROLE_CONV_BACKWARD,
                                    int hub_rows_role = -1) {
    ScratchLayout w;
    auto take = [&w](size_t bytes) { size_t at = w.total; w.total += bytes; return at; };
    // rows that the extra chunks of long segments write (forward-shaped kernels)
    if (hub_rows_role >= 0)
        if (size_t hb = hub_rows_bytes(k, hub_rows_role, nnz)) w.hub_rows = take(hb);
    if (arrivals)
        w.arrivals = take(align_up((size_t)node_count * (size_t)std::max(1, k->dims.n_chunks) * sizeof(int32_t), 256));
    if (terms && wpartial_role == OEQ_ROLE_CONV_BACKWARD && k->dims.dx_mode == OEQ_DX_SENDER_WALK) {
        // no terms: the sender-side walk forms the rows itself, and writes those of its extra chunks here
        if (int64_t su = hub_units(k, OEQ_ROLE_CONV_BACKWARD_DX, nnz))
            w.shub_rows = take(align_up((size_t)su * (size_t)k->dims.L1_dim * (size_t)k->dims.elem_size, 256));
    } else if (terms) {
        w.dx_tmp = take(align_up((size_t)nnz * (size_t)k->dims.L1_dim * (size_t)k->dims.elem_size, 256));
        // partial sums of the senders whose terms fixup_backward sums in chunks
        if (!arrivals)
            if (int64_t su = hub_units(k, OEQ_ROLE_CONV_FIXUP_BACKWARD, nnz))
                w.shub_rows = take(align_up((size_t)su * (size_t)k->dims.L1_dim * (size_t)k->dims.elem_size, 256));
    }
    if (wpartial)
        if (size_t wp = conv_wpartial_bytes(k, node_count + hub_units(k, wpartial_role, nnz), wpartial_role))
            w.wpartial = take(wp);
    return w;
}

struct WalkIndex {
    int64_t *rowptr = nullptr, *colptr = nullptr, *rperm = nullptr;
    const int64_t* sperm = nullptr;
    int64_t* order = nullptr;  // the order in which the walk kernels visit the nodes (NULL: by index)
    // extra walk positions of the nodes whose edge segments are cut into chunks (NULL / 0: none)
    int64_t *hubptr = nullptr, *hubnode = nullptr, *shubptr = nullptr, *shubnode = nullptr;
    int64_t hub_limit = 0;
};

struct WalkScratch {
    void *dx_tmp = nullptr, *wpartial = nullptr, *shub_rows = nullptr;
    int32_t* arrivals = nullptr;
};

static char* at_offset(const void* base, size_t off) { return off == SIZE_MAX ? nullptr : (char*)base + off; }

// Pointers into a built index buffer.
static int bind_index(const oeq_kernels* k, const char* who, const IndexLayout& w, const void* index,
                      size_t index_bytes, const int64_t* transpose_perm, WalkIndex* ix) {
    if (!index || index_bytes < w.keep)
        return fail(OEQ_ERR_INVALID, "%s: index buffer too small (%zu < %zu bytes)", who, index_bytes, w.keep);
    if (k->dims.deterministic == OEQ_CONV_SORTED && w.colptr != SIZE_MAX && !transpose_perm)
        return fail(OEQ_ERR_INVALID, "%s: deterministic mode needs transpose_perm", who);
    ix->rowptr = (int64_t*)at_offset(index, w.rowptr);
    ix->colptr = (int64_t*)at_offset(index, w.colptr);
    ix->rperm = (int64_t*)at_offset(index, w.rperm);
    ix->sperm = w.sperm != SIZE_MAX ? (const int64_t*)at_offset(index, w.sperm) : transpose_perm;
    ix->order = (int64_t*)at_offset(index, w.order);
    ix->hubptr = (int64_t*)at_offset(index, w.hubptr);
    ix->hubnode = (int64_t*)at_offset(index, w.hubnode);
    ix->shubptr = (int64_t*)at_offset(index, w.shubptr);
    ix->shubnode = (int64_t*)at_offset(index, w.shubnode);
    ix->hub_limit = ix->hubptr ? hub_limit_of(k) : 0;
    return OEQ_OK;
}

static int build_index(oeq_kernels* k, const char* who, const IndexLayout& w, int64_t node_count, int64_t nnz,
                       const int64_t* rows, const int64_t* cols, const int64_t* transpose_perm, void* index,
                       size_t index_bytes, void* stream) {
    if (!rows || !cols) return fail(OEQ_ERR_INVALID, "%s: NULL edge list", who);
    if (!index || index_bytes < w.total)
        return fail(OEQ_ERR_INVALID, "%s: workspace too small (%zu < %zu bytes)", who, index_bytes, w.total);
    WalkIndex ix;
    int rc = bind_index(k, who, w, index, index_bytes, transpose_perm, &ix);
    if (rc) return rc;
    const bool sender_side = w.colptr != SIZE_MAX;
    if (k->dims.deterministic == OEQ_CONV_SORTED) {
        rc = k->segment_ptr(nnz, node_count, rows, nullptr, ix.rowptr, stream);
        if (!rc && sender_side) rc = k->segment_ptr(nnz, node_count, cols, transpose_perm, ix.colptr, stream);
    } else {
        int64_t* cursor = (int64_t*)at_offset(index, w.cursor);
        int64_t* scratch = (int64_t*)at_offset(index, w.scratch);
        rc = k->group_by_key(nnz, node_count, rows, ix.rowptr, cursor, scratch, ix.rperm, stream);
        if (!rc && sender_side)
            rc = k->group_by_key(nnz, node_count, cols, ix.colptr, cursor, scratch, (int64_t*)ix.sperm, stream);
    }
    // extra positions of long segments: count per node, exclusive scan, list the nodes
    auto hub_table = [&](int64_t* segptr, int64_t* hubptr, int64_t* hubnode) {
        int64_t limit = ix.hub_limit, cap = hub_capacity(k, nnz), n1 = node_count + 1;
        int64_t* hubcur = (int64_t*)at_offset(index, w.hubcur);
        void* cargs[] = {&node_count, &nnz, &segptr, &limit, &hubptr};
        int r = k->launch(OEQ_ROLE_HUB_COUNT, n1, cargs, stream);
        void* sargs[] = {&n1, &hubptr, &hubcur};
        if (!r) r = k->launch(OEQ_ROLE_GROUP_SCAN, 1, sargs, stream);
        void* fargs[] = {&node_count, &cap, &hubptr, &hubnode};
        if (!r) r = k->launch(OEQ_ROLE_HUB_FILL, node_count, fargs, stream);
        return r;
    };
    if (!rc && ix.hubptr) rc = hub_table(ix.rowptr, ix.hubptr, ix.hubnode);
    if (!rc && ix.shubptr) rc = hub_table(ix.colptr, ix.shubptr, ix.shubnode);
    if (rc || !ix.order) return rc;
    // Walk order: cluster the nodes by the highest-priority node within `order_hops` edges, then list them
    // cluster by cluster (a counting sort by cluster key, ascending node index inside a cluster, so that the
    // order is a function of the edge list: with shared weights the walk kernels sum their weight gradients
    // per wave group over the nodes the group visits, and which nodes those are must not change between
    // two builds).
    int64_t* keys[2] = {(int64_t*)at_offset(index, w.key_a), (int64_t*)at_offset(index, w.key_b)};
    const int64_t* key_in = nullptr;
    const int64_t* cperm = ix.rperm;
    for (int h = 0; h < k->dims.order_hops; ++h) {
        int64_t* key_out = keys[h & 1];
        void* hargs[] = {&node_count, &nnz, &ix.rowptr, &cols, &cperm, &key_in, &key_out};
        rc = k->launch(OEQ_ROLE_ORDER_HOP, node_count, hargs, stream);
        if (rc) return rc;
        key_in = key_out;
    }
    return k->group_by_key(node_count, node_count, key_in, (int64_t*)at_offset(index, w.optr),
                           (int64_t*)at_offset(index, w.ocursor), (int64_t*)at_offset(index, w.oscratch), ix.order,
                           stream);
}

static bool walk_mode(const oeq_kernels* k) { return k->dims.deterministic != OEQ_CONV_ATOMIC; }

// L1_grad[s] = sum of the per-edge terms of sender s in sender-major order; senders with more than hub_limit
// edges in chunks whose partial sums (shub_rows) are added in chunk order afterwards.
static int sender_sum(oeq_kernels* k, int64_t node_count, int64_t nnz, void* dx_tmp, void* L1_grad,
                      const WalkIndex& ix, void* shub_rows, void* stream) {
    int64_t limit = (ix.shubptr && shub_rows) ? ix.hub_limit : 0;
    int64_t units = limit ? hub_units(k, OEQ_ROLE_CONV_FIXUP_BACKWARD, nnz) : 0;
    void* fargs[] = {&node_count, &nnz,         &dx_tmp, &L1_grad, (void*)&ix.sperm, (void*)&ix.colptr,
                     (void*)&ix.shubptr, (void*)&ix.shubnode, &limit, &units, &shub_rows};
    int rc = k->launch(OEQ_ROLE_CONV_FIXUP_BACKWARD, node_count + units, fargs, stream);
    if (rc || !units) return rc;
    int64_t row_len = k->dims.L1_dim;
    void* cargs[] = {&node_count, &units, (void*)&ix.shubptr, (void*)&ix.shubnode, &shub_rows, &L1_grad, &row_len};
    return k->launch(OEQ_ROLE_CONV_FIXUP_FORWARD, units, cargs, stream);
}
static bool backward_terms(const oeq_kernels* k) { return k->dims.dx_mode != OEQ_DX_ATOMIC; }

size_t oeq_conv_index_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz, int sender_side) {
    if (!k || !walk_mode(k) || node_count < 0 || nnz < 0) return 0;
    return index_layout(k, node_count, nnz, sender_side != 0).total;
}

int oeq_conv_index_piece(const oeq_kernels* k, int64_t node_count, int64_t nnz, int sender_side, int piece,
                         size_t* offset, size_t* entries) {
    if (!k || !offset || !entries) return fail(OEQ_ERR_INVALID, "oeq_conv_index_piece: NULL argument");
    if (!walk_mode(k) || node_count < 0 || nnz < 0) return fail(OEQ_ERR_INVALID, "oeq_conv_index_piece: no index");
    const IndexLayout w = index_layout(k, node_count, nnz, sender_side != 0);
    const size_t cap = (size_t)hub_capacity(k, nnz);
    const size_t n1 = (size_t)node_count + 1, n = (size_t)node_count, e = (size_t)nnz;
    const size_t at[] = {w.rowptr, w.colptr, w.rperm, w.sperm, w.order, w.hubptr, w.hubnode, w.shubptr, w.shubnode};
    const size_t len[] = {n1, n1, e, e, n, n1, cap, n1, cap};
    if (piece < 0 || piece >= (int)(sizeof(at) / sizeof(at[0])))
        return fail(OEQ_ERR_INVALID, "oeq_conv_index_piece: unknown piece %d", piece);
    if (at[piece] == SIZE_MAX) return fail(OEQ_ERR_INVALID, "oeq_conv_index_piece: piece %d is not part of this index", piece);
    *offset = at[piece];
    *entries = len[piece];
    return OEQ_OK;
}

int oeq_conv_index_build(oeq_kernels* k, int64_t node_count, int64_t nnz, const int64_t* rows, const int64_t* cols,
                         const int64_t* transpose_perm, int sender_side, void* index, size_t index_bytes,
                         void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_conv_index_build: NULL kernel set");
    if (int bad = check_graph_size("oeq_conv_index_build", node_count, nnz)) return bad;
    if (!walk_mode(k) || node_count == 0 || nnz == 0) return OEQ_OK;  // nothing to index
    if (sender_side && k->dims.deterministic == OEQ_CONV_SORTED && !transpose_perm)
        return fail(OEQ_ERR_INVALID, "oeq_conv_index_build: deterministic mode needs transpose_perm");
    return build_index(k, "oeq_conv_index_build", index_layout(k, node_count, nnz, sender_side != 0), node_count, nnz,
                       rows, cols, transpose_perm, index, index_bytes, stream);
}

size_t oeq_conv_forward_scratch_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz) {
    if (!k || !walk_mode(k) || node_count < 0 || nnz < 0) return 0;
    return scratch_layout(k, node_count, nnz, false, false, false, OEQ_ROLE_CONV_BACKWARD, OEQ_ROLE_CONV_FORWARD).total;
}

size_t oeq_conv_forward_workspace_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz) {
    return oeq_conv_index_bytes(k, node_count, nnz, 0) + oeq_conv_forward_scratch_bytes(k, node_count, nnz);
}

size_t oeq_conv_backward_scratch_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz) {
    if (!k || !walk_mode(k)) return 0;
    return scratch_layout(k, node_count, nnz, backward_terms(k), k->dims.dx_mode == OEQ_DX_ARRIVAL, true).total;
}

size_t oeq_conv_backward_workspace_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz) {
    if (!k || !walk_mode(k)) return 0;
    return oeq_conv_index_bytes(k, node_count, nnz, backward_terms(k)) +
           oeq_conv_backward_scratch_bytes(k, node_count, nnz);
}

// the second-order kernels always go through the per-edge terms and fixup_backward
size_t oeq_conv_double_backward_scratch_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz) {
    if (!k || !walk_mode(k)) return 0;
    return scratch_layout(k, node_count, nnz, true, false, true, OEQ_ROLE_DOUBLE_BACKWARD_B,
                          OEQ_ROLE_DOUBLE_BACKWARD_A).total;
}

size_t oeq_conv_double_backward_workspace_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz) {
    if (!k || !walk_mode(k)) return 0;
    return oeq_conv_index_bytes(k, node_count, nnz, 1) + oeq_conv_double_backward_scratch_bytes(k, node_count, nnz);
}

int oeq_conv_forward_indexed(oeq_kernels* k, int64_t node_count, int64_t nnz, const void* L1_in, const void* L2_in,
                             const void* W, void* L3_out, const int64_t* rows, const int64_t* cols, const void* index,
                             size_t index_bytes, int index_sender_side, void* scratch, size_t scratch_bytes,
                             void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_conv_forward: NULL kernel set");
    if (int bad = check_graph_size("oeq_conv_forward", node_count, nnz)) return bad;
    if (node_count == 0) return OEQ_OK;
    if (!L3_out) return fail(OEQ_ERR_INVALID, "oeq_conv_forward: NULL L3_out");
    const size_t out_bytes = (size_t)node_count * k->dims.L3_dim * k->dims.elem_size;
    if (nnz == 0) return k->fill_zero(L3_out, out_bytes, stream);
    if (!L1_in || !L2_in || !W || !rows || !cols) return fail(OEQ_ERR_INVALID, "oeq_conv_forward: NULL buffer");
    WalkIndex ix;
    int rc;
    int64_t units = 0;
    void* hub_rows = nullptr;
    if (walk_mode(k)) {
        // the forward reads the receiver side only; the caller's perm stands in where the layout wants one
        rc = bind_index(k, "oeq_conv_forward", index_layout(k, node_count, nnz, index_sender_side != 0), index,
                        index_bytes, rows, &ix);
        if (rc) return rc;
        if (ix.hub_limit) {
            units = hub_units(k, OEQ_ROLE_CONV_FORWARD, nnz);
            const size_t need = hub_rows_bytes(k, OEQ_ROLE_CONV_FORWARD, nnz);
            if (!scratch || scratch_bytes < need)
                return fail(OEQ_ERR_INVALID, "oeq_conv_forward: workspace too small (%zu < %zu bytes of scratch)",
                            scratch_bytes, need);
            hub_rows = scratch;
        }
    } else {
        rc = k->fill_zero(L3_out, out_bytes, stream);
        if (rc) return rc;
    }
    void* args[] = {&node_count, &nnz,      &L1_in,    &L2_in,      &W,           &L3_out,       &rows,  &cols,
                    &ix.rowptr,  &ix.rperm, &ix.order, &ix.hubptr, &ix.hubnode, &ix.hub_limit, &units, &hub_rows};
    rc = k->launch(OEQ_ROLE_CONV_FORWARD, walk_mode(k) ? node_count + units : nnz, args, stream);
    if (rc || !units) return rc;
    // the rows of the extra chunks, added to their nodes' rows in chunk order
    int64_t row_len = k->dims.L3_dim;
    void* fargs[] = {&node_count, &units, &ix.hubptr, &ix.hubnode, &hub_rows, &L3_out, &row_len};
    return k->launch(OEQ_ROLE_CONV_FIXUP_FORWARD, units, fargs, stream);
}

int oeq_conv_forward(oeq_kernels* k, int64_t node_count, int64_t nnz, const void* L1_in, const void* L2_in,
                     const void* W, void* L3_out, const int64_t* rows, const int64_t* cols, void* workspace,
                     size_t workspace_bytes, void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_conv_forward: NULL kernel set");
    if (int bad = check_graph_size("oeq_conv_forward", node_count, nnz)) return bad;
    size_t index_bytes = 0;
    if (!oeq_kernels::no_events) {
        // Where allocating is allowed: resolve the scratch array of oeq_conv_forward_static on this device
        // (the first look-up of a device symbol may load the library's own code object), so that the static
        // entry point, whose precondition is one call of this function, finds the address ready.
        void* unused = nullptr;
        (void)static_scratch(&unused);
    }
    if (walk_mode(k) && node_count > 0 && nnz > 0) {
        if (!L3_out) return fail(OEQ_ERR_INVALID, "oeq_conv_forward: NULL L3_out");
        if (!L1_in || !L2_in || !W || !rows || !cols) return fail(OEQ_ERR_INVALID, "oeq_conv_forward: NULL buffer");
        const IndexLayout w = index_layout(k, node_count, nnz, false);
        const size_t need = w.total + oeq_conv_forward_scratch_bytes(k, node_count, nnz);
        if (!workspace || workspace_bytes < need)
            return fail(OEQ_ERR_INVALID, "oeq_conv_forward: workspace too small (%zu < %zu bytes)", workspace_bytes,
                        need);
        int rc = build_index(k, "oeq_conv_forward", w, node_count, nnz, rows, cols, nullptr, workspace, w.total, stream);
        if (rc) return rc;
        index_bytes = w.total;
    }
    return oeq_conv_forward_indexed(k, node_count, nnz, L1_in, L2_in, W, L3_out, rows, cols, workspace, index_bytes, 0,
                                    workspace ? (char*)workspace + index_bytes : nullptr,
                                    workspace_bytes > index_bytes ? workspace_bytes - index_bytes : 0, stream);
}

size_t oeq_static_scratch_bytes(void) { return OEQ_STATIC_SCRATCH_BYTES; }

int oeq_conv_forward_static(oeq_kernels* k, int64_t node_count, int64_t nnz, const void* L1_in, const void* L2_in,
                            const void* W, void* L3_out, const int64_t* rows, const int64_t* cols, void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_conv_forward_static: NULL kernel set");
    if (node_count < 0 || nnz < 0) return fail(OEQ_ERR_INVALID, "oeq_conv_forward_static: negative size");
    oeq_kernels::no_hubs = true;  // whole segments: no rows of extra chunks to hold
    const size_t need = oeq_conv_forward_workspace_bytes(k, node_count, nnz);
    oeq_kernels::no_hubs = false;
    if (need > OEQ_STATIC_SCRATCH_BYTES)
        return fail(OEQ_ERR_INVALID,
                    "oeq_conv_forward_static: %lld nodes and %lld edges need %zu bytes of index scratch, the static "
                    "buffer holds %u; use oeq_conv_forward with a caller-provided workspace",
                    (long long)node_count, (long long)nnz, need, (unsigned)OEQ_STATIC_SCRATCH_BYTES);
    // loading a code object allocates device memory: that has to have happened before
    if (!k->loaded_on_current_device())
        return fail(OEQ_ERR_INVALID,
                    "oeq_conv_forward_static: the kernels are not loaded on this device yet; run oeq_conv_forward "
                    "once on it first");
    void* ws = nullptr;
    int rc = static_scratch(&ws);
    if (rc) return rc;
    oeq_kernels::no_events = oeq_kernels::no_hubs = true;
    rc = oeq_conv_forward(k, node_count, nnz, L1_in, L2_in, W, L3_out, rows, cols, ws, OEQ_STATIC_SCRATCH_BYTES, stream);
    oeq_kernels::no_events = oeq_kernels::no_hubs = false;
    return rc;
}

int oeq_conv_backward_indexed(oeq_kernels* k, int64_t node_count, int64_t nnz, const void* L1_in, void* L1_grad,
                              const void* L2_in, void* L2_grad, const void* W, void* W_grad, const void* L3_grad,
                              const int64_t* rows, const int64_t* cols, const int64_t* transpose_perm,
                              const void* index, size_t index_bytes, int index_sender_side, void* scratch,
                              size_t scratch_bytes, void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_conv_backward: NULL kernel set");
    if (int bad = check_graph_size("oeq_conv_backward", node_count, nnz)) return bad;
    const bool shared = k->dims.shared_weights != 0;
    const size_t es = (size_t)k->dims.elem_size;
    // shared weights: the float-atomics kernels add into a cleared W_grad; the walk kernels write partial
    // rows that are summed in order at the end (W_grad is cleared only when there is nothing to sum)
    const bool wrows = shared && walk_mode(k) && k->dims.wpartial_per_block > 0;
    int rc;
    if (shared && (!wrows || node_count == 0 || nnz == 0)) {
        if (!W_grad) return fail(OEQ_ERR_INVALID, "oeq_conv_backward: NULL W_grad");
        rc = k->fill_zero(W_grad, (size_t)k->dims.weight_numel * es, stream);
        if (rc) return rc;
    }
    if (node_count == 0) return OEQ_OK;
    if (!L1_grad) return fail(OEQ_ERR_INVALID, "oeq_conv_backward: NULL L1_grad");
    const size_t dx_bytes = (size_t)node_count * k->dims.L1_dim * es;
    if (nnz == 0) return k->fill_zero(L1_grad, dx_bytes, stream);
    if (!L1_in || !L2_in || !L2_grad || !W || !W_grad || !L3_grad || !rows || !cols)
        return fail(OEQ_ERR_INVALID, "oeq_conv_backward: NULL buffer");

    WalkIndex ix;
    WalkScratch sc;
    const int dx_mode = walk_mode(k) ? k->dims.dx_mode : (int)OEQ_DX_ATOMIC;
    if (walk_mode(k)) {
        if (backward_terms(k) && !index_sender_side)
            return fail(OEQ_ERR_INVALID, "oeq_conv_backward: this kernel set needs an index built with the sender side");
        rc = bind_index(k, "oeq_conv_backward", index_layout(k, node_count, nnz, index_sender_side != 0), index,
                        index_bytes, transpose_perm ? transpose_perm : rows, &ix);
        if (rc) return rc;
        if (backward_terms(k) && k->dims.deterministic == OEQ_CONV_SORTED && !transpose_perm)
            return fail(OEQ_ERR_INVALID, "oeq_conv_backward: deterministic mode needs transpose_perm");
        const ScratchLayout w =
            scratch_layout(k, node_count, nnz, backward_terms(k), dx_mode == OEQ_DX_ARRIVAL, true);
        if (w.total && (!scratch || scratch_bytes < w.total))
            return fail(OEQ_ERR_INVALID, "oeq_conv_backward: workspace too small (%zu < %zu bytes of scratch)",
                        scratch_bytes, w.total);
        sc.dx_tmp = at_offset(scratch, w.dx_tmp);
        sc.wpartial = at_offset(scratch, w.wpartial);
        sc.arrivals = (int32_t*)at_offset(scratch, w.arrivals);
        sc.shub_rows = at_offset(scratch, w.shub_rows);
    }
    if (dx_mode == OEQ_DX_ATOMIC || dx_mode == OEQ_DX_ARRIVAL) {
        // atomics accumulate into the rows; the arrival scheme never visits a node that sends nothing
        rc = k->fill_zero(L1_grad, dx_bytes, stream);
        if (rc) return rc;
    }
    if (dx_mode == OEQ_DX_ARRIVAL) {
        rc = k->fill_zero(sc.arrivals, (size_t)node_count * (size_t)std::max(1, k->dims.n_chunks) * sizeof(int32_t),
                          stream);
        if (rc) return rc;
    }
    int64_t units = ix.hub_limit ? hub_units(k, OEQ_ROLE_CONV_BACKWARD, nnz) : 0;
    void* args[] = {&node_count,  &nnz,      &L1_in,     &L1_grad,    &L2_in,        &L2_grad,     &W,         &W_grad,
                    &L3_grad,     &rows,     &cols,      &ix.rowptr,  &sc.dx_tmp,    &ix.rperm,    &sc.wpartial,
                    &ix.colptr,   &ix.sperm, &sc.arrivals, &ix.order, &ix.hubptr,    &ix.hubnode,  &ix.hub_limit,
                    &units};
    rc = k->launch(OEQ_ROLE_CONV_BACKWARD, walk_mode(k) ? node_count + units : nnz, args, stream);
    if (rc || !walk_mode(k)) return rc;
    if (dx_mode == OEQ_DX_TERMS) rc = sender_sum(k, node_count, nnz, sc.dx_tmp, L1_grad, ix, sc.shub_rows, stream);
    if (dx_mode == OEQ_DX_SENDER_WALK) {
        // The forward kernel of the adjoint problem over the sender side of the index: dZ rows of the receivers
        // for the rows of X, every sender's segment in sender-major order, long segments in chunks.
        int64_t limit = (ix.shubptr && sc.shub_rows) ? ix.hub_limit : 0;
        int64_t xunits = limit ? hub_units(k, OEQ_ROLE_CONV_BACKWARD_DX, nnz) : 0;
        void* xargs[] = {&node_count, &nnz,       &L3_grad,   &L2_in,     &W,           &L1_grad,      &cols,  &rows,
                         &ix.colptr,  &ix.sperm,  &ix.order,  &ix.shubptr, &ix.shubnode, &limit,        &xunits, &sc.shub_rows};
        rc = k->launch(OEQ_ROLE_CONV_BACKWARD_DX, node_count + xunits, xargs, stream);
        if (!rc && xunits) {
            int64_t row_len = k->dims.L1_dim;
            void* cargs[] = {&node_count, &xunits, &ix.shubptr, &ix.shubnode, &sc.shub_rows, &L1_grad, &row_len};
            rc = k->launch(OEQ_ROLE_CONV_FIXUP_FORWARD, xunits, cargs, stream);
        }
    }
    if (rc || !wrows) return rc;
    int64_t n_partials =
        (int64_t)k->grid_for(OEQ_ROLE_CONV_BACKWARD, node_count + units) * k->dims.wpartial_per_block;
    int64_t wn = k->dims.weight_numel;
    void* rargs[] = {&n_partials, &sc.wpartial, &W_grad, &wn};
    return k->launch(OEQ_ROLE_TP_BACKWARD_WREDUCE, wn, rargs, stream);
}

int oeq_conv_backward(oeq_kernels* k, int64_t node_count, int64_t nnz, const void* L1_in, void* L1_grad,
                      const void* L2_in, void* L2_grad, const void* W, void* W_grad, const void* L3_grad,
                      const int64_t* rows, const int64_t* cols, const int64_t* transpose_perm, void* workspace,
                      size_t workspace_bytes, void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_conv_backward: NULL kernel set");
    if (int bad = check_graph_size("oeq_conv_backward", node_count, nnz)) return bad;
    size_t index_bytes = 0;
    const bool sender_side = walk_mode(k) && backward_terms(k);
    if (walk_mode(k) && node_count > 0 && nnz > 0) {
        if (!L1_grad) return fail(OEQ_ERR_INVALID, "oeq_conv_backward: NULL L1_grad");
        if (!L1_in || !L2_in || !L2_grad || !W || !W_grad || !L3_grad || !rows || !cols)
            return fail(OEQ_ERR_INVALID, "oeq_conv_backward: NULL buffer");
        if (sender_side && k->dims.deterministic == OEQ_CONV_SORTED && !transpose_perm)
            return fail(OEQ_ERR_INVALID, "oeq_conv_backward: deterministic mode needs transpose_perm");
        const IndexLayout w = index_layout(k, node_count, nnz, sender_side);
        const size_t need = w.total + oeq_conv_backward_scratch_bytes(k, node_count, nnz);
        if (!workspace || workspace_bytes < need)
            return fail(OEQ_ERR_INVALID, "oeq_conv_backward: workspace too small (%zu < %zu bytes)", workspace_bytes,
                        need);
        int rc = build_index(k, "oeq_conv_backward", w, node_count, nnz, rows, cols, transpose_perm, workspace, w.total,
                             stream);
        if (rc) return rc;
        index_bytes = w.total;
    }
    return oeq_conv_backward_indexed(k, node_count, nnz, L1_in, L1_grad, L2_in, L2_grad, W, W_grad, L3_grad, rows, cols,
                                     transpose_perm, workspace, index_bytes, sender_side,
                                     workspace ? (char*)workspace + index_bytes : nullptr,
                                     workspace_bytes > index_bytes ? workspace_bytes - index_bytes : 0, stream);
}

// ---------------------------------------------------------------------------
// second-order kernels
// ---------------------------------------------------------------------------

// Kernel B alone is a complete set when it also produces kernel A's result (convolution, merged form).
int oeq_has_double_backward(const oeq_kernels* k) { return k && k->roles[OEQ_ROLE_DOUBLE_BACKWARD_B].present; }

size_t oeq_tp_double_backward_workspace_bytes(const oeq_kernels* k, int64_t num_batch) {
    if (!k || !k->dims.shared_weights || !k->roles[OEQ_ROLE_DOUBLE_BACKWARD_B].present) return 0;
    size_t rows = (size_t)k->grid_for(OEQ_ROLE_DOUBLE_BACKWARD_B, num_batch) * (size_t)k->dims.wpartial_per_block;
    return align_up(rows * (size_t)k->dims.weight_numel * (size_t)k->dims.elem_size, 256);
}

int oeq_tp_double_backward(oeq_kernels* k, int64_t num_batch, const void* L1_in, const void* L2_in, const void* W,
                           const void* L3_grad, const void* L1_dgrad, const void* L2_dgrad, const void* W_dgrad,
                           void* L1_grad, void* L2_grad, void* W_grad, void* L3_dgrad, void* workspace,
                           size_t workspace_bytes, void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_tp_double_backward: NULL kernel set");
    if (!oeq_has_double_backward(k) || !k->roles[OEQ_ROLE_DOUBLE_BACKWARD_A].present)
        return fail(OEQ_ERR_INVALID, "oeq_tp_double_backward: this kernel set has no second-order kernels");
    if (num_batch < 0) return fail(OEQ_ERR_INVALID, "oeq_tp_double_backward: negative batch");
    const bool shared = k->dims.shared_weights != 0;
    if (num_batch == 0) {
        // per-row weights: every operand is empty; shared weights: the weight gradient is a sum over no rows
        if (!shared) return OEQ_OK;
        if (!W_grad) return fail(OEQ_ERR_INVALID, "oeq_tp_double_backward: NULL W_grad");
        return k->fill_zero(W_grad, (size_t)k->dims.weight_numel * k->dims.elem_size, stream);
    }
    if (!L1_in || !L2_in || !W || !L3_grad || !L1_dgrad || !L2_dgrad || !W_dgrad || !L1_grad || !L2_grad || !W_grad ||
        !L3_dgrad)
        return fail(OEQ_ERR_INVALID, "oeq_tp_double_backward: NULL buffer");
    size_t need = oeq_tp_double_backward_workspace_bytes(k, num_batch);
    if (need && (!workspace || workspace_bytes < need))
        return fail(OEQ_ERR_INVALID, "oeq_tp_double_backward: workspace too small (%zu < %zu bytes)", workspace_bytes,
                    need);
    void* wpartial = need ? workspace : nullptr;
    void* a[] = {&num_batch, &L1_in, &L1_dgrad, &L2_in, &L2_dgrad, &W, &W_dgrad, &L3_dgrad};
    int rc = k->launch(OEQ_ROLE_DOUBLE_BACKWARD_A, num_batch, a, stream);
    if (rc) return rc;
    void* b[] = {&num_batch, &L1_in, &L1_dgrad, &L2_in, &L2_dgrad, &W, &W_dgrad, &L3_grad, &L1_grad, &L2_grad, &W_grad,
                 &wpartial};
    rc = k->launch(OEQ_ROLE_DOUBLE_BACKWARD_B, num_batch, b, stream);
    if (rc || !shared) return rc;
    // shared weights: the partial weight gradients of the wave groups, summed in block order
    int64_t n_partials = (int64_t)k->grid_for(OEQ_ROLE_DOUBLE_BACKWARD_B, num_batch) * k->dims.wpartial_per_block;
    int64_t wn = k->dims.weight_numel;
    void* rargs[] = {&n_partials, &wpartial, &W_grad, &wn};
    return k->launch(OEQ_ROLE_TP_BACKWARD_WREDUCE, wn, rargs, stream);
}

int oeq_conv_double_backward_indexed(oeq_kernels* k, int64_t node_count, int64_t nnz, const void* L1_in,
                                     const void* L2_in, const void* W, const void* L3_grad, const void* L1_dgrad,
                                     const void* L2_dgrad, const void* W_dgrad, void* L1_grad, void* L2_grad,
                                     void* W_grad, void* L3_dgrad, const int64_t* rows, const int64_t* cols,
                                     const int64_t* transpose_perm, const void* index, size_t index_bytes,
                                     void* scratch, size_t scratch_bytes, void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: NULL kernel set");
    if (!oeq_has_double_backward(k) || !walk_mode(k))
        return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: this kernel set has no second-order kernels");
    if (int bad = check_graph_size("oeq_conv_double_backward", node_count, nnz)) return bad;
    if (node_count == 0) return OEQ_OK;
    if (!L1_grad || !L3_dgrad) return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: NULL output");
    const size_t es = (size_t)k->dims.elem_size;
    if (nnz == 0) {
        int rc = k->fill_zero(L1_grad, (size_t)node_count * k->dims.L1_dim * es, stream);
        if (rc) return rc;
        if (k->dims.shared_weights) {  // a sum over no edges
            if (!W_grad) return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: NULL W_grad");
            rc = k->fill_zero(W_grad, (size_t)k->dims.weight_numel * es, stream);
            if (rc) return rc;
        }
        return k->fill_zero(L3_dgrad, (size_t)node_count * k->dims.L3_dim * es, stream);
    }
    if (!L1_in || !L2_in || !W || !L3_grad || !L1_dgrad || !L2_dgrad || !W_dgrad || !L2_grad || !W_grad || !rows ||
        !cols)
        return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: NULL buffer");
    WalkIndex ix;
    int rc = bind_index(k, "oeq_conv_double_backward", index_layout(k, node_count, nnz, true), index, index_bytes,
                        transpose_perm, &ix);
    if (rc) return rc;
    const ScratchLayout w = scratch_layout(k, node_count, nnz, true, false, true, OEQ_ROLE_DOUBLE_BACKWARD_B,
                                           OEQ_ROLE_DOUBLE_BACKWARD_A);
    if (!scratch || scratch_bytes < w.total)
        return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: workspace too small (%zu < %zu bytes of scratch)",
                    scratch_bytes, w.total);
    void* dx_tmp = at_offset(scratch, w.dx_tmp);
    // shared weights: kernel B leaves one partial weight-gradient row per wave group, summed in order at the end
    void* wpartial = at_offset(scratch, w.wpartial);
    void* hub_rows = at_offset(scratch, w.hub_rows);
    int64_t units_a = (ix.hub_limit && hub_rows) ? hub_units(k, OEQ_ROLE_DOUBLE_BACKWARD_A, nnz) : 0;
    int64_t units_b = ix.hub_limit ? hub_units(k, OEQ_ROLE_DOUBLE_BACKWARD_B, nnz) : 0;
    void* a[] = {&node_count, &nnz,  &L1_in,     &L1_dgrad, &L2_in,    &L2_dgrad,  &W,          &W_dgrad,      &L3_dgrad,
                 &rows,       &cols, &ix.rowptr, &ix.rperm, &ix.order, &ix.hubptr, &ix.hubnode, &ix.hub_limit, &units_a,
                 &hub_rows};
    if (k->roles[OEQ_ROLE_DOUBLE_BACKWARD_A].present) {
        rc = k->launch(OEQ_ROLE_DOUBLE_BACKWARD_A, node_count + units_a, a, stream);
        if (rc) return rc;
        if (units_a) {
            int64_t row_len = k->dims.L3_dim;
            void* fa[] = {&node_count, &units_a, &ix.hubptr, &ix.hubnode, &hub_rows, &L3_dgrad, &row_len};
            rc = k->launch(OEQ_ROLE_CONV_FIXUP_FORWARD, units_a, fa, stream);
            if (rc) return rc;
        }
    }
    void* b[] = {&node_count, &nnz,        &L1_in,      &L1_dgrad,     &L2_in,   &L2_dgrad,  &W,         &W_dgrad,
                 &L3_grad,    &L2_grad,    &W_grad,     &rows,         &cols,    &ix.rowptr, &dx_tmp,    &ix.rperm,
                 &L3_dgrad,   &ix.order,   &wpartial,   &ix.hubptr,    &ix.hubnode, &ix.hub_limit, &units_b};
    rc = k->launch(OEQ_ROLE_DOUBLE_BACKWARD_B, node_count + units_b, b, stream);
    if (rc) return rc;
    rc = sender_sum(k, node_count, nnz, dx_tmp, L1_grad, ix, at_offset(scratch, w.shub_rows), stream);
    if (rc || !wpartial) return rc;
    int64_t n_partials =
        (int64_t)k->grid_for(OEQ_ROLE_DOUBLE_BACKWARD_B, node_count + units_b) * k->dims.wpartial_per_block;
    int64_t wn = k->dims.weight_numel;
    void* rargs[] = {&n_partials, &wpartial, &W_grad, &wn};
    return k->launch(OEQ_ROLE_TP_BACKWARD_WREDUCE, wn, rargs, stream);
}

int oeq_conv_double_backward(oeq_kernels* k, int64_t node_count, int64_t nnz, const void* L1_in, const void* L2_in,
                             const void* W, const void* L3_grad, const void* L1_dgrad, const void* L2_dgrad,
                             const void* W_dgrad, void* L1_grad, void* L2_grad, void* W_grad, void* L3_dgrad,
                             const int64_t* rows, const int64_t* cols, const int64_t* transpose_perm, void* workspace,
                             size_t workspace_bytes, void* stream) {
    if (!k) return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: NULL kernel set");
    if (!oeq_has_double_backward(k) || !walk_mode(k))
        return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: this kernel set has no second-order kernels");
    if (int bad = check_graph_size("oeq_conv_double_backward", node_count, nnz)) return bad;
    size_t index_bytes = 0;
    if (node_count > 0 && nnz > 0) {
        if (!rows || !cols) return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: NULL buffer");
        if (k->dims.deterministic == OEQ_CONV_SORTED && !transpose_perm)
            return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: deterministic mode needs transpose_perm");
        const IndexLayout w = index_layout(k, node_count, nnz, true);
        const size_t need = w.total + oeq_conv_double_backward_scratch_bytes(k, node_count, nnz);
        if (!workspace || workspace_bytes < need)
            return fail(OEQ_ERR_INVALID, "oeq_conv_double_backward: workspace too small (%zu < %zu bytes)",
                        workspace_bytes, need);
        int rc = build_index(k, "oeq_conv_double_backward", w, node_count, nnz, rows, cols, transpose_perm, workspace,
                             w.total, stream);
        if (rc) return rc;
        index_bytes = w.total;
    }
    return oeq_conv_double_backward_indexed(k, node_count, nnz, L1_in, L2_in, W, L3_grad, L1_dgrad, L2_dgrad, W_dgrad,
                                            L1_grad, L2_grad, W_grad, L3_dgrad, rows, cols, transpose_perm, workspace,
                                            index_bytes, workspace ? (char*)workspace + index_bytes : nullptr,
                                            workspace_bytes > index_bytes ? workspace_bytes - index_bytes : 0, stream);
}

}  // extern "C"
