// Library state: device selection, error policy, the one persistent workspace.
// Counterpart of the reference's common_start / cudaCheck / cublaslt_workspace
// (train_gpt2.cu:1173-1200, llmc/cuda_common.h:52-58, llmc/cublas_common.h:28-31).
#include "common.hpp"
#include <algorithm>
#include "../../include/llmk.h"
#include <cstdarg>
#include <cstring>
#include <map>
#include <string>
#include <vector>

namespace llmk {

void attention_static_scratch_init();     // csrc/attention.hip

static DeviceInfo g_dev;
static int g_error_mode = 0;  // 0: print + exit, 1: record
static std::string g_last_error;
static bool g_failed = false;
static void* g_ws = nullptr;
static size_t g_ws_bytes = 0;

void fail(const char* file, int line, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    char msg[1200];
    snprintf(msg, sizeof msg, "%s at %s:%d", buf, file, line);
    if (g_error_mode == 0) {
        fprintf(stderr, "[llmk] %s\n", msg);
        exit(EXIT_FAILURE);
    }
    g_last_error = msg;
    g_failed = true;
}
bool failed() { return g_failed; }

const DeviceInfo& device_info() {
    if (!g_dev.ready) {
        int dev = 0;
        HIP_CHECK(hipGetDevice(&dev));
        hipDeviceProp_t p;
        HIP_CHECK(hipGetDeviceProperties(&p, dev));
        g_dev.device = dev;
        g_dev.num_cu = p.multiProcessorCount;
        g_dev.max_threads_per_cu = p.maxThreadsPerMultiProcessor;
        g_dev.lds_per_block = p.sharedMemPerBlock;
        snprintf(g_dev.name, sizeof g_dev.name, "%s (%s)", p.name, p.gcnArchName);
        g_dev.ready = true;
    }
    return g_dev;
}

void* workspace(size_t bytes) {
    if (bytes > g_ws_bytes) {
        // grow: happens a handful of times at the start of a run, never in steady state
        if (g_ws) { HIP_CHECK(hipDeviceSynchronize()); HIP_CHECK(hipFree(g_ws)); g_ws = nullptr; }
        size_t want = bytes + bytes / 8;
        HIP_CHECK(hipMalloc(&g_ws, want));
        g_ws_bytes = want;
    }
    return g_ws;
}

// ---- per-kernel event timing -------------------------------------------------------------------
struct ProfRec { const char* name; double flops, bytes; hipEvent_t e0, e1; };
struct ProfAgg { std::string name; int calls = 0; double ms = 0, flops = 0, bytes = 0; };
static bool g_prof_on = false;
static std::vector<ProfRec> g_prof_recs;
static std::vector<hipEvent_t> g_event_pool;
static std::vector<ProfAgg> g_prof_agg;

static std::string g_prof_only;   // when not empty: only this kernel family is timed
bool profiling(const char* name) { return g_prof_on && (g_prof_only.empty() || g_prof_only == name); }
static hipEvent_t take_event() {
    if (!g_event_pool.empty()) { hipEvent_t e = g_event_pool.back(); g_event_pool.pop_back(); return e; }
    hipEvent_t e;
    HIP_CHECK(hipEventCreate(&e));
    return e;
}
void prof_begin(const char* name, double flops, double bytes, hipStream_t st) {
    ProfRec r{name, flops, bytes, take_event(), take_event()};
    HIP_CHECK(hipEventRecord(r.e0, st));
    g_prof_recs.push_back(r);
}
void prof_end(hipStream_t st) { HIP_CHECK(hipEventRecord(g_prof_recs.back().e1, st)); }
static void prof_collect() {
    if (g_prof_recs.empty()) return;
    HIP_CHECK(hipDeviceSynchronize());
    std::map<std::string, size_t> index;
    for (size_t i = 0; i < g_prof_agg.size(); i++) index[g_prof_agg[i].name] = i;
    for (ProfRec& r : g_prof_recs) {
        float ms = 0.f;
        HIP_CHECK(hipEventElapsedTime(&ms, r.e0, r.e1));
        auto it = index.find(r.name);
        if (it == index.end()) { index[r.name] = g_prof_agg.size(); g_prof_agg.push_back(ProfAgg{r.name}); it = index.find(r.name); }
        ProfAgg& a = g_prof_agg[it->second];
        a.calls++; a.ms += ms; a.flops += r.flops; a.bytes += r.bytes;
        g_event_pool.push_back(r.e0);
        g_event_pool.push_back(r.e1);
    }
    g_prof_recs.clear();
}

}  // namespace llmk

namespace {
// 16-byte non-temporal zero stores, a few workgroups per CU striding the buffer
__global__ void __launch_bounds__(256) zero_kernel(float* __restrict__ p, size_t nvec) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const f4 z = {0.f, 0.f, 0.f, 0.f};
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += stride)
        __builtin_nontemporal_store(z, reinterpret_cast<f4*>(p) + i);
}
}  // namespace

extern "C" {

void llmk_profile_enable(int on) { llmk::prof_collect(); llmk::g_prof_on = on != 0; }
void llmk_profile_only(const char* family) { llmk::g_prof_only = family ? family : ""; }
void llmk_profile_reset(void) { llmk::prof_collect(); llmk::g_prof_agg.clear(); }
int llmk_profile_count(void) { llmk::prof_collect(); return (int)llmk::g_prof_agg.size(); }
void llmk_profile_get(int i, char* name64, int* calls, double* ms, double* flops, double* bytes) {
    llmk::prof_collect();
    if (i < 0 || i >= (int)llmk::g_prof_agg.size()) return;
    const llmk::ProfAgg& a = llmk::g_prof_agg[i];
    if (name64) { strncpy(name64, a.name.c_str(), 63); name64[63] = 0; }
    if (calls) *calls = a.calls;
    if (ms) *ms = a.ms;
    if (flops) *flops = a.flops;
    if (bytes) *bytes = a.bytes;
}

void llmk_init(int device) {
    HIP_CHECK(hipSetDevice(device));
    llmk::g_dev.ready = false;
    (void)llmk::device_info();
    llmk::attention_static_scratch_init();       // this device's address of the attention backward's static scratch
}

void llmk_shutdown(void) {
    if (llmk::g_ws) { (void)hipFree(llmk::g_ws); llmk::g_ws = nullptr; llmk::g_ws_bytes = 0; }
}

void llmk_workspace_reserve(size_t bytes) {
    if (llmk::failed()) return;
    (void)llmk::workspace(bytes);
}
size_t llmk_workspace_bytes(void) { return llmk::g_ws_bytes; }

const char* llmk_precision(void) { return LLMK_PRECISION_NAME; }
int llmk_sizeof_floatx(void) { return (int)sizeof(floatX); }

void llmk_device_props(int* num_cu, int* max_threads_per_cu, char* name256) {
    const llmk::DeviceInfo& d = llmk::device_info();
    if (num_cu) *num_cu = d.num_cu;
    if (max_threads_per_cu) *max_threads_per_cu = d.max_threads_per_cu;
    if (name256) { strncpy(name256, d.name, 255); name256[255] = 0; }
}

void llmk_set_error_mode(int record) { llmk::g_error_mode = record ? 1 : 0; }
const char* llmk_last_error(void) { return llmk::g_last_error.c_str(); }
void llmk_clear_error(void) { llmk::g_last_error.clear(); llmk::g_failed = false; }

void llmk_zero(void* ptr, size_t bytes, void* stream) {
    if (llmk::failed() || bytes == 0) return;
    hipStream_t st = (hipStream_t)stream;
    const size_t head = (16 - (uintptr_t)ptr % 16) % 16;          // bytes before the first 16-byte boundary
    if (bytes < head + 16) { HIP_CHECK(hipMemsetAsync(ptr, 0, bytes, st)); return; }
    char* p = (char*)ptr;
    if (head) HIP_CHECK(hipMemsetAsync(p, 0, head, st));
    const size_t nvec = (bytes - head) / 16, tail = bytes - head - nvec * 16;
    llmk::ProfScope prof("zero", 0, (double)nvec * 16, st);
    const size_t want = (nvec + 255) / 256;
    const unsigned grid = (unsigned)std::min(want, (size_t)llmk::device_info().num_cu * 16);
    zero_kernel<<<grid, 256, 0, st>>>((float*)(p + head), nvec);
    LAUNCH_CHECK();
    if (tail) HIP_CHECK(hipMemsetAsync(p + head + nvec * 16, 0, tail, st));
}

}  // extern "C"
