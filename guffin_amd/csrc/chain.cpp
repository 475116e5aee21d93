// The chain engine: an HSA queue of the library's own, the library's kernels loaded a second time as plain code
// objects (guffin_amd/hsaco/*.hsaco, built from the same sources with the same flags), and recorded launches
// replayed as AQL dispatch packets.  chain.hpp describes the role and the ordering protocol.
//
// A replay allocates nothing: kernel arguments and packets are laid down once by chain_end.
#include "common.hpp"

#include <dirent.h>
#include <dlfcn.h>
#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>

#include <algorithm>
#include <cstdio>
#include <fstream>
#include <mutex>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

namespace guffin {
namespace chain {
namespace {

constexpr uint32_t kHiddenBytes = 256;     // implicit kernel arguments behind the explicit ones (code object v5)
constexpr uint64_t kWaitNanoseconds = 30ull * 1000 * 1000 * 1000;

struct KernelInfo {
    uint64_t object = 0;
    uint32_t kernarg_size = 0, group = 0, priv = 0;
    int32_t explicit_end = -1, hidden_start = -1;   // from the build's kernarg table; hidden_start < 0: no implicit arguments
    std::string name;
};

struct Engine {
    bool ready = false;
    hsa_agent_t gpu {};
    hsa_queue_t* queue = nullptr;
    std::vector<hsa_executable_t> executables;
    std::unordered_map<std::string, KernelInfo> kernels;          // by mangled name
    std::unordered_map<const void*, const KernelInfo*> by_pointer;
    std::mutex mutex;
};
Engine g_engine;

std::string g_error;
int engine_fail(const std::string& what) {
    g_error = what;
    return fail(GUFFIN_E_HIP, g_error.c_str());
}

std::string hsa_text(hsa_status_t s) {
    const char* m = nullptr;
    hsa_status_string(s, &m);
    return m ? m : "unknown HSA error";
}

std::string library_directory() {
    Dl_info info {};
    if (!dladdr(reinterpret_cast<const void*>(&library_directory), &info) || !info.dli_fname) return ".";
    std::string path = info.dli_fname;
    const size_t slash = path.rfind('/');
    return slash == std::string::npos ? "." : path.substr(0, slash);
}

struct AgentSearch { int wanted, seen; hsa_agent_t found; bool ok; };
hsa_status_t agent_callback(hsa_agent_t agent, void* data) {
    auto* s = static_cast<AgentSearch*>(data);
    hsa_device_type_t type;
    if (hsa_agent_get_info(agent, HSA_AGENT_INFO_DEVICE, &type) != HSA_STATUS_SUCCESS) return HSA_STATUS_SUCCESS;
    if (type != HSA_DEVICE_TYPE_GPU) return HSA_STATUS_SUCCESS;
    if (s->seen++ == s->wanted) { s->found = agent; s->ok = true; }
    return HSA_STATUS_SUCCESS;
}

hsa_status_t symbol_callback(hsa_executable_t, hsa_agent_t, hsa_executable_symbol_t symbol, void* data) {
    auto* e = static_cast<Engine*>(data);
    hsa_symbol_kind_t kind;
    if (hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_TYPE, &kind) != HSA_STATUS_SUCCESS || kind != HSA_SYMBOL_KIND_KERNEL)
        return HSA_STATUS_SUCCESS;
    uint32_t length = 0;
    hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_NAME_LENGTH, &length);
    std::string name(length, '\0');
    hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_NAME, name.data());
    while (!name.empty() && name.back() == '\0') name.pop_back();
    if (name.size() > 3 && name.compare(name.size() - 3, 3, ".kd") == 0) name.resize(name.size() - 3);
    KernelInfo k;
    k.name = name;
    hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_OBJECT, &k.object);
    hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_KERNARG_SEGMENT_SIZE, &k.kernarg_size);
    hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_GROUP_SEGMENT_SIZE, &k.group);
    hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_PRIVATE_SEGMENT_SIZE, &k.priv);
    e->kernels.emplace(name, k);   // a kernel that two sources instantiate is the same code: the first one stays
    return HSA_STATUS_SUCCESS;
}

int load_code_object(Engine& e, const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) return engine_fail("chain: cannot read " + path);
    std::stringstream ss;
    ss << in.rdbuf();
    auto* image = new std::string(ss.str());   // the reader points into the image: it lives as long as the process
    hsa_code_object_reader_t reader;
    hsa_status_t rc = hsa_code_object_reader_create_from_memory(image->data(), image->size(), &reader);
    if (rc != HSA_STATUS_SUCCESS) return engine_fail("chain: code object reader: " + hsa_text(rc));
    hsa_executable_t exe;
    rc = hsa_executable_create_alt(HSA_PROFILE_FULL, HSA_DEFAULT_FLOAT_ROUNDING_MODE_DEFAULT, nullptr, &exe);
    if (rc != HSA_STATUS_SUCCESS) return engine_fail("chain: executable: " + hsa_text(rc));
    rc = hsa_executable_load_agent_code_object(exe, e.gpu, reader, nullptr, nullptr);
    if (rc != HSA_STATUS_SUCCESS) return engine_fail("chain: loading " + path + ": " + hsa_text(rc));
    rc = hsa_executable_freeze(exe, nullptr);
    if (rc != HSA_STATUS_SUCCESS) return engine_fail("chain: freezing " + path + ": " + hsa_text(rc));
    rc = hsa_executable_iterate_agent_symbols(exe, e.gpu, symbol_callback, &e);
    if (rc != HSA_STATUS_SUCCESS) return engine_fail("chain: symbols of " + path + ": " + hsa_text(rc));
    e.executables.push_back(exe);
    return GUFFIN_OK;
}

// the build's table: one line per kernel, "<mangled name> <end of the explicit arguments> <start of the implicit ones or -1>"
int load_kernarg_table(Engine& e, const std::string& path) {
    std::ifstream in(path);
    if (!in) return engine_fail("chain: cannot read " + path);
    std::string name;
    int explicit_end, hidden_start;
    while (in >> name >> explicit_end >> hidden_start) {
        auto it = e.kernels.find(name);
        if (it == e.kernels.end()) continue;
        it->second.explicit_end = explicit_end;
        it->second.hidden_start = hidden_start;
    }
    return GUFFIN_OK;
}

int engine_init() {
    Engine& e = g_engine;
    std::lock_guard<std::mutex> lock(e.mutex);
    if (e.ready) return GUFFIN_OK;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return engine_fail("chain: no current HIP device");
    hsa_status_t rc = hsa_init();   // counted: the HIP runtime holds the runtime open already
    if (rc != HSA_STATUS_SUCCESS) return engine_fail("chain: hsa_init: " + hsa_text(rc));
    AgentSearch search {device, 0, {}, false};
    hsa_iterate_agents(agent_callback, &search);
    if (!search.ok) return engine_fail("chain: no HSA agent for the current device");
    e.gpu = search.found;
    uint32_t max_size = 0;
    hsa_agent_get_info(e.gpu, HSA_AGENT_INFO_QUEUE_MAX_SIZE, &max_size);
    const uint32_t size = std::min<uint32_t>(max_size ? max_size : 4096u, 16384u);
    rc = hsa_queue_create(e.gpu, size, HSA_QUEUE_TYPE_SINGLE, nullptr, nullptr, UINT32_MAX, UINT32_MAX, &e.queue);
    if (rc != HSA_STATUS_SUCCESS) return engine_fail("chain: hsa_queue_create: " + hsa_text(rc));
    // dispatch timestamps for the packets that carry a signal (the first and the last of a replay)
    rc = hsa_amd_profiling_set_profiler_enabled(e.queue, 1);
    if (rc != HSA_STATUS_SUCCESS) return engine_fail("chain: dispatch timestamps: " + hsa_text(rc));
    const std::string dir = library_directory() + "/hsaco";
    DIR* d = opendir(dir.c_str());
    if (!d) return engine_fail("chain: no code objects under " + dir + " (run the build)");
    std::vector<std::string> files;
    while (dirent* entry = readdir(d)) {
        const std::string f = entry->d_name;
        if (f.size() > 6 && f.compare(f.size() - 6, 6, ".hsaco") == 0) files.push_back(dir + "/" + f);
    }
    closedir(d);
    std::sort(files.begin(), files.end());
    if (files.empty()) return engine_fail("chain: no code objects under " + dir + " (run the build)");
    for (const std::string& f : files)
        if (int err = load_code_object(e, f)) return err;
    if (int err = load_kernarg_table(e, dir + "/kernargs.txt")) return err;
    e.ready = true;
    return GUFFIN_OK;
}

struct Launch {
    const KernelInfo* kernel;
    dim3 grid, block;
    uint32_t lds;
    std::vector<uint8_t> args;
};

}  // namespace

struct Recorder {
    hipStream_t stream = nullptr;
    bool recording = false, built = false;
    std::string error;
    std::vector<Launch> launches;
    uint8_t* kernargs = nullptr;           // device
    std::vector<hsa_kernel_dispatch_packet_t> packets;   // headers zero (invalid) until they are copied into the ring
    std::vector<uint16_t> headers;
    hsa_signal_t done {}, started {};   // completion signals of the last and of the first packet
    bool have_signal = false;
    uint64_t replays = 0;
};

namespace {
Recorder* g_active = nullptr;
}  // namespace

Recorder* recorder_for(hipStream_t stream) {
    Recorder* r = g_active;
    return (r && r->recording && r->stream == stream) ? r : nullptr;
}

void record(Recorder* r, const void* host_function, dim3 grid, dim3 block, uint32_t lds_bytes, const void* args,
            uint32_t arg_bytes) {
    if (!r->error.empty()) return;
    Engine& e = g_engine;
    const KernelInfo* k = nullptr;
    auto it = e.by_pointer.find(host_function);
    if (it != e.by_pointer.end()) {
        k = it->second;
    } else {
        const char* name = hipKernelNameRefByPtr(host_function, nullptr);
        auto found = name ? e.kernels.find(name) : e.kernels.end();
        if (found == e.kernels.end()) { r->error = std::string("chain: kernel not in the code objects: ") + (name ? name : "(no name)"); return; }
        k = &found->second;
        e.by_pointer.emplace(host_function, k);
    }
    if (k->explicit_end < 0) { r->error = "chain: no kernarg table entry for " + k->name; return; }
    if (static_cast<int32_t>(arg_bytes) != k->explicit_end) {
        r->error = "chain: argument layout of " + k->name + " differs from the code object's (" + std::to_string(arg_bytes) + " vs "
                 + std::to_string(k->explicit_end) + " bytes)";
        return;
    }
    r->launches.push_back(Launch {k, grid, block, lds_bytes,
                                  std::vector<uint8_t>(static_cast<const uint8_t*>(args), static_cast<const uint8_t*>(args) + arg_bytes)});
}

namespace {

// implicit arguments of one dispatch (code object v5 layout): block counts, group sizes, remainders, global
// offsets (zero), grid dimensions and the dynamic LDS size; the kinds this library's kernels use
void fill_hidden(uint8_t* h, const Launch& l) {
    std::memset(h, 0, kHiddenBytes);
    const uint32_t counts[3] = {l.grid.x, l.grid.y, l.grid.z};
    const uint16_t sizes[3] = {static_cast<uint16_t>(l.block.x), static_cast<uint16_t>(l.block.y), static_cast<uint16_t>(l.block.z)};
    std::memcpy(h, counts, 12);
    std::memcpy(h + 12, sizes, 6);
    const uint16_t dims = l.grid.z > 1 || l.block.z > 1 ? 3 : (l.grid.y > 1 || l.block.y > 1 ? 2 : 1);
    std::memcpy(h + 64, &dims, 2);
    std::memcpy(h + 120, &l.lds, 4);
}

uint16_t packet_header(bool barrier, uint32_t acquire, uint32_t release) {
    return static_cast<uint16_t>((HSA_PACKET_TYPE_KERNEL_DISPATCH << HSA_PACKET_HEADER_TYPE) | ((barrier ? 1u : 0u) << HSA_PACKET_HEADER_BARRIER)
                                 | (acquire << HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE) | (release << HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE));
}

int build(Recorder& r) {
    Engine& e = g_engine;
    if (r.launches.empty()) return fail(GUFFIN_E_STATE, "chain_end: nothing was recorded");
    if (r.launches.size() + 1 > e.queue->size) return fail(GUFFIN_E_CAPACITY, "chain_end: more launches than the queue holds");
    // kernel arguments: explicit, then the implicit block where the kernel has one; 256-byte slots
    std::vector<size_t> offsets;
    size_t total = 0;
    for (const Launch& l : r.launches) {
        offsets.push_back(total);
        const size_t need = l.kernel->hidden_start >= 0 ? size_t(l.kernel->hidden_start) + kHiddenBytes : l.args.size();
        total += (std::max<size_t>(need, l.kernel->kernarg_size) + 255) & ~size_t{255};
    }
    std::vector<uint8_t> host(total, 0);
    for (size_t i = 0; i < r.launches.size(); ++i) {
        const Launch& l = r.launches[i];
        std::memcpy(host.data() + offsets[i], l.args.data(), l.args.size());
        if (l.kernel->hidden_start >= 0) fill_hidden(host.data() + offsets[i] + l.kernel->hidden_start, l);
    }
    if (hipMalloc(reinterpret_cast<void**>(&r.kernargs), total) != hipSuccess) return fail(GUFFIN_E_HIP, "chain_end: kernel argument buffer");
    if (hipMemcpy(r.kernargs, host.data(), total, hipMemcpyHostToDevice) != hipSuccess) return fail(GUFFIN_E_HIP, "chain_end: kernel argument upload");
    hsa_status_t rc = hsa_signal_create(0, 0, nullptr, &r.done);
    if (rc == HSA_STATUS_SUCCESS) rc = hsa_signal_create(0, 0, nullptr, &r.started);
    if (rc != HSA_STATUS_SUCCESS) return engine_fail("chain_end: signal: " + hsa_text(rc));
    r.have_signal = true;
    r.packets.assign(r.launches.size(), hsa_kernel_dispatch_packet_t {});
    r.headers.assign(r.launches.size(), 0);
    for (size_t i = 0; i < r.launches.size(); ++i) {
        const Launch& l = r.launches[i];
        hsa_kernel_dispatch_packet_t& p = r.packets[i];
        const bool three = l.grid.z > 1 || l.block.z > 1, two = l.grid.y > 1 || l.block.y > 1;
        p.setup = static_cast<uint16_t>((three ? 3 : two ? 2 : 1) << HSA_KERNEL_DISPATCH_PACKET_SETUP_DIMENSIONS);
        p.workgroup_size_x = static_cast<uint16_t>(l.block.x);
        p.workgroup_size_y = static_cast<uint16_t>(l.block.y);
        p.workgroup_size_z = static_cast<uint16_t>(l.block.z);
        p.grid_size_x = l.grid.x * l.block.x; p.grid_size_y = l.grid.y * l.block.y; p.grid_size_z = l.grid.z * l.block.z;
        p.private_segment_size = l.kernel->priv;
        p.group_segment_size = l.kernel->group + l.lds;
        p.kernel_object = l.kernel->object;
        p.kernarg_address = r.kernargs + offsets[i];
        p.completion_signal.handle = 0;
        const bool last = i + 1 == r.launches.size();
        if (last) p.completion_signal = r.done;
        else if (i == 0) p.completion_signal = r.started;   // carries the replay's first timestamp
        // the order and visibility of a stream: barrier bit, agent-scope fences; the last launch releases to the host
        r.headers[i] = packet_header(true, HSA_FENCE_SCOPE_AGENT, last ? HSA_FENCE_SCOPE_SYSTEM : HSA_FENCE_SCOPE_AGENT);
    }
    r.built = true;
    return GUFFIN_OK;
}

}  // namespace
}  // namespace chain
}  // namespace guffin

using namespace guffin;
using namespace guffin::chain;

extern "C" int guffin_hip_chain_begin(void* stream, void** out) {
    if (!out) return fail(GUFFIN_E_ARG, "chain_begin: null pointer");
    if (g_active && g_active->recording) return fail(GUFFIN_E_STATE, "chain_begin: another chain is being recorded");
    if (int rc = engine_init()) return rc;
    auto* r = new Recorder();
    r->stream = as_stream(stream);
    r->recording = true;
    g_active = r;
    *out = r;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_chain_end(void* chain) {
    auto* r = static_cast<Recorder*>(chain);
    if (!r || !r->recording) return fail(GUFFIN_E_STATE, "chain_end: the chain is not being recorded");
    r->recording = false;
    if (g_active == r) g_active = nullptr;
    if (!r->error.empty()) { g_error = r->error; return fail(GUFFIN_E_STATE, g_error.c_str()); }
    return build(*r);
}

extern "C" int guffin_hip_chain_launch(void* chain) {
    auto* r = static_cast<Recorder*>(chain);
    if (!r || !r->built) return fail(GUFFIN_E_STATE, "chain_launch: the chain has not been ended");
    Engine& e = g_engine;
    // everything the caller enqueued on the recorded stream before this call comes first
    if (hipStreamSynchronize(r->stream) != hipSuccess) return fail(GUFFIN_E_HIP, "chain_launch: the stream failed");
    hsa_queue_t* q = e.queue;
    const uint64_t n = r->packets.size();
    const uint64_t first = hsa_queue_add_write_index_relaxed(q, n);
    // room in the ring: earlier replays that are still queued are consumed first
    uint64_t spins = 0;
    while (first + n - hsa_queue_load_read_index_scacquire(q) > q->size) {
        if (++spins > (1ull << 34)) return fail(GUFFIN_E_HIP, "chain_launch: the queue does not drain");
    }
    hsa_signal_add_relaxed(r->done, 1);
    if (n > 1) hsa_signal_add_relaxed(r->started, 1);
    r->replays += 1;
    auto* ring = static_cast<hsa_kernel_dispatch_packet_t*>(q->base_address);
    const uint64_t mask = q->size - 1;
    for (uint64_t i = 0; i < n; ++i) {
        hsa_kernel_dispatch_packet_t* slot = ring + ((first + i) & mask);
        const hsa_kernel_dispatch_packet_t& p = r->packets[i];
        // body first, the header (which makes the packet valid) last
        std::memcpy(reinterpret_cast<uint8_t*>(slot) + 4, reinterpret_cast<const uint8_t*>(&p) + 4, sizeof(p) - 4);
        __atomic_store_n(reinterpret_cast<uint32_t*>(slot), uint32_t(r->headers[i]) | (uint32_t(p.setup) << 16), __ATOMIC_RELEASE);
    }
    hsa_signal_store_screlease(q->doorbell_signal, static_cast<hsa_signal_value_t>(first + n - 1));
    return GUFFIN_OK;
}

extern "C" int guffin_hip_chain_wait(void* chain) {
    auto* r = static_cast<Recorder*>(chain);
    if (!r || !r->built) return fail(GUFFIN_E_STATE, "chain_wait: the chain has not been ended");
    const hsa_signal_value_t v = hsa_signal_wait_scacquire(r->done, HSA_SIGNAL_CONDITION_LT, 1, kWaitNanoseconds, HSA_WAIT_STATE_BLOCKED);
    if (v >= 1) return fail(GUFFIN_E_HIP, "chain_wait: the replay did not complete in time");
    return GUFFIN_OK;
}

// Device time of the last replay, from the start of its first dispatch to the end of its last (the reference's
// gpu_duration_ns of a command buffer, metal_command_context.hpp:19-45: GPUEndTime - GPUStartTime).
extern "C" int guffin_hip_chain_gpu_ns(void* chain, uint64_t* nanoseconds) {
    auto* r = static_cast<Recorder*>(chain);
    if (!r || !nanoseconds) return fail(GUFFIN_E_ARG, "chain_gpu_ns: null pointer");
    if (!r->built || r->replays == 0) return fail(GUFFIN_E_STATE, "chain_gpu_ns: no replay has run");
    if (hsa_signal_load_scacquire(r->done) >= 1) return fail(GUFFIN_E_STATE, "chain_gpu_ns: a replay is still running (wait first)");
    hsa_amd_profiling_dispatch_time_t first {}, last {};
    hsa_status_t rc = hsa_amd_profiling_get_dispatch_time(g_engine.gpu, r->done, &last);
    if (rc == HSA_STATUS_SUCCESS) rc = r->packets.size() > 1 ? hsa_amd_profiling_get_dispatch_time(g_engine.gpu, r->started, &first) : rc;
    if (rc != HSA_STATUS_SUCCESS) return engine_fail("chain_gpu_ns: " + hsa_text(rc));
    if (r->packets.size() == 1) first = last;
    uint64_t frequency = 0;
    hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP_FREQUENCY, &frequency);
    if (frequency == 0 || last.end < first.start) return fail(GUFFIN_E_HIP, "chain_gpu_ns: no usable timestamps");
    *nanoseconds = static_cast<uint64_t>(static_cast<double>(last.end - first.start) * 1e9 / static_cast<double>(frequency));
    return GUFFIN_OK;
}

extern "C" int guffin_hip_chain_info(void* chain, uint32_t* launches) {
    auto* r = static_cast<Recorder*>(chain);
    if (!r || !launches) return fail(GUFFIN_E_ARG, "chain_info: null pointer");
    *launches = static_cast<uint32_t>(r->launches.size());
    return GUFFIN_OK;
}

extern "C" int guffin_hip_chain_destroy(void* chain) {
    auto* r = static_cast<Recorder*>(chain);
    if (!r) return GUFFIN_OK;
    if (r->recording) { r->recording = false; if (g_active == r) g_active = nullptr; }
    if (r->built) hsa_signal_wait_scacquire(r->done, HSA_SIGNAL_CONDITION_LT, 1, kWaitNanoseconds, HSA_WAIT_STATE_BLOCKED);
    if (r->have_signal) { hsa_signal_destroy(r->done); hsa_signal_destroy(r->started); }
    if (r->kernargs) (void)hipFree(r->kernargs);
    delete r;
    return GUFFIN_OK;
}
