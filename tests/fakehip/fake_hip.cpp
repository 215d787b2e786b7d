// Host-only model of the HIP runtime calls the backend makes; see fake_hip.h for what it checks.
#include "fake_hip.h"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace {

typedef std::map<int, uint64_t> Clock; // stream id -> position in that stream

void merge(Clock &into, const Clock &from) {
    for (const auto &kv : from) {
        uint64_t &v = into[kv.first];
        v = std::max(v, kv.second);
    }
}
struct Stamp {
    int stream = -1;
    uint64_t seq = 0;
};
bool ordered_before(const Stamp &s, const Clock &c) {
    if (s.stream < 0) return true;
    auto it = c.find(s.stream);
    return it != c.end() && it->second >= s.seq;
}

struct Op {
    std::string name;
    std::vector<FakeAccess> accesses;
};
struct Graph {
    std::vector<Op> ops;
};
struct Stream {
    int id;
    Clock clock;
    Graph *capture = nullptr;
};
struct Event {
    Clock clock;
    bool recorded = false;
};
struct Alloc {
    size_t bytes;
    Stamp writer;
    std::vector<Stamp> readers;
    bool owned; // malloc'ed here (false: a symbol's storage)
};
struct Function {
    std::string name;
    std::vector<int> params; // 0 scalar, 1 pointer read, 2 pointer written
};
struct Module {
    std::map<std::string, Function> fns;
};
struct RtcProgram {
    std::string source, log;
};

std::mutex g_mu;
std::map<uintptr_t, Alloc> g_allocs; // base address -> allocation
std::vector<Stream *> g_streams;
Stream g_null{0, {}, nullptr};
int g_next_stream = 1;
Clock g_host;
std::vector<std::string> g_hazards, g_log;
std::map<std::string, unsigned long> g_calls;
hipError_t g_last = hipSuccess;

void hazard(const std::string &m) { g_hazards.push_back(m); }
void count(const char *api) { g_calls[api]++; }

Stream *stream_of(hipStream_t s) { return s ? reinterpret_cast<Stream *>(s) : &g_null; }

Alloc *find_alloc(const void *p, uintptr_t *base = nullptr) {
    const uintptr_t a = (uintptr_t)p;
    auto it = g_allocs.upper_bound(a);
    if (it == g_allocs.begin()) return nullptr;
    --it;
    if (a >= it->first + std::max<size_t>(it->second.bytes, 1)) return nullptr;
    if (base) *base = it->first;
    return &it->second;
}

// One operation enters stream s: it is ordered after everything already in s and after everything the host has
// synchronised with. Checks and updates the allocations it touches.
bool enqueue(Stream *s, const std::string &name, const std::vector<FakeAccess> &acc) {
    if (s->capture) {
        s->capture->ops.push_back({name, acc});
        return true;
    }
    merge(s->clock, g_host);
    const uint64_t seq = ++s->clock[s->id];
    bool known = true;
    char where[96];
    snprintf(where, sizeof where, "%s on stream %d", name.c_str(), s->id);
    // writes after reads of the same allocation by one operation are one access: gather per allocation first
    std::map<Alloc *, bool> touched;
    for (const FakeAccess &a : acc) {
        if (!a.ptr) continue;
        Alloc *al = find_alloc(a.ptr);
        if (!al) {
            hazard(std::string(where) + ": pointer belongs to no live allocation");
            known = false;
            continue;
        }
        touched[al] = touched[al] || a.write;
    }
    for (auto &t : touched) {
        Alloc *al = t.first;
        if (!ordered_before(al->writer, s->clock))
            hazard(std::string(where) + (t.second ? ": write-after-write" : ": read-after-write") + " not ordered after the writer on stream " +
                   std::to_string(al->writer.stream));
        if (t.second) {
            for (const Stamp &r : al->readers)
                if (!ordered_before(r, s->clock))
                    hazard(std::string(where) + ": write-after-read not ordered after a reader on stream " + std::to_string(r.stream));
            al->writer = {s->id, seq};
            al->readers.clear();
        } else {
            al->readers.push_back({s->id, seq});
        }
    }
    return known;
}

void host_sync_all() {
    merge(g_host, g_null.clock);
    for (Stream *s : g_streams) merge(g_host, s->clock);
}

hipError_t fail(hipError_t e) {
    g_last = e;
    return e;
}

} // namespace

// ---- inspection -----------------------------------------------------------------------------------------------------
bool fakehip_launch(hipStream_t stream, const char *name, const std::vector<FakeAccess> &accesses) {
    std::lock_guard<std::mutex> lk(g_mu);
    Stream *s = stream_of(stream);
    if (!s->capture) g_log.push_back(std::string(name) + "@" + std::to_string(s->id));
    return enqueue(s, name, accesses);
}
std::vector<std::string> fakehip_hazards() {
    std::lock_guard<std::mutex> lk(g_mu);
    std::vector<std::string> out;
    out.swap(g_hazards);
    return out;
}
unsigned long fakehip_calls(const char *api) {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_calls.find(api);
    return it == g_calls.end() ? 0 : it->second;
}
std::vector<std::string> fakehip_launch_log() {
    std::lock_guard<std::mutex> lk(g_mu);
    return g_log;
}
void fakehip_live(size_t *n, size_t *bytes) {
    std::lock_guard<std::mutex> lk(g_mu);
    *n = 0;
    *bytes = 0;
    for (auto &kv : g_allocs)
        if (kv.second.owned) {
            ++*n;
            *bytes += kv.second.bytes;
        }
}

// ---- the HIP entry points the backend uses --------------------------------------------------------------------------
extern "C" {

const char *hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : e == hipErrorInvalidValue ? "invalid argument" : "fake HIP error"; }
hipError_t hipGetLastError(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    hipError_t e = g_last;
    g_last = hipSuccess;
    return e;
}
hipError_t hipGetDeviceCount(int *n) {
    *n = 1;
    return hipSuccess;
}
hipError_t hipSetDevice(int d) { return d == 0 ? hipSuccess : hipErrorInvalidDevice; }
hipError_t hipGetDeviceProperties(hipDeviceProp_t *p, int) {
    memset(p, 0, sizeof *p);
    snprintf(p->name, sizeof p->name, "fake MI355X");
    snprintf(p->gcnArchName, sizeof p->gcnArchName, "gfx950:sramecc+:xnack-");
    p->multiProcessorCount = 256;
    p->clockRate = 2400000;
    p->warpSize = 64;
    p->maxThreadsPerBlock = 1024;
    p->sharedMemPerBlock = 65536;
    p->totalGlobalMem = 288ull << 30;
    p->maxGridSize[0] = 2147483647;
    p->maxGridSize[1] = p->maxGridSize[2] = 65535;
    p->maxThreadsDim[0] = p->maxThreadsDim[1] = p->maxThreadsDim[2] = 1024;
    return hipSuccess;
}
hipError_t hipMemGetInfo(size_t *free_b, size_t *total) {
    *free_b = 280ull << 30;
    *total = 288ull << 30;
    return hipSuccess;
}
hipError_t hipMalloc(void **p, size_t bytes) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipMalloc");
    if (bytes > (4ull << 30)) return fail(hipErrorOutOfMemory); // host memory stands in for the device's
    void *m = malloc(bytes ? bytes : 1);
    if (!m) return fail(hipErrorOutOfMemory);
    memset(m, 0xcd, bytes);
    g_allocs[(uintptr_t)m] = Alloc{bytes, {}, {}, true};
    *p = m;
    return hipSuccess;
}
hipError_t hipFree(void *p) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipFree");
    if (!p) return hipSuccess;
    auto it = g_allocs.find((uintptr_t)p);
    if (it == g_allocs.end() || !it->second.owned) {
        hazard("hipFree of a pointer that is not a live allocation");
        return fail(hipErrorInvalidValue);
    }
    host_sync_all(); // hipFree waits for the device
    g_allocs.erase(it);
    free(p);
    return hipSuccess;
}
hipError_t hipGetSymbolAddress(void **p, const void *symbol) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipGetSymbolAddress");
    if (!g_allocs.count((uintptr_t)symbol)) g_allocs[(uintptr_t)symbol] = Alloc{1u << 20, {}, {}, false}; // size unknown here
    *p = const_cast<void *>(symbol);
    return hipSuccess;
}
hipError_t hipMemset(void *p, int v, size_t n) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipMemset");
    host_sync_all();
    if (n && !find_alloc(p)) return fail(hipErrorInvalidValue);
    memset(p, v, n);
    return hipSuccess;
}
hipError_t hipMemsetAsync(void *p, int v, size_t n, hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipMemsetAsync");
    Stream *s = stream_of(st);
    if (s->capture) hazard("hipMemsetAsync recorded into a graph capture (replays of such nodes have given wrong results)");
    enqueue(s, "memset", {{p, true}});
    if (!s->capture) memset(p, v, n);
    return hipSuccess;
}
hipError_t hipMemcpy(void *dst, const void *src, size_t n, hipMemcpyKind kind) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipMemcpy");
    host_sync_all();
    (void)kind;
    memcpy(dst, src, n);
    return hipSuccess;
}
hipError_t hipMemcpyAsync(void *dst, const void *src, size_t n, hipMemcpyKind kind, hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipMemcpyAsync");
    Stream *s = stream_of(st);
    std::vector<FakeAccess> acc;
    if (kind == hipMemcpyHostToDevice || kind == hipMemcpyDeviceToDevice) acc.push_back({dst, true});
    if (kind == hipMemcpyDeviceToHost || kind == hipMemcpyDeviceToDevice) acc.push_back({src, false});
    const bool ok = enqueue(s, kind == hipMemcpyHostToDevice ? "h2d" : kind == hipMemcpyDeviceToHost ? "d2h" : "d2d", acc);
    if (!ok) return fail(hipErrorInvalidValue);
    if (!s->capture) memmove(dst, src, n); // the data moves at once; only the ordering is modelled
    return hipSuccess;
}

hipError_t hipStreamCreateWithFlags(hipStream_t *out, unsigned) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipStreamCreate");
    Stream *s = new Stream{g_next_stream++, {}, nullptr};
    g_streams.push_back(s);
    *out = reinterpret_cast<hipStream_t>(s);
    return hipSuccess;
}
hipError_t hipStreamCreate(hipStream_t *out) { return hipStreamCreateWithFlags(out, 0); }
hipError_t hipStreamDestroy(hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_mu);
    Stream *s = stream_of(st);
    merge(g_host, s->clock);
    g_streams.erase(std::remove(g_streams.begin(), g_streams.end(), s), g_streams.end());
    delete s;
    return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipStreamSynchronize");
    Stream *s = stream_of(st);
    if (s->capture) {
        hazard("hipStreamSynchronize on a capturing stream");
        return fail(hipErrorStreamCaptureUnsupported);
    }
    merge(g_host, s->clock);
    return hipSuccess;
}
hipError_t hipDeviceSynchronize(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipDeviceSynchronize");
    host_sync_all();
    return hipSuccess;
}
hipError_t hipStreamWaitEvent(hipStream_t st, hipEvent_t ev, unsigned) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipStreamWaitEvent");
    Event *e = reinterpret_cast<Event *>(ev);
    if (!e) return fail(hipErrorInvalidValue);
    if (e->recorded) merge(stream_of(st)->clock, e->clock);
    return hipSuccess;
}

hipError_t hipEventCreateWithFlags(hipEvent_t *out, unsigned) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipEventCreate");
    *out = reinterpret_cast<hipEvent_t>(new Event());
    return hipSuccess;
}
hipError_t hipEventCreate(hipEvent_t *out) { return hipEventCreateWithFlags(out, 0); }
hipError_t hipEventDestroy(hipEvent_t ev) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipEventDestroy");
    delete reinterpret_cast<Event *>(ev);
    return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t ev, hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipEventRecord");
    Stream *s = stream_of(st);
    Event *e = reinterpret_cast<Event *>(ev);
    if (s->capture) {
        hazard("hipEventRecord on a capturing stream");
        return fail(hipErrorStreamCaptureUnsupported);
    }
    merge(s->clock, g_host);
    e->clock = s->clock;
    e->recorded = true;
    return hipSuccess;
}
hipError_t hipEventSynchronize(hipEvent_t ev) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipEventSynchronize");
    Event *e = reinterpret_cast<Event *>(ev);
    if (e->recorded) merge(g_host, e->clock);
    return hipSuccess;
}
hipError_t hipEventElapsedTime(float *ms, hipEvent_t, hipEvent_t) {
    *ms = 1.0f;
    return hipSuccess;
}

hipError_t hipStreamBeginCapture(hipStream_t st, hipStreamCaptureMode) {
    std::lock_guard<std::mutex> lk(g_mu);
    Stream *s = stream_of(st);
    if (s->capture) return fail(hipErrorIllegalState);
    s->capture = new Graph();
    return hipSuccess;
}
hipError_t hipStreamEndCapture(hipStream_t st, hipGraph_t *out) {
    std::lock_guard<std::mutex> lk(g_mu);
    Stream *s = stream_of(st);
    if (!s->capture) return fail(hipErrorIllegalState);
    *out = reinterpret_cast<hipGraph_t>(s->capture);
    s->capture = nullptr;
    return hipSuccess;
}
hipError_t hipGraphInstantiate(hipGraphExec_t *out, hipGraph_t g, hipGraphNode_t *, char *, size_t) {
    std::lock_guard<std::mutex> lk(g_mu);
    *out = reinterpret_cast<hipGraphExec_t>(new Graph(*reinterpret_cast<Graph *>(g)));
    return hipSuccess;
}
hipError_t hipGraphLaunch(hipGraphExec_t ex, hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipGraphLaunch");
    Stream *s = stream_of(st);
    bool ok = true;
    for (const Op &op : reinterpret_cast<Graph *>(ex)->ops) {
        g_log.push_back(op.name + "@" + std::to_string(s->id) + " (graph)");
        ok = enqueue(s, op.name, op.accesses) && ok;
    }
    return ok ? hipSuccess : fail(hipErrorInvalidValue);
}
hipError_t hipGraphExecDestroy(hipGraphExec_t ex) {
    delete reinterpret_cast<Graph *>(ex);
    return hipSuccess;
}
hipError_t hipGraphDestroy(hipGraph_t g) {
    delete reinterpret_cast<Graph *>(g);
    return hipSuccess;
}

// ---- run-time compilation: the "code object" is the source text; loading it reads the kernel's signature ----------
hiprtcResult hiprtcVersion(int *major, int *minor) {
    *major = 0;
    *minor = 1;
    return HIPRTC_SUCCESS;
}
const char *hiprtcGetErrorString(hiprtcResult r) { return r == HIPRTC_SUCCESS ? "success" : "fake hiprtc error"; }
hiprtcResult hiprtcCreateProgram(hiprtcProgram *out, const char *src, const char *, int, const char *const *, const char *const *) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hiprtcCreateProgram");
    *out = reinterpret_cast<hiprtcProgram>(new RtcProgram{src, ""});
    return HIPRTC_SUCCESS;
}
hiprtcResult hiprtcCompileProgram(hiprtcProgram p, int, const char *const *) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hiprtcCompileProgram");
    RtcProgram *r = reinterpret_cast<RtcProgram *>(p);
    if (r->source.find("__global__") == std::string::npos) {
        r->log = "no kernel in the source";
        return HIPRTC_ERROR_COMPILATION;
    }
    return HIPRTC_SUCCESS;
}
hiprtcResult hiprtcGetProgramLogSize(hiprtcProgram p, size_t *n) {
    *n = reinterpret_cast<RtcProgram *>(p)->log.size() + 1;
    return HIPRTC_SUCCESS;
}
hiprtcResult hiprtcGetProgramLog(hiprtcProgram p, char *out) {
    strcpy(out, reinterpret_cast<RtcProgram *>(p)->log.c_str());
    return HIPRTC_SUCCESS;
}
hiprtcResult hiprtcGetCodeSize(hiprtcProgram p, size_t *n) {
    *n = reinterpret_cast<RtcProgram *>(p)->source.size() + 1;
    return HIPRTC_SUCCESS;
}
hiprtcResult hiprtcGetCode(hiprtcProgram p, char *out) {
    strcpy(out, reinterpret_cast<RtcProgram *>(p)->source.c_str());
    return HIPRTC_SUCCESS;
}
hiprtcResult hiprtcDestroyProgram(hiprtcProgram *p) {
    delete reinterpret_cast<RtcProgram *>(*p);
    *p = nullptr;
    return HIPRTC_SUCCESS;
}

hipError_t hipModuleLoadData(hipModule_t *out, const void *image) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipModuleLoadData");
    const std::string src((const char *)image);
    Module *m = new Module();
    // every `__global__ ... name(params)`: a parameter with a `*` is a pointer, written unless it starts with `const`
    size_t at = 0;
    while ((at = src.find("__global__", at)) != std::string::npos) {
        const size_t open = src.find('(', src.find("void", at)), close = src.find(')', open);
        size_t name_open = open;
        // the launch-bounds attribute, when present, has its own parentheses before the name's
        const size_t lb = src.find("__launch_bounds__", at);
        if (lb != std::string::npos && lb < open) name_open = src.find('(', src.find(')', lb));
        const size_t name_close = src.find(')', name_open);
        size_t b = name_open;
        while (b > 0 && (isalnum((unsigned char)src[b - 1]) || src[b - 1] == '_')) b--;
        Function f;
        f.name = src.substr(b, name_open - b);
        std::string params = src.substr(name_open + 1, name_close - name_open - 1);
        size_t start = 0;
        while (start <= params.size()) {
            size_t comma = params.find(',', start);
            if (comma == std::string::npos) comma = params.size();
            std::string p = params.substr(start, comma - start);
            const size_t first = p.find_first_not_of(" \n\t");
            if (first != std::string::npos) {
                p = p.substr(first);
                f.params.push_back(p.find('*') == std::string::npos ? 0 : (p.compare(0, 5, "const") == 0 ? 1 : 2));
            }
            start = comma + 1;
        }
        m->fns[f.name] = f;
        at = std::max(close, name_close);
        (void)close;
    }
    *out = reinterpret_cast<hipModule_t>(m);
    return hipSuccess;
}
hipError_t hipModuleGetFunction(hipFunction_t *out, hipModule_t mod, const char *name) {
    std::lock_guard<std::mutex> lk(g_mu);
    Module *m = reinterpret_cast<Module *>(mod);
    auto it = m->fns.find(name);
    if (it == m->fns.end()) return fail(hipErrorNotFound);
    *out = reinterpret_cast<hipFunction_t>(&it->second);
    return hipSuccess;
}
hipError_t hipModuleUnload(hipModule_t mod) {
    std::lock_guard<std::mutex> lk(g_mu);
    count("hipModuleUnload");
    delete reinterpret_cast<Module *>(mod);
    return hipSuccess;
}
hipError_t hipModuleLaunchKernel(hipFunction_t fn, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by, unsigned bz, unsigned,
                                 hipStream_t st, void **args, void **) {
    Function *f = reinterpret_cast<Function *>(fn);
    if (!gx || !gy || !gz || !bx || !by || !bz || (uint64_t)bx * by * bz > 1024) return hipErrorInvalidValue;
    std::vector<FakeAccess> acc;
    for (size_t i = 0; i < f->params.size(); i++)
        if (f->params[i]) acc.push_back({*(void **)args[i], f->params[i] == 2});
    return fakehip_launch(st, f->name.c_str(), acc) ? hipSuccess : hipErrorInvalidValue;
}

} // extern "C"
