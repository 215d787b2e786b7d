// Host side of the MI355X HIP backend: the memory pool (caching allocator, async
// copies, scalar variables), the event table, the stream scheduler and the program
// registry behind the C ABI declared in include/zyx_hip.h.
//
// Design points that differ from the slot this fills (zyx/src/backend/hip.rs):
//   * Events are pooled: hipEventCreate/Destroy happen once per slot, a handle is
//     {slot, generation} so a stale or doubly consumed handle is an error, not a crash.
//   * Launch streams are chosen by affinity: a launch goes to the stream that
//     recorded the newest event of its wait list, so a dependency chain stays in one
//     in-order stream and needs no cross-stream wait; independent work round-robins
//     over the 8 launch streams.
//   * Freed blocks are cached by size class together with the events of their last
//     users; a reused block hands those events' completion to its next user through
//     the event zhip_alloc returns. hipMalloc/hipFree (device-wide synchronising)
//     leave the steady-state training step.
#include "../../include/zyx_hip.h"

#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <initializer_list>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "ir_compile.hpp"
#include "rtc_cache.hpp"
#include "kernels/kernels.hpp"

#define ZHIP_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

constexpr int kLaunchStreams = 8; // zyx/src/backend/hip.rs:242-274
constexpr int kMaxArgs = ZHIP_IR_MAX_PARAMS; // arguments of one launch (hand-written kernels take at most 8)
constexpr uint64_t kDefaultCacheBytes = 1ull << 30;
constexpr uint64_t kAllocAlign = 256;
constexpr uint64_t kStaticScratchBytes = 1ull << 20;

thread_local std::string g_init_error;

constexpr int kStreams = kLaunchStreams + 2; // launch streams, then the pool stream, then the plan stream

// Where in which stream a buffer was last written and, per stream, last read. The caller's events say what an
// operation must wait for -- but zyx files one event under ALL buffers of a kernel and consumes it on the first later
// use of ANY of them (zyx/src/runtime.rs:1-16, zyx/src/graph/plan.rs:311-327), so a buffer can lose its event to an
// operation that never touched it. The backend therefore keeps its own record and orders every operation after the
// conflicting accesses of its buffers, whatever the wait list holds; stream positions suffice (no event objects).
struct Stamp {
    int16_t stream = -3; // stream index as in stream_of(); -3 = none
    uint64_t seq = 0;
};
struct Access {
    Stamp writer;
    uint64_t read_seq[kStreams] = {0}; // latest read per stream slot, 0 = none since the last write
};

struct Buffer {
    enum Kind : uint8_t { Free, Memory, Variable } kind = Free;
    Access acc;
    void *ptr = nullptr;
    uint64_t bytes = 0;    // what the caller asked for (bookkeeping unit of free_bytes)
    uint64_t capacity = 0; // size class actually backing it
    int32_t var_dtype = 0;
    uint8_t var_value[8] = {0};
};

struct EventSlot {
    hipEvent_t ev = nullptr;
    uint32_t gen = 1;
    int16_t stream = -1; // launch stream index, -1 = pool stream
    uint64_t seq = 0;    // position in that stream's record order
    bool live = false;
    // An event handle first only names a position in its stream. The hipEvent is recorded when somebody has to wait
    // for it from another stream or from the host -- at the stream's end as it is then, which is at or after the
    // position and so waits for nothing less. Work chained on one stream (the common case: streams run in order and
    // a same-stream wait is skipped) never pays for a record. No wait cycle can arise: whatever was enqueued between
    // the position and the record only waits for events that existed before it, hence before the new waiter.
    bool recorded = false;
    uint64_t covers = 0; // once recorded: the position of its stream the record stands for (>= seq)
};

struct CachedBlock {
    void *ptr;
    std::vector<zhip_event> pending; // last users; owned by the cache
    Access acc;                      // and where they ran: the next owner's first operation is ordered after them
};

struct Program {
    bool live = false;
    zhip_kernel_desc desc{};
    int n_in = 0, n_out = 0;
    uint64_t need[kMaxArgs] = {0}; // minimum bytes per argument
    void *workspace = nullptr; // device scratch owned by the program (two-stage reductions)
    uint64_t workspace_bytes = 0;
    zk::EwJit *jit = nullptr;  // elementwise chains above the size threshold: code specialised at registration
    zk::IrProgram *ir = nullptr; // compiled from a linearized kernel (zhip_compile_ir); desc.kind is 0 then
    // A program's workspace is shared by all its launches: each launch waits for the previous one's event on
    // whatever stream that ran, so two launches with unrelated wait lists never overlap on the scratch memory.
    hipEvent_t ws_event = nullptr;
    int ws_last = 0;           // where the scratch was last used: 0 nowhere yet, 1 a launch (ws_event), 2 a plan (the context's plan_done)
    // A launch only notes its stream: the event is recorded when somebody else (another stream, a plan, the host) has to
    // wait for the scratch, at that stream's end as it is then. Back-to-back launches on one stream, the usual case, pay
    // no record (an event record after every two-kernel program left ~5.5 us between it and the next kernel).
    int ws_stream = 0;
    bool ws_recorded = false;
    int plan_refs = 0;         // live plans whose graphs hold this program's kernels, workspace and code
    // Direct convolution: which weights the re-laid copy in the workspace was made from (buffer, its device address and
    // the position of its last writer). A launch outside a plan that finds them unchanged skips the re-layout kernel.
    zhip_buf conv_w_buf = 0;
    const void *conv_w_ptr = nullptr;
    Stamp conv_w_writer{};
    bool conv_w_valid = false;
};

struct Plan {
    bool live = false;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    size_t n_nodes = 0;
    std::vector<zhip_prog> progs; // distinct programs of the plan
    std::vector<std::pair<zhip_buf, bool>> uses; // every memory buffer of the plan once; true = some node writes it
};

template <class T> struct Slab { // dense ids, lowest free id reused (zyx/src/slab.rs)
    std::vector<T> items;
    std::vector<uint32_t> free_ids;
    uint32_t push(T v) {
        if (!free_ids.empty()) {
            // lowest id first keeps ids dense and deterministic
            size_t best = 0;
            for (size_t i = 1; i < free_ids.size(); i++)
                if (free_ids[i] < free_ids[best]) best = i;
            uint32_t id = free_ids[best];
            free_ids.erase(free_ids.begin() + best);
            items[id] = std::move(v);
            return id;
        }
        items.push_back(std::move(v));
        return (uint32_t)items.size() - 1;
    }
    void remove(uint32_t id) { free_ids.push_back(id); }
};

} // namespace

// Partial results of zhip_reduce_static: device memory that exists from the moment the code object is loaded,
// one copy per GPU, so that entry point never allocates. In host code the name only stands for the symbol;
// its device address is looked up once per context (zhip_init) and kept in zhip_ctx::static_scratch.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

struct zhip_ctx {
    std::mutex mu;
    int device = 0;
    uint32_t debug = 0;
    int64_t ew_jit_min = 1 << 20; // elementwise chains of at least this many elements are compiled at registration
    std::string last_error;
    hipDeviceProp_t prop{};
    zhip_device_info info{};

    hipStream_t pool_stream = nullptr;
    hipStream_t launch_streams[kLaunchStreams] = {nullptr};
    uint64_t stream_seq[kStreams] = {0}; // [kLaunchStreams] = pool stream, [+1] = plan stream
    // seen[w][s]: stream w is ordered after everything stream s held up to this position (through a wait that was
    // enqueued in w); done[s]: the host has seen stream s complete up to this position
    uint64_t seen[kStreams][kStreams] = {{0}};
    uint64_t done[kStreams] = {0};
    hipEvent_t order_ev[kStreams] = {nullptr}; // one per source stream, re-recorded for every cross-stream ordering
    int rr = 0;

    uint64_t free_bytes = 0;
    uint64_t cache_limit = kDefaultCacheBytes, cached_bytes = 0;
    Slab<Buffer> buffers;
    std::map<uint64_t, std::vector<CachedBlock>> cache; // capacity -> blocks
    std::vector<EventSlot> events;
    std::vector<uint32_t> free_events;
    Slab<Program> programs;
    Slab<Plan> plans;
    hipStream_t plan_stream = nullptr; // plans are captured on and replayed into this stream
    hipEvent_t plan_done = nullptr;    // recorded after every plan launch that uses program scratch: one record for all of them
    hipEvent_t prof_a = nullptr, prof_b = nullptr;
    void *static_scratch = nullptr; // this device's copy of `scratch`

    int32_t fail(int32_t status, const char *fmt, ...) __attribute__((format(printf, 3, 4))) {
        char buf[512];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof buf, fmt, ap);
        va_end(ap);
        last_error = buf;
        if (debug & 1) fprintf(stderr, "[zyx-hip] error %d: %s\n", status, buf);
        return status;
    }
};

#define HIPCHK(ctx, call, status)                                                                                     \
    do {                                                                                                              \
        hipError_t e_ = (call);                                                                                       \
        if (e_ != hipSuccess) return (ctx)->fail((status), "%s failed: %s", #call, hipGetErrorString(e_));            \
    } while (0)

namespace {

int slot_of(int stream_idx);
hipStream_t stream_of(zhip_ctx *c, int idx);

uint64_t size_class(uint64_t bytes) {
    if (bytes < kAllocAlign) return kAllocAlign;
    // 8 classes per power of two: at most 12.5% slack, few distinct sizes to cache
    int msb = 63 - __builtin_clzll(bytes);
    uint64_t step = 1ull << (msb > 3 ? msb - 3 : 0);
    if (step < kAllocAlign) step = kAllocAlign;
    return (bytes + step - 1) / step * step;
}

// stream index: 0..7 launch streams, -1 pool stream, -2 plan stream
hipStream_t stream_of(zhip_ctx *c, int idx) {
    return idx == -1 ? c->pool_stream : idx == -2 ? c->plan_stream : c->launch_streams[idx];
}

// Stream slot w now runs after stream slot `from` up to position `upto`, hence also after whatever `from` had been
// ordered after by then. (What `from` waits for later does not carry over; the table only ever under-states.)
void note_ordered(zhip_ctx *c, int w, int from, uint64_t upto) {
    if (c->seen[w][from] < upto) c->seen[w][from] = upto;
    if (upto >= c->stream_seq[from]) // ordered after the stream's present end: its own waits carry over
        for (int k = 0; k < kStreams; k++)
            if (k != w && c->seen[w][k] < c->seen[from][k]) c->seen[w][k] = c->seen[from][k];
}

// Orders stream `stream_idx` after position `st`: nothing to do inside one stream, or when a wait already enqueued
// there, or the host, covers the position; else the source stream's ordering event is recorded at its present end
// (at or after the position) and waited for.
int32_t order_after(zhip_ctx *c, int stream_idx, const Stamp &st, int32_t status) {
    if (st.stream == -3 || st.stream == stream_idx) return ZHIP_OK;
    const int w = slot_of(stream_idx), from = slot_of(st.stream);
    if (c->seen[w][from] >= st.seq || c->done[from] >= st.seq) return ZHIP_OK;
    HIPCHK(c, hipEventRecord(c->order_ev[from], stream_of(c, st.stream)), status);
    HIPCHK(c, hipStreamWaitEvent(stream_of(c, stream_idx), c->order_ev[from], 0), status);
    note_ordered(c, w, from, c->stream_seq[from]);
    return ZHIP_OK;
}
// Before an operation in `stream_idx` reads (write == false) or writes a buffer: after its writer, and a write also
// after every reader.
int32_t order_access(zhip_ctx *c, int stream_idx, const Access &a, bool write, int32_t status) {
    int32_t rc = order_after(c, stream_idx, a.writer, status);
    for (int k = 0; k < kStreams && write && rc == ZHIP_OK; k++)
        if (a.read_seq[k]) rc = order_after(c, stream_idx, Stamp{(int16_t)(k == kLaunchStreams ? -1 : k == kLaunchStreams + 1 ? -2 : k), a.read_seq[k]}, status);
    return rc;
}
// After it was enqueued at position seq.
void stamp_access(Access &a, int stream_idx, uint64_t seq, bool write) {
    if (write) {
        a = Access();
        a.writer = Stamp{(int16_t)stream_idx, seq};
    } else {
        a.read_seq[slot_of(stream_idx)] = seq;
    }
}

int slot_of(int stream_idx) { return stream_idx == -1 ? kLaunchStreams : stream_idx == -2 ? kLaunchStreams + 1 : stream_idx; }

// --- events ---------------------------------------------------------------------
EventSlot *event_lookup(zhip_ctx *c, zhip_event h) {
    if (h == 0) return nullptr;
    uint32_t idx = (uint32_t)(h & 0xffffffffu) - 1, gen = (uint32_t)(h >> 32);
    if (idx >= c->events.size()) return nullptr;
    EventSlot &s = c->events[idx];
    return (s.live && s.gen == gen) ? &s : nullptr;
}
int32_t event_record(zhip_ctx *c, int stream_idx, int32_t status, zhip_event *out) {
    uint32_t idx;
    if (!c->free_events.empty()) {
        idx = c->free_events.back();
        c->free_events.pop_back();
    } else {
        EventSlot s;
        HIPCHK(c, hipEventCreateWithFlags(&s.ev, hipEventDisableTiming), status);
        c->events.push_back(s);
        idx = (uint32_t)c->events.size() - 1;
    }
    EventSlot &s = c->events[idx];
    s.live = true;
    s.recorded = false;
    s.stream = (int16_t)stream_idx;
    s.seq = ++c->stream_seq[slot_of(stream_idx)];
    s.covers = 0;
    *out = ((uint64_t)s.gen << 32) | (uint64_t)(idx + 1);
    return ZHIP_OK;
}
// Records the event if nobody needed it so far (see EventSlot::recorded).
hipError_t event_materialise(zhip_ctx *c, EventSlot *s) {
    if (s->recorded) return hipSuccess;
    hipError_t e = hipEventRecord(s->ev, stream_of(c, s->stream));
    if (e == hipSuccess) {
        s->recorded = true;
        s->covers = c->stream_seq[slot_of(s->stream)]; // the stream's end as it is now
    }
    return e;
}
void event_retire(zhip_ctx *c, EventSlot *s) {
    s->live = false;
    s->gen++;
    if (s->gen == 0) s->gen = 1;
    c->free_events.push_back((uint32_t)(s - c->events.data()));
}
// Makes `stream_idx` wait for every event of the list, then retires them (the call
// consumes its wait list). Events recorded on the same in-order stream need no wait.
int32_t wait_and_consume(zhip_ctx *c, int stream_idx, const zhip_event *evs, size_t n, int32_t status) {
    int32_t rc = ZHIP_OK;
    // Streams run in order: of several events recorded on one stream only the latest needs a wait (a cross-stream
    // wait is the expensive part of a launch on the host). Slot -1 / -2 are the pool and plan streams.
    EventSlot *latest[kStreams] = {nullptr};
    for (size_t i = 0; i < n; i++) {
        if (evs[i] == 0) continue;
        EventSlot *s = event_lookup(c, evs[i]);
        if (!s) {
            rc = c->fail(status, "wait list entry %zu is not a live event (stale or already consumed handle)", i);
            continue;
        }
        if (s->stream != stream_idx) {
            EventSlot *&l = latest[slot_of(s->stream)];
            if (!l || s->seq > l->seq) l = s;
        }
    }
    for (EventSlot *s : latest)
        if (s) {
            const int w = slot_of(stream_idx), from = slot_of(s->stream);
            if (c->seen[w][from] >= s->seq || c->done[from] >= s->seq) continue; // already ordered after that position
            hipError_t e = event_materialise(c, s);
            if (e == hipSuccess) e = hipStreamWaitEvent(stream_of(c, stream_idx), s->ev, 0);
            if (e != hipSuccess) rc = c->fail(status, "hipStreamWaitEvent failed: %s", hipGetErrorString(e));
            else note_ordered(c, w, from, s->covers);
        }
    for (size_t i = 0; i < n; i++)
        if (evs[i] != 0)
            if (EventSlot *s = event_lookup(c, evs[i])) event_retire(c, s);
    return rc;
}

// --- buffers --------------------------------------------------------------------
Buffer *buffer_lookup(zhip_ctx *c, zhip_buf id) {
    if (id >= c->buffers.items.size()) return nullptr;
    Buffer &b = c->buffers.items[id];
    return b.kind == Buffer::Free ? nullptr : &b;
}

// Direct convolution: true when the program's re-laid copy of the weights was made from this very buffer and nothing
// has written it since (same buffer id, same device address, same last writer); records the buffer as the source of
// the copy the coming launch makes otherwise. Call with the launch's arguments before enqueueing it.
bool conv_weights_current(zhip_ctx *c, Program &p, const zhip_buf *args, size_t n_args) {
    if (p.desc.kind != ZHIP_K_CONV2D || n_args < 2) return false;
    Buffer *w = buffer_lookup(c, args[1]);
    if (!w) return false;
    const bool same = p.conv_w_valid && p.conv_w_buf == args[1] && p.conv_w_ptr == w->ptr && p.conv_w_writer.stream == w->acc.writer.stream &&
                      p.conv_w_writer.seq == w->acc.writer.seq;
    p.conv_w_buf = args[1];
    p.conv_w_ptr = w->ptr;
    p.conv_w_writer = w->acc.writer;
    p.conv_w_valid = true;
    return same;
}

void trim_cache(zhip_ctx *c, uint64_t limit) {
    // Blocks go back to the driver largest first; their pending events are waited for
    // by hipFree's own device synchronisation.
    while (c->cached_bytes > limit && !c->cache.empty()) {
        auto it = std::prev(c->cache.end());
        CachedBlock blk = std::move(it->second.back());
        it->second.pop_back();
        uint64_t cap = it->first;
        if (it->second.empty()) c->cache.erase(it);
        for (zhip_event h : blk.pending)
            if (EventSlot *s = event_lookup(c, h)) {
                if (event_materialise(c, s) == hipSuccess) (void)hipEventSynchronize(s->ev);
                event_retire(c, s);
            }
        (void)hipFree(blk.ptr);
        c->cached_bytes -= cap;
    }
}

// --- program registry -----------------------------------------------------------
uint64_t dtype_bytes(int32_t dt) {
    switch (dt) {
    case ZHIP_BF16: case ZHIP_F16: case ZHIP_U16: case ZHIP_I16: return 2;
    case ZHIP_F32: case ZHIP_U32: case ZHIP_I32: return 4;
    case ZHIP_F64: case ZHIP_U64: case ZHIP_I64: return 8;
    case ZHIP_U8: case ZHIP_I8: case ZHIP_BOOL: return 1;
    default: return 0;
    }
}

// Fills arity and per-argument byte requirements; rejects shapes/dtypes no kernel covers.
// Shape parameters of a ZHIP_K_CONV2D descriptor, without pointers.
zk::Conv2d conv_args(const zhip_kernel_desc &d) {
    zk::Conv2d a{};
    a.N = (int)d.dims[0]; a.C = (int)d.dims[1]; a.H = (int)d.dims[2]; a.W = (int)d.dims[3];
    a.Cout = (int)d.dims[4]; a.KH = (int)d.dims[5]; a.KW = (int)d.dims[6];
    a.sy = d.iparams[0]; a.sx = d.iparams[1]; a.py = d.iparams[2]; a.px = d.iparams[3]; a.dy = d.iparams[4]; a.dx = d.iparams[5];
    // 64-bit: registration has bounded every term, the sums of a hostile descriptor must not wrap before it has
    a.OH = (int)(((int64_t)a.H + 2 * (int64_t)a.py - (int64_t)a.dy * (a.KH - 1) - 1) / a.sy + 1);
    a.OW = (int)(((int64_t)a.W + 2 * (int64_t)a.px - (int64_t)a.dx * (a.KW - 1) - 1) / a.sx + 1);
    a.dtype = d.dtype; a.out_dtype = d.out_dtype; a.relu = d.iparams[7]; a.pool = d.iparams[8];
    return a;
}
// the two int32 tap tables at the head of a conv program's workspace, rounded so what follows stays aligned
uint64_t conv_table_bytes(const zhip_kernel_desc &d) { return ((uint64_t)d.dims[1] * d.dims[5] * d.dims[6] * 8 + 255) / 256 * 256; }

// The chain program of a ZHIP_K_ELEMENTWISE descriptor, without pointers.
zk::Elementwise elementwise_args(const zhip_kernel_desc &d) {
    zk::Elementwise a{};
    a.rows = d.dims[0];
    a.cols = d.dims[1];
    a.n_in = d.iparams[0];
    a.n_instr = d.iparams[1];
    a.reg_class = d.dtype;
    a.out_dtype = d.out_dtype;
    for (int k = 0; k < a.n_in; k++) {
        a.in_dtype[k] = d.iparams[2 + k] & 0xff;
        a.in_bcast[k] = (d.iparams[2 + k] >> 8) & 0xff;
        if (a.in_bcast[k] == ZHIP_EW_ROW || a.in_bcast[k] == ZHIP_EW_COL) a.need_rowcol = 1;
    }
    for (int j = 0; j < a.n_instr; j++) a.code[j] = (uint32_t)d.iparams[6 + j];
    for (int k = 0; k < 8; k++) a.consts[k] = d.fparams[k];
    return a;
}

// bf16 problems of K a multiple of 64 and M, N of at least 64 (aligned for 128-bit loads) run on the 256-row
// LDS-tiled kernel, everything else on the general one.
// 16-bit problems (bf16, f16) of K a multiple of 64 and M, N of at least 64 run on the LDS-tiled kernels.
bool gemm_takes_fast_path(const zhip_kernel_desc &d) {
    const int64_t batch = d.dims[3] ? d.dims[3] : 1;
    const float alpha = d.fparams[0] == 0.0f ? 1.0f : d.fparams[0];
    return (d.dtype == ZHIP_BF16 || d.dtype == ZHIP_F16) && batch == 1 && alpha == 1.0f && d.iparams[2] != 2 &&
           zk::gemm_bf16_supported(d.dims[0], d.dims[1], d.dims[2], d.flags & ZHIP_GEMM_TRANS_A ? 1 : 0,
                                   d.flags & ZHIP_GEMM_TRANS_B ? 1 : 0, d.out_dtype != ZHIP_F32);
}

// Shape and scalar parameters of the two attention kinds.
zk::Attention attention_args(const zhip_kernel_desc &d) {
    zk::Attention a{};
    a.B = (int)d.dims[0];
    a.T = (int)d.dims[1];
    a.H = (int)d.dims[2];
    a.dh = (int)d.dims[3];
    a.dtype = d.dtype;
    a.scale = d.fparams[0] > 0.0f ? d.fparams[0] : (float)(1.0 / sqrt((double)a.dh));
    a.keep = 1.0f - d.fparams[1];
    a.causal = d.flags & ZHIP_ATTN_CAUSAL ? 1 : 0;
    return a;
}

// True when the product of the non-negative factors stays below 2^40 (elements; checked without overflowing), the
// bound every tensor of a kernel has to respect so that byte counts and indices fit their types.
bool elems_fit(std::initializer_list<int64_t> factors) {
    uint64_t n = 1;
    for (int64_t f : factors) {
        if (f < 0) return false;
        if (f == 0) return true;
        if ((uint64_t)f >= (1ull << 40) || n > (1ull << 40) / (uint64_t)f) return false;
        n *= (uint64_t)f;
    }
    return n < (1ull << 40);
}

int32_t program_from_desc(zhip_ctx *c, const zhip_kernel_desc &d, Program &p) {
    p.desc = d;
    switch (d.kind) {
    case ZHIP_K_SOFTMAX_ROWS: {
        int64_t rows = d.dims[0], cols = d.dims[1];
        if (d.dtype != ZHIP_F32 && d.dtype != ZHIP_BF16 && d.dtype != ZHIP_F16)
            return c->fail(ZHIP_KERNEL_COMPILATION, "softmax_rows: dtype must be f32, bf16 or f16");
        const uint64_t es = d.dtype == ZHIP_F32 ? 4 : 2;
        if (rows < 0 || cols < 0 || rows >= (1ll << 31) || cols >= (1ll << 31))
            return c->fail(ZHIP_KERNEL_COMPILATION, "softmax_rows: rows/cols out of range");
        if ((d.flags & 7) == 0 || (d.flags & ~7)) return c->fail(ZHIP_KERNEL_COMPILATION, "softmax_rows: bad output flags");
        p.n_in = 1;
        p.need[0] = (uint64_t)rows * cols * es;
        int o = 1;
        if (d.flags & ZHIP_SOFTMAX_Y) p.need[o++] = (uint64_t)rows * cols * es;
        if (d.flags & ZHIP_SOFTMAX_ROWSUM) p.need[o++] = (uint64_t)rows * es;
        if (d.flags & ZHIP_SOFTMAX_ARGMAX) p.need[o++] = (uint64_t)rows * 4;
        p.n_out = o - 1;
        return ZHIP_OK;
    }
    case ZHIP_K_ELEMENTWISE: {
        int64_t rows = d.dims[0], cols = d.dims[1];
        int n_in = d.iparams[0], n_instr = d.iparams[1];
        if (rows < 0 || cols < 0 || (cols && rows > (1ll << 40) / cols))
            return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise: rows/cols out of range");
        if (d.dtype != ZHIP_F32 && d.dtype != ZHIP_I32)
            return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise: register class must be F32 or I32");
        if (n_in < 1 || n_in > 4 || n_instr < 1 || n_instr > ZHIP_EW_MAX_INSTR)
            return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise: %d inputs / %d instructions not supported", n_in, n_instr);
        const bool ireg = d.dtype == ZHIP_I32;
        auto dtype_ok = [&](int dt, bool out) {
            if (ireg) return dt == ZHIP_I32 || dt == ZHIP_U8 || dt == ZHIP_BOOL;
            (void)out;
            return dt == ZHIP_F32 || dt == ZHIP_BF16 || dt == ZHIP_F16 || dt == ZHIP_I32 || dt == ZHIP_U8 || dt == ZHIP_BOOL;
        };
        for (int k = 0; k < n_in; k++) {
            int dt = d.iparams[2 + k] & 0xff, bc = (d.iparams[2 + k] >> 8) & 0xff;
            if (!dtype_ok(dt, false) || bc > ZHIP_EW_SCALAR)
                return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise: input %d has unsupported dtype %d / broadcast %d", k, dt, bc);
            uint64_t elems = bc == ZHIP_EW_FULL ? (uint64_t)rows * cols : bc == ZHIP_EW_ROW ? (uint64_t)cols
                             : bc == ZHIP_EW_COL ? (uint64_t)rows : 1;
            p.need[k] = elems * dtype_bytes(dt);
        }
        if (!dtype_ok(d.out_dtype, true)) return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise: unsupported output dtype %d", d.out_dtype);
        auto src_ok = [&](int s) { return s < n_in || s == ZHIP_EW_SRC_T || (s >= ZHIP_EW_SRC_CONST && s < ZHIP_EW_SRC_CONST + 8); };
        for (int j = 0; j < n_instr; j++) {
            uint32_t ins = (uint32_t)d.iparams[6 + j];
            int op = ins & 0xff, sa = (ins >> 8) & 0xff, sb = (ins >> 16) & 0xff;
            if (op >= ZHIP_EW_OP_COUNT_) return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise: instruction %d: unknown op %d", j, op);
            bool unary = (op >= ZHIP_EW_NEG && op <= ZHIP_EW_ABS) || op >= ZHIP_EW_RELU || op == ZHIP_EW_SAVE;
            if (!unary && !src_ok(sa)) return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise: instruction %d: bad operand %d", j, sa);
            if ((op == ZHIP_EW_WHERE || op == ZHIP_EW_MAD) && !src_ok(sb))
                return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise: instruction %d: bad second operand %d", j, sb);
            bool float_only = (op >= ZHIP_EW_EXP && op <= ZHIP_EW_TRUNC) || op == ZHIP_EW_POW || op == ZHIP_EW_TANH ||
                              op == ZHIP_EW_GELU || op == ZHIP_EW_SIGMOID || op == ZHIP_EW_RSQRT || op == ZHIP_EW_CAST_INT ||
                              op == ZHIP_EW_GELU_GRAD;
            bool int_only = op == ZHIP_EW_BITNOT || (op >= ZHIP_EW_BITXOR && op <= ZHIP_EW_SHR);
            if ((ireg && float_only) || (!ireg && int_only))
                return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise: instruction %d: op %d not defined for this register class", j, op);
            if (j == 0 && op != ZHIP_EW_LOAD) return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise: program must start with LOAD");
        }
        p.n_in = n_in;
        p.n_out = 1;
        p.need[n_in] = (uint64_t)rows * cols * dtype_bytes(d.out_dtype);
        return ZHIP_OK;
    }
    case ZHIP_K_REDUCE: {
        int64_t rows = d.dims[0], cols = d.dims[1];
        if (!zk::reduce_shape_ok(rows, cols, d.flags & 1))
            return c->fail(ZHIP_KERNEL_COMPILATION, "reduce: rows/cols out of range");
        if (d.dtype != ZHIP_F32 && d.dtype != ZHIP_BF16 && d.dtype != ZHIP_F16 && d.dtype != ZHIP_I32)
            return c->fail(ZHIP_KERNEL_COMPILATION, "reduce: dtype %d not implemented", d.dtype);
        if ((d.flags & ~1) || (d.iparams[0] != 0 && d.iparams[0] != 1)) return c->fail(ZHIP_KERNEL_COMPILATION, "reduce: bad flags/op");
        const bool base = d.iparams[1] != 0;
        if ((base || d.fparams[0] != 0.0f || d.fparams[1] != 0.0f) && d.dtype == ZHIP_I32)
            return c->fail(ZHIP_KERNEL_COMPILATION, "reduce: scale / base apply to float dtypes only");
        if (!std::isfinite(d.fparams[0]) || !std::isfinite(d.fparams[1])) return c->fail(ZHIP_KERNEL_COMPILATION, "reduce: scale is not finite");
        p.n_in = base ? 2 : 1;
        p.n_out = 1;
        p.need[0] = (uint64_t)rows * cols * dtype_bytes(d.dtype);
        p.need[1] = (uint64_t)((d.flags & 1) ? cols : rows) * dtype_bytes(d.dtype);
        p.need[2] = p.need[1];
        p.workspace_bytes = zk::reduce_workspace_bytes(rows, cols, d.flags & 1);
        return ZHIP_OK;
    }
    case ZHIP_K_ARGMAX: {
        const int64_t outer = d.dims[0], n = d.dims[1], inner = d.dims[2];
        if (d.dtype != ZHIP_F32 && d.dtype != ZHIP_BF16 && d.dtype != ZHIP_F16 && d.dtype != ZHIP_I32)
            return c->fail(ZHIP_KERNEL_COMPILATION, "argmax: dtype %d not implemented", d.dtype);
        if (d.flags) return c->fail(ZHIP_KERNEL_COMPILATION, "argmax: bad flags");
        if (!zk::argmax_shape_ok(outer, n, inner))
            return c->fail(ZHIP_KERNEL_COMPILATION, "argmax: shape out of range (axis length 1 .. 2^31 - 1)");
        p.n_in = 1;
        p.n_out = 1;
        p.need[0] = (uint64_t)outer * n * inner * dtype_bytes(d.dtype);
        p.need[1] = (uint64_t)outer * inner * 4;
        p.workspace_bytes = zk::argmax_workspace_bytes(outer, n, inner);
        return ZHIP_OK;
    }
    case ZHIP_K_GEMM: {
        int64_t M = d.dims[0], N = d.dims[1], K = d.dims[2], batch = d.dims[3] ? d.dims[3] : 1;
        int epi = d.iparams[0];
        if (M <= 0 || N <= 0 || K <= 0 || batch <= 0 || batch > 65535 || M >= (1ll << 31) || N >= (1ll << 31) || K >= (1ll << 31) ||
            !elems_fit({batch, M, K}) || !elems_fit({batch, K, N}) || !elems_fit({batch, M, N}))
            return c->fail(ZHIP_KERNEL_COMPILATION, "gemm: M, N, K, batch out of range");
        if (epi < 0 || epi > 3 || (d.flags & ~3) || d.iparams[2] < 0 || d.iparams[2] > 2)
            return c->fail(ZHIP_KERNEL_COMPILATION, "gemm: bad epilogue/flags");
        bool float_in = d.dtype == ZHIP_F32 || d.dtype == ZHIP_BF16 || d.dtype == ZHIP_F16;
        if (!float_in || (d.out_dtype != ZHIP_F32 && d.out_dtype != d.dtype))
            return c->fail(ZHIP_KERNEL_COMPILATION, "gemm: no kernel for dtype %d -> %d", d.dtype, d.out_dtype);
        if (epi && d.iparams[1] != ZHIP_BF16 && d.iparams[1] != ZHIP_F32 && d.iparams[1] != ZHIP_F16)
            return c->fail(ZHIP_KERNEL_COMPILATION, "gemm: bias must be bf16, f16 or f32");
        if ((M + 63) / 64 > 65535) return c->fail(ZHIP_KERNEL_COMPILATION, "gemm: M too large for the general kernel");
        int a = 0;
        p.need[a++] = (uint64_t)batch * M * K * dtype_bytes(d.dtype);
        p.need[a++] = (uint64_t)batch * K * N * dtype_bytes(d.dtype);
        if (epi) p.need[a++] = (uint64_t)N * dtype_bytes(d.iparams[1]);
        if (d.iparams[2]) p.need[a++] = (uint64_t)batch * M * N * dtype_bytes(d.out_dtype);
        p.n_in = a;
        p.need[a] = (uint64_t)batch * M * N * dtype_bytes(d.out_dtype);
        p.n_out = 1;
        p.workspace_bytes = gemm_takes_fast_path(d) ? zk::gemm_bf16_workspace_bytes(M, N, K) : zk::gemm_generic_workspace_bytes(M, N, K, batch);
        return ZHIP_OK;
    }
    case ZHIP_K_NORM_ROWS: {
        int64_t rows = d.dims[0], cols = d.dims[1];
        if (rows < 0 || cols < 0 || cols >= (1ll << 31) || (cols && rows > (1ll << 40) / cols))
            return c->fail(ZHIP_KERNEL_COMPILATION, "norm_rows: rows/cols out of range");
        if (d.dtype != ZHIP_F32 && d.dtype != ZHIP_BF16) return c->fail(ZHIP_KERNEL_COMPILATION, "norm_rows: dtype must be F32 or BF16");
        if (d.flags & ~7) return c->fail(ZHIP_KERNEL_COMPILATION, "norm_rows: bad flags");
        uint64_t e = dtype_bytes(d.dtype);
        int a = 0;
        p.need[a++] = (uint64_t)rows * cols * e;
        if (d.flags & ZHIP_NORM_WEIGHT) p.need[a++] = (uint64_t)cols * e;
        if (d.flags & ZHIP_NORM_BIAS) p.need[a++] = (uint64_t)cols * e;
        p.n_in = a;
        p.need[a] = (uint64_t)rows * cols * e;
        p.n_out = 1;
        return ZHIP_OK;
    }
    case ZHIP_K_NORM_ROWS_BWD: {
        int64_t rows = d.dims[0], cols = d.dims[1];
        if (rows < 0 || cols < 0 || cols >= (1ll << 31) || (cols && rows > (1ll << 40) / cols))
            return c->fail(ZHIP_KERNEL_COMPILATION, "norm_rows_bwd: rows/cols out of range");
        if (d.dtype != ZHIP_F32 && d.dtype != ZHIP_BF16) return c->fail(ZHIP_KERNEL_COMPILATION, "norm_rows_bwd: dtype must be F32 or BF16");
        if ((d.flags & ~15) || ((d.flags & ZHIP_NORM_RMS) && (d.flags & ZHIP_NORM_BIAS)))
            return c->fail(ZHIP_KERNEL_COMPILATION, "norm_rows_bwd: bad flags");
        const uint64_t e = dtype_bytes(d.dtype), full = (uint64_t)rows * cols * e;
        int a = 0;
        p.need[a++] = full;
        if (d.flags & ZHIP_NORM_WEIGHT) p.need[a++] = (uint64_t)cols * e;
        p.need[a++] = full;
        if (d.flags & ZHIP_NORM_ADD) p.need[a++] = full;
        p.n_in = a;
        p.need[a++] = full;
        if (d.flags & ZHIP_NORM_WEIGHT) p.need[a++] = (uint64_t)cols * e;
        if (d.flags & ZHIP_NORM_BIAS) p.need[a++] = (uint64_t)cols * e;
        p.n_out = a - p.n_in;
        p.workspace_bytes = zk::norm_rows_bwd_workspace_bytes(rows, cols);
        return ZHIP_OK;
    }
    case ZHIP_K_CROSS_ENTROPY: {
        int64_t rows = d.dims[0], cols = d.dims[1];
        if (rows < 0 || cols < 0 || cols >= (1ll << 31) || (cols && rows > (1ll << 40) / cols))
            return c->fail(ZHIP_KERNEL_COMPILATION, "cross_entropy: rows/cols out of range");
        if (d.dtype != ZHIP_F32) return c->fail(ZHIP_KERNEL_COMPILATION, "cross_entropy: logits must be F32");
        if ((d.flags & 7) == 0 || (d.flags & ~15)) return c->fail(ZHIP_KERNEL_COMPILATION, "cross_entropy: bad output flags");
        if ((d.flags & ZHIP_CE_MEAN) && (rows < 1 || rows > zk::kCrossEntropyMeanRows))
            return c->fail(ZHIP_KERNEL_COMPILATION, "cross_entropy: the mean output takes 1 to %lld rows", (long long)zk::kCrossEntropyMeanRows);
        p.n_in = 2;
        p.need[0] = (uint64_t)rows * cols * 4;
        p.need[1] = (d.flags & ZHIP_CE_DENSE) ? (uint64_t)rows * cols * 4 : (uint64_t)rows * 4;
        int o = 2;
        if (d.flags & ZHIP_CE_LOSS) p.need[o++] = (uint64_t)rows * 4;
        if (d.flags & ZHIP_CE_GRAD) p.need[o++] = (uint64_t)rows * cols * 4;
        if (d.flags & ZHIP_CE_MEAN) p.need[o++] = 4;
        p.n_out = o - 2;
        return ZHIP_OK;
    }
    case ZHIP_K_CONV2D: {
        const int64_t N = d.dims[0], C = d.dims[1], H = d.dims[2], W = d.dims[3], Co = d.dims[4], KH = d.dims[5], KW = d.dims[6];
        const int sy = d.iparams[0], sx = d.iparams[1], py = d.iparams[2], px = d.iparams[3], dy = d.iparams[4], dx = d.iparams[5];
        if (N < 0 || C <= 0 || H <= 0 || W <= 0 || Co <= 0 || KH <= 0 || KW <= 0 || sy <= 0 || sx <= 0 || py < 0 || px < 0 || dy <= 0 || dx <= 0)
            return c->fail(ZHIP_KERNEL_COMPILATION, "conv2d: bad shape or stride/padding/dilation");
        if ((d.dtype != ZHIP_F32 && d.dtype != ZHIP_BF16) || (d.out_dtype != d.dtype && !(d.dtype == ZHIP_BF16 && d.out_dtype == ZHIP_F32)))
            return c->fail(ZHIP_KERNEL_COMPILATION, "conv2d: dtype %d -> %d not implemented", d.dtype, d.out_dtype);
        if (H >= (1ll << 30) || W >= (1ll << 30) || KH >= (1ll << 20) || KW >= (1ll << 20) || sy >= (1 << 20) || sx >= (1 << 20) ||
            py >= (1 << 20) || px >= (1 << 20) || dy >= (1 << 20) || dx >= (1 << 20))
            return c->fail(ZHIP_KERNEL_COMPILATION, "conv2d: size, stride, padding or dilation out of range");
        const int64_t eh = H + 2 * (int64_t)py - (int64_t)dy * (KH - 1) - 1, ew = W + 2 * (int64_t)px - (int64_t)dx * (KW - 1) - 1;
        if (eh < 0 || ew < 0) return c->fail(ZHIP_KERNEL_COMPILATION, "conv2d: kernel larger than the padded input");
        const int64_t OH = eh / sy + 1, OW = ew / sx + 1;
        if (!elems_fit({C, H, W}) || !elems_fit({C, KH, KW}) || !elems_fit({N, OH, OW}) || !elems_fit({N, C, H, W}) ||
            !elems_fit({Co, C, KH, KW}) || !elems_fit({N, Co, OH, OW}) || Co >= (1ll << 31))
            return c->fail(ZHIP_KERNEL_COMPILATION, "conv2d: shape out of range");
        if (C * H * W >= (1ll << 31) || C * KH * KW >= (1ll << 24) || N * OH * OW >= (1ll << 37) || (KH - 1) * dy >= 32768 || (KW - 1) * dx >= 65536)
            return c->fail(ZHIP_KERNEL_COMPILATION, "conv2d: shape out of range");
        const uint64_t e = dtype_bytes(d.dtype);
        int a = 0;
        p.need[a++] = (uint64_t)N * C * H * W * e;
        p.need[a++] = (uint64_t)Co * C * KH * KW * e;
        if (d.iparams[6]) p.need[a++] = (uint64_t)Co * e;
        p.n_in = a;
        p.need[a] = (uint64_t)N * Co * OH * OW * dtype_bytes(d.out_dtype);
        if (d.iparams[8]) { // fused 2 x 2 / stride 2 max-pool: the direct 3 x 3 kernel's shapes with an even number of rows per tile
            if (d.iparams[8] != 1 || !zk::conv3x3_direct_ok(conv_args(d)))
                return c->fail(ZHIP_KERNEL_COMPILATION, "conv2d: the fused 2x2 max-pool needs a 3x3 / stride 1 / padding 1 shape of the direct kernel (C a multiple of 16, Cout of 128, W of 8 and a divisor of 224, H a multiple of 448 / W)");
            p.need[a] = (uint64_t)N * Co * (OH / 2) * (OW / 2) * dtype_bytes(d.out_dtype);
        }
        p.n_out = 1;
        // two int32 tables filled at registration, then (bf16 shapes that run on the tiled GEMM) a zero bias
        // and the patch matrix
        p.workspace_bytes = conv_table_bytes(d) + zk::conv2d_scratch_bytes(conv_args(d));
        return ZHIP_OK;
    }
    case ZHIP_K_MAX_POOL2D: {
        const int64_t planes = d.dims[0], H = d.dims[1], W = d.dims[2], KH = d.dims[3], KW = d.dims[4];
        const int sy = d.iparams[0], sx = d.iparams[1], py = d.iparams[2], px = d.iparams[3], dy = d.iparams[4], dx = d.iparams[5];
        if (planes < 0 || H <= 0 || W <= 0 || KH <= 0 || KW <= 0 || sy <= 0 || sx <= 0 || py < 0 || px < 0 || dy <= 0 || dx <= 0 ||
            H >= (1 << 30) || W >= (1 << 30))
            return c->fail(ZHIP_KERNEL_COMPILATION, "max_pool2d: bad shape or stride/padding/dilation");
        if (d.dtype != ZHIP_F32 && d.dtype != ZHIP_BF16) return c->fail(ZHIP_KERNEL_COMPILATION, "max_pool2d: dtype must be F32 or BF16");
        if (!elems_fit({planes, H, W}) || KH >= (1 << 30) || KW >= (1 << 30))
            return c->fail(ZHIP_KERNEL_COMPILATION, "max_pool2d: tensor too large");
        if (sy >= (1 << 20) || sx >= (1 << 20) || py >= (1 << 20) || px >= (1 << 20) || dy >= (1 << 20) || dx >= (1 << 20))
            return c->fail(ZHIP_KERNEL_COMPILATION, "max_pool2d: stride, padding or dilation out of range");
        const int64_t eh = H + 2 * (int64_t)py - (int64_t)dy * (KH - 1) - 1, ew = W + 2 * (int64_t)px - (int64_t)dx * (KW - 1) - 1;
        if (eh < 0 || ew < 0) return c->fail(ZHIP_KERNEL_COMPILATION, "max_pool2d: window larger than the padded input");
        const uint64_t e = dtype_bytes(d.dtype);
        p.n_in = 1;
        p.n_out = 1;
        p.need[0] = (uint64_t)planes * H * W * e;
        p.need[1] = (uint64_t)planes * (eh / sy + 1) * (ew / sx + 1) * e;
        return ZHIP_OK;
    }
    case ZHIP_K_INDEX: {
        const int axis = d.iparams[0], idt = d.iparams[1];
        if (axis < 0 || axis > 3 || (idt != ZHIP_I32 && idt != ZHIP_I64) || d.flags < 0 || d.flags > 2)
            return c->fail(ZHIP_KERNEL_COMPILATION, "index: bad axis, index dtype or mode");
        uint64_t nx = 1, no = 1;
        for (int k = 0; k < 4; k++) {
            if (d.dims[k] < 0 || d.dims[4 + k] < 0 || d.dims[k] >= (1ll << 31) || d.dims[4 + k] >= (1ll << 31))
                return c->fail(ZHIP_KERNEL_COMPILATION, "index: dimension out of range");
            if (k != axis && d.flags != ZHIP_INDEX_SELECT && d.dims[4 + k] > d.dims[k])
                return c->fail(ZHIP_KERNEL_COMPILATION, "Shape mismatch at dimension %d: self.shape = %lld < indices.shape = %lld", k,
                               (long long)d.dims[k], (long long)d.dims[4 + k]);
            if (k != axis && d.flags == ZHIP_INDEX_SELECT && d.dims[4 + k] != d.dims[k])
                return c->fail(ZHIP_KERNEL_COMPILATION, "index_select: output shape must equal the input's outside the axis");
            nx *= (uint64_t)d.dims[k];
            no *= (uint64_t)d.dims[4 + k];
            if (nx >= (1ull << 40) || no >= (1ull << 40)) return c->fail(ZHIP_KERNEL_COMPILATION, "index: tensor too large"); // < 2^71 here
        }
        const uint64_t e = dtype_bytes(d.dtype), ie = dtype_bytes(idt);
        if (e == 0) return c->fail(ZHIP_KERNEL_COMPILATION, "index: bad dtype");
        if (d.flags == ZHIP_INDEX_SCATTER) {
            if (d.dtype != ZHIP_F32 && d.dtype != ZHIP_F64 && d.dtype != ZHIP_I32 && d.dtype != ZHIP_U32 && d.dtype != ZHIP_I64 && d.dtype != ZHIP_U64)
                return c->fail(ZHIP_KERNEL_COMPILATION, "scatter: dtype %d not implemented", d.dtype);
            p.n_in = 3;
            p.need[0] = nx * e;
            p.need[1] = no * ie;
            p.need[2] = no * e;
            p.need[3] = nx * e;
        } else {
            p.n_in = 2;
            p.need[0] = nx * e;
            p.need[1] = (d.flags == ZHIP_INDEX_SELECT ? (uint64_t)d.dims[4 + axis] : no) * ie;
            p.need[2] = no * e;
        }
        p.n_out = 1;
        return ZHIP_OK;
    }
    case ZHIP_K_ATTENTION:
    case ZHIP_K_ATTENTION_BWD: {
        const int64_t B = d.dims[0], T = d.dims[1], H = d.dims[2], dh = d.dims[3];
        if (B < 0 || T < 0 || H <= 0 || dh <= 0 || dh > 256 || B > 65535 || H > 65535 || B * H > 65535 || T >= (1ll << 24) || B * T * 3 * H * dh >= (1ll << 40))
            return c->fail(ZHIP_KERNEL_COMPILATION, "attention: shape out of range (dh <= 256, B*H <= 65535)");
        if (d.dtype != ZHIP_F32 && d.dtype != ZHIP_BF16) return c->fail(ZHIP_KERNEL_COMPILATION, "attention: dtype must be F32 or BF16");
        if ((d.flags & ~(ZHIP_ATTN_LSE | ZHIP_ATTN_CAUSAL)) || d.fparams[0] < 0.0f || !(d.fparams[1] >= 0.0f && d.fparams[1] < 1.0f))
            return c->fail(ZHIP_KERNEL_COMPILATION, "attention: bad flags, scale or dropout probability");
        const uint64_t e = dtype_bytes(d.dtype);
        if (d.kind == ZHIP_K_ATTENTION_BWD) {
            if (d.flags & ~ZHIP_ATTN_CAUSAL) return c->fail(ZHIP_KERNEL_COMPILATION, "attention backward takes no flag but ZHIP_ATTN_CAUSAL");
            p.n_in = 4;
            p.need[0] = (uint64_t)(B * T * 3 * H * dh) * e;
            p.need[1] = p.need[2] = (uint64_t)(B * T * H * dh) * e;
            p.need[3] = (uint64_t)(B * H * T) * 4;
            p.need[4] = p.need[0];
            p.n_out = 1;
            p.workspace_bytes = zk::attention_bwd_workspace_bytes(attention_args(d));
            return ZHIP_OK;
        }
        p.n_in = 1;
        p.need[0] = (uint64_t)(B * T * 3 * H * dh) * e;
        p.need[1] = (uint64_t)(B * T * H * dh) * e;
        p.n_out = 1;
        if (d.flags & ZHIP_ATTN_LSE) p.need[p.n_out++ + 1] = (uint64_t)(B * H * T) * 4;
        return ZHIP_OK;
    }
    default: return c->fail(ZHIP_KERNEL_COMPILATION, "unknown kernel kind %d", d.kind);
    }
}

// Kinds whose workspace holds constant tables fill them here, once, at registration.
int32_t program_fill_workspace(zhip_ctx *c, Program &p) {
    const zhip_kernel_desc &d = p.desc;
    if (d.kind != ZHIP_K_CONV2D) return ZHIP_OK;
    const int64_t C = d.dims[1], H = d.dims[2], W = d.dims[3], KH = d.dims[5], KW = d.dims[6], K = C * KH * KW;
    const int dy = d.iparams[4], dx = d.iparams[5];
    std::vector<int32_t> tab(2 * K);
    for (int64_t ci = 0; ci < C; ci++)
        for (int64_t ky = 0; ky < KH; ky++)
            for (int64_t kx = 0; kx < KW; kx++) {
                const int64_t k = (ci * KH + ky) * KW + kx;
                tab[k] = (int32_t)(ci * H * W + ky * dy * W + kx * dx);
                tab[K + k] = (int32_t)(((ky * dy) << 16) | (kx * dx));
            }
    HIPCHK(c, hipMemcpy(p.workspace, tab.data(), tab.size() * 4, hipMemcpyHostToDevice), ZHIP_KERNEL_COMPILATION);
    if (p.workspace_bytes > conv_table_bytes(d)) // head of the scratch part: the all-zero bias
        HIPCHK(c, hipMemset((char *)p.workspace + conv_table_bytes(d), 0, 4096 * 4), ZHIP_KERNEL_COMPILATION);
    return ZHIP_OK;
}

hipError_t program_enqueue(const Program &p, void *const *ptr, hipStream_t st, bool conv_weights_ready = false) {
    const zhip_kernel_desc &d = p.desc;
    if (p.ir) {
        // kernel parameters are passed by address: a buffer's is the slot holding its device pointer, a
        // Variable's the bytes of its value (resolve_args left that address in the slot itself)
        void *slots[kMaxArgs];
        for (size_t i = 0; i < p.ir->params.size(); i++)
            slots[i] = p.ir->params[i].kind == ZHIP_IR_VARIABLE ? ptr[i] : (void *)&ptr[i];
        return zk::ir_launch(p.ir, slots, st, nullptr);
    }
    switch (d.kind) {
    case ZHIP_K_SOFTMAX_ROWS: {
        zk::SoftmaxRows a{};
        a.rows = d.dims[0];
        a.cols = d.dims[1];
        a.dtype = d.dtype;
        a.x = ptr[0];
        int o = 1;
        if (d.flags & ZHIP_SOFTMAX_Y) a.y = ptr[o++];
        if (d.flags & ZHIP_SOFTMAX_ROWSUM) a.rowsum = ptr[o++];
        if (d.flags & ZHIP_SOFTMAX_ARGMAX) a.arg = (int32_t *)ptr[o++];
        return zk::softmax_rows(a, st);
    }
    case ZHIP_K_ELEMENTWISE: {
        zk::Elementwise a = elementwise_args(d);
        for (int k = 0; k < a.n_in; k++) a.in[k] = ptr[k];
        a.out = ptr[a.n_in];
        if (zk::ew_jit_can_launch(p.jit, a)) return zk::ew_jit_launch(p.jit, a, st);
        return zk::elementwise(a, st);
    }
    case ZHIP_K_REDUCE: {
        zk::Reduce a{};
        a.rows = d.dims[0];
        a.cols = d.dims[1];
        a.dtype = d.dtype;
        a.op = d.iparams[0];
        a.axis0 = d.flags & 1;
        a.x = ptr[0];
        a.base = d.iparams[1] != 0 ? ptr[1] : nullptr;
        a.out = ptr[p.n_in];
        a.mul = d.fparams[0];
        a.div = d.fparams[1];
        a.workspace = p.workspace;
        a.workspace_bytes = p.workspace_bytes;
        return zk::reduce(a, st);
    }
    case ZHIP_K_ARGMAX: {
        zk::ArgMax a{};
        a.outer = d.dims[0];
        a.n = d.dims[1];
        a.inner = d.dims[2];
        a.dtype = d.dtype;
        a.x = ptr[0];
        a.out = (int32_t *)ptr[1];
        a.workspace = p.workspace;
        a.workspace_bytes = p.workspace_bytes;
        return zk::argmax(a, st);
    }
    case ZHIP_K_GEMM: {
        const int64_t batch = d.dims[3] ? d.dims[3] : 1;
        const float alpha = d.fparams[0] == 0.0f ? 1.0f : d.fparams[0];
        const void *residual = d.iparams[2] ? ptr[p.n_in - 1] : nullptr;
        if (gemm_takes_fast_path(d)) {
            zk::GemmBf16 a{};
            a.M = d.dims[0];
            a.N = d.dims[1];
            a.K = d.dims[2];
            a.trans_a = d.flags & ZHIP_GEMM_TRANS_A ? 1 : 0;
            a.trans_b = d.flags & ZHIP_GEMM_TRANS_B ? 1 : 0;
            a.epilogue = d.iparams[0];
            a.bias_dtype = d.iparams[1];
            a.A = ptr[0];
            a.B = ptr[1];
            a.bias = a.epilogue ? ptr[2] : nullptr;
            a.residual = residual;
            a.out_bf16 = d.out_dtype != ZHIP_F32;
            a.f16 = d.dtype == ZHIP_F16;
            a.C = ptr[p.n_in];
            a.workspace = p.workspace;
            return zk::gemm_bf16(a, st);
        }
        zk::GemmGeneric g{};
        g.M = d.dims[0];
        g.N = d.dims[1];
        g.K = d.dims[2];
        g.batch = batch;
        g.batch_a = g.M * g.K;
        g.batch_b = g.K * g.N;
        g.batch_c = g.M * g.N;
        g.dtype = d.dtype;
        g.out_dtype = d.out_dtype;
        g.trans_a = d.flags & ZHIP_GEMM_TRANS_A ? 1 : 0;
        g.trans_b = d.flags & ZHIP_GEMM_TRANS_B ? 1 : 0;
        g.epilogue = d.iparams[0];
        g.bias_dtype = d.iparams[1];
        g.alpha = alpha;
        g.A = ptr[0];
        g.B = ptr[1];
        g.bias = g.epilogue ? ptr[2] : nullptr;
        g.residual = residual;
        g.residual_is_mask = d.iparams[2] == 2;
        g.workspace = p.workspace;
        g.C = ptr[p.n_in];
        return zk::gemm_generic(g, st);
    }
    case ZHIP_K_NORM_ROWS: {
        zk::NormRows a{};
        a.rows = d.dims[0];
        a.cols = d.dims[1];
        a.dtype = d.dtype;
        a.rms = d.flags & ZHIP_NORM_RMS ? 1 : 0;
        a.eps = d.fparams[0];
        int i = 0;
        a.x = ptr[i++];
        if (d.flags & ZHIP_NORM_WEIGHT) a.w = ptr[i++];
        if (d.flags & ZHIP_NORM_BIAS) a.b = ptr[i++];
        a.y = ptr[i];
        return zk::norm_rows(a, st);
    }
    case ZHIP_K_NORM_ROWS_BWD: {
        zk::NormRowsBwd a{};
        a.rows = d.dims[0];
        a.cols = d.dims[1];
        a.dtype = d.dtype;
        a.rms = d.flags & ZHIP_NORM_RMS ? 1 : 0;
        a.eps = d.fparams[0];
        int i = 0;
        a.x = ptr[i++];
        if (d.flags & ZHIP_NORM_WEIGHT) a.w = ptr[i++];
        a.dy = ptr[i++];
        if (d.flags & ZHIP_NORM_ADD) a.add = ptr[i++];
        a.dx = ptr[i++];
        if (d.flags & ZHIP_NORM_WEIGHT) a.dw = ptr[i++];
        if (d.flags & ZHIP_NORM_BIAS) a.db = ptr[i++];
        a.workspace = p.workspace;
        a.workspace_bytes = p.workspace_bytes;
        return zk::norm_rows_bwd(a, st);
    }
    case ZHIP_K_CROSS_ENTROPY: {
        zk::CrossEntropy a{};
        a.rows = d.dims[0];
        a.cols = d.dims[1];
        a.gscale = d.fparams[0];
        a.x = (const float *)ptr[0];
        if (d.flags & ZHIP_CE_DENSE) a.dense = (const float *)ptr[1];
        else a.labels = (const int32_t *)ptr[1];
        int o = 2;
        if (d.flags & ZHIP_CE_LOSS) a.loss = (float *)ptr[o++];
        if (d.flags & ZHIP_CE_GRAD) a.grad = (float *)ptr[o++];
        if (d.flags & ZHIP_CE_MEAN) a.mean = (float *)ptr[o++];
        return zk::cross_entropy(a, st);
    }
    case ZHIP_K_CONV2D: {
        zk::Conv2d a = conv_args(d);
        a.x = ptr[0]; a.w = ptr[1]; a.bias = d.iparams[6] ? ptr[2] : nullptr; a.y = ptr[p.n_in];
        a.koff = (const int32_t *)p.workspace;
        a.kdyx = a.koff + (int64_t)a.C * a.KH * a.KW;
        if (zk::conv2d_scratch_bytes(a)) a.scratch = (char *)p.workspace + conv_table_bytes(d);
        a.weights_ready = conv_weights_ready;
        return zk::conv2d(a, st);
    }
    case ZHIP_K_MAX_POOL2D: {
        zk::MaxPool2d a{};
        a.planes = d.dims[0]; a.H = (int)d.dims[1]; a.W = (int)d.dims[2]; a.KH = (int)d.dims[3]; a.KW = (int)d.dims[4];
        a.sy = d.iparams[0]; a.sx = d.iparams[1]; a.py = d.iparams[2]; a.px = d.iparams[3]; a.dy = d.iparams[4]; a.dx = d.iparams[5];
        a.OH = (int)(((int64_t)a.H + 2 * (int64_t)a.py - (int64_t)a.dy * (a.KH - 1) - 1) / a.sy + 1);
        a.OW = (int)(((int64_t)a.W + 2 * (int64_t)a.px - (int64_t)a.dx * (a.KW - 1) - 1) / a.sx + 1);
        a.dtype = d.dtype; a.x = ptr[0]; a.y = ptr[1];
        return zk::max_pool2d(a, st);
    }
    case ZHIP_K_INDEX: {
        zk::IndexOp a{};
        for (int k = 0; k < 4; k++) {
            a.xs[k] = d.dims[k];
            a.os[k] = d.dims[4 + k];
        }
        a.axis = d.iparams[0];
        a.idx64 = d.iparams[1] == ZHIP_I64;
        a.dtype = d.dtype;
        a.select = d.flags == ZHIP_INDEX_SELECT;
        a.scatter = d.flags == ZHIP_INDEX_SCATTER;
        a.x = ptr[0];
        a.idx = ptr[1];
        a.src = a.scatter ? ptr[2] : nullptr;
        a.out = ptr[p.n_in];
        return zk::index_op(a, st);
    }
    case ZHIP_K_ATTENTION_BWD: {
        zk::AttentionBwd a{};
        a.fwd = attention_args(d);
        a.fwd.qkv = ptr[0];
        a.fwd.y = ptr[1];
        a.dy = ptr[2];
        a.fwd.lse = (float *)ptr[3];
        a.dqkv = ptr[4];
        a.workspace = p.workspace;
        return zk::attention_bwd(a, st);
    }
    case ZHIP_K_ATTENTION: {
        zk::Attention a = attention_args(d);
        a.qkv = ptr[0];
        a.y = ptr[1];
        a.lse = (d.flags & ZHIP_ATTN_LSE) ? (float *)ptr[2] : nullptr;
        return zk::attention_fwd(a, st);
    }
    default: return hipErrorInvalidValue;
    }
}

// Resolves and checks launch arguments: arity, liveness, kind and size.
int32_t resolve_args(zhip_ctx *c, zhip_prog prog, const zhip_buf *args, size_t n_args, Program **pp, void **ptr) {
    if (prog >= c->programs.items.size() || !c->programs.items[prog].live)
        return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "program %u does not exist", prog);
    Program &p = c->programs.items[prog];
    if (n_args != (size_t)(p.n_in + p.n_out))
        return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "program %u takes %d inputs + %d outputs, got %zu arguments", prog,
                       p.n_in, p.n_out, n_args);
    for (size_t i = 0; i < n_args; i++) {
        Buffer *b = buffer_lookup(c, args[i]);
        if (!b) return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "argument %zu: buffer %u does not exist", i, args[i]);
        if (p.ir && p.ir->params[i].kind == ZHIP_IR_VARIABLE) { // passed by value (cuda.rs:720-726)
            if (b->kind != Buffer::Variable)
                return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "argument %zu: buffer %u is memory, a scalar variable expected", i, args[i]);
            if (b->var_dtype != p.ir->params[i].dtype)
                return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "argument %zu: variable of dtype %d, the kernel takes dtype %d", i,
                               b->var_dtype, p.ir->params[i].dtype);
            ptr[i] = b->var_value;
            continue;
        }
        if (b->kind != Buffer::Memory)
            return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "argument %zu: buffer %u is a scalar variable, memory expected", i,
                           args[i]);
        if (b->bytes < p.need[i])
            return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "argument %zu: buffer %u holds %llu bytes, kernel needs %llu", i,
                           args[i], (unsigned long long)b->bytes, (unsigned long long)p.need[i]);
        ptr[i] = b->ptr;
    }
    // an output must not alias an input or another output: the hand-written kernels assume restrict
    // (generated kernels do not: zyx may hand one buffer to a kernel as source and destination)
    for (size_t i = p.n_in; i < n_args && !p.ir; i++)
        for (size_t j = 0; j < i; j++)
            if (ptr[i] == ptr[j] && p.need[i] && p.need[j])
                return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "arguments %zu and %zu are the same buffer", j, i);
    *pp = &p;
    return ZHIP_OK;
}

// The buffers of a launch: inputs are read, outputs written (a generated kernel may read its outputs as well: a write
// is ordered after everything anyway). Scalar variables are not memory.
int32_t order_args(zhip_ctx *c, int stream_idx, const Program &p, const zhip_buf *args, size_t n_args, int32_t status) {
    for (size_t i = 0; i < n_args; i++) {
        Buffer *b = buffer_lookup(c, args[i]);
        if (!b || b->kind != Buffer::Memory) continue;
        const bool write = p.ir ? p.ir->params[i].kind == ZHIP_IR_GLOBAL_MUT : i >= (size_t)p.n_in;
        int32_t rc = order_access(c, stream_idx, b->acc, write, status);
        if (rc != ZHIP_OK) return rc;
    }
    return ZHIP_OK;
}
void stamp_args(zhip_ctx *c, int stream_idx, uint64_t seq, const Program &p, const zhip_buf *args, size_t n_args) {
    for (int pass = 0; pass < 2; pass++) // reads first: a buffer that is input and output ends up written
        for (size_t i = 0; i < n_args; i++) {
            Buffer *b = buffer_lookup(c, args[i]);
            if (!b || b->kind != Buffer::Memory) continue;
            const bool write = p.ir ? p.ir->params[i].kind == ZHIP_IR_GLOBAL_MUT : i >= (size_t)p.n_in;
            if (write == (pass == 1)) stamp_access(b->acc, stream_idx, seq, write);
        }
}

int pick_stream(zhip_ctx *c, const zhip_event *evs, size_t n, const zhip_buf *args, size_t n_args) {
    int best = -1;
    uint64_t best_seq = 0;
    for (size_t i = 0; i < n; i++)
        if (EventSlot *s = event_lookup(c, evs[i]))
            if (s->stream >= 0 && s->seq >= best_seq) {
                best = s->stream;
                best_seq = s->seq;
            }
    if (best >= 0) return best;
    // no event names a launch stream: follow the stream that last wrote one of the buffers (outputs first), where the
    // launch needs no cross-stream wait for it
    for (size_t i = n_args; i-- > 0;)
        if (Buffer *b = buffer_lookup(c, args[i]))
            if (b->kind == Buffer::Memory && b->acc.writer.stream >= 0 && c->done[b->acc.writer.stream] < b->acc.writer.seq) return b->acc.writer.stream;
    c->rr = (c->rr + 1) % kLaunchStreams;
    return c->rr;
}

void fill_info(zhip_ctx *c) {
    const hipDeviceProp_t &p = c->prop;
    zhip_device_info &i = c->info;
    memset(&i, 0, sizeof i);
    i.compute_units = (uint32_t)p.multiProcessorCount;
    i.clock_khz = (uint32_t)p.clockRate;
    // 4 SIMDs x 16 lanes x 2 (fma) x 2 (dual-issue packed f32) per CU per clock
    i.compute = (uint64_t)p.multiProcessorCount * 256ull * (uint64_t)p.clockRate * 1000ull;
    for (int k = 0; k < 3; k++) {
        i.max_global_work_dims[k] = (uint64_t)p.maxGridSize[k];
        i.max_local_work_dims[k] = (uint32_t)p.maxThreadsDim[k];
    }
    i.max_local_threads = (uint32_t)p.maxThreadsPerBlock;
    i.preferred_vector_size = 16; // 128-bit global loads/stores
    i.local_mem_size = (uint64_t)p.sharedMemPerBlock;
    i.max_register_bytes = 512 * 4; // 512 unified VGPRs per lane
    i.tensor_cores = 1;
    i.warp_size = (uint32_t)p.warpSize;
    for (int d = 0; d < ZHIP_N_DTYPES; d++) i.dtype_capability[d] = 0;
    i.dtype_capability[ZHIP_F32] = 0xffffffffu;
    i.has_native_exp2 = 1;
    i.n_supported_vec_lens = 2;
    i.supported_vec_lens[0] = 2;
    i.supported_vec_lens[1] = 4;
    i.total_bytes = (uint64_t)p.totalGlobalMem;
    snprintf(i.name, sizeof i.name, "%s", p.name[0] ? p.name : "AMD Instinct (name not reported)");
    snprintf(i.arch, sizeof i.arch, "%s", p.gcnArchName);
}

} // namespace

// =================================================================================
// C ABI
// =================================================================================

ZHIP_EXPORT const char *zhip_last_error(zhip_ctx *ctx) { return ctx ? ctx->last_error.c_str() : g_init_error.c_str(); }

ZHIP_EXPORT int32_t zhip_device_count(int32_t *count) {
    if (!count) return ZHIP_DEVICE_ENUMERATION;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *count = 0;
        g_init_error = std::string("hipGetDeviceCount failed: ") + hipGetErrorString(e);
        return ZHIP_DEVICE_ENUMERATION;
    }
    *count = n;
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_init(const zhip_config *cfg, zhip_ctx **out) {
    if (!cfg || !out) {
        g_init_error = "zhip_init: null argument";
        return ZHIP_INITIALIZATION;
    }
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) {
        g_init_error = std::string("no HIP device: ") + (e != hipSuccess ? hipGetErrorString(e) : "device count is 0");
        return ZHIP_DEVICE_ENUMERATION;
    }
    if (cfg->device_id < 0 || cfg->device_id >= n) {
        g_init_error = "device_id " + std::to_string(cfg->device_id) + " out of range, " + std::to_string(n) + " devices";
        return ZHIP_DEVICE_ENUMERATION;
    }
    zhip_ctx *c = new zhip_ctx();
    c->device = cfg->device_id;
    c->debug = cfg->debug;
    if (const char *e = getenv("ZYX_HIP_EW_JIT_MIN")) c->ew_jit_min = atoll(e);
    c->cache_limit = cfg->cache_bytes ? cfg->cache_bytes : kDefaultCacheBytes;
    auto bail = [&](int32_t st, const char *what, hipError_t err) {
        g_init_error = std::string(what) + ": " + hipGetErrorString(err);
        delete c;
        return st;
    };
    if ((e = hipSetDevice(c->device)) != hipSuccess) return bail(ZHIP_INITIALIZATION, "hipSetDevice", e);
    if ((e = hipGetDeviceProperties(&c->prop, c->device)) != hipSuccess) return bail(ZHIP_DEVICE_QUERY, "hipGetDeviceProperties", e);
    if (strncmp(c->prop.gcnArchName, "gfx950", 6) != 0) {
        g_init_error = std::string("device is ") + c->prop.gcnArchName + ", this backend only carries gfx950 code";
        delete c;
        return ZHIP_INITIALIZATION;
    }
    size_t free_b = 0, total_b = 0;
    if ((e = hipMemGetInfo(&free_b, &total_b)) != hipSuccess) return bail(ZHIP_DEVICE_QUERY, "hipMemGetInfo", e);
    c->free_bytes = (uint64_t)free_b;
    if ((e = hipStreamCreateWithFlags(&c->pool_stream, hipStreamNonBlocking)) != hipSuccess)
        return bail(ZHIP_INITIALIZATION, "hipStreamCreate", e);
    for (int i = 0; i < kLaunchStreams; i++)
        if ((e = hipStreamCreateWithFlags(&c->launch_streams[i], hipStreamNonBlocking)) != hipSuccess)
            return bail(ZHIP_INITIALIZATION, "hipStreamCreate", e);
    if ((e = hipStreamCreateWithFlags(&c->plan_stream, hipStreamNonBlocking)) != hipSuccess)
        return bail(ZHIP_INITIALIZATION, "hipStreamCreate", e);
    if ((e = hipEventCreate(&c->prof_a)) != hipSuccess || (e = hipEventCreate(&c->prof_b)) != hipSuccess ||
        (e = hipEventCreateWithFlags(&c->plan_done, hipEventDisableTiming)) != hipSuccess)
        return bail(ZHIP_INITIALIZATION, "hipEventCreate", e);
    for (int k = 0; k < kStreams; k++)
        if ((e = hipEventCreateWithFlags(&c->order_ev[k], hipEventDisableTiming)) != hipSuccess) return bail(ZHIP_INITIALIZATION, "hipEventCreate", e);
    if ((e = hipGetSymbolAddress((void **)&c->static_scratch, HIP_SYMBOL(scratch))) != hipSuccess || !c->static_scratch)
        return bail(ZHIP_INITIALIZATION, "hipGetSymbolAddress of the static scratch array", e);
    if ((e = zk::gemm_bf16_init()) != hipSuccess || (e = zk::gemm_f16_init()) != hipSuccess)
        return bail(ZHIP_INITIALIZATION, "raising the LDS limit of the GEMM kernels", e);
    if ((e = zk::conv3x3_init()) != hipSuccess) return bail(ZHIP_INITIALIZATION, "raising the LDS limit of the convolution kernel", e);
    fill_info(c);
    if (c->debug & 1)
        fprintf(stderr, "[zyx-hip] device %d: %s (%s), %u CUs, %.1f GiB free\n", c->device, c->info.name, c->info.arch,
                c->info.compute_units, (double)c->free_bytes / (1 << 30));
    *out = c;
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_deinit(zhip_ctx *c) {
    if (!c) return ZHIP_DEINITIALIZATION;
    {
        std::lock_guard<std::mutex> lk(c->mu);
        (void)hipSetDevice(c->device);
        (void)hipStreamSynchronize(c->pool_stream);
        for (auto s : c->launch_streams) (void)hipStreamSynchronize(s);
        (void)hipStreamSynchronize(c->plan_stream);
        for (Plan &pl : c->plans.items)
            if (pl.live) {
                (void)hipGraphExecDestroy(pl.exec);
                (void)hipGraphDestroy(pl.graph);
            }
        (void)hipStreamDestroy(c->plan_stream);
        trim_cache(c, 0);
        for (Buffer &b : c->buffers.items)
            if (b.kind == Buffer::Memory) (void)hipFree(b.ptr);
        for (Program &p : c->programs.items) {
            if (p.live && p.workspace) (void)hipFree(p.workspace);
            if (p.live && p.jit) zk::ew_jit_destroy(p.jit);
            if (p.live && p.ir) zk::ir_destroy(p.ir);
            if (p.live && p.ws_event) (void)hipEventDestroy(p.ws_event);
        }
        for (EventSlot &s : c->events) (void)hipEventDestroy(s.ev);
        (void)hipEventDestroy(c->prof_a);
        (void)hipEventDestroy(c->prof_b);
        if (c->plan_done) (void)hipEventDestroy(c->plan_done);
        for (hipEvent_t ev : c->order_ev)
            if (ev) (void)hipEventDestroy(ev);
        (void)hipStreamDestroy(c->pool_stream);
        for (auto s : c->launch_streams) (void)hipStreamDestroy(s);
    }
    delete c;
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_get_device_info(zhip_ctx *c, zhip_device_info *info) {
    if (!c || !info) return ZHIP_DEVICE_QUERY;
    *info = c->info;
    return ZHIP_OK;
}

ZHIP_EXPORT uint64_t zhip_free_bytes(zhip_ctx *c) {
    std::lock_guard<std::mutex> lk(c->mu);
    return c->free_bytes;
}

ZHIP_EXPORT uint64_t zhip_free_compute(zhip_ctx *c) { return c->info.compute; }

ZHIP_EXPORT int32_t zhip_alloc(zhip_ctx *c, uint64_t bytes, zhip_buf *buf, zhip_event *ev) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!buf || !ev) return c->fail(ZHIP_MEMORY_ALLOCATION, "zhip_alloc: null out pointer");
    *buf = ZHIP_NULL_ID;
    *ev = 0;
    if (bytes > c->free_bytes) return c->fail(ZHIP_MEMORY_ALLOCATION, "Allocation failure");
    HIPCHK(c, hipSetDevice(c->device), ZHIP_MEMORY_ALLOCATION);
    uint64_t cap = size_class(bytes ? bytes : 1);
    Buffer b;
    b.kind = Buffer::Memory;
    b.bytes = bytes;
    b.capacity = cap;
    auto it = c->cache.find(cap);
    if (it != c->cache.end()) {
        CachedBlock blk = std::move(it->second.back());
        it->second.pop_back();
        if (it->second.empty()) c->cache.erase(it);
        c->cached_bytes -= cap;
        b.ptr = blk.ptr;
        b.acc = blk.acc; // the first operation on the new buffer is ordered after the block's last users
        if (!blk.pending.empty()) {
            // the previous users' completion becomes the new owner's first dependency
            int32_t rc = wait_and_consume(c, -1, blk.pending.data(), blk.pending.size(), ZHIP_MEMORY_ALLOCATION);
            if (rc == ZHIP_OK) rc = event_record(c, -1, ZHIP_MEMORY_ALLOCATION, ev);
            if (rc != ZHIP_OK) {
                (void)hipStreamSynchronize(c->pool_stream);
                *ev = 0;
            }
        }
    } else {
        hipError_t e = hipMalloc(&b.ptr, cap);
        if (e != hipSuccess) { // give cached blocks back and retry once
            (void)hipGetLastError();
            trim_cache(c, 0);
            e = hipMalloc(&b.ptr, cap);
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return c->fail(ZHIP_MEMORY_ALLOCATION, "hipMalloc(%llu) failed: %s", (unsigned long long)cap, hipGetErrorString(e));
        }
    }
    c->free_bytes -= bytes;
    *buf = c->buffers.push(b);
    if (c->debug & 64) fprintf(stderr, "[zyx-hip] alloc %llu B -> buffer %u @%p\n", (unsigned long long)bytes, *buf, b.ptr);
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_free(zhip_ctx *c, zhip_buf id, const zhip_event *evs, size_t n) {
    std::lock_guard<std::mutex> lk(c->mu);
    Buffer *b = buffer_lookup(c, id);
    if (!b) return c->fail(ZHIP_MEMORY_DEALLOCATION, "buffer %u does not exist", id);
    if (b->kind == Buffer::Variable) {
        for (size_t i = 0; i < n; i++)
            if (EventSlot *s = event_lookup(c, evs[i])) event_retire(c, s);
        b->kind = Buffer::Free;
        c->buffers.remove(id);
        return ZHIP_OK;
    }
    (void)hipSetDevice(c->device);
    CachedBlock blk{b->ptr, {}, b->acc};
    for (size_t i = 0; i < n; i++)
        if (evs[i] != 0 && event_lookup(c, evs[i])) blk.pending.push_back(evs[i]);
    c->free_bytes += b->bytes;
    uint64_t cap = b->capacity;
    b->kind = Buffer::Free;
    b->ptr = nullptr;
    c->buffers.remove(id);
    c->cache[cap].push_back(std::move(blk));
    c->cached_bytes += cap;
    if (c->cached_bytes > c->cache_limit) trim_cache(c, c->cache_limit);
    if (c->debug & 64) fprintf(stderr, "[zyx-hip] free buffer %u\n", id);
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_store_variable(zhip_ctx *c, int32_t dtype, const uint8_t value[8], zhip_buf *buf) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!buf || !value || dtype_bytes(dtype) == 0) return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "store_variable: bad argument");
    Buffer b;
    b.kind = Buffer::Variable;
    b.var_dtype = dtype;
    memcpy(b.var_value, value, 8);
    *buf = c->buffers.push(b);
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_get_variable(zhip_ctx *c, zhip_buf id, int32_t *found, int32_t *dtype, uint8_t value[8]) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!found) return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "get_variable: null out pointer");
    Buffer *b = buffer_lookup(c, id);
    *found = (b && b->kind == Buffer::Variable) ? 1 : 0; // None for memory buffers (backend/mod.rs:609-621)
    if (*found) {
        if (dtype) *dtype = b->var_dtype;
        if (value) memcpy(value, b->var_value, 8);
    }
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_h2d(zhip_ctx *c, const void *src, uint64_t bytes, zhip_buf dst, const zhip_event *evs, size_t n,
                             zhip_event *ev) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!ev) return c->fail(ZHIP_MEMORY_COPY_H2P, "zhip_h2d: null event out pointer");
    *ev = 0;
    HIPCHK(c, hipSetDevice(c->device), ZHIP_MEMORY_COPY_H2P);
    Buffer *b = buffer_lookup(c, dst);
    int32_t rc = wait_and_consume(c, -1, evs, n, ZHIP_MEMORY_COPY_H2P);
    if (rc != ZHIP_OK) return rc;
    if (!b || b->kind != Buffer::Memory) return c->fail(ZHIP_MEMORY_COPY_H2P, "buffer %u is not device memory", dst);
    if (bytes > b->bytes)
        return c->fail(ZHIP_MEMORY_COPY_H2P, "copy of %llu bytes into buffer %u of %llu bytes", (unsigned long long)bytes,
                       dst, (unsigned long long)b->bytes);
    rc = order_access(c, -1, b->acc, true, ZHIP_MEMORY_COPY_H2P);
    if (rc != ZHIP_OK) return rc;
    if (bytes) HIPCHK(c, hipMemcpyAsync(b->ptr, src, bytes, hipMemcpyHostToDevice, c->pool_stream), ZHIP_MEMORY_COPY_H2P);
    rc = event_record(c, -1, ZHIP_MEMORY_COPY_H2P, ev);
    stamp_access(b->acc, -1, c->stream_seq[kLaunchStreams], true);
    return rc;
}

ZHIP_EXPORT int32_t zhip_d2h(zhip_ctx *c, zhip_buf src, void *dst, uint64_t bytes, const zhip_event *evs, size_t n) {
    std::lock_guard<std::mutex> lk(c->mu);
    HIPCHK(c, hipSetDevice(c->device), ZHIP_MEMORY_COPY_P2H);
    Buffer *b = buffer_lookup(c, src);
    int32_t rc = wait_and_consume(c, -1, evs, n, ZHIP_MEMORY_COPY_P2H);
    if (rc != ZHIP_OK) return rc;
    if (!b || b->kind != Buffer::Memory) return c->fail(ZHIP_MEMORY_COPY_P2H, "buffer %u is not device memory", src);
    if (bytes > b->bytes)
        return c->fail(ZHIP_MEMORY_COPY_P2H, "copy of %llu bytes out of buffer %u of %llu bytes", (unsigned long long)bytes,
                       src, (unsigned long long)b->bytes);
    rc = order_access(c, -1, b->acc, false, ZHIP_MEMORY_COPY_P2H);
    if (rc != ZHIP_OK) return rc;
    if (bytes) HIPCHK(c, hipMemcpyAsync(dst, b->ptr, bytes, hipMemcpyDeviceToHost, c->pool_stream), ZHIP_MEMORY_COPY_P2H);
    HIPCHK(c, hipStreamSynchronize(c->pool_stream), ZHIP_MEMORY_COPY_P2H);
    // the pool stream has drained, and with it everything it was ordered after
    c->done[kLaunchStreams] = c->stream_seq[kLaunchStreams];
    for (int k = 0; k < kStreams; k++)
        if (c->done[k] < c->seen[kLaunchStreams][k]) c->done[k] = c->seen[kLaunchStreams][k];
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_d2d(zhip_ctx *c, zhip_buf src, uint64_t src_off, zhip_buf dst, uint64_t dst_off, uint64_t bytes,
                             const zhip_event *evs, size_t n, zhip_event *ev) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!ev) return c->fail(ZHIP_MEMORY_COPY_H2P, "zhip_d2d: null event out pointer");
    *ev = 0;
    HIPCHK(c, hipSetDevice(c->device), ZHIP_MEMORY_COPY_H2P);
    Buffer *s = buffer_lookup(c, src), *d = buffer_lookup(c, dst);
    int32_t rc = wait_and_consume(c, -1, evs, n, ZHIP_MEMORY_COPY_H2P);
    if (rc != ZHIP_OK) return rc;
    if (!s || !d || s->kind != Buffer::Memory || d->kind != Buffer::Memory)
        return c->fail(ZHIP_MEMORY_COPY_H2P, "d2d: buffers %u -> %u are not both device memory", src, dst);
    if (src_off > s->bytes || bytes > s->bytes - src_off || dst_off > d->bytes || bytes > d->bytes - dst_off)
        return c->fail(ZHIP_MEMORY_COPY_H2P, "d2d: %llu bytes at offsets %llu -> %llu exceed a buffer", (unsigned long long)bytes,
                       (unsigned long long)src_off, (unsigned long long)dst_off);
    rc = order_access(c, -1, s->acc, false, ZHIP_MEMORY_COPY_H2P);
    if (rc == ZHIP_OK) rc = order_access(c, -1, d->acc, true, ZHIP_MEMORY_COPY_H2P);
    if (rc != ZHIP_OK) return rc;
    if (bytes) {
        char *to = (char *)d->ptr + dst_off;
        const char *from = (const char *)s->ptr + src_off;
        // small moves go through a copy kernel (cheaper to issue); overlapping ranges of one buffer and large moves
        // through the runtime's copy
        const bool overlap = s == d && src_off < dst_off + bytes && dst_off < src_off + bytes;
        if (bytes <= (4u << 20) && !overlap) HIPCHK(c, zk::copy_range(to, from, bytes, c->pool_stream), ZHIP_MEMORY_COPY_H2P);
        else HIPCHK(c, hipMemcpyAsync(to, from, bytes, hipMemcpyDeviceToDevice, c->pool_stream), ZHIP_MEMORY_COPY_H2P);
    }
    rc = event_record(c, -1, ZHIP_MEMORY_COPY_H2P, ev);
    if (s != d) stamp_access(s->acc, -1, c->stream_seq[kLaunchStreams], false);
    stamp_access(d->acc, -1, c->stream_seq[kLaunchStreams], true);
    return rc;
}

ZHIP_EXPORT int32_t zhip_sync_events(zhip_ctx *c, const zhip_event *evs, size_t n) {
    std::lock_guard<std::mutex> lk(c->mu);
    int32_t rc = ZHIP_OK;
    for (size_t i = 0; i < n; i++) {
        if (evs[i] == 0) continue;
        EventSlot *s = event_lookup(c, evs[i]);
        if (!s) {
            rc = c->fail(ZHIP_KERNEL_SYNC, "event %zu is not live (stale or already consumed handle)", i);
            continue;
        }
        hipError_t e = event_materialise(c, s);
        if (e == hipSuccess) e = hipEventSynchronize(s->ev);
        if (e != hipSuccess) rc = c->fail(ZHIP_KERNEL_SYNC, "hipEventSynchronize failed: %s", hipGetErrorString(e));
        else {
            const int from = slot_of(s->stream);
            if (c->done[from] < s->covers) c->done[from] = s->covers;
        }
        event_retire(c, s);
    }
    return rc;
}

ZHIP_EXPORT int32_t zhip_release_events(zhip_ctx *c, const zhip_event *evs, size_t n) {
    std::lock_guard<std::mutex> lk(c->mu);
    int32_t rc = ZHIP_OK;
    for (size_t i = 0; i < n; i++) {
        if (evs[i] == 0) continue;
        EventSlot *s = event_lookup(c, evs[i]);
        if (!s) rc = c->fail(ZHIP_DEINITIALIZATION, "event %zu is not live (stale or already consumed handle)", i);
        else event_retire(c, s);
    }
    return rc;
}

ZHIP_EXPORT int32_t zhip_buffer_ptr(zhip_ctx *c, zhip_buf id, void **ptr, uint64_t *bytes) {
    std::lock_guard<std::mutex> lk(c->mu);
    Buffer *b = buffer_lookup(c, id);
    if (!b || b->kind != Buffer::Memory) return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "buffer %u is not device memory", id);
    if (ptr) *ptr = b->ptr;
    if (bytes) *bytes = b->bytes;
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_register_kernel(zhip_ctx *c, const zhip_kernel_desc *desc, zhip_prog *prog) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!desc || !prog) return c->fail(ZHIP_KERNEL_COMPILATION, "register_kernel: null argument");
    *prog = ZHIP_NULL_ID;
    Program p;
    int32_t rc = program_from_desc(c, *desc, p);
    if (rc != ZHIP_OK) return rc;
    if (p.workspace_bytes) {
        HIPCHK(c, hipSetDevice(c->device), ZHIP_KERNEL_COMPILATION);
        HIPCHK(c, hipMalloc(&p.workspace, p.workspace_bytes), ZHIP_KERNEL_COMPILATION);
        rc = program_fill_workspace(c, p);
        if (rc != ZHIP_OK) {
            (void)hipFree(p.workspace);
            return rc;
        }
        if (hipEventCreateWithFlags(&p.ws_event, hipEventDisableTiming) != hipSuccess) {
            (void)hipFree(p.workspace);
            return c->fail(ZHIP_KERNEL_COMPILATION, "register_kernel: cannot create the workspace event");
        }
    }
    // Large chains get code generated for exactly this program (zyx compiles every fused kernel at run time,
    // zyx/src/backend/mod.rs:899-933); small ones run on the interpreting kernel, where the ~0.3 s compile
    // would not pay. ZYX_HIP_EW_JIT_MIN overrides the element-count threshold (0 = always, -1 = never).
    if (desc->kind == ZHIP_K_ELEMENTWISE) {
        const zk::Elementwise a = elementwise_args(*desc);
        int v;
        if (c->ew_jit_min >= 0 && a.rows * a.cols >= c->ew_jit_min && zk::ew_jit_eligible(a, &v)) {
            std::string err;
            (void)hipSetDevice(c->device);
            p.jit = zk::ew_jit_compile(a, err);
            if (!p.jit) return c->fail(ZHIP_KERNEL_COMPILATION, "elementwise chain: %s", err.c_str());
        }
    }
    p.live = true;
    *prog = c->programs.push(p);
    if (c->debug & 128) fprintf(stderr, "[zyx-hip] program %u = kind %d\n", *prog, desc->kind);
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_compile_ir(zhip_ctx *c, const void *ir, uint64_t ir_bytes, zhip_prog *prog) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!prog) return c->fail(ZHIP_KERNEL_COMPILATION, "compile_ir: null out pointer");
    *prog = ZHIP_NULL_ID;
    HIPCHK(c, hipSetDevice(c->device), ZHIP_KERNEL_COMPILATION);
    std::string err;
    zk::IrProgram *k = zk::ir_compile(ir, ir_bytes, err);
    if (!k) return c->fail(ZHIP_KERNEL_COMPILATION, "%s", err.c_str());
    if (c->debug & 16) fprintf(stderr, "[zyx-hip] generated kernel:\n%s\n", k->source.substr(k->source.find("extern \"C\"")).c_str());
    Program p;
    p.ir = k;
    for (size_t i = 0; i < k->params.size(); i++) {
        const zk::IrParam &q = k->params[i];
        p.need[i] = q.kind == ZHIP_IR_VARIABLE ? 0 : q.elems * dtype_bytes(q.dtype);
        if (q.kind == ZHIP_IR_GLOBAL_MUT) p.n_out++;
        else p.n_in++;
    }
    p.live = true;
    *prog = c->programs.push(p);
    if (c->debug & 128) fprintf(stderr, "[zyx-hip] program %u = generated kernel, %zu parameters\n", *prog, k->params.size());
    return ZHIP_OK;
}

ZHIP_EXPORT void zhip_compile_cache_stats(uint64_t counts[3]) {
    const zk::RtcCacheStats s = zk::rtc_cache_stats();
    counts[0] = s.compiled;
    counts[1] = s.memory_hits;
    counts[2] = s.disk_hits;
}

ZHIP_EXPORT int32_t zhip_ir_generate(const void *ir, uint64_t ir_bytes, char *buf, uint64_t cap, uint64_t *len) {
    zk::IrProgram k;
    std::string err;
    const bool ok = zk::ir_generate(ir, ir_bytes, k, err);
    const std::string &text = ok ? k.source : err;
    if (len) *len = text.size();
    if (buf && cap) {
        const size_t n = std::min<uint64_t>(cap - 1, text.size());
        memcpy(buf, text.data(), n);
        buf[n] = 0;
    }
    return ok ? ZHIP_OK : ZHIP_KERNEL_COMPILATION;
}

ZHIP_EXPORT int32_t zhip_program_source(zhip_ctx *c, zhip_prog prog, char *buf, uint64_t cap, uint64_t *len) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (prog >= c->programs.items.size() || !c->programs.items[prog].live)
        return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "program %u does not exist", prog);
    const Program &p = c->programs.items[prog];
    const std::string empty;
    const std::string &src = p.ir ? p.ir->source : empty;
    if (len) *len = src.size();
    if (buf && cap) {
        const size_t n = std::min<uint64_t>(cap - 1, src.size());
        memcpy(buf, src.data(), n);
        buf[n] = 0;
    }
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_release_program(zhip_ctx *c, zhip_prog prog) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (prog >= c->programs.items.size() || !c->programs.items[prog].live)
        return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "program %u does not exist", prog);
    Program &p = c->programs.items[prog];
    if (p.plan_refs > 0) return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "program %u is part of %d live plan(s): destroy them first", prog, p.plan_refs);
    if (p.ws_event) {
        (void)hipEventDestroy(p.ws_event);
        p.ws_event = nullptr;
    }
    if (p.workspace) { // hipFree waits for the device, so no launch still uses it
        (void)hipSetDevice(c->device);
        (void)hipFree(p.workspace);
        p.workspace = nullptr;
    }
    if (p.ir) {
        (void)hipSetDevice(c->device);
        (void)hipDeviceSynchronize(); // a launch of the module may still be running
        zk::ir_destroy(p.ir);
        p.ir = nullptr;
    }
    if (p.jit) {
        (void)hipSetDevice(c->device);
        (void)hipDeviceSynchronize(); // a launch of the module may still be running
        zk::ew_jit_destroy(p.jit);
        p.jit = nullptr;
    }
    p.live = false;
    c->programs.remove(prog);
    return ZHIP_OK;
}

// The event somebody else waits on for a program's scratch (ws_last != 0): the context's plan_done, or the program's own
// event, recorded now on the stream of its last launch if that has not been done since.
static hipError_t ws_wait_event(zhip_ctx *c, Program &p, hipEvent_t *out) {
    if (p.ws_last == 2) {
        *out = c->plan_done;
        return hipSuccess;
    }
    if (!p.ws_recorded) {
        hipError_t e = hipEventRecord(p.ws_event, c->launch_streams[p.ws_stream]);
        if (e != hipSuccess) return e;
        p.ws_recorded = true;
    }
    *out = p.ws_event;
    return hipSuccess;
}

ZHIP_EXPORT int32_t zhip_launch(zhip_ctx *c, zhip_prog prog, const zhip_buf *args, size_t n_args, const zhip_event *evs,
                                size_t n_evs, zhip_event *ev) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!ev) return c->fail(ZHIP_KERNEL_LAUNCH, "zhip_launch: null event out pointer");
    *ev = 0;
    Program *p = nullptr;
    void *ptr[kMaxArgs] = {nullptr};
    int32_t rc = resolve_args(c, prog, args, n_args, &p, ptr);
    if (rc != ZHIP_OK) { // nothing enqueued; the wait list is still consumed so no event leaks
        (void)hipSetDevice(c->device);
        for (size_t i = 0; i < n_evs; i++)
            if (EventSlot *s = event_lookup(c, evs[i])) event_retire(c, s);
        return rc;
    }
    HIPCHK(c, hipSetDevice(c->device), ZHIP_KERNEL_LAUNCH);
    int si = pick_stream(c, evs, n_evs, args, n_args);
    rc = wait_and_consume(c, si, evs, n_evs, ZHIP_KERNEL_LAUNCH);
    if (rc == ZHIP_OK) rc = order_args(c, si, *p, args, n_args, ZHIP_KERNEL_LAUNCH);
    if (rc != ZHIP_OK) return rc;
    if (c->debug & 32) fprintf(stderr, "[zyx-hip] launch program %u (kind %d) on stream %d\n", prog, p->desc.kind, si);
    if (p->ws_event && p->ws_last && !(p->ws_last == 1 && p->ws_stream == si)) { // the same stream is ordered by itself
        hipEvent_t w;
        HIPCHK(c, ws_wait_event(c, *p, &w), ZHIP_KERNEL_LAUNCH);
        HIPCHK(c, hipStreamWaitEvent(c->launch_streams[si], w, 0), ZHIP_KERNEL_LAUNCH);
    }
    hipError_t e = program_enqueue(*p, ptr, c->launch_streams[si], conv_weights_current(c, *p, args, n_args));
    if (e != hipSuccess) {
        p->conv_w_valid = false;
        return c->fail(ZHIP_KERNEL_LAUNCH, "launch of program %u failed: %s", prog, hipGetErrorString(e));
    }
    if (p->ws_event) {
        p->ws_last = 1;
        p->ws_stream = si;
        p->ws_recorded = false;
    }
    rc = event_record(c, si, ZHIP_KERNEL_LAUNCH, ev);
    stamp_args(c, si, c->stream_seq[si], *p, args, n_args);
    return rc;
}

ZHIP_EXPORT int32_t zhip_reduce_static(zhip_ctx *c, int32_t dtype, int32_t op, int32_t axis0, int64_t rows, int64_t cols,
                                       const void *x, void *out, void *stream) {
    if (!c) return ZHIP_KERNEL_LAUNCH;
    std::lock_guard<std::mutex> lk(c->mu);
    if (dtype != ZHIP_F32 && dtype != ZHIP_BF16 && dtype != ZHIP_F16 && dtype != ZHIP_I32)
        return c->fail(ZHIP_KERNEL_COMPILATION, "reduce_static: dtype %d not implemented", dtype);
    if ((op != 0 && op != 1) || (axis0 != 0 && axis0 != 1)) return c->fail(ZHIP_KERNEL_COMPILATION, "reduce_static: bad op/axis");
    if (!zk::reduce_shape_ok(rows, cols, axis0)) return c->fail(ZHIP_KERNEL_COMPILATION, "reduce_static: rows/cols out of range");
    const uint64_t need = zk::reduce_workspace_bytes(rows, cols, axis0);
    if (need > kStaticScratchBytes)
        return c->fail(ZHIP_KERNEL_COMPILATION,
                       "reduce_static: a %lld x %lld reduce over axis %d needs %llu bytes of partial results, the static "
                       "scratch holds %llu; use zhip_register_kernel + zhip_launch for this shape",
                       (long long)rows, (long long)cols, axis0 ? 0 : 1, (unsigned long long)need, (unsigned long long)kStaticScratchBytes);
    const int64_t n_in = rows * cols, n_out = axis0 ? cols : rows;
    if ((n_in && !x) || (n_out && !out)) return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "reduce_static: null device pointer");
    HIPCHK(c, hipSetDevice(c->device), ZHIP_KERNEL_LAUNCH);
    zk::Reduce a{};
    a.rows = rows;
    a.cols = cols;
    a.dtype = dtype;
    a.op = op;
    a.axis0 = axis0;
    a.x = x;
    a.out = out;
    a.workspace = c->static_scratch;
    a.workspace_bytes = kStaticScratchBytes;
    hipError_t e = zk::reduce(a, (hipStream_t)stream);
    if (e != hipSuccess) return c->fail(ZHIP_KERNEL_LAUNCH, "reduce_static: launch failed: %s", hipGetErrorString(e));
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_measure_ceilings(zhip_ctx *c, uint64_t bytes, zhip_ceilings *out) {
    static_assert(sizeof(zhip_ceilings) == sizeof(zk::Ceilings), "zhip_ceilings and zk::Ceilings are one layout");
    if (!c) return ZHIP_DEVICE_QUERY;
    std::lock_guard<std::mutex> lk(c->mu);
    if (!out || bytes < (1u << 20)) return c->fail(ZHIP_DEVICE_QUERY, "measure_ceilings: null result or fewer than 1 MiB");
    HIPCHK(c, hipSetDevice(c->device), ZHIP_DEVICE_QUERY);
    HIPCHK(c, hipStreamSynchronize(c->launch_streams[0]), ZHIP_KERNEL_SYNC);
    zk::Ceilings r{};
    hipError_t e = zk::measure_ceilings(bytes, (int)c->info.compute_units, &r, c->launch_streams[0]);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return c->fail(ZHIP_DEVICE_QUERY, "measure_ceilings failed: %s", hipGetErrorString(e));
    }
    memcpy(out, &r, sizeof r);
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_time_kernel(zhip_ctx *c, zhip_prog prog, const zhip_buf *args, size_t n_args, uint64_t *ns) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!ns) return c->fail(ZHIP_KERNEL_LAUNCH, "zhip_time_kernel: null out pointer");
    Program *p = nullptr;
    void *ptr[kMaxArgs] = {nullptr};
    int32_t rc = resolve_args(c, prog, args, n_args, &p, ptr);
    if (rc != ZHIP_OK) return rc;
    HIPCHK(c, hipSetDevice(c->device), ZHIP_KERNEL_LAUNCH);
    hipStream_t st = c->launch_streams[0];
    if (p->ws_event && p->ws_last) {
        hipEvent_t w;
        HIPCHK(c, ws_wait_event(c, *p, &w), ZHIP_KERNEL_SYNC);
        HIPCHK(c, hipEventSynchronize(w), ZHIP_KERNEL_SYNC);
    }
    rc = order_args(c, 0, *p, args, n_args, ZHIP_KERNEL_LAUNCH);
    if (rc != ZHIP_OK) return rc;
    HIPCHK(c, hipStreamSynchronize(st), ZHIP_KERNEL_SYNC);
    p->conv_w_valid = false; // timed in full, re-layout included
    (void)conv_weights_current(c, *p, args, n_args);
    auto t0 = std::chrono::steady_clock::now();
    hipError_t e = program_enqueue(*p, ptr, st);
    if (e != hipSuccess) return c->fail(ZHIP_KERNEL_LAUNCH, "launch of program %u failed: %s", prog, hipGetErrorString(e));
    HIPCHK(c, hipStreamSynchronize(st), ZHIP_KERNEL_SYNC);
    stamp_args(c, 0, ++c->stream_seq[0], *p, args, n_args);
    c->done[0] = c->stream_seq[0];
    *ns = (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t0).count();
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_profile_kernel(zhip_ctx *c, zhip_prog prog, const zhip_buf *args, size_t n_args, size_t arg_sets,
                                        int32_t iters, float *avg_us) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!avg_us || iters <= 0 || arg_sets == 0 || arg_sets > 64)
        return c->fail(ZHIP_KERNEL_LAUNCH, "zhip_profile_kernel: bad argument");
    std::vector<void *> ptrs(arg_sets * kMaxArgs, nullptr);
    Program *p = nullptr;
    for (size_t s = 0; s < arg_sets; s++) {
        int32_t rc = resolve_args(c, prog, args + s * n_args, n_args, &p, &ptrs[s * kMaxArgs]);
        if (rc != ZHIP_OK) return rc;
    }
    HIPCHK(c, hipSetDevice(c->device), ZHIP_KERNEL_LAUNCH);
    hipStream_t st = c->launch_streams[0];
    if (p->ws_event && p->ws_last) {
        hipEvent_t w;
        HIPCHK(c, ws_wait_event(c, *p, &w), ZHIP_KERNEL_SYNC);
        HIPCHK(c, hipEventSynchronize(w), ZHIP_KERNEL_SYNC);
    }
    for (size_t s = 0; s < arg_sets; s++) {
        int32_t rc = order_args(c, 0, *p, args + s * n_args, n_args, ZHIP_KERNEL_LAUNCH);
        if (rc != ZHIP_OK) return rc;
    }
    HIPCHK(c, hipStreamSynchronize(st), ZHIP_KERNEL_SYNC);
    HIPCHK(c, hipEventRecord(c->prof_a, st), ZHIP_KERNEL_LAUNCH);
    for (int32_t i = 0; i < iters; i++) {
        // what a chain of zhip_launch calls with these arguments would do: nothing writes the weights in between
        const bool ready = conv_weights_current(c, *p, args + (i % arg_sets) * n_args, n_args);
        hipError_t e = program_enqueue(*p, &ptrs[(i % arg_sets) * kMaxArgs], st, ready);
        if (e != hipSuccess) {
            p->conv_w_valid = false;
            return c->fail(ZHIP_KERNEL_LAUNCH, "launch of program %u failed: %s", prog, hipGetErrorString(e));
        }
    }
    HIPCHK(c, hipEventRecord(c->prof_b, st), ZHIP_KERNEL_LAUNCH);
    HIPCHK(c, hipEventSynchronize(c->prof_b), ZHIP_KERNEL_SYNC);
    float ms = 0.0f;
    HIPCHK(c, hipEventElapsedTime(&ms, c->prof_a, c->prof_b), ZHIP_KERNEL_SYNC);
    *avg_us = ms * 1000.0f / (float)iters;
    ++c->stream_seq[0];
    for (size_t s = 0; s < arg_sets; s++) stamp_args(c, 0, c->stream_seq[0], *p, args + s * n_args, n_args);
    c->done[0] = c->stream_seq[0]; // the second event was waited for
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_plan_create(zhip_ctx *c, const zhip_prog *progs, const zhip_buf *args_flat, const uint32_t *n_args,
                                     size_t n_nodes, zhip_plan *plan) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!progs || !args_flat || !n_args || !plan || n_nodes == 0) return c->fail(ZHIP_KERNEL_COMPILATION, "plan_create: bad argument");
    *plan = ZHIP_NULL_ID;
    // resolve every node before anything is captured: a bad node must not leave a capture open
    std::vector<Program *> ps(n_nodes);
    std::vector<void *> ptrs(n_nodes * kMaxArgs, nullptr);
    size_t off = 0;
    for (size_t i = 0; i < n_nodes; i++) {
        int32_t rc = resolve_args(c, progs[i], args_flat + off, n_args[i], &ps[i], &ptrs[i * kMaxArgs]);
        if (rc != ZHIP_OK) return rc;
        off += n_args[i];
    }
    HIPCHK(c, hipSetDevice(c->device), ZHIP_KERNEL_COMPILATION);
    HIPCHK(c, hipStreamSynchronize(c->plan_stream), ZHIP_KERNEL_SYNC);
    HIPCHK(c, hipStreamBeginCapture(c->plan_stream, hipStreamCaptureModeThreadLocal), ZHIP_KERNEL_COMPILATION);
    hipError_t bad = hipSuccess;
    for (size_t i = 0; i < n_nodes && bad == hipSuccess; i++) bad = program_enqueue(*ps[i], &ptrs[i * kMaxArgs], c->plan_stream);
    Plan pl;
    hipError_t e = hipStreamEndCapture(c->plan_stream, &pl.graph);
    if (bad != hipSuccess || e != hipSuccess) {
        if (pl.graph) (void)hipGraphDestroy(pl.graph);
        (void)hipGetLastError();
        return c->fail(ZHIP_KERNEL_COMPILATION, "plan capture failed: %s", hipGetErrorString(bad != hipSuccess ? bad : e));
    }
    e = hipGraphInstantiate(&pl.exec, pl.graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(pl.graph);
        return c->fail(ZHIP_KERNEL_COMPILATION, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    }
    pl.live = true;
    pl.n_nodes = n_nodes;
    for (size_t i = 0; i < n_nodes; i++)
        if (std::find(pl.progs.begin(), pl.progs.end(), progs[i]) == pl.progs.end()) pl.progs.push_back(progs[i]);
    for (zhip_prog q : pl.progs) c->programs.items[q].plan_refs++;
    off = 0;
    for (size_t i = 0; i < n_nodes; i++) {
        const Program &pr = *ps[i];
        for (size_t a = 0; a < n_args[i]; a++) {
            const zhip_buf id = args_flat[off + a];
            Buffer *b = buffer_lookup(c, id);
            if (!b || b->kind != Buffer::Memory) continue;
            const bool write = pr.ir ? pr.ir->params[a].kind == ZHIP_IR_GLOBAL_MUT : a >= (size_t)pr.n_in;
            auto it = std::find_if(pl.uses.begin(), pl.uses.end(), [id](const std::pair<zhip_buf, bool> &u) { return u.first == id; });
            if (it == pl.uses.end()) pl.uses.push_back({id, write});
            else it->second = it->second || write;
        }
        off += n_args[i];
    }
    *plan = c->plans.push(pl);
    return ZHIP_OK;
}

ZHIP_EXPORT int32_t zhip_plan_launch(zhip_ctx *c, zhip_plan plan, const zhip_event *evs, size_t n_evs, zhip_event *ev) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!ev) return c->fail(ZHIP_KERNEL_LAUNCH, "plan_launch: null event out pointer");
    *ev = 0;
    if (plan >= c->plans.items.size() || !c->plans.items[plan].live) {
        for (size_t i = 0; i < n_evs; i++)
            if (EventSlot *s = event_lookup(c, evs[i])) event_retire(c, s);
        return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "plan %u does not exist", plan);
    }
    HIPCHK(c, hipSetDevice(c->device), ZHIP_KERNEL_LAUNCH);
    int32_t rc = wait_and_consume(c, -2, evs, n_evs, ZHIP_KERNEL_LAUNCH);
    if (rc != ZHIP_OK) return rc;
    Plan &pl = c->plans.items[plan];
    // Program scratch: a program last used by a single launch on another stream is waited for; one last used by a
    // plan needs nothing (plans replay in order on one stream). Afterwards one event covers every program of the plan.
    bool any_ws = false;
    for (zhip_prog q : pl.progs) {
        Program &pr = c->programs.items[q];
        if (!pr.ws_event) continue;
        any_ws = true;
        if (pr.ws_last == 1) {
            hipEvent_t w;
            HIPCHK(c, ws_wait_event(c, pr, &w), ZHIP_KERNEL_LAUNCH);
            HIPCHK(c, hipStreamWaitEvent(c->plan_stream, w, 0), ZHIP_KERNEL_LAUNCH);
        }
    }
    for (const auto &u : pl.uses)
        if (Buffer *b = buffer_lookup(c, u.first)) {
            rc = order_access(c, -2, b->acc, u.second, ZHIP_KERNEL_LAUNCH);
            if (rc != ZHIP_OK) return rc;
        }
    for (zhip_prog q : pl.progs) c->programs.items[q].conv_w_valid = false; // a plan always re-lays, from its own weights
    HIPCHK(c, hipGraphLaunch(pl.exec, c->plan_stream), ZHIP_KERNEL_LAUNCH);
    if (any_ws) {
        HIPCHK(c, hipEventRecord(c->plan_done, c->plan_stream), ZHIP_KERNEL_LAUNCH);
        for (zhip_prog q : pl.progs)
            if (c->programs.items[q].ws_event) c->programs.items[q].ws_last = 2;
    }
    // A plan is a coarse unit whose end other streams typically wait for while the next plan is already queued (batch
    // copies of a training loop): its event is recorded right here, so that such a wait covers this plan only.
    int32_t rc2 = event_record(c, -2, ZHIP_KERNEL_LAUNCH, ev);
    for (const auto &u : pl.uses)
        if (Buffer *b = buffer_lookup(c, u.first)) stamp_access(b->acc, -2, c->stream_seq[kLaunchStreams + 1], u.second);
    if (rc2 == ZHIP_OK)
        if (EventSlot *s = event_lookup(c, *ev))
            if (event_materialise(c, s) != hipSuccess) return c->fail(ZHIP_KERNEL_LAUNCH, "hipEventRecord failed");
    return rc2;
}

ZHIP_EXPORT int32_t zhip_plan_destroy(zhip_ctx *c, zhip_plan plan) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (plan >= c->plans.items.size() || !c->plans.items[plan].live) return c->fail(ZHIP_INCORRECT_KERNEL_ARG, "plan %u does not exist", plan);
    Plan &pl = c->plans.items[plan];
    (void)hipSetDevice(c->device);
    (void)hipStreamSynchronize(c->plan_stream);
    (void)hipGraphExecDestroy(pl.exec);
    (void)hipGraphDestroy(pl.graph);
    for (zhip_prog q : pl.progs)
        if (q < c->programs.items.size() && c->programs.items[q].plan_refs > 0) c->programs.items[q].plan_refs--;
    pl = Plan();
    c->plans.remove(plan);
    return ZHIP_OK;
}
