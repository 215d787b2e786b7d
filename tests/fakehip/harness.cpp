// Drives the backend's C ABI (include/zyx_hip.h) against the host-only HIP model of fake_hip.cpp, the way zyx's runtime
// drives a backend, and asserts that no launch, copy or free was enqueued without being ordered after the accesses it
// conflicts with. The sequences replayed are the reference's own:
//   * Runtime::execute_plan (zyx/src/graph/plan.rs:271-361): Allocate (+1 trash element) -> Launch with the wait list
//     drained from the event map -> Deallocate with the drained events;
//   * Runtime::materialize_kernel (zyx/src/runtime.rs:2262-2300): allocate stores, wait list = their allocation events
//     + the drained events of every buffer, launch, insert the event under the set of all buffers;
//   * the event map rule itself (zyx/src/runtime.rs:1-16): an event is stored under the set of buffers its kernel
//     touched and is consumed by the first later operation that touches any of them.
// Built by tests/test_runtime_on_fake_hip.py with g++ and AddressSanitizer + UBSan, and once more with ThreadSanitizer.
#include "../../include/zyx_hip.h"
#include "fake_hip.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <random>
#include <set>
#include <string>
#include <thread>
#include <vector>

static int g_failures = 0;
#define EXPECT(cond)                                                                         \
    do {                                                                                     \
        if (!(cond)) {                                                                       \
            printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                       \
            g_failures++;                                                                    \
        }                                                                                    \
    } while (0)
#define OK(call) EXPECT((call) == ZHIP_OK)

static bool no_hazards(const char *what) {
    const std::vector<std::string> h = fakehip_hazards();
    for (const std::string &m : h) printf("  hazard in %s: %s\n", what, m.c_str());
    if (!h.empty()) g_failures++;
    return h.empty();
}

// ---- a miniature of zyx's runtime state: the event map -------------------------------------------------------------
struct EventMap {
    std::vector<std::pair<std::set<zhip_buf>, zhip_event>> entries;
    // drain_events_for_bufs (zyx/src/graph/plan.rs:366-390): every event whose key contains one of the buffers
    std::vector<zhip_event> drain(const std::set<zhip_buf> &bufs) {
        std::vector<zhip_event> out;
        for (size_t i = 0; i < entries.size();) {
            bool hit = false;
            for (zhip_buf b : bufs) hit = hit || entries[i].first.count(b);
            if (hit) {
                out.push_back(entries[i].second);
                entries.erase(entries.begin() + (long)i);
            } else i++;
        }
        return out;
    }
    void insert(const std::set<zhip_buf> &bufs, zhip_event ev) {
        if (ev) entries.push_back({bufs, ev});
    }
    std::vector<zhip_event> all() {
        std::vector<zhip_event> out;
        for (auto &e : entries) out.push_back(e.second);
        entries.clear();
        return out;
    }
};

static zhip_kernel_desc desc(int kind, int dtype, int64_t d0, int64_t d1) {
    zhip_kernel_desc d;
    memset(&d, 0, sizeof d);
    d.kind = kind;
    d.dtype = d.out_dtype = dtype;
    d.dims[0] = d0;
    d.dims[1] = d1;
    return d;
}
// y = x * 2 + 1 as an elementwise chain over [rows, cols] f32: 1 input, 3 instructions
static zhip_kernel_desc chain_desc(int64_t rows, int64_t cols) {
    zhip_kernel_desc d = desc(ZHIP_K_ELEMENTWISE, ZHIP_F32, rows, cols);
    d.iparams[0] = 1;
    d.iparams[1] = 3;
    d.iparams[2] = ZHIP_F32 | (ZHIP_EW_FULL << 8);
    d.iparams[6] = ZHIP_EW_LOAD | (0 << 8);
    d.iparams[7] = ZHIP_EW_MUL | (ZHIP_EW_SRC_CONST << 8);
    d.iparams[8] = ZHIP_EW_ADD | ((ZHIP_EW_SRC_CONST + 1) << 8);
    d.fparams[0] = 2.0f;
    d.fparams[1] = 1.0f;
    return d;
}
// z = x + y: 2 inputs
static zhip_kernel_desc add_desc(int64_t rows, int64_t cols) {
    zhip_kernel_desc d = desc(ZHIP_K_ELEMENTWISE, ZHIP_F32, rows, cols);
    d.iparams[0] = 2;
    d.iparams[1] = 2;
    d.iparams[2] = d.iparams[3] = ZHIP_F32 | (ZHIP_EW_FULL << 8);
    d.iparams[6] = ZHIP_EW_LOAD | (0 << 8);
    d.iparams[7] = ZHIP_EW_ADD | (1 << 8);
    return d;
}

static zhip_ctx *new_ctx(uint64_t cache_bytes = 0) {
    zhip_config cfg;
    memset(&cfg, 0, sizeof cfg);
    cfg.cache_bytes = cache_bytes;
    zhip_ctx *ctx = nullptr;
    if (zhip_init(&cfg, &ctx) != ZHIP_OK) {
        printf("zhip_init failed: %s\n", zhip_last_error(nullptr));
        exit(2);
    }
    return ctx;
}

// ---- scenarios -----------------------------------------------------------------------------------------------------
static void execute_plan_sequence() {
    printf("execute_plan sequence\n");
    zhip_ctx *ctx = new_ctx();
    EventMap events;
    const int64_t R = 64, Cc = 256, n = R * Cc;
    std::vector<float> host(n, 1.5f), back(n);
    // leaf: Runtime::new_tensor = allocate + host_to_pool, event kept in the map
    zhip_buf x;
    zhip_event ev;
    OK(zhip_alloc(ctx, (n + 1) * 4, &x, &ev));
    zhip_event up;
    OK(zhip_h2d(ctx, host.data(), n * 4, x, &ev, 1, &up));
    events.insert({x}, up);
    zhip_prog chain, add, sum;
    zhip_kernel_desc d1 = chain_desc(R, Cc), d2 = add_desc(R, Cc), d3 = desc(ZHIP_K_REDUCE, ZHIP_F32, R, Cc);
    OK(zhip_register_kernel(ctx, &d1, &chain));
    OK(zhip_register_kernel(ctx, &d2, &add));
    OK(zhip_register_kernel(ctx, &d3, &sum));
    for (int round = 0; round < 3; round++) { // a cached plan is executed again and again
        // Allocate nodes
        zhip_buf y, z, s;
        zhip_event ey, ez, es;
        OK(zhip_alloc(ctx, (n + 1) * 4, &y, &ey));
        events.insert({y}, ey);
        OK(zhip_alloc(ctx, (n + 1) * 4, &z, &ez));
        events.insert({z}, ez);
        OK(zhip_alloc(ctx, (R + 1) * 4, &s, &es));
        events.insert({s}, es);
        // Launch nodes: args = load classes then store classes, wait list drained from the map
        auto launch = [&](zhip_prog p, std::vector<zhip_buf> args) {
            std::set<zhip_buf> bufs(args.begin(), args.end());
            std::vector<zhip_event> waits = events.drain(bufs);
            zhip_event done = 0;
            OK(zhip_launch(ctx, p, args.data(), args.size(), waits.data(), waits.size(), &done));
            events.insert(bufs, done);
        };
        launch(chain, {x, y});    // y = f(x)
        launch(add, {x, y, z});   // z = x + y
        launch(sum, {z, s});      // s = rowsum(z)
        launch(chain, {x, y});    // overwrites y, which `add` read: that launch's event went to `sum`, the map holds nothing for y
        // read a result back (Tensor -> Vec): pool_to_host with the drained events
        std::vector<zhip_event> w = events.drain({s});
        OK(zhip_d2h(ctx, s, back.data(), R * 4, w.data(), w.size()));
        // Deallocate nodes
        for (zhip_buf b : {y, z, s}) {
            std::vector<zhip_event> wl = events.drain({b});
            OK(zhip_free(ctx, b, wl.data(), wl.size()));
        }
        no_hazards("execute_plan round");
    }
    std::vector<zhip_event> rest = events.all();
    OK(zhip_sync_events(ctx, rest.data(), rest.size()));
    OK(zhip_free(ctx, x, nullptr, 0));
    OK(zhip_deinit(ctx));
    no_hazards("execute_plan teardown");
    size_t live, bytes;
    fakehip_live(&live, &bytes);
    EXPECT(live == 0);
}

// The event of a kernel is stored under ALL its buffers and consumed by the first later operation touching ANY of them
// (zyx/src/runtime.rs:1-16). k1: x -> y; k2: x -> z consumes k1's event; k3: y -> w then finds no event for y and
// launches with an empty wait list. The backend must still order k3 after k1: it remembers who wrote each buffer.
static void consumed_event_still_orders() {
    printf("consumed event still orders\n");
    zhip_ctx *ctx = new_ctx();
    EventMap events;
    const int64_t n = 4096;
    zhip_buf b[4];
    for (int i = 0; i < 4; i++) {
        zhip_event e;
        OK(zhip_alloc(ctx, (n + 1) * 4, &b[i], &e));
        events.insert({b[i]}, e);
    }
    zhip_prog chain;
    zhip_kernel_desc d = chain_desc(16, 256);
    OK(zhip_register_kernel(ctx, &d, &chain));
    auto launch = [&](zhip_buf in, zhip_buf out) {
        std::set<zhip_buf> bufs = {in, out};
        std::vector<zhip_event> waits = events.drain(bufs);
        zhip_event done = 0;
        zhip_buf args[2] = {in, out};
        OK(zhip_launch(ctx, chain, args, 2, waits.data(), waits.size(), &done));
        events.insert(bufs, done);
    };
    for (int rep = 0; rep < 20; rep++) {
        launch(b[0], b[1]); // k1
        launch(b[0], b[2]); // k2 consumes k1's event (shared input)
        launch(b[1], b[3]); // k3 reads k1's output with nothing to wait for
        launch(b[3], b[1]); // k4 overwrites what k3... and so on
    }
    no_hazards("consumed event");
    std::vector<zhip_event> rest = events.all();
    OK(zhip_sync_events(ctx, rest.data(), rest.size()));
    for (zhip_buf x : b) OK(zhip_free(ctx, x, nullptr, 0));
    OK(zhip_deinit(ctx));
}

static void program_scratch_is_serialised() {
    printf("launches sharing a program's scratch\n");
    zhip_ctx *ctx = new_ctx();
    const int64_t R = 64, Cc = 8192;
    zhip_prog sum;
    zhip_kernel_desc d = desc(ZHIP_K_REDUCE, ZHIP_F32, R, Cc);
    OK(zhip_register_kernel(ctx, &d, &sum));
    zhip_buf x[4], s[4];
    std::vector<zhip_event> done;
    for (int i = 0; i < 4; i++) {
        zhip_event e1, e2, ev;
        OK(zhip_alloc(ctx, (R * Cc + 1) * 4, &x[i], &e1));
        OK(zhip_alloc(ctx, (R + 1) * 4, &s[i], &e2));
        zhip_buf args[2] = {x[i], s[i]};
        zhip_event w[2] = {e1, e2};
        OK(zhip_launch(ctx, sum, args, 2, w, 2, &ev)); // unrelated wait lists: four streams, one scratch buffer
        done.push_back(ev);
    }
    // the same program inside a plan and as single launches, alternating
    zhip_plan plan;
    zhip_buf pargs[2] = {x[0], s[0]};
    uint32_t cnt = 2;
    OK(zhip_sync_events(ctx, done.data(), done.size()));
    OK(zhip_plan_create(ctx, &sum, pargs, &cnt, 1, &plan));
    for (int i = 0; i < 3; i++) {
        zhip_event pe, le;
        OK(zhip_plan_launch(ctx, plan, nullptr, 0, &pe));
        zhip_buf args[2] = {x[1], s[1]};
        OK(zhip_launch(ctx, sum, args, 2, nullptr, 0, &le));
        zhip_event both[2] = {pe, le};
        OK(zhip_release_events(ctx, both, 2));
    }
    EXPECT(zhip_release_program(ctx, sum) == ZHIP_INCORRECT_KERNEL_ARG); // a live plan holds it
    OK(zhip_plan_destroy(ctx, plan));
    OK(zhip_release_program(ctx, sum));
    no_hazards("program scratch");
    for (int i = 0; i < 4; i++) {
        OK(zhip_free(ctx, x[i], nullptr, 0));
        OK(zhip_free(ctx, s[i], nullptr, 0));
    }
    OK(zhip_deinit(ctx));
    no_hazards("program scratch teardown");
}

static void freed_blocks_are_reused_in_order() {
    printf("block cache\n");
    zhip_ctx *ctx = new_ctx();
    zhip_prog chain;
    zhip_kernel_desc d = chain_desc(16, 256);
    OK(zhip_register_kernel(ctx, &d, &chain));
    zhip_buf x;
    zhip_event ex;
    OK(zhip_alloc(ctx, 4097 * 4, &x, &ex));
    const unsigned long mallocs0 = fakehip_calls("hipMalloc");
    for (int i = 0; i < 50; i++) {
        zhip_buf y;
        zhip_event ey, done;
        OK(zhip_alloc(ctx, 4097 * 4, &y, &ey)); // from the second round on: the block freed below, still in use
        zhip_buf args[2] = {x, y};
        zhip_event w[2] = {ex, ey};
        OK(zhip_launch(ctx, chain, args, 2, w, 2, &done));
        ex = 0;
        // the reference frees with the kernel's event in the wait list: the block goes back while the kernel runs
        OK(zhip_free(ctx, y, &done, 1));
    }
    EXPECT(fakehip_calls("hipMalloc") - mallocs0 <= 1);
    no_hazards("block cache");
    const uint64_t free_before = zhip_free_bytes(ctx);
    zhip_buf big;
    zhip_event e;
    EXPECT(zhip_alloc(ctx, free_before + 1, &big, &e) == ZHIP_MEMORY_ALLOCATION); // hip.rs:355-357
    EXPECT(big == ZHIP_NULL_ID);
    OK(zhip_free(ctx, x, nullptr, 0));
    OK(zhip_deinit(ctx));
}

static void plans_and_batch_copies() {
    printf("plan replays with batch uploads in between\n");
    zhip_ctx *ctx = new_ctx();
    const int64_t R = 64, Cc = 784, n = R * Cc;
    std::vector<float> batch(n, 0.25f);
    zhip_buf x, h, s;
    zhip_event e[3];
    OK(zhip_alloc(ctx, (n + 1) * 4, &x, &e[0]));
    OK(zhip_alloc(ctx, (n + 1) * 4, &h, &e[1]));
    OK(zhip_alloc(ctx, (R + 1) * 4, &s, &e[2]));
    OK(zhip_sync_events(ctx, e, 3));
    zhip_prog chain, sum;
    zhip_kernel_desc d1 = chain_desc(R, Cc), d2 = desc(ZHIP_K_REDUCE, ZHIP_F32, R, Cc);
    OK(zhip_register_kernel(ctx, &d1, &chain));
    OK(zhip_register_kernel(ctx, &d2, &sum));
    zhip_prog progs[2] = {chain, sum};
    zhip_buf flat[4] = {x, h, h, s};
    uint32_t counts[2] = {2, 2};
    zhip_plan plan;
    OK(zhip_plan_create(ctx, progs, flat, counts, 2, &plan));
    zhip_event last = 0;
    for (int step = 0; step < 10; step++) {
        zhip_event up, done;
        OK(zhip_h2d(ctx, batch.data(), n * 4, x, &last, last ? 1 : 0, &up)); // the upload waits for the step that read x
        OK(zhip_plan_launch(ctx, plan, &up, 1, &done));
        last = done;
    }
    std::vector<float> out(R);
    OK(zhip_d2h(ctx, s, out.data(), R * 4, &last, 1));
    no_hazards("plans");
    OK(zhip_plan_destroy(ctx, plan));
    for (zhip_buf b : {x, h, s}) OK(zhip_free(ctx, b, nullptr, 0));
    OK(zhip_deinit(ctx));
}

static void misuse_is_an_error_not_a_crash() {
    printf("error paths\n");
    zhip_ctx *ctx = new_ctx();
    zhip_buf x;
    zhip_event e;
    OK(zhip_alloc(ctx, 1024, &x, &e));
    OK(zhip_sync_events(ctx, &e, 1)); // a fresh block is ready at once: the null event, which may be synced any number of times
    const char bytes[16] = "fifteen letters";
    OK(zhip_h2d(ctx, bytes, sizeof bytes, x, nullptr, 0, &e));
    EXPECT(e != 0);
    OK(zhip_sync_events(ctx, &e, 1));
    EXPECT(zhip_sync_events(ctx, &e, 1) == ZHIP_KERNEL_SYNC);              // consumed twice
    zhip_event bogus = 0x7777000000000009ull;
    EXPECT(zhip_release_events(ctx, &bogus, 1) == ZHIP_DEINITIALIZATION); // never existed
    zhip_prog chain;
    zhip_kernel_desc d = chain_desc(16, 256);
    OK(zhip_register_kernel(ctx, &d, &chain));
    zhip_buf args[2] = {x, x};
    zhip_event done;
    EXPECT(zhip_launch(ctx, chain, args, 2, nullptr, 0, &done) == ZHIP_INCORRECT_KERNEL_ARG); // too small, and aliased
    EXPECT(zhip_launch(ctx, chain, args, 1, nullptr, 0, &done) == ZHIP_INCORRECT_KERNEL_ARG); // arity
    EXPECT(zhip_launch(ctx, 12345, args, 2, nullptr, 0, &done) == ZHIP_INCORRECT_KERNEL_ARG);
    OK(zhip_free(ctx, x, nullptr, 0));
    EXPECT(zhip_free(ctx, x, nullptr, 0) == ZHIP_MEMORY_DEALLOCATION);                         // double free
    zhip_kernel_desc bad = desc(99, ZHIP_F32, 1, 1);
    EXPECT(zhip_register_kernel(ctx, &bad, &chain) == ZHIP_KERNEL_COMPILATION);
    const char junk[64] = "not a kernel image";
    zhip_prog p;
    EXPECT(zhip_compile_ir(ctx, junk, sizeof junk, &p) == ZHIP_KERNEL_COMPILATION);
    EXPECT(strlen(zhip_last_error(ctx)) > 0);
    // scalar variables share the buffer id space (backend/mod.rs:597-621)
    uint8_t v[8] = {42, 0, 0, 0, 0, 0, 0, 0}, r[8];
    zhip_buf var;
    int32_t found = 0, dt = -1;
    OK(zhip_store_variable(ctx, ZHIP_U64, v, &var));
    OK(zhip_get_variable(ctx, var, &found, &dt, r));
    EXPECT(found == 1 && dt == ZHIP_U64 && r[0] == 42);
    OK(zhip_free(ctx, var, nullptr, 0));
    no_hazards("error paths");
    OK(zhip_deinit(ctx));
}

// A generated kernel: y[i] = x[i] * x[i] over 4 groups of 64 lanes, written as the image Device::compile receives.
static std::vector<uint8_t> square_image() {
    std::vector<zhip_ir_op> ops;
    auto push = [&](uint16_t opcode, uint16_t dtype, uint32_t a, uint32_t b, uint32_t c, uint32_t aux, uint64_t imm) {
        zhip_ir_op o;
        memset(&o, 0, sizeof o);
        o.id = (uint32_t)ops.size();
        o.opcode = opcode;
        o.dtype = dtype;
        o.a = a;
        o.b = b;
        o.c = c;
        o.aux = aux;
        o.imm = imm;
        ops.push_back(o);
        return o.id;
    };
    const uint32_t N = ZHIP_IR_NULL;
    uint32_t x = push(ZHIP_IR_PARAM, ZHIP_F32, N, N, N, ZHIP_IR_GLOBAL, 256);
    uint32_t y = push(ZHIP_IR_PARAM, ZHIP_F32, N, N, N, ZHIP_IR_GLOBAL_MUT, 256);
    uint32_t four = push(ZHIP_IR_CONST, ZHIP_I64, N, N, N, 0, 4);
    uint32_t g = push(ZHIP_IR_INDEX, 0, four, N, N, 0 | (ZHIP_IR_IDX_GROUP << 8), 0);
    uint32_t l = push(ZHIP_IR_INDEX, 0, N, N, N, 0 | (ZHIP_IR_IDX_LOCAL << 8), 64);
    uint32_t c64 = push(ZHIP_IR_CONST, ZHIP_I64, N, N, N, 0, 64);
    uint32_t base = push(ZHIP_IR_BINARY, 0, g, c64, N, ZHIP_IR_MUL, 0);
    uint32_t i = push(ZHIP_IR_BINARY, 0, base, l, N, ZHIP_IR_ADD, 0);
    uint32_t v = push(ZHIP_IR_LOAD, 0, x, i, N, 0, 0);
    uint32_t sq = push(ZHIP_IR_BINARY, 0, v, v, N, ZHIP_IR_MUL, 0);
    push(ZHIP_IR_STORE, 0, y, sq, i, 0, 0);
    zhip_ir_header h = {ZHIP_IR_MAGIC, (uint32_t)ops.size(), 0, 0};
    std::vector<uint8_t> img(sizeof h + ops.size() * sizeof(zhip_ir_op));
    memcpy(img.data(), &h, sizeof h);
    memcpy(img.data() + sizeof h, ops.data(), ops.size() * sizeof(zhip_ir_op));
    return img;
}

static void generated_kernels_and_the_code_cache() {
    printf("generated kernels\n");
    zhip_ctx *ctx = new_ctx();
    const std::vector<uint8_t> img = square_image();
    uint64_t before[3], after[3];
    zhip_compile_cache_stats(before);
    zhip_prog p1, p2;
    OK(zhip_compile_ir(ctx, img.data(), img.size(), &p1));
    OK(zhip_compile_ir(ctx, img.data(), img.size(), &p2));
    zhip_compile_cache_stats(after);
    EXPECT(after[0] + after[2] == before[0] + before[2] + 1 && after[1] == before[1] + 1); // built (or found on disk) once
    zhip_buf x, y, z;
    zhip_event e[3], d1, d2;
    OK(zhip_alloc(ctx, 257 * 4, &x, &e[0]));
    OK(zhip_alloc(ctx, 257 * 4, &y, &e[1]));
    OK(zhip_alloc(ctx, 257 * 4, &z, &e[2]));
    zhip_buf a1[2] = {x, y}, a2[2] = {y, z};
    zhip_event w1[2] = {e[0], e[1]};
    OK(zhip_launch(ctx, p1, a1, 2, w1, 2, &d1));
    zhip_event w2[2] = {d1, e[2]};
    OK(zhip_launch(ctx, p2, a2, 2, w2, 2, &d2));
    zhip_buf small;
    zhip_event es;
    OK(zhip_alloc(ctx, 16, &small, &es));
    zhip_buf a3[2] = {x, small};
    zhip_event dz;
    EXPECT(zhip_launch(ctx, p1, a3, 2, &es, 1, &dz) == ZHIP_INCORRECT_KERNEL_ARG); // the image says 256 elements
    char src[64];
    uint64_t len = 0;
    OK(zhip_program_source(ctx, p1, src, sizeof src, &len));
    EXPECT(len > 64 && strlen(src) == 63);
    OK(zhip_sync_events(ctx, &d2, 1));
    no_hazards("generated kernels");
    OK(zhip_release_program(ctx, p1));
    OK(zhip_release_program(ctx, p2));
    for (zhip_buf b : {x, y, z, small}) OK(zhip_free(ctx, b, nullptr, 0));
    OK(zhip_deinit(ctx));
}

static void reduce_static_allocates_nothing() {
    printf("zhip_reduce_static\n");
    zhip_ctx *ctx = new_ctx();
    zhip_buf x, s;
    zhip_event e[2];
    OK(zhip_alloc(ctx, 64 * 8192 * 4, &x, &e[0]));
    OK(zhip_alloc(ctx, 8192 * 4, &s, &e[1]));
    OK(zhip_sync_events(ctx, e, 2));
    void *xp, *sp;
    OK(zhip_buffer_ptr(ctx, x, &xp, nullptr));
    OK(zhip_buffer_ptr(ctx, s, &sp, nullptr));
    hipStream_t st;
    EXPECT(hipStreamCreate(&st) == hipSuccess);
    const unsigned long m0 = fakehip_calls("hipMalloc"), f0 = fakehip_calls("hipFree"), ev0 = fakehip_calls("hipEventCreate");
    OK(zhip_reduce_static(ctx, ZHIP_F32, 0, 1, 64, 8192, xp, sp, st));
    OK(zhip_reduce_static(ctx, ZHIP_F32, 1, 0, 32, 4096, xp, sp, st));
    // inside somebody else's capture: nothing but kernel nodes may be recorded
    hipGraph_t graph;
    EXPECT(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal) == hipSuccess);
    OK(zhip_reduce_static(ctx, ZHIP_F32, 0, 1, 64, 8192, xp, sp, st));
    EXPECT(hipStreamEndCapture(st, &graph) == hipSuccess);
    EXPECT(fakehip_calls("hipMalloc") == m0 && fakehip_calls("hipFree") == f0 && fakehip_calls("hipEventCreate") == ev0);
    EXPECT(zhip_reduce_static(ctx, ZHIP_F64, 0, 1, 4, 4, xp, sp, st) == ZHIP_KERNEL_COMPILATION);
    // partial results beyond the static scratch: refused with the sizes, before any pointer is looked at
    EXPECT(zhip_reduce_static(ctx, ZHIP_F32, 0, 1, 7777, 64, nullptr, nullptr, st) == ZHIP_KERNEL_COMPILATION);
    EXPECT(strstr(zhip_last_error(ctx), "67108864") && strstr(zhip_last_error(ctx), "1048576"));
    // null pointers are an argument error, not a launch
    EXPECT(zhip_reduce_static(ctx, ZHIP_F32, 0, 1, 64, 64, nullptr, sp, st) == ZHIP_INCORRECT_KERNEL_ARG);
    EXPECT(zhip_reduce_static(ctx, ZHIP_F32, 0, 1, 64, 64, xp, nullptr, st) == ZHIP_INCORRECT_KERNEL_ARG);
    no_hazards("reduce_static");
    (void)hipGraphDestroy(graph);
    (void)hipStreamSynchronize(st);
    (void)hipStreamDestroy(st);
    OK(zhip_free(ctx, x, nullptr, 0));
    OK(zhip_free(ctx, s, nullptr, 0));
    OK(zhip_deinit(ctx));
}

// A random program under zyx's event discipline: launches over random buffers, uploads, downloads, frees and
// re-allocations in any order. Whatever the order, the fake must see no unordered conflicting accesses.
static void random_schedules(unsigned seed, int steps) {
    printf("random schedule, seed %u\n", seed);
    std::mt19937 rng(seed);
    zhip_ctx *ctx = new_ctx(1 << 20); // a small cache: blocks also go back to the driver
    EventMap events;
    const int64_t R = 16, Cc = 256, n = R * Cc;
    std::vector<float> host(n, 1.0f), back(n);
    zhip_prog chain, add, sum, soft;
    zhip_kernel_desc d1 = chain_desc(R, Cc), d2 = add_desc(R, Cc), d3 = desc(ZHIP_K_REDUCE, ZHIP_F32, R, Cc), d4 = desc(ZHIP_K_SOFTMAX_ROWS, ZHIP_F32, R, Cc);
    d4.flags = ZHIP_SOFTMAX_Y;
    OK(zhip_register_kernel(ctx, &d1, &chain));
    OK(zhip_register_kernel(ctx, &d2, &add));
    OK(zhip_register_kernel(ctx, &d3, &sum));
    OK(zhip_register_kernel(ctx, &d4, &soft));
    std::vector<zhip_buf> bufs;
    auto alloc = [&] {
        zhip_buf b;
        zhip_event e;
        OK(zhip_alloc(ctx, (n + 1) * 4, &b, &e));
        events.insert({b}, e);
        bufs.push_back(b);
    };
    for (int i = 0; i < 6; i++) alloc();
    auto pick = [&] { return bufs[rng() % bufs.size()]; };
    for (int step = 0; step < steps; step++) {
        const unsigned what = rng() % 100;
        if (what < 55 && bufs.size() >= 3) {
            zhip_buf a = pick(), b = pick(), c = pick();
            std::vector<zhip_buf> args;
            zhip_prog p;
            switch (rng() % 4) {
            case 0: p = chain; if (a == c) continue; args = {a, c}; break;
            case 1: p = add; if (a == c || b == c) continue; args = {a, b, c}; break;
            case 2: p = sum; if (a == c) continue; args = {a, c}; break;
            default: p = soft; if (a == c) continue; args = {a, c}; break;
            }
            std::set<zhip_buf> key(args.begin(), args.end());
            std::vector<zhip_event> waits = events.drain(key);
            zhip_event done = 0;
            OK(zhip_launch(ctx, p, args.data(), args.size(), waits.data(), waits.size(), &done));
            events.insert(key, done);
        } else if (what < 65) {
            zhip_buf b = pick();
            std::vector<zhip_event> waits = events.drain({b});
            zhip_event up = 0;
            OK(zhip_h2d(ctx, host.data(), n * 4, b, waits.data(), waits.size(), &up));
            events.insert({b}, up);
        } else if (what < 75) {
            zhip_buf b = pick();
            std::vector<zhip_event> waits = events.drain({b});
            OK(zhip_d2h(ctx, b, back.data(), n * 4, waits.data(), waits.size()));
        } else if (what < 82 && bufs.size() >= 2) {
            zhip_buf a = pick(), b = pick();
            if (a == b) continue;
            std::vector<zhip_event> waits = events.drain({a, b});
            zhip_event ev = 0;
            OK(zhip_d2d(ctx, a, 0, b, 0, n * 4, waits.data(), waits.size(), &ev));
            events.insert({a, b}, ev);
        } else if (what < 92 && bufs.size() > 3) {
            const size_t i = rng() % bufs.size();
            std::vector<zhip_event> waits = events.drain({bufs[i]});
            OK(zhip_free(ctx, bufs[i], waits.data(), waits.size()));
            bufs.erase(bufs.begin() + (long)i);
        } else if (bufs.size() < 12) {
            alloc();
        }
        if (!no_hazards("random schedule")) {
            printf("  at step %d\n", step);
            break;
        }
    }
    std::vector<zhip_event> rest = events.all();
    OK(zhip_sync_events(ctx, rest.data(), rest.size()));
    OK(zhip_deinit(ctx)); // frees what is left
    no_hazards("random schedule teardown");
}

// The detector itself: two launches that conflict and are not ordered must be reported.
static void the_detector_detects() {
    printf("negative control\n");
    void *p = nullptr;
    hipStream_t a, b;
    EXPECT(hipMalloc(&p, 1024) == hipSuccess && hipStreamCreate(&a) == hipSuccess && hipStreamCreate(&b) == hipSuccess);
    fakehip_launch(a, "writer", {{p, true}});
    fakehip_launch(b, "reader", {{p, false}}); // no event between the streams
    EXPECT(fakehip_hazards().size() == 1);
    hipEvent_t ev;
    EXPECT(hipEventCreate(&ev) == hipSuccess);
    fakehip_launch(a, "writer", {{p, true}}); // write-after-read across streams, unordered as well
    EXPECT(fakehip_hazards().size() == 1);
    EXPECT(hipEventRecord(ev, a) == hipSuccess && hipStreamWaitEvent(b, ev, 0) == hipSuccess);
    fakehip_launch(b, "reader", {{p, false}});
    EXPECT(fakehip_hazards().empty());
    char q[8];
    EXPECT(!fakehip_launch(a, "stray", {{q, true}})); // not device memory
    EXPECT(fakehip_hazards().size() == 1);
    (void)hipEventDestroy(ev);
    (void)hipStreamDestroy(a);
    (void)hipStreamDestroy(b);
    (void)hipFree(p);
}

// Calls may come from any thread (zyx serialises its own under one mutex, other hosts may not): several threads
// work on one context at once.
static void threads_share_a_context() {
    printf("threads\n");
    zhip_ctx *ctx = new_ctx();
    zhip_prog chain;
    zhip_kernel_desc d = chain_desc(16, 256);
    OK(zhip_register_kernel(ctx, &d, &chain));
    std::vector<std::thread> ts;
    for (int t = 0; t < 4; t++)
        ts.emplace_back([ctx, chain] {
            std::vector<float> host(4096, 2.0f), back(4096);
            for (int i = 0; i < 40; i++) {
                zhip_buf x, y;
                zhip_event ex, ey, up, done;
                if (zhip_alloc(ctx, 4097 * 4, &x, &ex) != ZHIP_OK || zhip_alloc(ctx, 4097 * 4, &y, &ey) != ZHIP_OK) abort();
                if (zhip_h2d(ctx, host.data(), 4096 * 4, x, &ex, 1, &up) != ZHIP_OK) abort();
                zhip_buf args[2] = {x, y};
                zhip_event w[2] = {up, ey};
                if (zhip_launch(ctx, chain, args, 2, w, 2, &done) != ZHIP_OK) abort();
                if (zhip_d2h(ctx, y, back.data(), 4096 * 4, &done, 1) != ZHIP_OK) abort();
                if (zhip_free(ctx, x, nullptr, 0) != ZHIP_OK || zhip_free(ctx, y, nullptr, 0) != ZHIP_OK) abort();
            }
        });
    for (auto &t : ts) t.join();
    no_hazards("threads");
    OK(zhip_deinit(ctx));
}

int main(int argc, char **argv) {
    const std::string only = argc > 1 ? argv[1] : "";
    auto want = [&](const char *name) { return only.empty() || only == name; };
    if (want("detector")) the_detector_detects();
    if (want("plan")) execute_plan_sequence();
    if (want("consumed")) consumed_event_still_orders();
    if (want("scratch")) program_scratch_is_serialised();
    if (want("cache")) freed_blocks_are_reused_in_order();
    if (want("plans")) plans_and_batch_copies();
    if (want("errors")) misuse_is_an_error_not_a_crash();
    if (want("ir")) generated_kernels_and_the_code_cache();
    if (want("static")) reduce_static_allocates_nothing();
    if (want("random"))
        for (unsigned seed = 1; seed <= 12; seed++) random_schedules(seed, 400);
    if (want("threads")) threads_share_a_context();
    printf(g_failures ? "FAILED: %d\n" : "all scenarios passed\n", g_failures);
    return g_failures ? 1 : 0;
}
