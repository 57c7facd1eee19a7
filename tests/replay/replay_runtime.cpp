// The runtime behind tests/replay/hip/hip_runtime.h: fibres, the workgroup scheduler, "device" memory and the few
// runtime calls the library's host side makes.  Test infrastructure; see the header for what is modelled.
#include <hip/hip_runtime.h>

#include <dlfcn.h>
#include <sys/mman.h>

#include <atomic>
#include <condition_variable>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define REPLAY_ASAN 1
#include <sanitizer/common_interface_defs.h>
#endif
#endif
// functions whose frames are abandoned when a fibre ends must leave no poisoned red zones on a stack that is used again
#define REPLAY_NO_ASAN __attribute__((no_sanitize("address")))

// ---- context switch (x86-64 System V): callee-saved registers on the old stack, swap stack pointers -----------------
extern "C" void replay_switch(void** save_sp, void* load_sp);
asm(R"(
.text
.globl replay_switch
.type replay_switch,@function
replay_switch:
    pushq %rbp
    pushq %rbx
    pushq %r12
    pushq %r13
    pushq %r14
    pushq %r15
    movq %rsp, (%rdi)
    movq %rsi, %rsp
    popq %r15
    popq %r14
    popq %r13
    popq %r12
    popq %rbx
    popq %rbp
    ret
.size replay_switch,.-replay_switch
)");

namespace replay {

thread_local Lane* cur = nullptr;
int late_loads = 0;

namespace {

constexpr size_t STACK_BYTES = 256 * 1024;
constexpr int MAX_LANES = 1024;

std::mutex g_mem_mutex;
std::map<uintptr_t, size_t> g_allocs; // every hipMalloc'ed block and every range the test registered
std::atomic<int> g_failed{0};
char g_failure[1024];
std::mutex g_fail_mutex;

// per OS thread: the fibres of the workgroup it is running
struct Worker {
    char* stacks = nullptr;
    Lane lanes[MAX_LANES];
    Wave waves[MAX_LANES / WAVE];
    Workgroup wg;
    int n = 0;
    void* main_sp = nullptr;
    const std::function<void()>* body = nullptr;
#ifdef REPLAY_ASAN
    const void* main_stack_bottom = nullptr;
    size_t main_stack_size = 0;
#endif
};
thread_local Worker* tl_worker = nullptr;

REPLAY_NO_ASAN void switch_to(Worker* w, Lane* from, Lane* to, bool from_is_finished = false) { // `to` == nullptr: back to the thread's own stack
    void** save = from ? &from->sp : &w->main_sp;
    void* load = to ? to->sp : w->main_sp;
    cur = to;
#ifdef REPLAY_ASAN
    void* fake = nullptr;
    void** fake_save = from_is_finished ? nullptr : &fake; // a fibre that never runs again gives its fake stack back
    if (to) __sanitizer_start_switch_fiber(fake_save, w->stacks + (size_t)to->index * STACK_BYTES, STACK_BYTES);
    else __sanitizer_start_switch_fiber(fake_save, w->main_stack_bottom, w->main_stack_size);
    replay_switch(save, load);
    const void* old_bottom;
    size_t old_size;
    __sanitizer_finish_switch_fiber(fake, &old_bottom, &old_size);
#else
    replay_switch(save, load);
#endif
}

bool runnable(const Lane& l) {
    if (l.state == 0) return true;
    if (l.state == 1) return l.wave->gen != l.wait_gen;
    if (l.state == 2) return l.wg->gen != l.wait_gen;
    return false;
}

// hands the processor to the next lane that can run; returns when this lane can
void yield_lane() {
    Worker* w = tl_worker;
    Lane* me = cur;
    for (int step = 1; step <= w->n; ++step) {
        Lane* cand = &w->lanes[(me->index + step) % w->n];
        if (cand == me) break;
        if (runnable(*cand)) {
            cand->state = 0;
            switch_to(w, me, cand);
            // resumed: whoever switched here saw this lane runnable
            return;
        }
    }
    if (runnable(*me)) { me->state = 0; return; }
    // nobody can run: the workgroup is stuck
    int at_wave = 0, at_wg = 0, done = 0;
    for (int i = 0; i < w->n; ++i) { at_wave += w->lanes[i].state == 1; at_wg += w->lanes[i].state == 2; done += w->lanes[i].state == 3; }
    fail("deadlock in kernel %s, workgroup (%u,%u,%u): %d lanes wait for their wavefront, %d at a workgroup barrier, %d have finished "
         "(a barrier or a wavefront-wide operation that not every live lane reaches)",
         w->wg.kernel, w->wg.bid.x, w->wg.bid.y, w->wg.bid.z, at_wave, at_wg, done);
}

REPLAY_NO_ASAN void lane_exit() {
    Worker* w = tl_worker;
    Lane* me = cur;
    complete_loads(0);
    me->state = 3;
    Wave* wv = me->wave;
    wv->alive[me->lane] = false;
    if (--wv->live > 0 && wv->arrived == wv->live) { wv->arrived = 0; ++wv->gen; }
    if (--w->wg.live > 0 && w->wg.arrived == w->wg.live) { w->wg.arrived = 0; ++w->wg.gen; }
    if (w->wg.live == 0) { switch_to(w, me, nullptr, true); }
    for (int step = 1; step < w->n; ++step) {
        Lane* cand = &w->lanes[(me->index + step) % w->n];
        if (runnable(*cand)) { cand->state = 0; switch_to(w, me, cand, true); }
    }
    int at_wave = 0, at_wg = 0;
    for (int i = 0; i < w->n; ++i) { at_wave += w->lanes[i].state == 1; at_wg += w->lanes[i].state == 2; }
    fail("deadlock in kernel %s, workgroup (%u,%u,%u): a lane finished while %d lanes wait for their wavefront and %d at a workgroup barrier",
         w->wg.kernel, w->wg.bid.x, w->wg.bid.y, w->wg.bid.z, at_wave, at_wg);
}

extern "C" REPLAY_NO_ASAN void replay_fibre_entry() {
#ifdef REPLAY_ASAN
    {
        const void* bottom;
        size_t size;
        __sanitizer_finish_switch_fiber(nullptr, &bottom, &size);
        if (cur->index == 0) { tl_worker->main_stack_bottom = bottom; tl_worker->main_stack_size = size; } // lane 0 is entered from the thread's own stack
    }
#endif
    (*tl_worker->body)();
    lane_exit();
    __builtin_trap(); // a finished fibre is never resumed
}

void run_workgroup(Worker* w, const char* name, dim3 grid, dim3 block, dim3 bid, const std::function<void()>& body) {
    const int n = (int)(block.x * block.y * block.z);
    w->n = n;
    w->body = &body;
    w->wg.bid = bid; w->wg.bdim = block; w->wg.gdim = grid;
    w->wg.live = n; w->wg.arrived = 0; w->wg.gen = 0; w->wg.kernel = name;
    const int nw = (n + WAVE - 1) / WAVE;
    for (int i = 0; i < nw; ++i) {
        w->waves[i].live = std::min(WAVE, n - i * WAVE); w->waves[i].arrived = 0; w->waves[i].gen = 0;
        for (int j = 0; j < WAVE; ++j) w->waves[i].alive[j] = j < w->waves[i].live;
    }
    for (int i = 0; i < n; ++i) {
        Lane& l = w->lanes[i];
        l.index = i; l.lane = i % WAVE; l.wave = &w->waves[i / WAVE]; l.wg = &w->wg;
        l.tid = dim3(i % block.x, (i / block.x) % block.y, i / (block.x * block.y));
        l.state = 0; l.wait_gen = 0; l.turn = 0; l.pend_head = 0; l.pend_count = 0;
        // a fresh stack: [return address of the entry function = 0][entry][six zeroed registers]
        uintptr_t top = (uintptr_t)(w->stacks + (size_t)(i + 1) * STACK_BYTES);
        top &= ~(uintptr_t)15;
        uint64_t* sp = (uint64_t*)top;
        *--sp = 0;
        *--sp = (uint64_t)(uintptr_t)&replay_fibre_entry;
        for (int r = 0; r < 6; ++r) *--sp = 0;
        l.sp = sp;
    }
    switch_to(w, nullptr, &w->lanes[0]);
    cur = nullptr;
}

Worker* make_worker() {
    Worker* w = new Worker();
    w->stacks = (char*)mmap(nullptr, (size_t)MAX_LANES * STACK_BYTES, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (w->stacks == MAP_FAILED) { perror("mmap"); abort(); }
    return w;
}

int worker_threads() {
    static int n = [] {
        const char* e = getenv("REPLAY_THREADS");
        int v = e ? atoi(e) : (int)std::thread::hardware_concurrency();
        return std::max(1, std::min(v, 64));
    }();
    return n;
}

} // namespace

void fail(const char* fmt, ...) {
    {
        std::lock_guard<std::mutex> lock(g_fail_mutex);
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(g_failure, sizeof(g_failure), fmt, ap);
        va_end(ap);
        g_failed = 1;
        fprintf(stderr, "replay: %s\n", g_failure);
        fflush(stderr);
    }
    // a kernel cannot be unwound from inside a fibre: the process ends here, as a faulting GPU program would
    _Exit(97);
}

void wave_sync() {
    Lane* l = cur;
    Wave* w = l->wave;
    if (++w->arrived == w->live) { w->arrived = 0; ++w->gen; return; }
    l->wait_gen = w->gen;
    l->state = 1;
    yield_lane();
}

void wg_barrier() {
    Lane* l = cur;
    Workgroup* g = l->wg;
    if (++g->arrived == g->live) { g->arrived = 0; ++g->gen; return; }
    l->wait_gen = g->gen;
    l->state = 2;
    yield_lane();
}

void complete_loads(int leave) {
    Lane* l = cur;
    while (l->pend_count > leave) {
        const PendingLoad& p = l->pending[l->pend_head];
        if (p.dst) std::memcpy(p.dst, p.src, 16);
        l->pend_head = (l->pend_head + 1) % MAX_PENDING;
        --l->pend_count;
    }
}

void check_global(const void* p, size_t bytes, bool write, const char* what) {
    // REPLAY_STRICT=0: operands come from an allocator this runtime does not see (a test that passes its own arrays);
    // the direct loads are then as unchecked as the plain ones
    static const bool strict = [] { const char* e = getenv("REPLAY_STRICT"); return !(e && e[0] == '0'); }();
    if (!strict) return;
    const uintptr_t a = (uintptr_t)p;
    bool ok = false;
    size_t count;
    {
        std::lock_guard<std::mutex> lock(g_mem_mutex);
        count = g_allocs.size();
        auto it = g_allocs.upper_bound(a);
        if (it != g_allocs.begin()) {
            --it;
            ok = a >= it->first && a + bytes <= it->first + it->second;
        }
    }
    if (ok || count == 0) return; // (nothing registered: the caller works on plain host memory and relies on the sanitizer)
    Lane* l = cur;
    fail("%s of %zu bytes at %p lies outside every device allocation: kernel %s, workgroup (%u,%u,%u), thread %u%s", what, bytes, p,
         l ? l->wg->kernel : "?", l ? l->wg->bid.x : 0, l ? l->wg->bid.y : 0, l ? l->wg->bid.z : 0, l ? l->tid.x : 0, write ? " (write)" : "");
}

namespace {
// a pool of threads that lives as long as the process (never joined: the process may end while they wait)
struct Pool {
    std::mutex m;
    std::condition_variable work_cv, done_cv;
    std::function<void()> job;
    uint64_t job_id = 0;
    int running = 0, size = 0;
};
Pool* g_pool = nullptr;

void pool_thread(Pool* p) {
    tl_worker = make_worker();
    uint64_t seen = 0;
    for (;;) {
        std::function<void()> job;
        {
            std::unique_lock<std::mutex> lock(p->m);
            p->work_cv.wait(lock, [&] { return p->job_id != seen; });
            seen = p->job_id;
            job = p->job;
        }
        job();
        {
            std::lock_guard<std::mutex> lock(p->m);
            if (--p->running == 0) p->done_cv.notify_all();
        }
    }
}

void run_on_pool(const std::function<void()>& job) {
    static std::mutex launch_mutex; // one launch at a time
    std::lock_guard<std::mutex> one(launch_mutex);
    if (!g_pool) {
        g_pool = new Pool();
        g_pool->size = worker_threads();
        for (int i = 0; i < g_pool->size; ++i) std::thread(pool_thread, g_pool).detach();
    }
    Pool* p = g_pool;
    std::unique_lock<std::mutex> lock(p->m);
    p->job = job;
    p->running = p->size;
    ++p->job_id;
    p->work_cv.notify_all();
    p->done_cv.wait(lock, [&] { return p->running == 0; });
}
} // namespace

std::atomic<long> g_launches{0};
std::string g_last_kernel; // (launches are serialized)

// REPLAY_DUMP_DIR: every launch leaves what is needed to run the same launch elsewhere (the emulator of the generated GPU code,
// tests/isa/): the kernel function (its offset in the file it lives in, for the symbol table), grid and block, the argument block, and
// every device allocation before and after the launch.
// (pages that are all 0x00 or all 0xFF are left out: the library's workspace is tens of megabytes of which a launch touches little; and the whole
// process writes at most REPLAY_DUMP_LIMIT_MB, 4096 by default, after which it records no further launch)
std::atomic<uint64_t> g_dumped{0};
bool dump_memory(const std::string& path) {
    static const uint64_t limit = (uint64_t)(getenv("REPLAY_DUMP_LIMIT_MB") ? atoll(getenv("REPLAY_DUMP_LIMIT_MB")) : 4096) << 20;
    if (g_dumped.load() > limit) return false;
    FILE* f = fopen(path.c_str(), "wb");
    if (!f) return false;
    constexpr size_t PAGE = 4096;
    static unsigned char fill[2][PAGE];
    std::memset(fill[0], 0x00, PAGE);
    std::memset(fill[1], 0xFF, PAGE); // (what hipMalloc leaves in an allocation here)
    std::lock_guard<std::mutex> lock(g_mem_mutex);
    for (const auto& a : g_allocs) {
        const unsigned char* base = (const unsigned char*)a.first;
        // pages that are all 0x00 or all 0xFF are not written: whichever kind there is more of is the allocation's background
        std::vector<uint64_t> plain[2], pages;
        for (size_t off = 0; off < a.second; off += PAGE) {
            const size_t n = std::min(PAGE, a.second - off);
            if (std::memcmp(base + off, fill[0], n) == 0) plain[0].push_back(off);
            else if (std::memcmp(base + off, fill[1], n) == 0) plain[1].push_back(off);
            else pages.push_back(off);
        }
        const int background = plain[1].size() > plain[0].size() ? 1 : 0;
        pages.insert(pages.end(), plain[1 - background].begin(), plain[1 - background].end());
        const uint64_t head[4] = {(uint64_t)a.first, (uint64_t)a.second, (uint64_t)pages.size(), background ? 0xFFull : 0ull};
        fwrite(head, sizeof(head), 1, f);
        for (uint64_t off : pages) {
            fwrite(&off, sizeof(off), 1, f);
            fwrite(base + off, 1, std::min(PAGE, a.second - (size_t)off), f);
        }
        g_dumped += sizeof(head) + pages.size() * (PAGE + 8);
    }
    fclose(f);
    return true;
}

void launch(const char* name, dim3 grid, dim3 block, std::function<void()> body, const KernelArgs& args) {
    const long index = g_launches++;
    g_last_kernel = name;
    const char* dump_dir = getenv("REPLAY_DUMP_DIR");
    char stem[512] = "";
    if (dump_dir && args.fn) {
        std::snprintf(stem, sizeof(stem), "%s/launch_%04ld", dump_dir, index);
        Dl_info info{};
        dladdr(args.fn, &info);
        FILE* f = fopen((std::string(stem) + ".txt").c_str(), "w");
        if (f) {
            fprintf(f, "kernel %s\nfile %s\noffset %llu\nsymbol %s\ngrid %u %u %u\nblock %u %u %u\nargs ", name, info.dli_fname ? info.dli_fname : "?",
                    (unsigned long long)((uintptr_t)args.fn - (uintptr_t)info.dli_fbase), info.dli_sname ? info.dli_sname : "?", grid.x, grid.y, grid.z,
                    block.x, block.y, block.z);
            for (unsigned char b : args.bytes) fprintf(f, "%02x", b);
            fprintf(f, "\n");
            fclose(f);
        }
        if (!dump_memory(std::string(stem) + ".before")) { remove((std::string(stem) + ".txt").c_str()); stem[0] = 0; }
    }
    const int64_t total = (int64_t)grid.x * grid.y * grid.z;
    if ((int64_t)block.x * block.y * block.z > MAX_LANES || total <= 0) fail("launch of %s: bad grid or block", name);
    // what the HIP runtime refuses: more than 65535 workgroups along y or z, 2^32 or more threads along one dimension
    if (grid.y > 65535u || grid.z > 65535u || (uint64_t)grid.x * block.x > 0xffffffffull || (uint64_t)grid.y * block.y > 0xffffffffull ||
        (uint64_t)grid.z * block.z > 0xffffffffull)
        fail("launch of %s: grid (%u,%u,%u) x block (%u,%u,%u) is beyond what a HIP launch takes", name, grid.x, grid.y, grid.z, block.x, block.y, block.z);
    std::atomic<int64_t> next{0};
    run_on_pool([&]() {
        for (;;) {
            const int64_t b = next.fetch_add(1);
            if (b >= total) break;
            const dim3 bid((unsigned)(b % grid.x), (unsigned)((b / grid.x) % grid.y), (unsigned)(b / ((int64_t)grid.x * grid.y)));
            run_workgroup(tl_worker, name, grid, block, bid, body);
        }
    });
    if (stem[0]) dump_memory(std::string(stem) + ".after");
}

} // namespace replay

// ---- runtime API --------------------------------------------------------------------------------------------------
struct replayStream { bool capturing = false; struct replayGraph* graph = nullptr; };
struct replayEvent { int dummy; };
struct LaunchRecord { std::string name; dim3 grid, block; std::function<void()> body; replay::KernelArgs args; };
struct replayGraph { std::vector<LaunchRecord> nodes; };
struct replayGraphExec { std::vector<LaunchRecord> nodes; };

namespace {
replayStream g_null_stream;
replayStream* stream_of(hipStream_t s) { return s ? s : &g_null_stream; }
} // namespace

namespace replay {
void enqueue(hipStream_t s, const char* name, dim3 grid, dim3 block, std::function<void()> body, KernelArgs args) {
    replayStream* st = stream_of(s);
    if (st->capturing) { st->graph->nodes.push_back(LaunchRecord{name, grid, block, std::move(body), std::move(args)}); return; }
    launch(name, grid, block, std::move(body), args);
}
} // namespace replay

hipError_t hipGetDeviceCount(int* n) { *n = 1; return hipSuccess; }
hipError_t hipSetDevice(int d) { return d == 0 ? hipSuccess : hipErrorInvalidValue; }
hipError_t hipGetDeviceProperties(hipDeviceProp_t* p, int) {
    std::memset(p, 0, sizeof(*p));
    std::snprintf(p->name, sizeof(p->name), "CPU replay of gfx950");
    std::snprintf(p->gcnArchName, sizeof(p->gcnArchName), "gfx950:replay");
    const char* e = getenv("REPLAY_CUS");
    p->multiProcessorCount = e ? atoi(e) : 256;
    p->totalGlobalMem = (size_t)1 << 36;
    return hipSuccess;
}
// Device memory is plain heap memory (under AddressSanitizer: with red zones on both sides).
hipError_t hipMalloc(void** p, size_t bytes) {
    void* q = nullptr;
    if (posix_memalign(&q, 256, bytes ? bytes : 1) != 0) return hipErrorOutOfMemory;
    std::memset(q, 0xFF, bytes); // device memory comes with whatever was there: NaNs here, so that nothing can lean on fresh pages being zero
    std::lock_guard<std::mutex> lock(replay::g_mem_mutex);
    replay::g_allocs[(uintptr_t)q] = bytes;
    *p = q;
    return hipSuccess;
}
hipError_t hipFree(void* p) {
    if (!p) return hipSuccess;
    {
        std::lock_guard<std::mutex> lock(replay::g_mem_mutex);
        replay::g_allocs.erase((uintptr_t)p);
    }
    free(p);
    return hipSuccess;
}
hipError_t hipMemcpy(void* dst, const void* src, size_t bytes, hipMemcpyKind) { std::memmove(dst, src, bytes); return hipSuccess; }
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind, hipStream_t s) {
    replayStream* st = stream_of(s);
    if (st->capturing) { st->graph->nodes.push_back(LaunchRecord{"memcpy", dim3(0), dim3(0), [=]() { std::memmove(dst, src, bytes); }, {}}); return hipSuccess; }
    std::memmove(dst, src, bytes);
    return hipSuccess;
}
hipError_t hipMemcpy2DAsync(void* dst, size_t dpitch, const void* src, size_t spitch, size_t width, size_t height, hipMemcpyKind, hipStream_t) {
    for (size_t r = 0; r < height; ++r) std::memmove((char*)dst + r * dpitch, (const char*)src + r * spitch, width);
    return hipSuccess;
}
hipError_t hipMemset(void* dst, int value, size_t bytes) { std::memset(dst, value, bytes); return hipSuccess; }
hipError_t hipMemsetAsync(void* dst, int value, size_t bytes, hipStream_t s) {
    replayStream* st = stream_of(s);
    if (st->capturing) { st->graph->nodes.push_back(LaunchRecord{"memset", dim3(0), dim3(0), [=]() { std::memset(dst, value, bytes); }, {}}); return hipSuccess; }
    std::memset(dst, value, bytes);
    return hipSuccess;
}
hipError_t hipStreamCreate(hipStream_t* s) { *s = new replayStream(); return hipSuccess; }
hipError_t hipStreamDestroy(hipStream_t s) { delete s; return hipSuccess; }
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipDeviceSynchronize() { return hipSuccess; }
hipError_t hipEventCreate(hipEvent_t* e) { *e = new replayEvent(); return hipSuccess; }
hipError_t hipEventDestroy(hipEvent_t e) { delete e; return hipSuccess; }
hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) { *ms = 1.0f; return hipSuccess; }
hipError_t hipGetLastError() { return hipSuccess; }
const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "error (CPU replay)"; }
hipError_t hipGetSymbolAddress(void** p, const void* symbol) { *p = const_cast<void*>(symbol); return hipSuccess; }
hipError_t hipStreamBeginCapture(hipStream_t s, hipStreamCaptureMode) {
    replayStream* st = stream_of(s);
    st->capturing = true;
    st->graph = new replayGraph();
    return hipSuccess;
}
hipError_t hipStreamEndCapture(hipStream_t s, hipGraph_t* g) {
    replayStream* st = stream_of(s);
    st->capturing = false;
    *g = st->graph;
    st->graph = nullptr;
    return hipSuccess;
}
hipError_t hipGraphInstantiate(hipGraphExec_t* exec, hipGraph_t g, void*, void*, size_t) {
    *exec = new replayGraphExec{g->nodes};
    return hipSuccess;
}
hipError_t hipGraphDestroy(hipGraph_t g) { delete g; return hipSuccess; }
hipError_t hipGraphExecDestroy(hipGraphExec_t e) { delete e; return hipSuccess; }
hipError_t hipGraphLaunch(hipGraphExec_t e, hipStream_t) {
    for (const LaunchRecord& n : e->nodes) {
        if (n.grid.x == 0) n.body();
        else replay::launch(n.name.c_str(), n.grid, n.block, n.body, n.args);
    }
    return hipSuccess;
}

// ---- for the tests ------------------------------------------------------------------------------------------------
extern "C" {
// a range of host memory that kernels may touch (operands the test allocated itself); 0 bytes: forget it
void replay_register(const void* p, size_t bytes) {
    std::lock_guard<std::mutex> lock(replay::g_mem_mutex);
    if (bytes) replay::g_allocs[(uintptr_t)p] = bytes;
    else replay::g_allocs.erase((uintptr_t)p);
}
void replay_set_late_loads(int on) { replay::late_loads = on; }
long replay_launch_count() { return replay::g_launches.load(); } // kernel launches executed so far
const char* replay_last_kernel() { return replay::g_last_kernel.c_str(); } // the kernel expression of the last launch, as the source spells it
}
