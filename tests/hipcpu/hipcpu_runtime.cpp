/*
 * Test infrastructure: the runtime behind tests/hipcpu/hip/hip_runtime.h.
 * Work-items are ucontext fibers on one OS thread; workgroups run one after the other.
 */
#include <hip/hip_runtime.h>
#include <sys/mman.h>
#include <ucontext.h>
#include <unistd.h>
#include <functional>
#include <map>
#include <vector>

extern "C" {
HipCpuItem *hipcpu_cur = nullptr;
dim3 hipcpu_block_idx, hipcpu_block_dim, hipcpu_grid_dim;
}

namespace {

constexpr size_t STACK_BYTES = 512 * 1024;
constexpr size_t PAGE = 4096;

struct Fiber {
    HipCpuItem item;
    ucontext_t ctx;
    char *stack = nullptr;
    bool done = false;
};

struct Wave {
    uint32_t table[64 * 16];
    int arrived = 0, gen = 0;   /* barrier of the live lanes */
    int live = 0;
};

std::vector<Fiber> g_fibers;
std::vector<Wave> g_waves;
ucontext_t g_sched;
int g_n = 0, g_live = 0, g_block_arrived = 0, g_block_gen = 0;
void (*g_entry)(void *) = nullptr;
void *g_closure = nullptr;
void *g_lds = nullptr;
long g_switches_without_progress = 0;
/* HIPCPU_ORDER=reverse runs the work-items of a workgroup, and the workgroups of a grid, from
   the last to the first.  Results must not change: between two barriers every order is one
   the hardware may choose, so a difference is a missing barrier (or a workgroup that relies
   on another one of the same launch). */
const bool g_reverse = getenv("HIPCPU_ORDER") && !strcmp(getenv("HIPCPU_ORDER"), "reverse");

void die(const char *msg)
{
    fprintf(stderr, "hipcpu: %s\n", msg);
    abort();
}

/* ---- guarded allocations: the block ends at a PROT_NONE page ------------------------- */
struct Guarded { void *map; size_t map_len; };
std::map<void *, Guarded> g_allocs;

void *guarded_alloc(size_t n)
{
    if (n == 0) n = 1;
    const size_t body = (n + PAGE - 1) / PAGE * PAGE;
    const size_t len = body + 2 * PAGE;
    char *m = (char *)mmap(nullptr, len, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
    if (m == MAP_FAILED) return nullptr;
    mprotect(m, PAGE, PROT_NONE);
    mprotect(m + PAGE + body, PAGE, PROT_NONE);
    /* right-aligned to 16 bytes (what the widest vector access needs): an access that
       starts 16 bytes or more past the end faults */
    char *p = m + PAGE + body - (n + 15) / 16 * 16;
    memset(p, 0xA5, (n + 15) / 16 * 16); /* fresh device memory is not zero */
    g_allocs[p] = Guarded{ m, len };
    return p;
}

/* ---- the stream: a queue of launches and copies, drained at the waits ---------------------- */
std::vector<std::function<void()>> g_queue;
bool g_draining = false;
const bool g_sync = getenv("HIPCPU_SYNC") && atoi(getenv("HIPCPU_SYNC")) != 0;

bool in_runtime_block(const void *q)
{
    auto it = g_allocs.upper_bound(const_cast<void *>(q));
    if (it == g_allocs.begin()) return false;
    --it;
    const char *end = (const char *)it->second.map + it->second.map_len - PAGE;
    return (const char *)q >= (const char *)it->first && (const char *)q < end;
}

void flush_copies()
{
    if (g_draining) return;
    g_draining = true;
    for (size_t i = 0; i < g_queue.size(); i++) g_queue[i]();
    g_queue.clear();
    g_draining = false;
}

void guarded_free(void *p)
{
    if (!p) return;
    flush_copies(); /* the runtime waits for the device before it releases memory */
    auto it = g_allocs.find(p);
    if (it == g_allocs.end()) die("free of a pointer that hipMalloc did not return");
    munmap(it->second.map, it->second.map_len);
    g_allocs.erase(it);
}

/* ---- fibers ------------------------------------------------------------------------------ */
void yield_to_scheduler()
{
    Fiber *f = &g_fibers[hipcpu_cur->linear];
    swapcontext(&f->ctx, &g_sched);
}

void fiber_main()
{
    Fiber *f = &g_fibers[hipcpu_cur->linear];
    g_entry(g_closure);
    f->done = true;
    g_live--;
    g_waves[f->item.wave].live--;
    g_switches_without_progress = 0;
    /* a barrier that only waited for this work-item completes now */
    if (g_live > 0 && g_block_arrived == g_live && g_block_arrived > 0) {
        g_block_arrived = 0;
        g_block_gen++;
    }
    Wave &w = g_waves[f->item.wave];
    if (w.live > 0 && w.arrived == w.live && w.arrived > 0) {
        w.arrived = 0;
        w.gen++;
    }
    swapcontext(&f->ctx, &g_sched);
}

void run_block()
{
    g_live = g_n;
    g_block_arrived = 0;
    for (Wave &w : g_waves) { w.arrived = 0; w.live = 0; }
    for (int i = 0; i < g_n; i++) {
        Fiber &f = g_fibers[i];
        f.done = false;
        g_waves[f.item.wave].live++;
        getcontext(&f.ctx);
        f.ctx.uc_stack.ss_sp = f.stack;
        f.ctx.uc_stack.ss_size = STACK_BYTES;
        f.ctx.uc_link = nullptr;
        makecontext(&f.ctx, fiber_main, 0);
    }
    g_switches_without_progress = 0;
    while (g_live > 0) {
        for (int k = 0; k < g_n && g_live > 0; k++) {
            Fiber &f = g_fibers[g_reverse ? g_n - 1 - k : k];
            if (f.done) continue;
            hipcpu_cur = &f.item;
            swapcontext(&g_sched, &f.ctx);
            if (++g_switches_without_progress > 64L * g_n + 1000000)
                die("deadlock: every work-item waits (a barrier or a wavefront collective inside divergent code?)");
        }
    }
    hipcpu_cur = nullptr;
}

} // namespace

extern "C" {

void *hipcpu_dynamic_lds(void) { return g_lds; }

void hipcpu_syncthreads(void)
{
    const int gen = g_block_gen;
    if (++g_block_arrived == g_live) {
        g_block_arrived = 0;
        g_block_gen++;
        g_switches_without_progress = 0;
        return;
    }
    while (g_block_gen == gen) yield_to_scheduler();
}

void hipcpu_wave_barrier(void)
{
    Wave &w = g_waves[hipcpu_cur->wave];
    const int gen = w.gen;
    if (++w.arrived == w.live) {
        w.arrived = 0;
        w.gen++;
        g_switches_without_progress = 0;
        return;
    }
    while (w.gen == gen) yield_to_scheduler();
}

const uint32_t *hipcpu_wave_exchange(const uint32_t *words, int n)
{
    Wave &w = g_waves[hipcpu_cur->wave];
    if (n > 16) die("wave exchange of more than 16 words");
    memcpy(w.table + hipcpu_cur->lane * 16, words, sizeof(uint32_t) * n);
    hipcpu_wave_barrier();
    return w.table;
}

void hipcpu_launch(dim3 grid, dim3 block, size_t shmem, void (*entry)(void *), void *closure)
{
    if (hipcpu_cur) die("a kernel launched a kernel");
    const int n = (int)(block.x * block.y * block.z);
    if (n < 1 || n > 1024) die("workgroup size outside [1, 1024]");
    if (shmem > 160 * 1024) die("more than 160 KiB of dynamic LDS");
    if ((int)g_fibers.size() < n) {
        size_t old = g_fibers.size();
        g_fibers.resize(n);
        for (size_t i = old; i < (size_t)n; i++) {
            g_fibers[i].stack = (char *)mmap(nullptr, STACK_BYTES, PROT_READ | PROT_WRITE,
                                             MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
            if (g_fibers[i].stack == MAP_FAILED) die("cannot map a fiber stack");
        }
    }
    g_n = n;
    g_waves.assign((n + 63) / 64, Wave());
    for (int i = 0; i < n; i++) {
        HipCpuItem &it = g_fibers[i].item;
        it.linear = i;
        it.tid = dim3(i % block.x, (i / block.x) % block.y, i / (block.x * block.y));
        it.wave = i / 64;
        it.lane = i % 64;
    }
    g_entry = entry;
    g_closure = closure;
    g_lds = shmem ? guarded_alloc(shmem) : nullptr;
    hipcpu_block_dim = block;
    hipcpu_grid_dim = grid;
    const uint64_t n_blocks = (uint64_t)grid.x * grid.y * grid.z;
    for (uint64_t k = 0; k < n_blocks; k++) {
        const uint64_t b = g_reverse ? n_blocks - 1 - k : k;
        hipcpu_block_idx = dim3((unsigned)(b % grid.x), (unsigned)(b / grid.x % grid.y),
                                (unsigned)(b / ((uint64_t)grid.x * grid.y)));
        run_block();
    }
    if (g_lds) guarded_free(g_lds);
    g_lds = nullptr;
}

hipError_t hipMalloc(void **p, size_t n)
{
    *p = guarded_alloc(n);
    return *p ? hipSuccess : hipErrorOutOfMemory;
}
hipError_t hipFree(void *p) { guarded_free(p); return hipSuccess; }
hipError_t hipHostMalloc(void **p, size_t n, unsigned) { return hipMalloc(p, n); }
hipError_t hipHostFree(void *p) { return hipFree(p); }
void hipcpu_flush_copies(void) { flush_copies(); }
hipError_t hipcpu_memcpy_async(void *d, const void *s, size_t n)
{
    if (in_runtime_block(d) && in_runtime_block(s)) {
        hipcpu_enqueue([d, s, n]() { memmove(d, s, n); });
    } else if (in_runtime_block(d)) {
        /* pageable source: staged before the call returns, written in stream order */
        std::vector<char> staged((const char *)s, (const char *)s + n);
        hipcpu_enqueue([d, staged]() { memcpy(d, staged.data(), staged.size()); });
    } else {
        flush_copies(); /* pageable destination: the call waits */
        memmove(d, s, n);
    }
    return hipSuccess;
}

} // extern "C"

void hipcpu_enqueue(std::function<void()> op)
{
    if (g_sync || g_draining) { op(); return; }
    g_queue.push_back(std::move(op));
    if (g_queue.size() >= 100000) flush_copies();
}
