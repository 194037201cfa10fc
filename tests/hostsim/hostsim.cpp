// Runtime of the host execution model declared in hip/hip_runtime.h — TEST INFRASTRUCTURE.
//
// * launch(): the workgroups of a grid are dealt to a pool of OS threads; a launch returns when
//   all of them have finished (launches are therefore in stream order by construction).
// * A workgroup runs on one OS thread: each of its lanes is a fiber with its own stack; a fiber
//   runs until it reaches a rendezvous (wavefront operation or workgroup barrier) or returns.
// * hostsim_alloc(): buffers between inaccessible pages, filled with 0xFF (NaN in bf16 and fp32),
//   so an access outside a buffer faults and a read of never-written scratch shows in results.
// * Controls for walking large shapes: hostsim_set_block_filter() runs only some workgroups of
//   each launch, hostsim_set_skip_math() makes the MFMA a no-op (addresses and control flow only).
#include "hip/hip_runtime.h"

#include <signal.h>
#include <time.h>
#include <sys/mman.h>
#include <unistd.h>

#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <mutex>
#include <thread>
#include <dlfcn.h>
#include <link.h>
#include <string>
#include <vector>

namespace hostsim {

// ---------------------------------------------------------------------------------------------
// fibers
// ---------------------------------------------------------------------------------------------
extern "C" void hostsim_switch(void** save_sp, void* load_sp);
asm(R"(
.text
.globl hostsim_switch
.type hostsim_switch,@function
hostsim_switch:
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
.size hostsim_switch,.-hostsim_switch
)");

constexpr size_t kStackBytes = 512 * 1024;
constexpr int kMaxThreadsPerBlock = 1024;

struct Fiber {
    void* sp = nullptr;
    bool done = false;
    int wait_kind = 0;          // 0 runnable, 1 wavefront rendezvous, 2 workgroup barrier
    unsigned wait_gen = 0;
    Lane lane;
};

struct Wave {
    void* slot[64];
    unsigned long long mask = 0;
    int arrived = 0, alive = 0, tag = 0;
    unsigned gen = 0;
    Thunk thunk = nullptr;
    void* fnobj = nullptr;
};

struct Block {
    int arrived = 0, alive = 0;
    unsigned gen = 0;
};

struct Worker {
    char* stacks = nullptr;                 // kMaxThreadsPerBlock stacks
    char* lds = nullptr;                    // dynamic LDS
    void* sched_sp = nullptr;
    Fiber fibers[kMaxThreadsPerBlock];
    Wave waves[kMaxThreadsPerBlock / 64];
    Block block;
    const std::function<void()>* body = nullptr;
    const char* kernel = "";
};

static thread_local Worker* t_worker = nullptr;
static thread_local Lane* t_cur = nullptr;

Lane* cur() { return t_cur; }
char* dynamic_lds() { return t_worker->lds; }

static std::atomic<int> g_skip_math{0};
static std::atomic<int> g_schedule{0};      // order in which runnable lanes are resumed (see hostsim_set_schedule)
static std::atomic<int> g_fill{1};
static std::atomic<int> g_strict_lanes{1};   // see wave_complete
static std::atomic<int> g_poison_lds{0};    // overwrite all LDS with 0xFF before every workgroup (see hostsim_set_poison_lds)

// This thread's copy of the library's zero-initialised thread-local block: where every `__shared__`
// array of the kernels lives in this build (one copy per worker thread, as a CU has one LDS).
struct TlsSpan { char* base = nullptr; size_t bytes = 0; };
static int find_tls(dl_phdr_info* info, size_t, void* out) {
    const uintptr_t me = reinterpret_cast<uintptr_t>(&find_tls);
    bool mine = false;
    for (int i = 0; i < info->dlpi_phnum; ++i) {
        const ElfW(Phdr)& ph = info->dlpi_phdr[i];
        if (ph.p_type == PT_LOAD && me >= info->dlpi_addr + ph.p_vaddr && me < info->dlpi_addr + ph.p_vaddr + ph.p_memsz)
            mine = true;
    }
    if (!mine) return 0;
    for (int i = 0; i < info->dlpi_phnum; ++i) {
        const ElfW(Phdr)& ph = info->dlpi_phdr[i];
        if (ph.p_type == PT_TLS && info->dlpi_tls_data) {
            TlsSpan* t = static_cast<TlsSpan*>(out);
            t->base = static_cast<char*>(info->dlpi_tls_data) + ph.p_filesz;     // the part without initialisers
            t->bytes = ph.p_memsz - ph.p_filesz;
        }
    }
    return 1;
}
static void poison_lds(Worker* wk) {
    static thread_local TlsSpan span;
    static thread_local bool looked = false;
    Worker* const w = t_worker;
    Lane* const c = t_cur;
    if (!looked) {
        TlsSpan found;                  // a local: `span` itself lies in the block that is overwritten below
        dl_iterate_phdr(find_tls, &found);
        span = found;
        looked = true;
        if (getenv("HOSTSIM_DEBUG")) fprintf(stderr, "[hostsim] tls zero-init block %p + %zu (t_worker at %p)\n", (void*)found.base, found.bytes, (void*)&t_worker);
    }
    const TlsSpan keep = span;
    if (keep.base) memset(keep.base, 0xFF, keep.bytes);
    // the runtime's own thread-locals lie in the same block: let their addresses escape, so that the
    // compiler takes the memset to have changed them and keeps the stores that put them back
    asm volatile("" : : "r"(&t_worker), "r"(&t_cur), "r"(&span), "r"(&looked) : "memory");
    span = keep;
    looked = true;
    t_worker = w;
    t_cur = c;
    memset(wk->lds, 0xFF, 160 * 1024);
}

[[noreturn]] static void die(const char* what) {
    Lane* c = t_cur;
    fprintf(stderr, "\n[hostsim] %s", what);
    if (t_worker) fprintf(stderr, " in kernel %s", t_worker->kernel);
    if (c)
        fprintf(stderr, ", block (%u,%u,%u) thread %u", c->bidx.x, c->bidx.y, c->bidx.z, c->tidx.x);
    fprintf(stderr, "\n");
    fflush(stderr);
    abort();
}

static void yield_to_scheduler() {
    Fiber* f = static_cast<Fiber*>(t_cur->fiber);
    hostsim_switch(&f->sp, t_worker->sched_sp);
}

static void wave_complete(Wave* w) {
    // Matrix and cross-lane data operations of a wavefront some of whose lanes have already left the
    // kernel: the hardware takes the operands of such lanes from whatever their registers hold (MFMA
    // does not look at the execution mask), so the result of the remaining lanes is not defined.
    // Votes, readfirstlane and the wave barrier are defined for any set of active lanes.
    if (w->alive != 64 && (w->tag == 1 || w->tag == 4 || w->tag == 6) && g_strict_lanes.load(std::memory_order_relaxed))
        die("MFMA / shuffle / permlane in a wavefront with lanes that have exited");
    w->thunk(w->fnobj, w->slot, w->mask);
    for (int l = 0; l < 64; ++l) w->slot[l] = nullptr;
    w->mask = 0;
    w->arrived = 0;
    w->gen++;
}

void wave_rendezvous(int tag, void* mine, Thunk thunk, void* fnobj) {
    Lane* c = t_cur;
    Wave* w = c->wave;
    if (w->arrived == 0) {
        w->tag = tag;
        w->thunk = thunk;
        w->fnobj = fnobj;
    } else if (w->tag != tag) {
        char msg[128];
        snprintf(msg, sizeof msg, "divergent wavefront operation (op %d meets op %d)", tag, w->tag);
        die(msg);
    }
    w->slot[c->lane] = mine;
    w->mask |= 1ull << c->lane;
    if (++w->arrived == w->alive) {
        wave_complete(w);
        return;
    }
    Fiber* f = static_cast<Fiber*>(c->fiber);
    f->wait_kind = 1;
    f->wait_gen = w->gen;
    yield_to_scheduler();
}

void block_barrier() {
    Lane* c = t_cur;
    Block* b = c->block;
    if (++b->arrived == b->alive) {
        b->arrived = 0;
        b->gen++;
        return;
    }
    Fiber* f = static_cast<Fiber*>(c->fiber);
    f->wait_kind = 2;
    f->wait_gen = b->gen;
    yield_to_scheduler();
}

static void fiber_main() {
    Worker* wk = t_worker;
    (*wk->body)();
    Fiber* f = static_cast<Fiber*>(t_cur->fiber);
    f->done = true;
    yield_to_scheduler();
    die("finished fiber resumed");
}

static void worker_init(Worker* wk) {
    wk->stacks = static_cast<char*>(mmap(nullptr, kStackBytes * kMaxThreadsPerBlock, PROT_READ | PROT_WRITE,
                                         MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0));
    wk->lds = static_cast<char*>(mmap(nullptr, 160 * 1024, PROT_READ | PROT_WRITE,
                                      MAP_PRIVATE | MAP_ANONYMOUS, -1, 0));
    if (wk->stacks == MAP_FAILED || wk->lds == MAP_FAILED) die("mmap of fiber stacks failed");
}

static void run_block(Worker* wk, dim3 grid, dim3 block, dim3 bidx) {
    const int nt = (int)(block.x * block.y * block.z);
    if (nt > kMaxThreadsPerBlock || nt <= 0) die("workgroup size out of range");
    const int nw = (nt + 63) / 64;
    if (g_poison_lds.load(std::memory_order_relaxed)) poison_lds(wk);
    wk->block = Block{};
    wk->block.alive = nt;
    for (int w = 0; w < nw; ++w) {
        wk->waves[w] = Wave{};
        for (int l = 0; l < 64; ++l) wk->waves[w].slot[l] = nullptr;
        wk->waves[w].alive = (w + 1) * 64 <= nt ? 64 : nt - w * 64;
    }
    for (int t = 0; t < nt; ++t) {
        Fiber& f = wk->fibers[t];
        f.done = false;
        f.wait_kind = 0;
        f.lane.tidx = dim3(t % block.x, (t / block.x) % block.y, t / (block.x * block.y));
        f.lane.bidx = bidx;
        f.lane.bdim = block;
        f.lane.gdim = grid;
        f.lane.lane = t & 63;
        f.lane.wave = &wk->waves[t >> 6];
        f.lane.block = &wk->block;
        f.lane.fiber = &f;
        // initial frame: six callee-saved registers, then the entry point as return address;
        // after `ret` the stack pointer is 8 below a 16-byte boundary, as after a call
        char* top = wk->stacks + (size_t)(t + 1) * kStackBytes;
        void** sp = reinterpret_cast<void**>(top - 64);
        sp -= 1;                                  // alignment slot
        *--sp = reinterpret_cast<void*>(&fiber_main);
        for (int i = 0; i < 6; ++i) *--sp = nullptr;
        f.sp = sp;
    }
    int remaining = nt;
    const int schedule = g_schedule.load(std::memory_order_relaxed);
    unsigned pass = 0;
    while (remaining > 0) {
        bool progress = false;
        ++pass;
        for (int k = 0; k < nt; ++k) {
            // 0: lanes in order; 1: in reverse; 2: wavefronts in an order that rotates from pass to
            // pass.  A kernel free of races between wavefronts gives the same bits under all three.
            int t = k;
            if (schedule == 1) t = nt - 1 - k;
            else if (schedule == 2) t = (int)((((k >> 6) + pass * 7) % (unsigned)nw) << 6 | (k & 63));
            if (t >= nt) continue;
            Fiber& f = wk->fibers[t];
            if (f.done) continue;
            if (f.wait_kind == 1 && f.lane.wave->gen == f.wait_gen) continue;
            if (f.wait_kind == 2 && wk->block.gen == f.wait_gen) continue;
            f.wait_kind = 0;
            progress = true;
            t_cur = &f.lane;
            hostsim_switch(&wk->sched_sp, f.sp);
            if (f.done) {
                --remaining;
                Wave* w = f.lane.wave;
                --w->alive;
                if (w->arrived > 0 && w->arrived == w->alive) wave_complete(w);
                Block* b = &wk->block;
                --b->alive;
                if (b->arrived > 0 && b->arrived == b->alive) {
                    b->arrived = 0;
                    b->gen++;
                }
            }
        }
        if (!progress) die("deadlock: lanes wait at a rendezvous that the others never reach");
    }
    t_cur = nullptr;
}

// ---------------------------------------------------------------------------------------------
// thread pool
// ---------------------------------------------------------------------------------------------
struct Job {
    const char* name;
    dim3 grid, block;
    const std::function<void()>* body;
    std::atomic<long long> next{0};
    long long total = 0;
    std::atomic<int> pending{0};
};

// the pool's threads are detached and outlive static destruction: these objects are never destroyed
static std::mutex& g_mu = *new std::mutex;
static std::condition_variable& g_cv = *new std::condition_variable;
static std::condition_variable& g_done_cv = *new std::condition_variable;
static Job* g_job = nullptr;
static unsigned long long g_job_seq = 0;
static std::vector<std::thread>& g_pool = *new std::vector<std::thread>;
static int g_threads = 0;
static bool g_stop = false;
static long long g_filter_stride = 1, g_filter_edge = 0;

static bool block_selected(long long i, long long total) {
    if (g_filter_stride <= 1) return true;
    return i < g_filter_edge || i >= total - g_filter_edge || i % g_filter_stride == 0;
}

static void work_on(Job* j, Worker* wk) {
    wk->body = j->body;
    wk->kernel = j->name;
    for (;;) {
        long long i = j->next.fetch_add(1);
        if (i >= j->total) break;
        // schedule 3: the workgroups of a launch in descending order (results may not depend on the
        // order in which workgroups run: nothing orders them on the GPU)
        if (g_schedule.load(std::memory_order_relaxed) == 3) i = j->total - 1 - i;
        if (!block_selected(i, j->total)) continue;
        dim3 b((unsigned)(i % j->grid.x), (unsigned)((i / j->grid.x) % j->grid.y),
               (unsigned)(i / ((long long)j->grid.x * j->grid.y)));
        run_block(wk, j->grid, j->block, b);
    }
}

static void pool_main() {
    Worker* wk = new Worker;
    worker_init(wk);
    t_worker = wk;
    unsigned long long seen = 0;
    for (;;) {
        Job* j;
        {
            std::unique_lock<std::mutex> lk(g_mu);
            g_cv.wait(lk, [&] { return g_stop || (g_job && g_job_seq != seen); });
            if (g_stop) return;
            j = g_job;
            seen = g_job_seq;
        }
        work_on(j, wk);
        if (j->pending.fetch_sub(1) == 1) {
            std::lock_guard<std::mutex> lk(g_mu);
            g_done_cv.notify_all();
        }
    }
}

static void ensure_pool() {
    if (g_threads) return;
    const char* e = getenv("HOSTSIM_THREADS");
    int n = e ? atoi(e) : (int)std::thread::hardware_concurrency();
    if (n < 1) n = 1;
    if (n > 16) n = 16;
    g_threads = n;
    for (int i = 0; i < n; ++i) g_pool.emplace_back(pool_main);
    for (auto& t : g_pool) t.detach();
}

static std::mutex& g_launch_mu = *new std::mutex;
static std::atomic<long long> g_launches{0};
struct KernelStat { const char* name; long long launches, blocks; double seconds; };
// largest workgroup each kernel was ever launched with (kept for the life of the process)
struct KernelShape { const char* name; unsigned threads; };
static std::vector<KernelShape>& g_shapes = *new std::vector<KernelShape>;
static std::vector<KernelStat>& g_stats = *new std::vector<KernelStat>;
static double now_s() {
    timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return ts.tv_sec + 1e-9 * ts.tv_nsec;
}

void launch(const char* name, dim3 grid, dim3 block, size_t dyn_lds, const std::function<void()>& body) {
    std::lock_guard<std::mutex> launch_lock(g_launch_mu);
    if (dyn_lds > 160 * 1024) die("dynamic LDS request above 160 KiB");
    // what hipLaunchKernel refuses on the GPU
    if (grid.y > 65535u || grid.z > 65535u || grid.x > 0x7fffffffu) die("grid dimension above the launch limit");
    const unsigned long long nthreads = (unsigned long long)block.x * block.y * block.z;
    if (nthreads == 0 || nthreads > (unsigned long long)kMaxThreadsPerBlock) die("workgroup size outside 1..1024");
    {
        bool seen = false;
        for (KernelShape& k : g_shapes)
            if (k.name == name || strcmp(k.name, name) == 0) {
                if (k.threads < nthreads) k.threads = (unsigned)nthreads;
                seen = true;
                break;
            }
        if (!seen) g_shapes.push_back({name, (unsigned)nthreads});
    }
    ensure_pool();
    g_launches++;
    Job j;
    j.name = name;
    j.grid = grid;
    j.block = block;
    j.body = &body;
    j.total = (long long)grid.x * grid.y * grid.z;
    if (j.total <= 0) return;
    j.pending = g_threads;
    const double t0 = now_s();
    {
        std::lock_guard<std::mutex> lk(g_mu);
        g_job = &j;
        ++g_job_seq;
    }
    g_cv.notify_all();
    {
        std::unique_lock<std::mutex> lk(g_mu);
        g_done_cv.wait(lk, [&] { return j.pending.load() == 0; });
        g_job = nullptr;
    }
    const double dt = now_s() - t0;
    for (KernelStat& k : g_stats)
        if (k.name == name || strcmp(k.name, name) == 0) {
            k.launches++; k.blocks += j.total; k.seconds += dt;
            return;
        }
    g_stats.push_back({name, 1, j.total, dt});
}

// ---------------------------------------------------------------------------------------------
// MFMA
// ---------------------------------------------------------------------------------------------
void mfma_32x32x16_bf16_all(MfmaArgs** s) {
    if (g_skip_math.load(std::memory_order_relaxed)) return;
    float A[32][16], Bm[16][32], D[32][32];
    for (int l = 0; l < 64; ++l) {
        const int col = l & 31, half = l >> 5;
        if (!s[l]) {
            for (int e = 0; e < 8; ++e) { A[col][8 * half + e] = 0.f; Bm[8 * half + e][col] = 0.f; }
            for (int v = 0; v < 16; ++v) D[8 * (v >> 2) + 4 * half + (v & 3)][col] = 0.f;
            continue;
        }
        for (int e = 0; e < 8; ++e) {
            A[col][8 * half + e] = (float)s[l]->a[e];
            Bm[8 * half + e][col] = (float)s[l]->b[e];
        }
        for (int v = 0; v < 16; ++v) D[8 * (v >> 2) + 4 * half + (v & 3)][col] = s[l]->c[v];
    }
    for (int i = 0; i < 32; ++i)
        for (int k = 0; k < 16; ++k) {
            const float a = A[i][k];
            for (int j = 0; j < 32; ++j) D[i][j] += a * Bm[k][j];
        }
    for (int l = 0; l < 64; ++l) {
        if (!s[l]) continue;
        const int col = l & 31, half = l >> 5;
        for (int v = 0; v < 16; ++v) s[l]->c[v] = D[8 * (v >> 2) + 4 * half + (v & 3)][col];
    }
}

// ---------------------------------------------------------------------------------------------
// guard-paged buffers
// ---------------------------------------------------------------------------------------------
struct Alloc { char* base; size_t map_bytes; char* user; size_t bytes; };
static std::mutex& g_alloc_mu = *new std::mutex;
static std::vector<Alloc>& g_allocs = *new std::vector<Alloc>;
static struct sigaction g_old_segv, g_old_bus;

static void segv_handler(int sig, siginfo_t* info, void*) {
    char* addr = static_cast<char*>(info->si_addr);
    fprintf(stderr, "\n[hostsim] invalid memory access at %p", (void*)addr);
    if (t_worker) fprintf(stderr, " in kernel %s", t_worker->kernel);
    if (t_cur)
        fprintf(stderr, ", block (%u,%u,%u) thread %u", t_cur->bidx.x, t_cur->bidx.y, t_cur->bidx.z,
                t_cur->tidx.x);
    for (const Alloc& a : g_allocs)
        if (addr >= a.base && addr < a.base + a.map_bytes)
            fprintf(stderr, ": %lld bytes past the start of a %zu-byte buffer", (long long)(addr - a.user), a.bytes);
    fprintf(stderr, "\n");
    fflush(stderr);
    // hand over to whoever handled the signal before (Python's faulthandler, or the default
    // action): returning re-executes the faulting access under that handler
    sigaction(sig, sig == SIGSEGV ? &g_old_segv : &g_old_bus, nullptr);
}

// A trap of a checking build (HOSTSIM_EXTRA_FLAGS with the compiler's checks in trapping mode): say where, as an offset
// into this library that `llvm-symbolizer -e libkfold_hostsim.so` resolves when built with -g.
static struct sigaction g_old_ill;
static void ill_handler(int sig, siginfo_t* info, void*) {
    Dl_info dl;
    memset(&dl, 0, sizeof dl);
    dladdr(info->si_addr, &dl);
    fprintf(stderr, "\n[hostsim] trap at %p (library offset 0x%llx)", info->si_addr,
            (unsigned long long)(static_cast<char*>(info->si_addr) - static_cast<char*>(dl.dli_fbase)));
    if (t_worker) fprintf(stderr, " in kernel %s", t_worker->kernel);
    if (t_cur)
        fprintf(stderr, ", block (%u,%u,%u) thread %u", t_cur->bidx.x, t_cur->bidx.y, t_cur->bidx.z, t_cur->tidx.x);
    fprintf(stderr, "\n");
    fflush(stderr);
    sigaction(sig, &g_old_ill, nullptr);
}

__attribute__((constructor)) static void install_handler() {
    // the handler runs on the faulting fiber's own stack, which is ordinary mapped memory
    struct sigaction sa;
    memset(&sa, 0, sizeof sa);
    sa.sa_sigaction = segv_handler;
    sa.sa_flags = SA_SIGINFO;
    sigaction(SIGSEGV, &sa, &g_old_segv);
    sigaction(SIGBUS, &sa, &g_old_bus);
    sa.sa_sigaction = ill_handler;
    sigaction(SIGILL, &sa, &g_old_ill);
}

}  // namespace hostsim

extern "C" {

// `bytes` of memory whose last byte (rounded up to `align`) is followed by an inaccessible page
// and whose first byte is preceded by one (at a distance below a page); filled with 0xFF unless
// hostsim_set_fill(0) was called.
void* hostsim_alloc(size_t bytes, size_t align) {
    using namespace hostsim;
    const size_t page = (size_t)sysconf(_SC_PAGESIZE);
    if (align == 0) align = 256;
    const size_t padded = (bytes + align - 1) / align * align;
    const size_t body = (padded + page - 1) / page * page;
    char* base = static_cast<char*>(mmap(nullptr, body + 2 * page, PROT_READ | PROT_WRITE,
                                         MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0));
    if (base == MAP_FAILED) return nullptr;
    mprotect(base, page, PROT_NONE);
    mprotect(base + page + body, page, PROT_NONE);
    char* user = base + page + (body - padded);
    if (hostsim::g_fill.load()) memset(base + page, 0xFF, body);
    std::lock_guard<std::mutex> lk(g_alloc_mu);
    g_allocs.push_back({base, body + 2 * page, user, bytes});
    return user;
}

void hostsim_free(void* p) {
    using namespace hostsim;
    std::lock_guard<std::mutex> lk(g_alloc_mu);
    for (size_t i = 0; i < g_allocs.size(); ++i)
        if (g_allocs[i].user == p) {
            munmap(g_allocs[i].base, g_allocs[i].map_bytes);
            g_allocs.erase(g_allocs.begin() + i);
            return;
        }
}

// Run only workgroups whose linear index is below `edge`, within `edge` of the end, or a multiple
// of `stride` (stride <= 1: all).
void hostsim_set_block_filter(long long stride, long long edge) {
    hostsim::g_filter_stride = stride;
    hostsim::g_filter_edge = edge;
}

// 1 (default): new buffers are filled with 0xFF; 0: left as the zero pages the kernel maps
void hostsim_set_fill(int on) { hostsim::g_fill.store(on); }
void hostsim_set_strict_lanes(int on) { hostsim::g_strict_lanes.store(on); }
// 1: every workgroup starts with all of its LDS (static arrays and the dynamic part) set to 0xFF
// bytes, NaN as bf16 and as fp32, so a read of LDS that the workgroup has not written shows in the
// result; costs a few MB of memset per workgroup, so it is for small problems
void hostsim_set_poison_lds(int on) { hostsim::g_poison_lds.store(on); }
// Order in which the lanes of a workgroup are resumed: 0 ascending, 1 descending, 2 wavefronts
// rotating.  Results of a correctly synchronised kernel do not depend on it.
void hostsim_set_schedule(int mode) { hostsim::g_schedule.store(mode); }
void hostsim_set_skip_math(int on) { hostsim::g_skip_math.store(on); }
// per-kernel launch counts and host seconds since the last call, to stderr
void hostsim_report(void) {
    for (const hostsim::KernelStat& k : hostsim::g_stats)
        fprintf(stderr, "[hostsim] %-60s launches %5lld  blocks %9lld  %8.3f s\n", k.name, k.launches, k.blocks, k.seconds);
    hostsim::g_stats.clear();
}
long long hostsim_launch_count(void) { return hostsim::g_launches.load(); }
// "name\tthreads\n" per kernel launched so far: the largest workgroup it was launched with;
// returns the length needed (the text is cut to `cap` bytes including the final NUL)
size_t hostsim_launch_shapes(char* buf, size_t cap) {
    std::lock_guard<std::mutex> lk(hostsim::g_launch_mu);
    std::string out;
    for (const hostsim::KernelShape& k : hostsim::g_shapes) out += std::string(k.name) + "\t" + std::to_string(k.threads) + "\n";
    if (buf && cap) {
        const size_t n = out.size() < cap - 1 ? out.size() : cap - 1;
        memcpy(buf, out.data(), n);
        buf[n] = 0;
    }
    return out.size() + 1;
}
int hostsim_threads(void) { hostsim::ensure_pool(); return hostsim::g_threads; }

}  // extern "C"
