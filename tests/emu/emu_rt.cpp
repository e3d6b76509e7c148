// Runtime of the host-side kernel build (see include/hip/hip_runtime.h).  TEST INFRASTRUCTURE ONLY.
//
// Every GPU thread of a workgroup is a fiber (its own stack, switched in user space) on ONE OS
// thread; a scheduler runs the fibers round robin and a fiber leaves the CPU only at a barrier that
// is not complete yet.  Workgroups of a launch run on a few OS threads side by side (`__shared__`
// is thread-local storage).  A launch in which every live fiber waits and nothing can run is
// reported as a deadlock, with the barrier kinds, instead of hanging.  The dynamic LDS of a
// workgroup ends at an inaccessible page.
#include <hip/hip_runtime.h>

#include <stdlib.h>
#include <sys/mman.h>
#include <unistd.h>

#include <atomic>
#include <condition_variable>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

// void emu_ctx_switch(void** save_sp, void* load_sp): saves the callee-saved registers on the current
// stack, leaves the stack pointer in *save_sp and continues on the stack load_sp (System V x86-64).
asm(R"(
.text
.globl emu_ctx_switch
.type emu_ctx_switch,@function
emu_ctx_switch:
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
.size emu_ctx_switch,.-emu_ctx_switch
)");
extern "C" void emu_ctx_switch(void** save_sp, void* load_sp);

namespace emu {

Idx g_block_dim, g_grid_dim;

// Order in which a sweep of the scheduler visits the fibers of a workgroup: 0 ascending thread index, 1 descending,
// 2 a fresh random permutation per sweep.  Between two barriers the threads of a workgroup run one after the other
// in that order, so a pair of accesses that needs a barrier and has none sees the writer first under one order and
// the reader first under another: results that differ between orders are a race.
std::atomic<int> g_order_mode{0};
std::atomic<uint64_t> g_order_seed{1};
// QK_EMU_ORDER=reverse | random[:seed] sets the order for a whole process (a test file run on the host-side build)
static const bool g_order_from_env = [] {
    const char* e = getenv("QK_EMU_ORDER");
    if (!e) return false;
    const std::string v(e);
    if (v == "reverse") g_order_mode = 1;
    else if (v.rfind("random", 0) == 0) {
        g_order_mode = 2;
        if (v.size() > 7) g_order_seed = strtoull(v.c_str() + 7, nullptr, 10) | 1u;
    }
    return true;
}();

namespace {
constexpr int MAX_WAVES = 16;
constexpr size_t STACK_BYTES = 512 * 1024;

struct Fiber {
    void* sp = nullptr;
    uint8_t* stack = nullptr; // mapping of STACK_BYTES + one guard page below
    Idx tid{};
    bool done = false;
    int wait_kind = 0; // 0 runnable, 1 wave barrier, 2 block barrier
    uint64_t wait_gen = 0;
    uint32_t xn = 0; // cross-lane operations done so far: the same in every lane of a wave (they run in lockstep)
};

// n bytes that END at an inaccessible page: an access behind the buffer faults at once.
struct GuardBuf {
    uint8_t* map = nullptr;
    size_t map_bytes = 0;
    uint8_t* p = nullptr;
    explicit GuardBuf(size_t n, size_t align = 16)
    {
        const size_t page = (size_t)sysconf(_SC_PAGESIZE);
        const size_t body = (n + page - 1) / page * page;
        map_bytes = body + page;
        map = (uint8_t*)mmap(nullptr, map_bytes, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
        if (map == MAP_FAILED) abort();
        mprotect(map + body, page, PROT_NONE);
        p = map + body - (n + align - 1) / align * align; // aligned; for sizes that are multiples of `align` the end is exact
    }
    ~GuardBuf() { munmap(map, map_bytes); }
    GuardBuf(const GuardBuf&) = delete;
};

struct Workgroup {
    std::vector<Fiber> f;
    int n = 0;
    void* main_sp = nullptr;
    Fiber* cur = nullptr;
    Idx block{};
    const std::function<void()>* body = nullptr;
    uint64_t block_gen = 0, wave_gen[MAX_WAVES] = {};
    int block_arrived = 0, block_expected = 0, wave_arrived[MAX_WAVES] = {}, wave_expected[MAX_WAVES] = {};
    // Two buffers in turn: operation n + 2 writes where operation n was read, and a lane reaches it only through
    // the barrier of operation n + 1, which every lane passes after it has read n -- so one barrier per
    // operation is enough.
    uint64_t xbuf[MAX_WAVES][2][64];
    float mfma_a[MAX_WAVES][2][64][8], mfma_b[MAX_WAVES][2][64][8]; // the halves, widened once by the lane that owns them
    GuardBuf* dyn = nullptr;
    ~Workgroup()
    {
        for (auto& x : f)
            if (x.stack) munmap(x.stack, STACK_BYTES + 4096);
        delete dyn;
    }
};
thread_local Workgroup* t_wg = nullptr;

void yield_to_scheduler()
{
    Workgroup& g = *t_wg;
    emu_ctx_switch(&g.cur->sp, g.main_sp);
}

void fiber_entry()
{
    Workgroup& g = *t_wg;
    Fiber* me = g.cur;
    (*g.body)();
    // a thread that has left the kernel takes no further part in its barriers
    me->done = true;
    const int w = me->tid.x >> 6;
    if (--g.wave_expected[w] > 0 && g.wave_arrived[w] >= g.wave_expected[w]) {
        g.wave_arrived[w] = 0;
        g.wave_gen[w]++;
    }
    if (--g.block_expected > 0 && g.block_arrived >= g.block_expected) {
        g.block_arrived = 0;
        g.block_gen++;
    }
    yield_to_scheduler();
    abort(); // never resumed
}

void prepare_fiber(Fiber& fb, uint32_t tid)
{
    if (!fb.stack) {
        fb.stack = (uint8_t*)mmap(nullptr, STACK_BYTES + 4096, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
        if (fb.stack == MAP_FAILED) abort();
        mprotect(fb.stack, 4096, PROT_NONE);
    }
    uint64_t* top = (uint64_t*)(fb.stack + 4096 + STACK_BYTES); // 16-byte aligned
    top[-1] = 0;                                                // what fiber_entry would return to
    top[-2] = (uint64_t)(void*)&fiber_entry;
    for (int i = 3; i <= 8; i++) top[-i] = 0; // rbp, rbx, r12..r15
    fb.sp = top - 8;
    fb.tid = Idx{tid, 0, 0};
    fb.done = false;
    fb.wait_kind = 0;
    fb.xn = 0;
}

void run_workgroup(Workgroup& g, Idx block, int n, size_t lds, const std::function<void()>& body)
{
    t_wg = &g;
    g.block = block;
    g.body = &body;
    g.n = n;
    if ((int)g.f.size() < n) g.f.resize(n);
    for (int t = 0; t < n; t++) prepare_fiber(g.f[t], (uint32_t)t);
    g.block_arrived = 0;
    g.block_expected = n;
    for (int w = 0; w < n / 64; w++) {
        g.wave_arrived[w] = 0;
        g.wave_expected[w] = 64;
    }
    delete g.dyn;
    g.dyn = new GuardBuf(lds ? lds : 16);
    int live = n;
    const int mode = g_order_mode.load();
    uint64_t rng = g_order_seed.load() * 0x9E3779B97F4A7C15ull + (((uint64_t)block.z << 40) ^ ((uint64_t)block.y << 20) ^ block.x) + 1;
    std::vector<int> order((size_t)n);
    for (int t = 0; t < n; t++) order[(size_t)t] = mode == 1 ? n - 1 - t : t;
    // mode 2 also holds waves back: now and then a wave sits out up to 48 sweeps (a sweep is about one
    // cross-lane operation or matrix instruction of every other wave), so the waves of a workgroup drift apart
    // between two workgroup barriers as far as they may on a device
    int hold[MAX_WAVES] = {};
    while (live > 0) {
        bool ran = false, held = false;
        if (mode == 2) {
            for (int t = n - 1; t > 0; t--) { // Fisher-Yates on a xorshift stream
                rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17;
                std::swap(order[(size_t)t], order[(size_t)(rng % (uint64_t)(t + 1))]);
            }
            for (int w = 0; w < n / 64; w++) {
                rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17;
                if (hold[w] > 0) hold[w]--;
                else if ((rng & 7u) == 0) hold[w] = 1 + (int)((rng >> 8) % 48u);
            }
        }
        for (int k = 0; k < n; k++) {
            const int t = order[(size_t)k];
            Fiber& fb = g.f[t];
            if (fb.done) continue;
            if (fb.wait_kind == 1 && g.wave_gen[t >> 6] == fb.wait_gen) continue;
            if (fb.wait_kind == 2 && g.block_gen == fb.wait_gen) continue;
            if (hold[t >> 6] > 0) { held = true; continue; }
            fb.wait_kind = 0;
            g.cur = &fb;
            emu_ctx_switch(&g.main_sp, fb.sp);
            ran = true;
            if (fb.done) live--;
        }
        if (!ran && held) { // only held waves could run: let them
            for (int w = 0; w < MAX_WAVES; w++) hold[w] = 0;
            continue;
        }
        if (!ran) {
            int at_wave = 0, at_block = 0;
            for (int t = 0; t < n; t++)
                if (!g.f[t].done) (g.f[t].wait_kind == 1 ? at_wave : at_block)++;
            fprintf(stderr, "emu: deadlock in workgroup (%u,%u,%u): %d threads wait at a wave barrier or cross-lane operation, "
                            "%d at __syncthreads(), none can run\n", block.x, block.y, block.z, at_wave, at_block);
            abort();
        }
    }
    t_wg = nullptr;
}

std::mutex g_launch_mu; // one launch at a time
} // namespace


const Idx& cur_thread() { return t_wg->cur->tid; }
const Idx& cur_block() { return t_wg->block; }
void* dyn_lds() { return t_wg->dyn->p; }

void block_barrier()
{
    Workgroup& g = *t_wg;
    if (++g.block_arrived >= g.block_expected) {
        g.block_arrived = 0;
        g.block_gen++;
        return;
    }
    g.cur->wait_kind = 2;
    g.cur->wait_gen = g.block_gen;
    yield_to_scheduler();
}
void wave_barrier()
{
    Workgroup& g = *t_wg;
    const int w = g.cur->tid.x >> 6;
    if (++g.wave_arrived[w] >= g.wave_expected[w]) {
        g.wave_arrived[w] = 0;
        g.wave_gen[w]++;
        return;
    }
    g.cur->wait_kind = 1;
    g.cur->wait_gen = g.wave_gen[w];
    yield_to_scheduler();
}
const uint64_t* exchange(uint64_t v)
{
    Workgroup& g = *t_wg;
    const uint32_t t = g.cur->tid.x, par = g.cur->xn++ & 1u;
    g.xbuf[t >> 6][par][t & 63u] = v;
    wave_barrier();
    return t_wg->xbuf[t >> 6][par];
}
void exchange_done() {} // the values stay valid until the wave's next operation but one

// ---- LDS bank model ------------------------------------------------------------------------------
bool g_lds_probe_on = false;
constexpr int PROBE_SITES = 8;
static std::atomic<uint64_t> g_probe[PROBE_SITES][3]; // wave instructions, cycles in the model, cycles without conflicts
void lds_probe(int site, const void* p, int bytes)
{
    const uint32_t t = t_wg->cur->tid.x;
    const uint64_t* all = exchange((uint64_t)(uintptr_t)p);
    if ((t & 63u) == 0 && site >= 0 && site < PROBE_SITES) {
        const uint32_t lanes = std::min<uint32_t>(64, g_block_dim.x - (t & ~63u));
        const uint32_t per_pass = bytes <= 4 ? 64 : bytes == 8 ? 32 : 16, dwords = (uint32_t)(bytes + 3) / 4;
        uint64_t cycles = 0, ideal = 0;
        for (uint32_t l0 = 0; l0 < lanes; l0 += per_pass) {
            uint64_t seen[64][16];
            uint32_t n[64] = {0};
            for (uint32_t l = l0; l < std::min(lanes, l0 + per_pass); l++)
                for (uint32_t d = 0; d < dwords; d++) {
                    const uint64_t dw = (all[l] >> 2) + d;
                    const uint32_t bank = (uint32_t)(dw & 63u);
                    bool dup = false;
                    for (uint32_t k = 0; k < n[bank]; k++) dup = dup || seen[bank][k] == dw;
                    if (!dup && n[bank] < 16) seen[bank][n[bank]++] = dw; // the same dword is one broadcast read
                }
            uint32_t worst = 1;
            for (uint32_t b = 0; b < 64; b++) worst = std::max(worst, n[b]);
            cycles += worst;
            ideal += 1;
        }
        g_probe[site][0]++;
        g_probe[site][1] += cycles;
        g_probe[site][2] += ideal;
    }
    exchange_done();
}

// Helper threads that live as long as the process (QK_EMU_THREADS, default the host's cores, minus the caller).
struct Pool {
    unsigned size = 0;
    std::mutex m;
    std::condition_variable wake, idle;
    uint64_t gen = 0;
    unsigned wanted = 0, taken = 0, running = 0;
    const std::function<void()>* job = nullptr;
    void loop()
    {
        uint64_t seen = 0;
        for (;;) {
            const std::function<void()>* j = nullptr;
            {
                std::unique_lock<std::mutex> l(m);
                wake.wait(l, [&] { return gen != seen && taken < wanted; });
                seen = gen;
                taken++;
                j = job;
            }
            (*j)();
            {
                std::lock_guard<std::mutex> l(m);
                if (--running == 0) idle.notify_all();
            }
        }
    }
    void start(const std::function<void()>& j, unsigned n)
    {
        std::lock_guard<std::mutex> l(m);
        job = &j;
        wanted = running = n;
        taken = 0;
        gen++;
        wake.notify_all();
    }
    void wait()
    {
        std::unique_lock<std::mutex> l(m);
        idle.wait(l, [&] { return running == 0; });
        wanted = 0;
    }
};
static Pool& the_pool()
{
    static Pool* p = [] {
        Pool* q = new Pool; // never destroyed: its threads outlive main's statics
        const char* e = getenv("QK_EMU_THREADS");
        const unsigned v = e ? (unsigned)atoi(e) : std::thread::hardware_concurrency();
        q->size = v > 1 ? v - 1 : 0;
        for (unsigned i = 0; i < q->size; i++) std::thread([q] { q->loop(); }).detach();
        return q;
    }();
    return *p;
}

void run(dim3 grid, dim3 block, size_t lds, const std::function<void()>& body)
{
    std::lock_guard<std::mutex> launch(g_launch_mu);
    const int n = (int)(block.x * block.y * block.z);
    if (n <= 0 || n > 64 * MAX_WAVES || (n % 64) != 0 || block.y != 1 || block.z != 1) {
        fprintf(stderr, "emu: workgroup of %ux%ux%u threads not modelled (multiples of 64 up to %d)\n", block.x, block.y, block.z, 64 * MAX_WAVES);
        abort();
    }
    g_block_dim = Idx{block.x, block.y, block.z};
    g_grid_dim = Idx{grid.x, grid.y, grid.z};
    const uint64_t total = (uint64_t)grid.x * grid.y * grid.z;
    std::atomic<uint64_t> next{0};
    // Every OS thread keeps its Workgroup (the fibers' stacks) from launch to launch: mapping a thousand stacks
    // per launch cost more than small kernels themselves.
    auto worker = [&] {
        static thread_local Workgroup* mine = new Workgroup; // lives as long as the thread
        for (;;) {
            const uint64_t b = next.fetch_add(1);
            if (b >= total) break;
            const Idx bi{(uint32_t)(b % grid.x), (uint32_t)(b / grid.x % grid.y), (uint32_t)(b / ((uint64_t)grid.x * grid.y))};
            run_workgroup(*mine, bi, n, lds, body);
        }
    };
    Pool& pool = the_pool();
    const unsigned helpers = (unsigned)std::min<uint64_t>(pool.size, total > 1 ? total - 1 : 0);
    const std::function<void()> job = worker; // outlives the helpers' use of it: wait() returns after the last one
    if (helpers) pool.start(job, helpers);
    worker();
    if (helpers) pool.wait();
}

// ---- stream capture ---------------------------------------------------------------------------
static thread_local Graph* t_capture = nullptr;

void submit(std::function<void()> op)
{
    if (t_capture) t_capture->ops.push_back(std::move(op));
    else op();
}

bool capture_begin()
{
    if (t_capture) return false;
    t_capture = new Graph;
    return true;
}

Graph* capture_end()
{
    Graph* g = t_capture;
    t_capture = nullptr;
    return g;
}

} // namespace emu

emu_float4 emu_mfma_16x16x32_f16(emu_half8 a, emu_half8 b, emu_float4 c)
{
    using namespace emu;
    Workgroup& g = *t_wg;
    const uint32_t t = g.cur->tid.x, w = t >> 6, lane = t & 63u, par = g.cur->xn++ & 1u;
    for (int i = 0; i < 8; i++) {
        g.mfma_a[w][par][lane][i] = (float)a[i];
        g.mfma_b[w][par][lane][i] = (float)b[i];
    }
    wave_barrier();
    const uint32_t col = lane & 15u, rq = lane >> 4;
    emu_float4 d = c;
    for (int i = 0; i < 4; i++) {
        const uint32_t row = 4 * rq + i;
        float s = 0.f;
        for (uint32_t kq = 0; kq < 4; kq++)
            for (int j = 0; j < 8; j++) s += g.mfma_a[w][par][row + 16 * kq][j] * g.mfma_b[w][par][col + 16 * kq][j];
        d[i] += s;
    }
    return d;
}

// Device allocations of the library itself (the engine's tensors): guarded like the tests' buffers.
static std::mutex g_alloc_mu;
static std::vector<std::pair<void*, emu::GuardBuf*>> g_allocs;
hipError_t hipMalloc(void** p, size_t n)
{
    auto* g = new emu::GuardBuf(n ? n : 16);
    std::lock_guard<std::mutex> l(g_alloc_mu);
    g_allocs.emplace_back(g->p, g);
    *p = g->p;
    return hipSuccess;
}
hipError_t hipFree(void* p)
{
    if (!p) return hipSuccess;
    std::lock_guard<std::mutex> l(g_alloc_mu);
    for (size_t i = 0; i < g_allocs.size(); i++)
        if (g_allocs[i].first == p) {
            delete g_allocs[i].second;
            g_allocs.erase(g_allocs.begin() + i);
            return hipSuccess;
        }
    return hipErrorInvalidValue;
}

// C entry points for the tests: buffers that end at a guard page.
extern "C" {
// mode 0: threads of a workgroup run in ascending order between barriers, 1: descending, 2: random per sweep (seed)
void emu_set_schedule(int mode, uint64_t seed)
{
    emu::g_order_mode = mode < 0 || mode > 2 ? 0 : mode;
    emu::g_order_seed = seed ? seed : 1;
}
void emu_lds_probe_enable(int on)
{
    emu::g_lds_probe_on = on != 0;
    if (on)
        for (auto& site : emu::g_probe)
            for (auto& v : site) v = 0;
}
// out[0..2] = wave instructions, modelled cycles, conflict-free cycles of the lookups marked `site`
void emu_lds_probe_read(int site, uint64_t* out)
{
    for (int i = 0; i < 3; i++) out[i] = site >= 0 && site < emu::PROBE_SITES ? emu::g_probe[site][i].load() : 0;
}
void* emu_guard_alloc(size_t n, size_t align, void** handle)
{
    auto* g = new emu::GuardBuf(n ? n : 16, align < 16 ? 16 : align);
    *handle = g;
    return g->p;
}
void emu_guard_free(void* handle) { delete (emu::GuardBuf*)handle; }
}
