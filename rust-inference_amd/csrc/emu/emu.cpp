// The CPU stand-in's machinery: the threads of a workgroup as coroutines, their meeting points, buffers
// between guard pages, and the report when a kernel touches memory outside them.
#include <hip/hip_runtime.h>

#include <signal.h>
#include <stdio.h>
#include <stdlib.h>
#include <sys/mman.h>
#include <ucontext.h>
#include <unistd.h>

#include <vector>

namespace emu {

Thread* self = nullptr;
dim3 block_idx, block_dim, grid_dim;

namespace {
constexpr size_t STACK_BYTES = 512 * 1024;

enum State { READY, AT_BARRIER, AT_WAVE, DONE };

struct Fiber {
    Thread t;
    ucontext_t ctx;
    State state = READY;
    char* stack = nullptr;
    uint64_t wave_seq = 0;           // collectives of its wavefront this thread has been through
};

struct Wave {
    unsigned char buf[2][64][64];    // two meeting points in turn
    int arrived[2] = {0, 0}, left[2] = {0, 0};
    uint64_t mask[2] = {0, 0};
    int live = 0;                    // lanes that exist and have not ended
};

std::vector<Fiber> fibers;
std::vector<Wave> waves;
std::vector<char*> stack_pool;
ucontext_t scheduler;
Fiber* current = nullptr;
Body* running_body = nullptr;
int live_threads = 0, at_barrier = 0;
std::vector<unsigned char> dyn;
const char* kernel_name = "";

void yield() { swapcontext(&current->ctx, &scheduler); }

void trampoline() {
    running_body->run();
    current->state = DONE;
    --live_threads;
    --waves[current->t.wave].live;
    swapcontext(&current->ctx, &scheduler);
}

// ---- guarded buffers and the fault report
struct Region { char* base; size_t mapped; char* data; size_t bytes; char name[48]; };
std::vector<Region> regions;
long page_size() { static long p = sysconf(_SC_PAGESIZE); return p; }

void on_fault(int, siginfo_t* info, void*) {
    char msg[512];
    const char* addr = (const char*)info->si_addr;
    int n = snprintf(msg, sizeof msg, "[emu] kernel %s, workgroup (%u, %u, %u), thread %d: access at %p outside every buffer\n",
                     kernel_name, block_idx.x, block_idx.y, block_idx.z, current ? current->t.linear : -1, (const void*)addr);
    for (const Region& r : regions) {
        if (addr >= r.base && addr < r.base + r.mapped) {
            const long past = addr - (r.data + r.bytes), before = r.data - addr;
            if (past >= 0)
                n = snprintf(msg, sizeof msg, "[emu] kernel %s, workgroup (%u, %u, %u), thread %d: access %ld bytes past the end of buffer '%s' (%zu bytes)\n",
                             kernel_name, block_idx.x, block_idx.y, block_idx.z, current ? current->t.linear : -1, past, r.name, r.bytes);
            else
                n = snprintf(msg, sizeof msg, "[emu] kernel %s, workgroup (%u, %u, %u), thread %d: access %ld bytes before buffer '%s' (%zu bytes)\n",
                             kernel_name, block_idx.x, block_idx.y, block_idx.z, current ? current->t.linear : -1, before, r.name, r.bytes);
            break;
        }
    }
    if (write(2, msg, (size_t)n) < 0) {}
    _exit(86);
}

void install_handler() {
    static bool done = false;
    if (done) return;
    done = true;
    static char alt[64 * 1024];
    stack_t ss = {};
    ss.ss_sp = alt;
    ss.ss_size = sizeof alt;
    sigaltstack(&ss, nullptr);
    struct sigaction sa = {};
    sa.sa_sigaction = on_fault;
    sa.sa_flags = SA_SIGINFO | SA_ONSTACK;
    sigaction(SIGSEGV, &sa, nullptr);
    sigaction(SIGBUS, &sa, nullptr);
}
}  // namespace

void* dyn_shared() { return dyn.data(); }

void barrier() {
    current->state = AT_BARRIER;
    ++at_barrier;
    yield();
}

uint64_t wave_gather(const void* mine, size_t bytes, void* all) {
    if (bytes > 64) {
        fprintf(stderr, "[emu] a lane hands %zu bytes to its wavefront (64 at most)\n", bytes);
        abort();
    }
    Wave& w = waves[current->t.wave];
    const int slot = (int)(current->wave_seq++ & 1);
    memcpy(w.buf[slot][current->t.lane], mine, bytes);
    w.mask[slot] |= 1ull << current->t.lane;
    ++w.arrived[slot];
    while (w.arrived[slot] < w.live) {
        current->state = AT_WAVE;
        yield();
    }
    current->state = READY;
    const uint64_t mask = w.mask[slot];
    for (int l = 0; l < 64; ++l) {
        if ((mask >> l) & 1) memcpy((char*)all + (size_t)l * bytes, w.buf[slot][l], bytes);
        else memset((char*)all + (size_t)l * bytes, 0, bytes);
    }
    if (++w.left[slot] == w.arrived[slot]) {         // the last to leave clears the meeting point for its next use
        w.arrived[slot] = w.left[slot] = 0;
        w.mask[slot] = 0;
    }
    return mask;
}

void launch(const char* name, dim3 grid, dim3 block, size_t dyn_bytes, Body& body) {
    install_handler();
    kernel_name = name;
    const int threads = (int)(block.x * block.y * block.z);
    if (threads < 1 || threads > 1024) {
        fprintf(stderr, "[emu] kernel %s launched with %d threads a workgroup\n", name, threads);
        abort();
    }
    grid_dim = grid;
    block_dim = block;
    running_body = &body;
    dyn.assign(dyn_bytes + 64, 0);
    while ((int)stack_pool.size() < threads) {
        char* s = (char*)mmap(nullptr, STACK_BYTES, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
        if (s == MAP_FAILED) { perror("[emu] mmap of a stack"); abort(); }
        stack_pool.push_back(s);
    }
    for (unsigned bz = 0; bz < grid.z; ++bz)
    for (unsigned by = 0; by < grid.y; ++by)
    for (unsigned bx = 0; bx < grid.x; ++bx) {
        block_idx = dim3(bx, by, bz);
        fibers.assign((size_t)threads, Fiber());
        waves.assign((size_t)(threads + 63) / 64, Wave());
        live_threads = threads;
        at_barrier = 0;
        for (int i = 0; i < threads; ++i) {
            Fiber& f = fibers[i];
            f.t.linear = i;
            f.t.idx = dim3(i % block.x, (i / block.x) % block.y, i / (block.x * block.y));
            f.t.lane = i & 63;
            f.t.wave = i >> 6;
            ++waves[f.t.wave].live;
            f.stack = stack_pool[i];
            getcontext(&f.ctx);
            f.ctx.uc_stack.ss_sp = f.stack;
            f.ctx.uc_stack.ss_size = STACK_BYTES;
            f.ctx.uc_link = &scheduler;
            makecontext(&f.ctx, trampoline, 0);
        }
        while (live_threads > 0) {
            bool ran = false;
            for (int i = 0; i < threads; ++i) {
                Fiber& f = fibers[i];
                if (f.state == DONE || f.state == AT_BARRIER) continue;
                if (f.state == AT_WAVE) {
                    const Wave& w = waves[f.t.wave];
                    const int slot = (int)((f.wave_seq - 1) & 1);
                    if (w.arrived[slot] < w.live) continue;          // its wavefront is not complete yet
                }
                current = &f;
                self = &f.t;
                ran = true;
                swapcontext(&scheduler, &f.ctx);
            }
            if (live_threads > 0 && at_barrier == live_threads) {    // everyone who is left has arrived
                for (Fiber& f : fibers)
                    if (f.state == AT_BARRIER) f.state = READY;
                at_barrier = 0;
                ran = true;
            }
            if (!ran) {
                fprintf(stderr, "[emu] kernel %s, workgroup (%u, %u, %u): the threads wait for one another for ever "
                        "(%d live, %d at the barrier): a barrier or a lane exchange that not every thread reaches\n",
                        name, bx, by, bz, live_threads, at_barrier);
                _exit(87);
            }
        }
    }
    current = nullptr;
    self = nullptr;
}

}  // namespace emu

// ---- C interface for the tests
extern "C" {

// A buffer of `bytes` bytes between two pages that may not be touched.  `flush_end`: its last byte lies
// against the page behind it (what catches a read past the end; sizes are rounded up to 16 bytes, the widest
// load there is); else its first byte against the page before it.
void* ri_emu_alloc(size_t bytes, int flush_end, const char* name) {
    emu::install_handler();
    const size_t page = (size_t)emu::page_size();
    const size_t padded = (bytes + 15) / 16 * 16;
    const size_t body = (padded + page - 1) / page * page;
    char* base = (char*)mmap(nullptr, body + 2 * page, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
    if (base == MAP_FAILED) return nullptr;
    mprotect(base, page, PROT_NONE);
    mprotect(base + page + body, page, PROT_NONE);
    char* data = flush_end ? base + page + body - padded : base + page;
    emu::Region r = {};
    r.base = base;
    r.mapped = body + 2 * page;
    r.data = data;
    r.bytes = padded;
    snprintf(r.name, sizeof r.name, "%s", name ? name : "?");
    emu::regions.push_back(r);
    return data;
}

void ri_emu_free_all(void) {
    for (const emu::Region& r : emu::regions) munmap(r.base, r.mapped);
    emu::regions.clear();
}

}  // extern "C"
