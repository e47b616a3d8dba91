// Fibre scheduler behind emu.h (TEST INFRASTRUCTURE ONLY): one fibre per lane, cooperative, single OS thread.
#include "emu.h"

#include <stdio.h>
#include <stdlib.h>
#include <ucontext.h>
#include <random>
#include <vector>

namespace emu {

emu_dim3 g_block = {0, 0, 0}, g_grid = {1, 1, 1};
int g_late_dma = 0;
char* g_lds = nullptr;

namespace {

constexpr size_t kStack = 512 * 1024;
constexpr size_t kLds = 160 * 1024;
constexpr size_t kMaxExchange = 64;   // bytes per lane

struct Dma { const void* src; uint32_t off; int bytes; long seq; };

struct Fiber {
    ucontext_t ctx;
    char* stack = nullptr;
    emu_dim3 tid = {0, 0, 0};
    bool done = false;
    // what the fibre waits for: a generation counter to move past `seen`
    const long* wait_gen = nullptr;
    long seen = 0;
    std::vector<Dma> pending;
    long issued = 0;
};

struct Wave {
    long gen = 0;
    int arrived = 0;
    alignas(16) char buf[2][kLanes * kMaxExchange];
};

std::vector<Fiber> fibers;
std::vector<Wave> waves;
ucontext_t sched_ctx;
int cur = -1;
long block_gen = 0;
int block_arrived = 0;
kernel_fn g_fn = nullptr;
void* g_arg = nullptr;

void yield_until(const long* gen, long seen) {
    Fiber& f = fibers[cur];
    f.wait_gen = gen;
    f.seen = seen;
    swapcontext(&f.ctx, &sched_ctx);
}

void trampoline() {
    g_fn(g_arg);
    fibers[cur].done = true;
    swapcontext(&fibers[cur].ctx, &sched_ctx);
}

}  // namespace

const emu_dim3& thread_idx() { return fibers[cur].tid; }

void block_barrier() {
    const long seen = block_gen;
    if (++block_arrived == (int)fibers.size()) {
        block_arrived = 0;
        ++block_gen;
        return;
    }
    yield_until(&block_gen, seen);
}

const void* wave_exchange(const void* mine, size_t bytes) {
    if (bytes > kMaxExchange) abort();
    Wave& w = waves[fibers[cur].tid.x / kLanes];
    const int lane = fibers[cur].tid.x % kLanes;
    const long seen = w.gen;
    char* table = w.buf[seen & 1];
    if (bytes) memcpy(table + lane * bytes, mine, bytes);
    if (++w.arrived == kLanes) {
        w.arrived = 0;
        ++w.gen;
    } else {
        yield_until(&w.gen, seen);
    }
    return table;
}

void wave_barrier() { wave_exchange(nullptr, 0); }

void dma_issue(const void* src, uint32_t lds_offset, int bytes) {
    if (lds_offset + (size_t)bytes > kLds) {
        fprintf(stderr, "emu: transfer to LDS offset %u + %d is outside the 160 KB\n", lds_offset, bytes);
        abort();
    }
    Fiber& f = fibers[cur];
    if (!g_late_dma) memcpy(g_lds + lds_offset, src, bytes);
    else f.pending.push_back({src, lds_offset, bytes, f.issued});
    ++f.issued;
}

void dma_wait(int allowed) {
    Fiber& f = fibers[cur];
    size_t done = 0;
    while (done < f.pending.size() && f.pending[done].seq < f.issued - allowed) {
        const Dma& d = f.pending[done];
        memcpy(g_lds + d.off, d.src, d.bytes);
        ++done;
    }
    f.pending.erase(f.pending.begin(), f.pending.begin() + done);
}

int run_grid(kernel_fn fn, void* arg, unsigned blocks, unsigned threads, unsigned seed, int late_dma, char* lds) {
    if (threads % kLanes) return 2;
    g_fn = fn;
    g_arg = arg;
    g_late_dma = late_dma;
    g_grid = {blocks, 1, 1};
    std::mt19937 rng(seed);
    g_lds = lds;
    std::vector<char*> stacks(threads);
    for (auto& s : stacks) s = (char*)malloc(kStack);
    int status = 0;
    for (unsigned b = 0; b < blocks && !status; ++b) {
        g_block = {b, 0, 0};
        memset(g_lds, 0xff, kLds);   // fp16 / fp32 NaN patterns: a read of bytes nobody wrote shows in the result
        fibers.assign(threads, Fiber());
        waves.assign(threads / kLanes, Wave());
        block_gen = 0;
        block_arrived = 0;
        for (unsigned t = 0; t < threads; ++t) {
            Fiber& f = fibers[t];
            f.tid = {t, 0, 0};
            f.stack = stacks[t];
            getcontext(&f.ctx);
            f.ctx.uc_stack.ss_sp = f.stack;
            f.ctx.uc_stack.ss_size = kStack;
            f.ctx.uc_link = nullptr;
            makecontext(&f.ctx, trampoline, 0);
        }
        std::vector<int> order(threads / kLanes);
        for (size_t i = 0; i < order.size(); ++i) order[i] = (int)i;
        size_t finished = 0;
        while (finished < threads) {
            std::shuffle(order.begin(), order.end(), rng);
            bool progress = false;
            for (int w : order) {
                // this wavefront runs until every lane of it is blocked on something another wavefront must provide
                bool moved = true;
                while (moved) {
                    moved = false;
                    for (int l = 0; l < kLanes; ++l) {
                        Fiber& f = fibers[w * kLanes + l];
                        if (f.done || (f.wait_gen && *f.wait_gen == f.seen)) continue;
                        f.wait_gen = nullptr;
                        cur = w * kLanes + l;
                        swapcontext(&sched_ctx, &f.ctx);
                        cur = -1;
                        moved = progress = true;
                        if (f.done) ++finished;
                    }
                }
            }
            if (!progress) {
                fprintf(stderr, "emu: deadlock in block %u (%zu of %u lanes finished)\n", b, finished, threads);
                status = 1;
                break;
            }
        }
    }
    for (auto s : stacks) free(s);
    fibers.clear();
    g_lds = nullptr;
    return status;
}

}  // namespace emu
