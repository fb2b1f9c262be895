// Fiber scheduler of the wave64 emulator (test infrastructure; see emu_runtime.h).
#include "emu_runtime.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>

#include <vector>

namespace emu {

thread_local Lane* cur = nullptr;

namespace {

constexpr size_t kStack = 512 << 10;
constexpr size_t kLdsBytes = 160 << 10;
constexpr int kMaxThreads = 1024;

struct Fiber {
    Lane lane;
    void* sp;
    bool done;
};

struct WaveState {
    int live, arrived;
    unsigned gen;
    // global -> LDS instruction slots in flight through the wave's lanes (a lane's n-th request is slot n): how many lanes
    // have passed each, and how many of them with a real request
    unsigned char slot_lanes[1024], slot_real[1024];
    int lanes0;                  // lanes the wave started with
    unsigned max_requests;       // most requests any lane has made
    unsigned ended_after[64];    // requests made by each lane that has ended
    int n_ended;
    alignas(64) char buf[2][64][256];
};

struct Group {
    std::vector<Fiber> fibers;
    std::vector<WaveState> waves;
    char* stacks = nullptr;
    char* lds_region = nullptr;  // kLdsBytes, then one inaccessible page
    char* lds = nullptr;         // the launch's dynamic LDS: ends where the inaccessible page begins
    int n = 0, live = 0, running = -1;
    int bar_arrived = 0;
    unsigned bar_gen = 0;
    void* main_sp = nullptr;
    const std::function<void()>* body = nullptr;
    long idle = 0;  // consecutive yields without progress
    bool failed = false;
    char why[256];
};

Group g;
hipError_t last_error = hipSuccess;

extern "C" void emu_switch(void** save_sp, void* to_sp);
asm(R"(
    .text
    .globl emu_switch
    .type emu_switch,@function
emu_switch:
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
)");

void fail(const char* what)
{
    if (!g.failed) {
        g.failed = true;
        snprintf(g.why, sizeof(g.why), "%s (workgroup %u,%u,%u thread %u)", what, cur->bid.x, cur->bid.y, cur->bid.z, cur->tid.x);
        fprintf(stderr, "emu: %s\n", g.why);
    }
}

// Instruction slot n of a wave is complete when every lane that gets that far has passed it: the lanes the wave started
// with minus those that ended after fewer than n + 1 requests.  A complete slot must have had a real request.
void close_slot(WaveState& w, unsigned n)
{
    int expected = w.lanes0;
    for (int i = 0; i < w.n_ended; ++i)
        if (w.ended_after[i] <= n) --expected;
    const unsigned slot = n & 1023u;
    if (w.slot_lanes[slot] == 0 || (int)w.slot_lanes[slot] < expected) return;
    if (w.slot_real[slot] == 0) fail("a global -> LDS instruction with every lane of the wave masked off: the hardware would not issue it");
    w.slot_lanes[slot] = w.slot_real[slot] = 0;
}

// run the next fiber that has not finished; back to the launcher when none is left
void schedule()
{
    const int from = g.running;
    void** save = from >= 0 ? &g.fibers[from].sp : &g.main_sp;
    if (g.live == 0 || g.failed) {
        g.running = -1;
        cur = nullptr;
        if (from >= 0) emu_switch(save, g.main_sp);
        return;
    }
    // Fibers take turns in thread order, or in the opposite order with EMU_ORDER=reverse: between two barriers the
    // waves of a workgroup then run last to first, so a wave that reads what an earlier wave wrote without a barrier in
    // between - which the forward order lets pass - sees the poison instead.
    static const bool reverse = [] {
        const char* e = getenv("EMU_ORDER");
        return e && strcmp(e, "reverse") == 0;
    }();
    int next = from < 0 && reverse ? 0 : from;
    do {
        next = reverse ? (next + g.n - 1) % g.n : (next + 1) % g.n;
    } while (g.fibers[next].done);
    if (next == from) return;
    g.running = next;
    cur = &g.fibers[next].lane;
    emu_switch(save, g.fibers[next].sp);
}

void yield_waiting()
{
    // every live fiber waiting and nobody making progress for several rounds: the kernel deadlocked (lanes of a wave took
    // different paths to a cross-lane instruction, or a barrier that not every wave reaches)
    if (++g.idle > 8L * g.n + 64) fail("deadlock: a rendezvous that not every live lane reaches");
    schedule();
}

void fiber_exit()
{
    Fiber& f = g.fibers[g.running];
    f.done = true;
    --g.live;
    WaveState& w = g.waves[f.lane.wave];
    --w.live;
    if (w.n_ended < 64) w.ended_after[w.n_ended++] = f.lane.requests;
    for (unsigned n = f.lane.requests; n < w.max_requests; ++n) close_slot(w, n);  // slots this lane will never reach
    if (w.arrived > 0 && w.arrived >= w.live) fail("a lane ended while other lanes of its wave wait in a cross-lane instruction");
    if (g.bar_arrived > 0 && g.bar_arrived >= g.live) {  // the hardware barrier does not wait for ended waves
        g.bar_arrived = 0;
        ++g.bar_gen;
    }
    g.idle = 0;
    schedule();
    abort();  // a finished fiber is never resumed
}

void fiber_main()
{
    (*g.body)();
    if (cur->pending_count) fail("a lane ended with global -> LDS copies still in flight (no wait before the workgroup retires)");
    fiber_exit();
}

}  // namespace

hipError_t take_error()
{
    const hipError_t e = last_error;
    last_error = hipSuccess;
    return e;
}

char* dynamic_lds() { return g.lds; }

void barrier()
{
    const unsigned gen = g.bar_gen;
    if (++g.bar_arrived >= g.live) {
        g.bar_arrived = 0;
        ++g.bar_gen;
        g.idle = 0;
        return;
    }
    while (g.bar_gen == gen && !g.failed) yield_waiting();
}

const char* exchange(const void* mine, size_t n)
{
    WaveState& w = g.waves[cur->wave];
    const unsigned gen = w.gen;
    char(*slots)[256] = w.buf[gen & 1];
    memcpy(slots[cur->lane], mine, n);
    if (++w.arrived >= w.live) {
        if (w.live != 64 && w.live != (int)(g.n - cur->wave * 64))
            fail("cross-lane instruction with lanes of the wave already ended");
        w.arrived = 0;
        ++w.gen;
        g.idle = 0;
    } else {
        while (w.gen == gen && !g.failed) yield_waiting();
    }
    return &slots[0][0];
}

bool late_loads()
{
    static const bool late = [] {
        const char* e = getenv("EMU_LATE_LOADS");
        return !(e && e[0] == '0');
    }();
    return late;
}

void request_copy(char* dst, const char* src)
{
    // The waits count INSTRUCTIONS per wave.  An instruction that every lane of a wave skips is not issued at all (the
    // compiler branches around it when no lane is active), so the wave's count of outstanding copies would be one lower
    // than the wait was written for, and an older copy could still be in flight behind it.  A kernel that masks lanes
    // off (padded head dims) must therefore keep at least one lane on every instruction.
    {
        Lane& l = *cur;
        WaveState& w = g.waves[l.wave];
        const unsigned n = l.requests++;
        if (l.requests > w.max_requests) w.max_requests = l.requests;
        ++w.slot_lanes[n & 1023u];
        if (dst) ++w.slot_real[n & 1023u];
        close_slot(w, n);
    }
    if (!late_loads()) {
        if (dst) memcpy(dst, src, 16);
        return;
    }
    Lane& l = *cur;
    if (l.pending_count == 256) land_copies(255);  // more than the hardware counter holds: the oldest must have landed
    l.pending[(l.pending_head + l.pending_count) & 255] = PendingCopy{dst, src};
    ++l.pending_count;
}

void land_copies(int keep)
{
    Lane& l = *cur;
    while (l.pending_count > keep) {
        const PendingCopy& c = l.pending[l.pending_head];
        if (c.dst) memcpy(c.dst, c.src, 16);  // null: the lane was masked off for this instruction
        l.pending_head = (l.pending_head + 1) & 255;
        --l.pending_count;
    }
}

int readfirstlane(int x) { return lane_value<int>(exchange(&x, 4), 0); }

uint64_t ballot(bool p)
{
    const char c = p ? 1 : 0;
    const char* all = exchange(&c, 1);
    const int lanes = g.n - cur->wave * 64 < 64 ? g.n - cur->wave * 64 : 64;
    uint64_t m = 0;
    for (int i = 0; i < lanes; ++i) m |= (uint64_t)(all[(size_t)i * 256] != 0) << i;
    return m;
}

void note_launch(const char* tag)
{
    static const char* path = getenv("EMU_COVERAGE");
    if (!path) return;
    static std::vector<const char*> seen;  // type_info names: one address per instantiation
    for (const char* s : seen)
        if (s == tag) return;
    seen.push_back(tag);
    if (FILE* f = fopen(path, "a")) {
        fprintf(f, "%s\n", tag);
        fclose(f);
    }
}

void launch(dim3 grid, dim3 block, size_t lds_bytes, const std::function<void()>& body)
{
    const int n = (int)(block.x * block.y * block.z);
    if (n <= 0 || n > kMaxThreads || lds_bytes > kLdsBytes) {
        last_error = hipErrorInvalidValue;
        return;
    }
    if (!g.stacks) {
        g.stacks = (char*)mmap(nullptr, kStack * kMaxThreads, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
        g.lds_region = (char*)mmap(nullptr, kLdsBytes + 4096, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_32BIT, -1, 0);
        if (g.stacks == MAP_FAILED || g.lds_region == MAP_FAILED || mprotect(g.lds_region + kLdsBytes, 4096, PROT_NONE) != 0) {
            fprintf(stderr, "emu: cannot map fiber stacks / LDS\n");
            abort();
        }
    }
    // an access past the end of the launch's LDS allocation runs into the inaccessible page
    g.lds = g.lds_region + kLdsBytes - ((lds_bytes + 15) & ~(size_t)15);
    g.fibers.resize(n);
    g.waves.resize((n + 63) / 64);
    g.n = n;
    g.body = &body;
    g.failed = false;
    for (unsigned bz = 0; bz < grid.z && !g.failed; ++bz)
        for (unsigned by = 0; by < grid.y && !g.failed; ++by)
            for (unsigned bx = 0; bx < grid.x && !g.failed; ++bx) {
                // LDS content of the previous workgroup is poison, as on the hardware where it is whatever was there
                memset(g.lds, 0xff, lds_bytes);
                for (auto& w : g.waves) {
                    w.live = 0;
                    w.arrived = 0;
                    w.gen = 0;
                    memset(w.slot_lanes, 0, sizeof(w.slot_lanes));
                    memset(w.slot_real, 0, sizeof(w.slot_real));
                    w.lanes0 = w.n_ended = 0;
                    w.max_requests = 0;
                }
                for (int t = 0; t < n; ++t) {
                    Fiber& f = g.fibers[t];
                    f.lane.tid = dim3(t % block.x, (t / block.x) % block.y, t / (block.x * block.y));
                    f.lane.bid = dim3(bx, by, bz);
                    f.lane.bdim = block;
                    f.lane.gdim = grid;
                    f.lane.lane = t & 63;
                    f.lane.wave = t >> 6;
                    f.lane.pending_head = f.lane.pending_count = 0;
                    f.lane.requests = 0;
                    f.done = false;
                    ++g.waves[t >> 6].live;
                    ++g.waves[t >> 6].lanes0;
                    // initial frame: six callee-saved registers, then the entry point as return address; the stack
                    // pointer is 8 modulo 16 when fiber_main starts, as after a call
                    uintptr_t top = (uintptr_t)(g.stacks + (size_t)(t + 1) * kStack) & ~(uintptr_t)15;
                    void** sp = (void**)(top - 8);
                    *--sp = (void*)&fiber_main;
                    for (int r = 0; r < 6; ++r) *--sp = nullptr;
                    f.sp = sp;
                }
                g.live = n;
                g.bar_arrived = 0;
                g.bar_gen = 0;
                g.idle = 0;
                g.running = -1;
                schedule();  // returns when every fiber has finished (or the kernel failed)
            }
    if (g.failed) last_error = hipErrorLaunchFailure;
    g.body = nullptr;
}

}  // namespace emu
