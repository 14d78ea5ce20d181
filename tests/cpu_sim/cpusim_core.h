// The core of the CPU stand-in for the GPU (tests only): runs a kernel launch work-item by work-item.
//
// Every work-item of a workgroup is a fiber (its own stack, switched by hand: x86-64 only) of the calling OS thread;
// workgroups run one after another, by default in the order x fastest, then y, then z (so the workgroup that is
// numbered last is the one that "arrives last" at a counter; CPUSIM_SCHEDULE chooses other orders of workgroups and
// of work-items).  A work-item runs until it has to wait for others: at a workgroup barrier or at an operation that
// crosses the lanes of its wave (a shuffle, an MFMA).  When no work-item can run, the waiting ones are let go: first
// all that wait at a wave operation (every lane that took part has arrived, since all ran until they had to wait: the
// lanes that did not arrive are masked out, as the hardware's EXEC mask would have them), otherwise all that wait at
// the barrier.  A work-item that returns takes part in nothing afterwards.
//
// Data crosses lanes through per-wave slots: a lane deposits its operands, waits, reads what the others deposited.
// Two sets of slots alternate between consecutive operations of a wave, so a lane that is already at the next
// operation cannot overwrite what a slower lane has yet to read.
#pragma once
#include <sys/mman.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <string>
#include <vector>

#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define CPUSIM_ASAN 1
extern "C" void __sanitizer_start_switch_fiber(void **fake_stack_save, const void *bottom, size_t size);
extern "C" void __sanitizer_finish_switch_fiber(void *fake_stack_save, const void **bottom_old, size_t *size_old);
extern "C" void __asan_unpoison_memory_region(void const volatile *addr, size_t size);
#endif
#if __has_feature(thread_sanitizer)
#define CPUSIM_TSAN 1
extern "C" void *__tsan_get_current_fiber(void);
extern "C" void *__tsan_create_fiber(unsigned flags);
extern "C" void __tsan_destroy_fiber(void *fiber);
extern "C" void __tsan_switch_to_fiber(void *fiber, unsigned flags);
#endif
#endif

namespace cpusim {

struct Dim3u {
    uint32_t x = 1, y = 1, z = 1;
};

constexpr uint32_t WAVE_LANES = 64;
constexpr size_t SLOT_BYTES = 64;         // per lane and operand
constexpr size_t STACK_BYTES = 512 << 10;  // per work-item (mapped on demand)

// Saves the callee-saved registers on the current stack, leaves the stack pointer in *from_sp and continues on to_sp
// (a stack that was left by this function, or one prepared by prepare_stack).
__attribute__((naked, noinline)) static void switch_stack(void **from_sp, void *to_sp) {
    asm volatile(
        "pushq %rbp\n pushq %rbx\n pushq %r12\n pushq %r13\n pushq %r14\n pushq %r15\n"
        "movq %rsp, (%rdi)\n movq %rsi, %rsp\n"
        "popq %r15\n popq %r14\n popq %r13\n popq %r12\n popq %rbx\n popq %rbp\n ret\n");
}
// A fresh stack on which switch_stack "returns" into entry()
inline void *prepare_stack(char *stack, size_t bytes, void (*entry)()) {
    void **sp = reinterpret_cast<void **>(reinterpret_cast<uintptr_t>(stack + bytes) & ~(uintptr_t)15);
    *--sp = nullptr;                             // where entry() would return to: it never does
    *--sp = reinterpret_cast<void *>(entry);     // popped by ret
    for (int r = 0; r < 6; ++r) *--sp = nullptr;  // the six registers
    return sp;
}

enum class ItemState { Runnable, AtWaveOp, AtBarrier, Done };

struct WaveSlots {
    uint32_t generation = 0;  // operations of this wave that have been let go
    alignas(16) unsigned char slot[2][2][WAVE_LANES][SLOT_BYTES];  // [set][operand][lane]
};

struct Item {
    void *sp = nullptr;
    Dim3u tid;
    uint32_t flat = 0;
    ItemState state = ItemState::Done;
    char *stack = nullptr;
    uint32_t site = 0;  // where in the source the wave operation it waits at was written
    void *asan_fake = nullptr;
    void *tsan_fiber = nullptr;
};

struct Worker {
    std::vector<Item *> items;  // grows to the largest workgroup seen; stacks are kept
    std::vector<WaveSlots> waves;
    void *sched_sp = nullptr;
    void *asan_fake = nullptr;
    void *tsan_sched = nullptr;
    const void *sched_stack = nullptr;
    size_t sched_stack_size = 0;
    Item *cur = nullptr;
    Dim3u block_idx, block_dim, grid_dim;
    const std::function<void()> *body = nullptr;
    // statistics of the launches so far
    uint64_t launches = 0, workgroups = 0, out_of_range_loads = 0, out_of_range_stores = 0;
    // bytes moved by buffer accesses inside their resources, by cache policy: [0] plain, [1] non-temporal, [2] sc1
    uint64_t buffer_load_bytes[3] = {0, 0, 0}, buffer_store_bytes[3] = {0, 0, 0};
    ~Worker() {
        for (Item *it : items) {
            munmap(it->stack - 4096, STACK_BYTES + 4096);
            delete it;
        }
    }
};

struct Schedule {
    enum Kind { Forward, Reverse, Shuffle } kind = Forward;
    uint64_t seed = 0;
};
inline const Schedule &schedule() {
    static const Schedule s = [] {
        Schedule out;
        const char *e = std::getenv("CPUSIM_SCHEDULE");
        if (e && std::strcmp(e, "reverse") == 0) out.kind = Schedule::Reverse;
        else if (e && std::strncmp(e, "shuffle", 7) == 0) out.kind = Schedule::Shuffle, out.seed = e[7] == ':' ? std::strtoull(e + 8, nullptr, 0) : 1;
        else if (e && *e && std::strcmp(e, "forward") != 0) {
            std::fprintf(stderr, "cpusim: CPUSIM_SCHEDULE=%s is none of forward, reverse, shuffle[:seed]\n", e);
            std::abort();
        }
        return out;
    }();
    return s;
}

inline Worker &worker() {
    static thread_local Worker w;
    return w;
}

inline void to_scheduler() {
    Worker &w = worker();
    Item *it = w.cur;
#ifdef CPUSIM_ASAN
    __sanitizer_start_switch_fiber(it->state == ItemState::Done ? nullptr : &it->asan_fake, w.sched_stack, w.sched_stack_size);
#endif
#ifdef CPUSIM_TSAN
    __tsan_switch_to_fiber(w.tsan_sched, 0);
#endif
    switch_stack(&it->sp, w.sched_sp);
#ifdef CPUSIM_ASAN
    __sanitizer_finish_switch_fiber(it->asan_fake, &w.sched_stack, &w.sched_stack_size);
#endif
}

inline void item_entry() {
    Worker &w = worker();
#ifdef CPUSIM_ASAN
    __sanitizer_finish_switch_fiber(nullptr, &w.sched_stack, &w.sched_stack_size);
#endif
    (*w.body)();
    w.cur->state = ItemState::Done;
    to_scheduler();
    std::abort();  // a finished work-item is never resumed
}

inline void barrier() {
    worker().cur->state = ItemState::AtBarrier;
    to_scheduler();
}

// Deposit up to two operands, wait for the wave, and return the slots of the set that was deposited into.
struct WaveView {
    const unsigned char (*a)[SLOT_BYTES];
    const unsigned char (*b)[SLOT_BYTES];
};
inline WaveView wave_exchange(uint32_t site, const void *op_a, size_t bytes_a, const void *op_b = nullptr, size_t bytes_b = 0) {
    Worker &w = worker();
    Item *it = w.cur;
    it->site = site;
    WaveSlots &ws = w.waves[it->flat / WAVE_LANES];
    const uint32_t set = ws.generation & 1, lane = it->flat % WAVE_LANES;
    if (bytes_a > SLOT_BYTES || bytes_b > SLOT_BYTES) std::abort();
    if (bytes_a) std::memcpy(ws.slot[set][0][lane], op_a, bytes_a);
    if (bytes_b) std::memcpy(ws.slot[set][1][lane], op_b, bytes_b);
    it->state = ItemState::AtWaveOp;
    to_scheduler();
    return {ws.slot[set][0], ws.slot[set][1]};
}
inline uint32_t lane_id() { return worker().cur->flat % WAVE_LANES; }

inline void run_workgroup(Worker &w, uint32_t threads) {
    for (uint32_t t = 0; t < threads; ++t) {
        Item *it = w.items[t];
        it->flat = t;
        it->tid = Dim3u{t % w.block_dim.x, (t / w.block_dim.x) % w.block_dim.y, t / (w.block_dim.x * w.block_dim.y)};
        it->state = ItemState::Runnable;
        it->asan_fake = nullptr;
#ifdef CPUSIM_ASAN
        __asan_unpoison_memory_region(it->stack, STACK_BYTES);  // what the stack's last user left poisoned
#endif
        it->sp = prepare_stack(it->stack, STACK_BYTES, item_entry);
#ifdef CPUSIM_TSAN
        if (it->tsan_fiber) __tsan_destroy_fiber(it->tsan_fiber);
        it->tsan_fiber = __tsan_create_fiber(0);
#endif
    }
    for (auto &ws : w.waves) ws.generation = 0;
#ifdef CPUSIM_TSAN
    w.tsan_sched = __tsan_get_current_fiber();
#endif
    const Schedule &sch = schedule();
    uint64_t rnd = sch.seed * 0x9E3779B97F4A7C15ull + w.workgroups;
    for (;;) {
        // The order in which the runnable work-items get their turn: a correct kernel gives the same result for every
        // order (between barriers the hardware interleaves waves as it likes).  CPUSIM_SCHEDULE=reverse or
        // shuffle:<seed> (a new order of the waves, and a rotation of the lanes inside them, on every pass) tests that.
        uint32_t wave_xor = 0, lane_rot = 0;
        bool backwards = sch.kind == Schedule::Reverse;
        if (sch.kind == Schedule::Shuffle) {
            rnd = rnd * 6364136223846793005ull + 1442695040888963407ull;
            wave_xor = (uint32_t)(rnd >> 33), lane_rot = (uint32_t)(rnd >> 40) % WAVE_LANES, backwards = (rnd >> 60) & 1;
        }
        const uint32_t nwaves = threads / WAVE_LANES;
        uint32_t wave_mask = 1;
        while (wave_mask < nwaves) wave_mask <<= 1;
        wave_mask -= 1;
        for (uint32_t n = 0; n < (wave_mask + 1) * WAVE_LANES; ++n) {
            const uint32_t m = backwards ? (wave_mask + 1) * WAVE_LANES - 1 - n : n;
            const uint32_t wv = (m / WAVE_LANES) ^ (wave_xor & wave_mask);
            if (wv >= nwaves) continue;
            const uint32_t t = wv * WAVE_LANES + (m % WAVE_LANES + lane_rot) % WAVE_LANES;
            Item *it = w.items[t];
            if (it->state != ItemState::Runnable) continue;
            w.cur = it;
#ifdef CPUSIM_ASAN
            __sanitizer_start_switch_fiber(&w.asan_fake, it->stack, STACK_BYTES);
#endif
#ifdef CPUSIM_TSAN
            __tsan_switch_to_fiber(it->tsan_fiber, 0);
#endif
            switch_stack(&w.sched_sp, it->sp);
#ifdef CPUSIM_ASAN
            __sanitizer_finish_switch_fiber(w.asan_fake, nullptr, nullptr);
#endif
            w.cur = nullptr;
        }
        // nobody can run: let the wave operations go, else the barrier
        bool any = false;
        for (uint32_t t = 0; t < threads; ++t)
            if (w.items[t]->state == ItemState::AtWaveOp) {
                w.items[t]->state = ItemState::Runnable;
                any = true;
            }
        if (any) {
            // (a wave none of whose lanes waited did no operation: its generation stays)
            for (uint32_t v = 0; v < threads / WAVE_LANES; ++v) {
                bool woke = false;
                uint32_t site = 0;
                for (uint32_t l = 0; l < WAVE_LANES; ++l) {
                    const Item *it = w.items[v * WAVE_LANES + l];
                    if (it->state != ItemState::Runnable) continue;
                    // The lanes that meet must be at one and the same operation of the source: lanes of a wave that
                    // took different branches would execute their operations one after the other on the hardware,
                    // each under its own mask, and pairing them here would hand them each other's operands.
                    if (woke && it->site != site) {
                        std::fprintf(stderr, "cpusim: lanes of wave %u of workgroup (%u, %u, %u) met at different wave operations (source lines %u and %u)\n",
                                     v, w.block_idx.x, w.block_idx.y, w.block_idx.z, site, it->site);
                        std::abort();
                    }
                    woke = true, site = it->site;
                }
                if (woke) w.waves[v].generation++;
            }
            continue;
        }
        for (uint32_t t = 0; t < threads; ++t)
            if (w.items[t]->state == ItemState::AtBarrier) {
                w.items[t]->state = ItemState::Runnable;
                any = true;
            }
        if (!any) break;  // every work-item has returned
    }
}

// Runs body() once per work-item of the grid.  Workgroups of whole waves only.
inline void launch(Dim3u grid, Dim3u block, size_t dynamic_lds_bytes, const std::function<void()> &body) {
    Worker &w = worker();
    const uint32_t threads = block.x * block.y * block.z;
    if (threads == 0 || threads % WAVE_LANES || threads > 1024) {
        std::fprintf(stderr, "cpusim: a workgroup of %u work-items (whole waves, at most 1024)\n", threads);
        std::abort();
    }
    if (w.cur) {
        std::fprintf(stderr, "cpusim: a launch from inside a kernel\n");
        std::abort();
    }
    while (w.items.size() < threads) {
        Item *it = new Item;
        // a stack with an inaccessible page below it
        char *m = static_cast<char *>(mmap(nullptr, STACK_BYTES + 4096, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0));
        if (m == MAP_FAILED) {
            std::perror("cpusim: mmap of a work-item stack");
            std::abort();
        }
        mprotect(m, 4096, PROT_NONE);
        it->stack = m + 4096;
        w.items.push_back(it);
    }
    if (w.waves.size() < threads / WAVE_LANES) w.waves.resize(threads / WAVE_LANES);
    w.block_dim = block;
    w.grid_dim = grid;
    w.body = &body;
    (void)dynamic_lds_bytes;  // dynamic LDS is a thread-local array of the module, of the largest size a launch may ask for
    w.launches++;
    // Workgroups in ascending order (x fastest); backwards under CPUSIM_SCHEDULE=reverse, in a pseudo-random order under
    // shuffle: a kernel must not depend on which workgroup runs first or last.
    const Schedule &sch = schedule();
    const uint64_t total = (uint64_t)grid.x * grid.y * grid.z;
    uint64_t mul = 1, add = 0;
    if (sch.kind == Schedule::Shuffle && total > 2) {
        auto gcd = [](uint64_t a, uint64_t b) {
            while (b) {
                const uint64_t t = a % b;
                a = b, b = t;
            }
            return a;
        };
        mul = (sch.seed * 2654435761ull + w.launches * 40503ull) % total;
        while (mul < 2 || gcd(mul, total) != 1) mul = (mul + 1) % total;
        add = (sch.seed + 7 * w.launches) % total;
    }
    for (uint64_t n = 0; n < total; ++n) {
        uint64_t b = sch.kind == Schedule::Reverse ? total - 1 - n : (uint64_t)((unsigned __int128)n * mul % total + add) % total;
        w.block_idx = Dim3u{(uint32_t)(b % grid.x), (uint32_t)(b / grid.x % grid.y), (uint32_t)(b / ((uint64_t)grid.x * grid.y))};
        w.workgroups++;
        run_workgroup(w, threads);
    }
    w.body = nullptr;
}

// ---- the kernels of the library's modules, by name (filled by the generated registration code of each module)
using KernelEntry = void (*)(const void *params);
struct KernelInfo {
    KernelEntry entry;
    size_t params_size;
    std::string module;
};
inline std::map<std::string, KernelInfo> &registry() {
    static std::map<std::string, KernelInfo> r;
    return r;
}
template <class P>
struct KernelOf;
template <class P>
struct KernelOf<void (*)(P)> {
    using Params = P;
};

}  // namespace cpusim
