// Host model of a gfx950 workgroup: fibres, wavefront-wide operations, checked memory and an interpreter for the
// library's assembly statements.  See sim.h.  Test infrastructure only.
#include "sim.h"

#include <dlfcn.h>
#include <signal.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <ucontext.h>
#include <unistd.h>

#include <map>
#include <string>
#include <unordered_map>
#include <vector>

namespace sim {

// ---- report ---------------------------------------------------------------------------------------------------
static std::vector<std::string> g_viol;
static std::vector<std::string> g_launches;
static int g_launch_error = 0;
static int g_cus = 8;
static const char *g_kernel = "(no kernel)";
static uint64_t g_asm_instructions = 0;
static bool g_abort_launch = false;
static bool g_lds_reads_clamped = false;  // LDS reads beyond the launch's LDS give 0, as on the hardware, instead of a violation
static bool g_any_memory = false;  // addresses outside the model's own arrays are taken on trust (arrays of the caller's)
static uint64_t g_schedule = 0;  // 0: wavefronts run in index order; else the seed of a new order every round

struct Fiber;
static Fiber *g_cur = nullptr;
static std::string where();

static void violation(const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (g_viol.size() < 64) g_viol.push_back(where() + buf);
    g_launch_error = 719;
}

// ---- global memory --------------------------------------------------------------------------------------------
struct Alloc {
    uint8_t *map;
    size_t map_bytes;
    uint8_t *ptr;
    size_t bytes;
};
static std::vector<Alloc> g_allocs;
static std::vector<Alloc> g_symbols;  // (no mapping of their own)

static const Alloc g_trusted = {nullptr, 0, nullptr, 0};

static const Alloc *find_alloc(uint64_t addr, size_t n) {
    if (g_any_memory && addr >= 4096) return &g_trusted;
    for (const Alloc &a : g_allocs)
        if (addr >= (uint64_t)a.ptr && addr + n <= (uint64_t)a.ptr + a.bytes) return &a;
    for (const Alloc &a : g_symbols)
        if (addr >= (uint64_t)a.ptr && addr + n <= (uint64_t)a.ptr + a.bytes) return &a;
    return nullptr;
}

static std::string describe_address(uint64_t addr) {
    char buf[256];
    const Alloc *best = nullptr;
    int64_t best_d = INT64_MAX;
    for (const Alloc &a : g_allocs) {
        int64_t d = addr < (uint64_t)a.ptr ? (int64_t)((uint64_t)a.ptr - addr)
                                           : addr >= (uint64_t)a.ptr + a.bytes ? (int64_t)(addr - ((uint64_t)a.ptr + a.bytes) + 1) : 0;
        if (d < best_d) {
            best_d = d;
            best = &a;
        }
    }
    if (!best) return "no allocation";
    snprintf(buf, sizeof buf, "nearest allocation #%zu of %zu bytes, offset %lld", (size_t)(best - g_allocs.data()), best->bytes,
             (long long)((int64_t)addr - (int64_t)(uint64_t)best->ptr));
    return buf;
}

void *register_symbol(void *p, size_t bytes) {
    for (const Alloc &a : g_symbols)
        if (a.ptr == p) return p;
    g_symbols.push_back(Alloc{nullptr, 0, (uint8_t *)p, bytes});
    return p;
}

// ---- LDS ------------------------------------------------------------------------------------------------------
constexpr size_t kLdsBytes = 160 * 1024;
static uint8_t *g_lds = nullptr;
static size_t g_lds_open = kLdsBytes;  // bytes of the LDS area that are accessible: the running launch's dynamic LDS, to the page
static size_t g_lds_launch = 0;  // dynamic LDS the running launch asked for

uint8_t *lds_base() { return g_lds; }

static void map_lds() {
    if (g_lds) return;
    for (uint64_t at = 0x2000000000ull; at < 0x7000000000ull; at += 0x100000000ull) {
        void *p = mmap((void *)at, kLdsBytes + 4096, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_FIXED_NOREPLACE, -1, 0);
        if (p == (void *)at) {
            mprotect(p, kLdsBytes, PROT_READ | PROT_WRITE);
            g_lds = (uint8_t *)p;
            return;
        }
        if (p != MAP_FAILED) munmap(p, kLdsBytes + 4096);
    }
    fprintf(stderr, "host model: no address with 32 zero low bits is free for the LDS\n");
    abort();
}

// ---- fibres ---------------------------------------------------------------------------------------------------
enum St : uint8_t { RUN, WAIT_WAVE, WAIT_WG, DONE };
enum Op : int { OP_CATCHUP = 100, OP_SYNC = 1, OP_BALLOT, OP_READLANE, OP_READFIRST, OP_DPP, OP_PERMSWAP, OP_SHFL, OP_SHFL_UP, OP_MFMA, OP_ASM };

struct Fiber {
    void *sp;
    St st;
    bool yielded;
    int op;
    const void *site;
    void *args;
    LaneCtx ctx;
};

constexpr int kMaxThreads = 1024;
constexpr size_t kStackBytes = 256 * 1024;
static Fiber g_fib[kMaxThreads];
static uint8_t *g_stacks = nullptr;
static void *g_sched_sp = nullptr;
static const std::function<void()> *g_body = nullptr;
static LaneCtx g_host_ctx;

const LaneCtx &lane_ctx() { return g_cur ? g_cur->ctx : g_host_ctx; }

static std::string where() {
    char buf[256];
    if (!g_cur) {
        snprintf(buf, sizeof buf, "[%s] ", g_kernel);
        return buf;
    }
    const LaneCtx &c = g_cur->ctx;
    snprintf(buf, sizeof buf, "[%s block (%u,%u,%u) thread %u] ", g_kernel, c.block_idx.x, c.block_idx.y, c.block_idx.z,
             c.thread_idx.x);
    return buf;
}

// ---- ordering between wavefronts -------------------------------------------------------------------------------
// In the build whose kernel sources are compiled with the compiler's thread-sanitizer instrumentation (build.py,
// `order=True`) every plain memory access of the kernels calls one of the __tsan_* hooks at the end of this file, and
// the interpreter reports its own accesses here as well.  What is checked is what the fibres cannot show by
// themselves, since they run one after the other: two wavefronts that touch the same byte, at least one of them
// writing, with nothing between the two accesses that orders them on the GPU.
//   * LDS (and `__shared__` arrays): a wavefront counts as one thread -- its lanes run in step, and its LDS
//     operations complete in order -- with a vector clock over the wavefronts of the workgroup.  A workgroup barrier
//     joins the clocks of the wavefronts that wait at it; an atomic with release semantics leaves the wavefront's
//     clock at its address, one with acquire semantics takes what was left there.
//   * arrays from sim_alloc: the same inside a workgroup; between workgroups of one launch nothing orders anything, so
//     a byte written by one workgroup and read or written by another is reported.  Launches are ordered by the stream.
//   * inside one wavefront: on the GPU the lanes run in step, so an LDS write that comes earlier in the program than a
//     read has happened for every lane before any lane reads.  Here the lanes are fibres that run one after the other
//     between two wavefront-wide operations, so a lane can see a later lane's byte too early or an earlier lane's too
//     late -- and a result that only comes out right in lane order (a sum handed from lane to lane through the LDS,
//     say) would pass here and fail on the GPU.  So: two different lanes of a wavefront that touch the same byte, at
//     least one writing, with no wavefront-wide operation between the two accesses, are reported.  (The interpreter's
//     accesses are those of the whole wavefront in step and are exempt.)
//   * arrays from sim_alloc, second check: a byte that nothing has written -- no upload (sim_mark_written), no host code
//     of the library (hipMemsetAsync, hipMemcpyAsync), no kernel -- and that a kernel reads.  On the GPU such a byte
//     holds what an earlier launch left there.  The fill pattern of sim_alloc is a tiny number both as fp32 and as
//     bf16, so a sum that includes such bytes passes every tolerance; here the read itself is the violation.
// Atomic accesses themselves are not recorded (they do not race with each other).
constexpr int kMaxWaves = kMaxThreads / 64;
static bool g_order_on = false;
static uint32_t g_vc[kMaxWaves][kMaxWaves];
static uint8_t *g_sh_wwave = nullptr;   // per LDS byte: the wavefront that wrote it last (0xFF: none in this workgroup)
static uint32_t *g_sh_wclk = nullptr;   //   ... at this value of its own clock
static uint32_t *g_sh_rclk = nullptr;   // per LDS byte and wavefront: its clock when it last read the byte (0: never)
struct LaneMark {  // per LDS byte: the last plain write and the last plain read, for the check inside a wavefront
    uint8_t wlane, rwave, rlane;
    uint32_t wepoch, repoch;
};
static LaneMark *g_sh_lane = nullptr;
static uint32_t g_wave_epoch[kMaxThreads / 64];  // counts the wavefront-wide operations (and barriers) of each wavefront
static std::unordered_map<uint64_t, std::vector<uint32_t>> g_sync;  // address of an atomic -> clock left by releases
struct SharedStatic {  // a `__shared__` array of a kernel, with a shadow of its own (emptied when a new workgroup first touches it)
    uint64_t ptr;
    size_t bytes;
    uint64_t workgroup;
    std::vector<uint8_t> wwave;
    std::vector<uint32_t> wclk, rclk;
    std::vector<LaneMark> lane;
};
static std::vector<SharedStatic> g_shared_statics;
static uint32_t g_wg_index = 0, g_order_reports = 0;
static uint64_t g_launch_seq = 0, g_workgroup_seq = 0;
struct GlobalShadow {
    uint64_t launch = 0;  // the launch its contents belong to
    std::vector<uint32_t> w_id, w_clk, r_id, r_clk;  // per byte: (workgroup + 1) << 4 | wavefront, and that wavefront's clock
    std::vector<uint8_t> written;  // per byte, for the life of the array: something has written it
    std::vector<uint8_t> w_lane, r_lane;  // the lanes of the last plain write and read (the check inside a wavefront) ...
    std::vector<uint32_t> w_epoch, r_epoch;  // ... and their wavefront's count of wavefront-wide operations then
};
static bool g_check_unwritten = true;
static std::unordered_map<uint64_t, GlobalShadow> g_global_shadow;  // by Alloc::ptr

static void order_report(const char *fmt, ...) {
    if (++g_order_reports > 6) return;  // per launch
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    violation("ordering: %s", buf);
}

static void order_start_workgroup(uint32_t n_waves, size_t lds_open) {
    if (!g_order_on) return;
    ++g_workgroup_seq;
    if (!g_sh_wwave) {
        const size_t n = kLdsBytes + 16;  // (an access that starts at the last byte: it faults, after the check)
        g_sh_wwave = (uint8_t *)malloc(n);
        g_sh_wclk = (uint32_t *)malloc(n * 4);
        g_sh_rclk = (uint32_t *)malloc(n * 4 * kMaxWaves);
        g_sh_lane = (LaneMark *)malloc(n * sizeof(LaneMark));
        if (!g_sh_wwave || !g_sh_wclk || !g_sh_rclk || !g_sh_lane) abort();
        lds_open = kLdsBytes;
    }
    memset(g_sh_wwave, 0xFF, lds_open);
    memset(g_sh_rclk, 0, lds_open * 4 * kMaxWaves);
    memset(g_sh_lane, 0xFF, lds_open * sizeof(LaneMark));
    memset(g_wave_epoch, 0, sizeof g_wave_epoch);
    memset(g_vc, 0, sizeof g_vc);
    for (uint32_t w = 0; w < n_waves; ++w) g_vc[w][w] = 1;
    g_sync.clear();
}

// The wavefronts in `mask` leave a workgroup barrier together.
static void order_barrier(uint32_t mask) {
    if (!g_order_on) return;
    uint32_t joined[kMaxWaves] = {0};
    for (int w = 0; w < kMaxWaves; ++w)
        if (mask >> w & 1)
            for (int k = 0; k < kMaxWaves; ++k) joined[k] = joined[k] > g_vc[w][k] ? joined[k] : g_vc[w][k];
    for (int w = 0; w < kMaxWaves; ++w)
        if (mask >> w & 1) {
            memcpy(g_vc[w], joined, sizeof joined);
            ++g_vc[w][w];
        }
}

static inline uint32_t cur_wave() { return g_cur->ctx.thread_idx.x / 64; }

// The shadow of one area of shared memory.
struct SharedShadow {
    uint8_t *wwave;
    uint32_t *wclk, *rclk;
    LaneMark *lane;
};
constexpr uint32_t kWholeWave = 0xFE;  // an access of the interpreter: every lane in step

static void order_shared(const SharedShadow &sh, size_t off, size_t n, bool write, const char *what, uint32_t lane) {
    const uint32_t w = cur_wave(), epoch = g_wave_epoch[w];
    for (size_t b = off; b < off + n; ++b) {
        const uint8_t ww = sh.wwave[b];
        LaneMark &lm = sh.lane[b];
        if (lane != kWholeWave) {
            if (ww == w && lm.wlane < 64 && lm.wlane != lane && lm.wepoch == epoch) {
                order_report("lane %u of wavefront %u %s byte 0x%zx of %s (an access of %zu bytes) that lane %u of the same wavefront wrote, and "
                             "no wavefront-wide operation lies between the two: what this lane sees depends on the order in which the "
                             "model runs the lanes", lane, w, write ? "overwrites" : "reads", b, what, n, (unsigned)lm.wlane);
                return;
            }
            if (write && lm.rwave == w && lm.rlane < 64 && lm.rlane != lane && lm.repoch == epoch) {
                order_report("lane %u of wavefront %u writes byte 0x%zx of %s (an access of %zu bytes) that lane %u of the same wavefront read, "
                             "and no wavefront-wide operation lies between the two: what that lane saw depends on the order in which the "
                             "model runs the lanes", lane, w, b, what, n, (unsigned)lm.rlane);
                return;
            }
        }
        if (write) {
            lm.wlane = (uint8_t)lane;
            lm.wepoch = epoch;
        } else {
            lm.rwave = (uint8_t)w;
            lm.rlane = (uint8_t)lane;
            lm.repoch = epoch;
        }
        if (ww != 0xFF && ww != w && sh.wclk[b] > g_vc[w][ww]) {
            order_report("wavefront %u %s byte 0x%zx of %s (an access of %zu bytes) that wavefront %u wrote, and no barrier or "
                         "release/acquire pair lies between the two", w, write ? "overwrites" : "reads", b, what, n, ww);
            return;
        }
        if (write) {
            for (uint32_t r = 0; r < (uint32_t)kMaxWaves; ++r)
                if (r != w && sh.rclk[b * kMaxWaves + r] > g_vc[w][r]) {
                    order_report("wavefront %u writes byte 0x%zx of %s (an access of %zu bytes) that wavefront %u read, and no barrier or "
                                 "release/acquire pair lies between the two", w, b, what, n, r);
                    return;
                }
            sh.wwave[b] = (uint8_t)w;
            sh.wclk[b] = g_vc[w][w];
        } else {
            sh.rclk[b * kMaxWaves + w] = g_vc[w][w];
        }
    }
}

// An access to the LDS or to a `__shared__` array: checked, and true.
static bool order_shared_access(uint64_t addr, size_t n, bool write, uint32_t lane) {
    if (addr - (uint64_t)g_lds < kLdsBytes) {
        order_shared(SharedShadow{g_sh_wwave, g_sh_wclk, g_sh_rclk, g_sh_lane}, (size_t)(addr - (uint64_t)g_lds), n, write, "the LDS", lane);
        return true;
    }
    for (SharedStatic &s : g_shared_statics)
        if (addr - s.ptr < s.bytes) {
            if (s.workgroup != g_workgroup_seq) {
                s.workgroup = g_workgroup_seq;
                s.wwave.assign(s.bytes + 16, 0xFF);
                s.wclk.assign(s.bytes + 16, 0);
                s.rclk.assign((s.bytes + 16) * kMaxWaves, 0);
                s.lane.assign(s.bytes + 16, LaneMark{0xFF, 0xFF, 0xFF, 0, 0});
            }
            order_shared(SharedShadow{s.wwave.data(), s.wclk.data(), s.rclk.data(), s.lane.data()}, (size_t)(addr - s.ptr), n, write,
                         "a __shared__ array", lane);
            return true;
        }
    return false;
}

static bool is_shared(uint64_t addr) {
    if (addr - (uint64_t)g_lds < kLdsBytes) return true;
    for (const SharedStatic &s : g_shared_statics)
        if (addr - s.ptr < s.bytes) return true;
    return false;
}

static void order_global(const Alloc &a, uint64_t addr, size_t n, bool write, uint32_t lane) {
    GlobalShadow &s = g_global_shadow[(uint64_t)a.ptr];
    if (s.launch != g_launch_seq || s.w_id.size() != a.bytes) {
        s.launch = g_launch_seq;
        s.w_id.assign(a.bytes, 0);
        s.w_clk.assign(a.bytes, 0);
        s.r_id.assign(a.bytes, 0);
        s.r_clk.assign(a.bytes, 0);
        s.w_lane.assign(a.bytes, 0xFF);
        s.r_lane.assign(a.bytes, 0xFF);
        s.w_epoch.assign(a.bytes, 0);
        s.r_epoch.assign(a.bytes, 0);
    }
    if (s.written.size() != a.bytes) s.written.assign(a.bytes, 0);
    const uint32_t w = cur_wave(), me = (g_wg_index + 1) << 4 | w;
    // did the access `id` at clock `clk` happen before what this wavefront does now?
    auto before = [&](uint32_t id, uint32_t clk) { return id == 0 || id == me || (id >> 4 == me >> 4 && clk <= g_vc[w][id & 15]); };
    const size_t o = (size_t)(addr - (uint64_t)a.ptr);
    const uint32_t epoch = g_wave_epoch[w];
    for (size_t i = 0; i < n && o + i < a.bytes; ++i) {
        const size_t b = o + i;
        if (lane != kWholeWave) {  // inside the wavefront, as for the LDS
            if (s.w_id[b] == me && s.w_lane[b] < 64 && s.w_lane[b] != lane && s.w_epoch[b] == epoch) {
                order_report("lane %u of workgroup %u wavefront %u %s byte %zu of allocation #%zu (%zu bytes) that lane %u of the same "
                             "wavefront wrote, and no wavefront-wide operation lies between the two: what this lane sees depends on the "
                             "order in which the model runs the lanes", lane, g_wg_index, w, write ? "overwrites" : "reads", b,
                             (size_t)(&a - g_allocs.data()), a.bytes, (unsigned)s.w_lane[b]);
                return;
            }
            if (write && s.r_id[b] == me && s.r_lane[b] < 64 && s.r_lane[b] != lane && s.r_epoch[b] == epoch) {
                order_report("lane %u of workgroup %u wavefront %u writes byte %zu of allocation #%zu (%zu bytes) that lane %u of the same "
                             "wavefront read, and no wavefront-wide operation lies between the two: what that lane saw depends on the "
                             "order in which the model runs the lanes", lane, g_wg_index, w, b, (size_t)(&a - g_allocs.data()), a.bytes,
                             (unsigned)s.r_lane[b]);
                return;
            }
        }
        if (write) {
            s.w_lane[b] = (uint8_t)lane;
            s.w_epoch[b] = epoch;
        } else {
            s.r_lane[b] = (uint8_t)lane;
            s.r_epoch[b] = epoch;
        }
        if (!before(s.w_id[b], s.w_clk[b])) {
            order_report("workgroup %u wavefront %u %s byte %zu of allocation #%zu (%zu bytes) that workgroup %u wavefront %u wrote in the "
                         "same launch, and nothing orders the two", g_wg_index, w, write ? "overwrites" : "reads", b,
                         (size_t)(&a - g_allocs.data()), a.bytes, (s.w_id[b] >> 4) - 1, s.w_id[b] & 15);
            return;
        }
        if (!write && !s.written[b] && g_check_unwritten) {
            order_report("workgroup %u wavefront %u reads byte %zu of allocation #%zu (%zu bytes; an access of %zu bytes at offset %zu), "
                         "which nothing has written: no upload, no host code of the library, no kernel", g_wg_index, w, b,
                         (size_t)(&a - g_allocs.data()), a.bytes, n, o);
            return;
        }
        if (write) {
            s.written[b] = 1;
            if (!before(s.r_id[b], s.r_clk[b])) {
                order_report("workgroup %u wavefront %u writes byte %zu of allocation #%zu (%zu bytes) that workgroup %u wavefront %u read in "
                             "the same launch, and nothing orders the two", g_wg_index, w, b, (size_t)(&a - g_allocs.data()), a.bytes,
                             (s.r_id[b] >> 4) - 1, s.r_id[b] & 15);
                return;
            }
            s.w_id[b] = me;
            s.w_clk[b] = g_vc[w][w];
        } else {
            s.r_id[b] = me;
            s.r_clk[b] = g_vc[w][w];
        }
    }
}

// Every access of kernel code: plain C++ through the compiler's hooks, the interpreter's by its own calls.
static void mark_written(uint64_t addr, size_t n) {
    for (const Alloc &a : g_allocs)
        if (addr - (uint64_t)a.ptr < a.bytes) {
            GlobalShadow &s = g_global_shadow[(uint64_t)a.ptr];
            if (s.written.size() != a.bytes) s.written.assign(a.bytes, 0);
            const size_t o = (size_t)(addr - (uint64_t)a.ptr);
            memset(s.written.data() + o, 1, n < a.bytes - o ? n : a.bytes - o);
            return;
        }
}

static inline void order_access(uint64_t addr, size_t n, bool write, bool whole_wave = false) {
    if (!g_order_on || n == 0) return;
    if (!g_cur) return;  // host code
    if (addr - (uint64_t)g_stacks < (uint64_t)kMaxThreads * kStackBytes) return;  // a fibre's own stack
    const uint32_t lane = whole_wave ? kWholeWave : g_cur->ctx.thread_idx.x % 64;
    if (order_shared_access(addr, n, write, lane)) return;
    static size_t last = 0;
    if (last < g_allocs.size() && addr - (uint64_t)g_allocs[last].ptr < g_allocs[last].bytes) {
        order_global(g_allocs[last], addr, n, write, lane);
        return;
    }
    for (size_t k = 0; k < g_allocs.size(); ++k)
        if (addr - (uint64_t)g_allocs[k].ptr < g_allocs[k].bytes) {
            last = k;
            order_global(g_allocs[k], addr, n, write, lane);
            return;
        }
}

// An atomic access of kernel code (the stand-ins of hip_runtime.h call this): no access is recorded; release and
// acquire move clocks through the address.  Device-scope atomics on arrays order nothing between workgroups here.
void order_atomic(const void *p, bool acquire, bool release) {
    if (!g_order_on || !g_cur) return;
    if (!is_shared((uint64_t)p)) return;
    const uint32_t w = cur_wave();
    std::vector<uint32_t> &left = g_sync[(uint64_t)p];
    if (left.empty()) left.assign(kMaxWaves, 0);
    if (acquire)
        for (int k = 0; k < kMaxWaves; ++k) g_vc[w][k] = g_vc[w][k] > left[k] ? g_vc[w][k] : left[k];
    if (release) {
        for (int k = 0; k < kMaxWaves; ++k) left[k] = left[k] > g_vc[w][k] ? left[k] : g_vc[w][k];
        ++g_vc[w][w];
    }
}

void shared_static(const void *p, size_t bytes) {
    if (!g_order_on) return;
    for (const SharedStatic &s : g_shared_statics)
        if (s.ptr == (uint64_t)p) return;
    g_shared_statics.push_back(SharedStatic{(uint64_t)p, bytes, 0, {}, {}, {}, {}});
}

extern "C" void sim_switch(void **from_sp, void *to_sp);
asm(R"(
.text
.globl sim_switch
.type sim_switch,@function
sim_switch:
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
.size sim_switch, .-sim_switch
)");

static void to_scheduler() {
    Fiber *f = g_cur;
    sim_switch(&f->sp, g_sched_sp);
}

static void fiber_main() {
    (*g_body)();
    g_cur->st = DONE;
    to_scheduler();
    abort();
}

static void fiber_reset(Fiber &f, int index) {
    uint64_t top = ((uint64_t)(g_stacks + (size_t)(index + 1) * kStackBytes)) & ~(uint64_t)15;
    uint64_t *s = (uint64_t *)top;
    *--s = 0;                      // the address fiber_main would return to (it never returns)
    *--s = (uint64_t)&fiber_main;  // taken by sim_switch's ret
    for (int i = 0; i < 6; ++i) *--s = 0;
    f.sp = s;
    f.st = RUN;
    f.yielded = false;
    f.op = 0;
    f.site = nullptr;
    f.args = nullptr;
}

static void meet(int op, void *args, const void *site) {
    Fiber *f = g_cur;
    if (!f) {
        fprintf(stderr, "host model: a wavefront-wide operation outside a kernel\n");
        abort();
    }
    f->op = op;
    f->args = args;
    f->site = site;
    f->st = WAIT_WAVE;
    to_scheduler();
}

// ---- wavefront-wide operations: what a lane hands in -----------------------------------------------------------
struct BallotArgs {
    int pred;
    uint64_t out;
};
struct LaneArgs {  // readlane, readfirstlane, shuffles
    int v, sel, width, out;
};
struct DppArgs {
    int old, src, ctrl, row_mask, bank_mask;
    bool bound_ctrl;
    int out;
};
struct SwapArgs {
    uint32_t a, b;
    int rows;
    uint32_t out_a, out_b;
};
struct MfmaArgs {
    const void *a, *b;
    void *c;
};
struct AsmArgs {
    const char *tmpl;
    AsmOperand *ops;
    int n;
};

__attribute__((noinline)) uint64_t ballot(int pred) {
    BallotArgs a{pred, 0};
    meet(OP_BALLOT, &a, __builtin_return_address(0));
    return a.out;
}
__attribute__((noinline)) int readlane(int v, int lane) {
    LaneArgs a{v, lane, 64, 0};
    meet(OP_READLANE, &a, __builtin_return_address(0));
    return a.out;
}
__attribute__((noinline)) int readfirstlane(int v) {
    LaneArgs a{v, 0, 64, 0};
    meet(OP_READFIRST, &a, __builtin_return_address(0));
    return a.out;
}
__attribute__((noinline)) int update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
    DppArgs a{old, src, ctrl, row_mask, bank_mask, bound_ctrl, 0};
    meet(OP_DPP, &a, __builtin_return_address(0));
    return a.out;
}
__attribute__((noinline)) u32x2v permlane_swap(uint32_t x, uint32_t y, int rows) {
    SwapArgs a{x, y, rows, 0, 0};
    meet(OP_PERMSWAP, &a, __builtin_return_address(0));
    u32x2v r;
    r[0] = a.out_a;
    r[1] = a.out_b;
    return r;
}
__attribute__((noinline)) int shfl(int v, int src, int width) {
    LaneArgs a{v, src, width, 0};
    meet(OP_SHFL, &a, __builtin_return_address(0));
    return a.out;
}
__attribute__((noinline)) int shfl_up(int v, unsigned delta, int width) {
    LaneArgs a{v, (int)delta, width, 0};
    meet(OP_SHFL_UP, &a, __builtin_return_address(0));
    return a.out;
}
__attribute__((noinline)) void wave_sync() { meet(OP_SYNC, nullptr, __builtin_return_address(0)); }
// A lane about to publish something (a store or read-modify-write with release semantics) waits until every other
// lane of its wavefront has run up to its next meeting point: on the GPU the lanes of a wavefront run in step, so
// what the other lanes did earlier in the program has happened before one lane's later store.
void wave_catch_up() { meet(OP_CATCHUP, nullptr, nullptr); }
__attribute__((noinline)) void mfma_impl(const void *a, const void *b, void *c) {
    MfmaArgs m{a, b, c};
    meet(OP_MFMA, &m, __builtin_return_address(0));
}
__attribute__((noinline)) void run_asm(const char *tmpl, AsmOperand *ops, int n) {
    bool any = false;  // a statement without instructions (a compiler barrier) is no meeting point
    for (const char *p = tmpl; *p; ++p) any = any || (*p != ' ' && *p != '\n' && *p != '\t');
    if (!any) return;
    AsmArgs a{tmpl, ops, n};
    meet(OP_ASM, &a, tmpl);
}
void syncthreads() {
    Fiber *f = g_cur;
    f->st = WAIT_WG;
    to_scheduler();
}
void yield() {
    Fiber *f = g_cur;
    f->yielded = true;
    to_scheduler();
}

uint32_t v_perm(uint32_t s0, uint32_t s1, uint32_t sel) {
    const uint64_t src = ((uint64_t)s0 << 32) | s1;
    uint32_t out = 0;
    for (int i = 0; i < 4; ++i) {
        const uint32_t s = (sel >> (8 * i)) & 0xFFu;
        uint32_t byte;
        if (s <= 7)
            byte = (uint32_t)(src >> (8 * s)) & 0xFFu;
        else if (s <= 11)  // sign of a 16-bit half
            byte = ((src >> (16 * (s - 8) + 15)) & 1u) ? 0xFFu : 0u;
        else if (s == 12)
            byte = 0;
        else
            byte = 0xFFu;
        out |= byte << (8 * i);
    }
    return out;
}

static inline float bf16_f32(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }

// D = C + A B for v_mfma_f32_32x32x16_bf16.  A: lane l holds row l % 32, k = 8 (l / 32) .. + 7; B: lane l holds
// column l % 32, the same k; C / D: register v of lane l is row 8 (v / 4) + 4 (l / 32) + v % 4, column l % 32.
// Products are exact in fp32; they are added to the accumulator in ascending k (the hardware's order is its own).
static void mfma_compute(const uint16_t (*a)[8], const uint16_t (*b)[8], float (*c)[16]) {
    float af[32][16], bf[32][16];  // [row i][k], [column j][k]
    for (int l = 0; l < 64; ++l)
        for (int t = 0; t < 8; ++t) {
            af[l % 32][8 * (l / 32) + t] = bf16_f32(a[l][t]);
            bf[l % 32][8 * (l / 32) + t] = bf16_f32(b[l][t]);
        }
    for (int l = 0; l < 64; ++l)
        for (int v = 0; v < 16; ++v) {
            const int i = 8 * (v / 4) + 4 * (l / 32) + v % 4, j = l % 32;
            float s = c[l][v];
            for (int k = 0; k < 16; ++k) s += af[i][k] * bf[j][k];
            c[l][v] = s;
        }
}

// ---- the interpreter of assembly statements -------------------------------------------------------------------
enum OpdKind : uint8_t { K_NONE, K_V, K_S, K_VCC, K_EXEC, K_LIT, K_LABEL };
struct Opd {
    OpdKind k = K_NONE;
    uint16_t reg = 0;
    uint8_t n = 1;
    uint32_t lit = 0;
    std::string label;
};
enum Code : int {
    I_V_AND, I_V_LSHRREV, I_V_LSHLREV, I_V_MAD_U24, I_V_CMP_GT_U32, I_V_CMPX_GT_U32, I_S_AND_SAVEEXEC, I_V_LSHL_OR,
    I_V_SUBREV, I_V_ADD, I_V_MOV, I_V_PERM, I_V_AND_OR, I_DS_READ_U8, I_DS_READ_B64, I_GLOAD_DWORD, I_GLOAD_X4,
    I_GSTORE_BYTE, I_MFMA, I_S_MOV32, I_S_MOV64, I_S_ADD, I_S_SUB, I_S_LSHR, I_S_CMP_EQ, I_S_CMP_LG, I_S_CSELECT,
    I_S_WAITCNT, I_S_NOP, I_S_BRANCH, I_S_CBRANCH_SCC1, I_S_CBRANCH_SCC0, I_S_CBRANCH_EXECNZ, I_END
};
static const std::map<std::string, Code> kMnemonics = {
    {"v_and_b32", I_V_AND}, {"v_lshrrev_b32", I_V_LSHRREV}, {"v_lshlrev_b32", I_V_LSHLREV},
    {"v_mad_u32_u24", I_V_MAD_U24}, {"v_cmp_gt_u32", I_V_CMP_GT_U32}, {"v_cmpx_gt_u32", I_V_CMPX_GT_U32},
    {"s_and_saveexec_b64", I_S_AND_SAVEEXEC}, {"v_lshl_or_b32", I_V_LSHL_OR}, {"v_subrev_u32", I_V_SUBREV},
    {"v_add_u32", I_V_ADD}, {"v_mov_b32", I_V_MOV}, {"v_perm_b32", I_V_PERM}, {"v_and_or_b32", I_V_AND_OR},
    {"ds_read_u8", I_DS_READ_U8}, {"ds_read_b64", I_DS_READ_B64}, {"global_load_dword", I_GLOAD_DWORD},
    {"global_load_dwordx4", I_GLOAD_X4}, {"global_store_byte", I_GSTORE_BYTE},
    {"v_mfma_f32_32x32x16_bf16", I_MFMA}, {"s_mov_b32", I_S_MOV32}, {"s_mov_b64", I_S_MOV64}, {"s_add_u32", I_S_ADD},
    {"s_sub_u32", I_S_SUB}, {"s_lshr_b32", I_S_LSHR}, {"s_cmp_eq_u32", I_S_CMP_EQ}, {"s_cmp_lg_u32", I_S_CMP_LG},
    {"s_cselect_b32", I_S_CSELECT}, {"s_waitcnt", I_S_WAITCNT}, {"s_nop", I_S_NOP}, {"s_branch", I_S_BRANCH},
    {"s_cbranch_scc1", I_S_CBRANCH_SCC1}, {"s_cbranch_scc0", I_S_CBRANCH_SCC0}, {"s_cbranch_execnz", I_S_CBRANCH_EXECNZ},
};

struct Ins {
    Code c;
    Opd o[4];
    int nops = 0;
    int32_t offset = 0;         // offset:N of a memory instruction
    int wait_vm = -1, wait_lgkm = -1;
    int target = -1;
    int seq = 0;                // position in the text (for numeric labels)
    std::string text;
};
struct Binding {
    std::string name;
    bool vector, written, read;
    int reg, nregs;
};
struct Program {
    std::vector<Ins> ins;
    std::vector<Binding> bind;  // one per operand of the statement, in order
    bool ok = true;
};

static std::string trim(const std::string &s) {
    size_t a = s.find_first_not_of(" \t\r"), b = s.find_last_not_of(" \t\r");
    return a == std::string::npos ? "" : s.substr(a, b - a + 1);
}

static bool parse_operand(const std::string &tok, Opd &o) {
    unsigned a = 0, b = 0;
    char c = 0;
    if (sscanf(tok.c_str(), "%c[%u:%u]", &c, &a, &b) == 3 && (c == 'v' || c == 's') && tok.back() == ']') {
        o.k = c == 'v' ? K_V : K_S;
        o.reg = (uint16_t)a;
        o.n = (uint8_t)(b - a + 1);
        return true;
    }
    if ((tok[0] == 'v' || tok[0] == 's') && tok.size() > 1 && isdigit((unsigned char)tok[1])) {
        char *end = nullptr;
        const unsigned long r = strtoul(tok.c_str() + 1, &end, 10);
        if (*end == 0) {
            o.k = tok[0] == 'v' ? K_V : K_S;
            o.reg = (uint16_t)r;
            o.n = 1;
            return true;
        }
    }
    if (tok == "vcc") {
        o.k = K_VCC;
        return true;
    }
    if (tok == "exec") {
        o.k = K_EXEC;
        return true;
    }
    if (isdigit((unsigned char)tok[0]) || tok[0] == '-') {
        char *end = nullptr;
        const long long v = strtoll(tok.c_str(), &end, 0);
        if (*end == 0) {
            o.k = K_LIT;
            o.lit = (uint32_t)v;
            return true;
        }
    }
    o.k = K_LABEL;
    o.label = tok;
    return true;
}

static std::unordered_map<const char *, Program> g_programs;

static const Program &compile(const AsmArgs &st) {
    auto it = g_programs.find(st.tmpl);
    if (it != g_programs.end()) return it->second;
    Program &p = g_programs[st.tmpl];
    // registers for the operands: vector operands from v0 up (the statements' own registers start at v72),
    // scalar ones from s40 (theirs are s20..s25)
    int next_v = 0, next_s = 40;
    for (int i = 0; i < st.n; ++i) {
        const AsmOperand &op = st.ops[i];
        Binding b;
        b.name = op.name;
        b.vector = strchr(op.constraint, 'v') != nullptr;
        b.written = strchr(op.constraint, '=') || strchr(op.constraint, '+');
        b.read = !strchr(op.constraint, '=');
        b.nregs = (int)((op.bytes + 3) / 4);
        if (b.vector) {
            b.reg = next_v;
            next_v += b.nregs;
        } else {
            if (b.nregs > 1) next_s = (next_s + 1) & ~1;
            b.reg = next_s;
            next_s += b.nregs;
        }
        p.bind.push_back(b);
    }
    if (next_v > 72 || next_s > 100) {
        violation("asm statement: too many operands for the model's register plan");
        p.ok = false;
        return p;
    }
    auto reg_text = [&](const Binding &b) {
        char buf[32];
        const char c = b.vector ? 'v' : 's';
        if (b.nregs == 1)
            snprintf(buf, sizeof buf, "%c%d", c, b.reg);
        else
            snprintf(buf, sizeof buf, "%c[%d:%d]", c, b.reg, b.reg + b.nregs - 1);
        return std::string(buf);
    };
    // substitute %[name], %N and %=
    std::string text;
    for (const char *s = st.tmpl; *s;) {
        if (s[0] == '%' && s[1] == '[') {
            const char *e = strchr(s, ']');
            const std::string name(s + 2, e);
            bool found = false;
            for (const Binding &b : p.bind)
                if (b.name == name) {
                    text += reg_text(b);
                    found = true;
                }
            if (!found) {
                violation("asm statement names an operand it does not have: %s", name.c_str());
                p.ok = false;
            }
            s = e + 1;
        } else if (s[0] == '%' && s[1] == '=') {
            text += "U";
            s += 2;
        } else if (s[0] == '%' && isdigit((unsigned char)s[1])) {
            char *e = nullptr;
            const long n = strtol(s + 1, &e, 10);
            if (n < (long)p.bind.size()) text += reg_text(p.bind[n]);
            s = e;
        } else {
            text += *s++;
        }
    }
    // lines -> two sections of instructions and the labels
    struct Label {
        std::string name;
        int seq, section, pos;
    };
    std::vector<Ins> sec[2];
    std::vector<Label> labels;
    int section = 0, seq = 0;
    size_t at = 0;
    while (at <= text.size()) {
        size_t nl = text.find('\n', at);
        if (nl == std::string::npos) nl = text.size();
        std::string line = trim(text.substr(at, nl - at));
        at = nl + 1;
        const size_t cm = line.find("//");
        if (cm != std::string::npos) line = trim(line.substr(0, cm));
        if (line.empty()) continue;
        ++seq;
        if (line.rfind(".subsection", 0) == 0) {
            section = atoi(line.c_str() + 11) ? 1 : 0;
            continue;
        }
        if (line.back() == ':') {
            labels.push_back(Label{line.substr(0, line.size() - 1), seq, section, (int)sec[section].size()});
            continue;
        }
        Ins in;
        in.text = line;
        in.seq = seq;
        const size_t sp = line.find_first_of(" \t");
        const std::string mn = line.substr(0, sp);
        auto m = kMnemonics.find(mn);
        if (m == kMnemonics.end()) {
            violation("the interpreter does not know the instruction `%s`", line.c_str());
            p.ok = false;
            continue;
        }
        in.c = m->second;
        std::string rest = sp == std::string::npos ? "" : trim(line.substr(sp));
        if (in.c == I_S_WAITCNT) {
            const char *v = strstr(rest.c_str(), "vmcnt("), *l = strstr(rest.c_str(), "lgkmcnt(");
            if (v) in.wait_vm = atoi(v + 6);
            if (l) in.wait_lgkm = atoi(l + 8);
        } else if (!rest.empty()) {
            size_t a2 = 0;
            while (a2 <= rest.size()) {
                size_t c2 = rest.find(',', a2);
                // (a comma inside v[a:b] does not occur: ranges use a colon)
                if (c2 == std::string::npos) c2 = rest.size();
                std::string tok = trim(rest.substr(a2, c2 - a2));
                a2 = c2 + 1;
                const size_t off = tok.find("offset:");
                if (off != std::string::npos) {
                    in.offset = (int32_t)strtol(tok.c_str() + off + 7, nullptr, 0);
                    tok = trim(tok.substr(0, off));
                }
                if (tok.empty()) continue;
                if (in.nops >= 4) {
                    violation("instruction with more than four operands: `%s`", line.c_str());
                    p.ok = false;
                    break;
                }
                parse_operand(tok, in.o[in.nops++]);
            }
        }
        sec[section].push_back(in);
    }
    // linear program: section 0, END, section 1, END
    const int base1 = (int)sec[0].size() + 1;
    for (const Ins &in : sec[0]) p.ins.push_back(in);
    Ins end;
    end.c = I_END;
    end.text = "(end of the statement)";
    p.ins.push_back(end);
    for (const Ins &in : sec[1]) p.ins.push_back(in);
    end.text = "(end of the out-of-line code: falls off)";
    p.ins.push_back(end);
    for (Ins &in : p.ins) {
        if (in.c != I_S_BRANCH && in.c != I_S_CBRANCH_SCC0 && in.c != I_S_CBRANCH_SCC1 && in.c != I_S_CBRANCH_EXECNZ) continue;
        const std::string &l = in.o[0].label;
        const Label *hit = nullptr;
        const bool numeric = l.size() >= 2 && isdigit((unsigned char)l[0]) && (l.back() == 'f' || l.back() == 'b');
        for (const Label &lb : labels) {
            if (numeric) {
                if (lb.name != l.substr(0, l.size() - 1)) continue;
                if (l.back() == 'f' && lb.seq > in.seq && (!hit || lb.seq < hit->seq)) hit = &lb;
                if (l.back() == 'b' && lb.seq < in.seq && (!hit || lb.seq > hit->seq)) hit = &lb;
            } else if (lb.name == l) {
                hit = &lb;
            }
        }
        if (!hit) {
            violation("branch to an unknown label: `%s`", in.text.c_str());
            p.ok = false;
            continue;
        }
        in.target = (hit->section ? base1 : 0) + hit->pos;
    }
    return p;
}

struct WaveRegs {
    uint32_t v[256][64];
    uint32_t s[128];
    uint64_t vcc, exec;
    bool scc;
    // loads in flight: per VGPR the kind (1 LDS, 2 global) and the issue number of the load that will write it
    uint8_t pend_kind[256];
    uint64_t pend_seq[256];
    uint64_t issued[3], done[3];
};
static WaveRegs g_w;

static bool reg_ready(int r) { return g_w.pend_kind[r] == 0 || g_w.pend_seq[r] <= g_w.done[g_w.pend_kind[r]]; }

static void exec_asm(Fiber **lanes, int n_lanes_total, uint64_t part) {
    // `lanes[i]` = fibre of lane i or null; `part` = mask of the lanes that take part
    const AsmArgs *first = nullptr;
    for (int l = 0; l < 64; ++l)
        if (part >> l & 1) {
            first = (const AsmArgs *)lanes[l]->args;
            break;
        }
    const Program &p = compile(*first);
    if (!p.ok) {
        g_abort_launch = true;
        return;
    }
    WaveRegs &w = g_w;
    memset(w.pend_kind, 0, sizeof w.pend_kind);
    memset(w.issued, 0, sizeof w.issued);
    memset(w.done, 0, sizeof w.done);
    w.exec = part;
    w.vcc = 0;
    w.scc = false;
    for (int r = 72; r < 128; ++r)
        for (int l = 0; l < 64; ++l) w.v[r][l] = 0xDEAD0000u + r;  // the statement's own registers start undefined
    // operands in
    for (size_t k = 0; k < p.bind.size(); ++k) {
        const Binding &b = p.bind[k];
        if (b.vector) {
            for (int l = 0; l < 64; ++l) {
                if (!(part >> l & 1)) {
                    for (int j = 0; j < b.nregs; ++j) w.v[b.reg + j][l] = 0;
                    continue;
                }
                const AsmOperand &op = ((const AsmArgs *)lanes[l]->args)->ops[k];
                uint32_t tmp[16] = {0};
                memcpy(tmp, op.ptr, op.bytes);
                for (int j = 0; j < b.nregs; ++j) w.v[b.reg + j][l] = b.read ? tmp[j] : 0xDEADBEEFu;
            }
        } else {
            uint32_t ref[4] = {0};
            bool have = false;
            for (int l = 0; l < 64; ++l) {
                if (!(part >> l & 1)) continue;
                const AsmOperand &op = ((const AsmArgs *)lanes[l]->args)->ops[k];
                uint32_t tmp[4] = {0};
                memcpy(tmp, op.ptr, op.bytes);
                if (!have) {
                    memcpy(ref, tmp, sizeof ref);
                    have = true;
                } else if (memcmp(ref, tmp, sizeof ref) != 0) {
                    g_cur = lanes[l];
                    violation("asm operand %%[%s] sits in a scalar register but differs between lanes (lane %d: 0x%x, first lane: 0x%x)",
                              b.name.c_str(), l, tmp[0], ref[0]);
                    g_abort_launch = true;
                    return;
                }
            }
            for (int j = 0; j < b.nregs; ++j) w.s[b.reg + j] = ref[j];
        }
    }
    g_cur = lanes[__builtin_ctzll(part)];

    auto sval = [&](const Opd &o) -> uint32_t {  // scalar source
        if (o.k == K_S) return w.s[o.reg];
        if (o.k == K_LIT) return o.lit;
        violation("scalar instruction with an operand the model does not read");
        return 0;
    };
    auto vsrc = [&](const Opd &o, int l) -> uint32_t {  // vector-instruction source
        switch (o.k) {
            case K_V: return w.v[o.reg][l];
            case K_S: return w.s[o.reg];
            case K_LIT: return o.lit;
            default: return 0;
        }
    };
    auto need_ready = [&](const Ins &in, const Opd &o) {
        if (o.k != K_V) return;
        for (int j = 0; j < o.n; ++j)
            if (!reg_ready(o.reg + j))
                violation("`%s` uses v%d before the s_waitcnt that covers its load", in.text.c_str(), o.reg + j);
    };
    auto s64 = [&](const Opd &o) -> uint64_t { return (uint64_t)w.s[o.reg] | ((uint64_t)w.s[o.reg + 1] << 32); };

    uint64_t steps = 0;
    int pc = 0;
    for (;;) {
        const Ins &in = p.ins[pc];
        if (in.c == I_END) {
            if (pc == (int)p.ins.size() - 1) violation("asm statement: the out-of-line code runs off its end");
            break;
        }
        if (++steps > 50000000ull) {
            violation("asm statement does not end (50 M instructions)");
            g_abort_launch = true;
            return;
        }
        ++g_asm_instructions;
        int next = pc + 1;
        const Opd *o = in.o;
        switch (in.c) {
            case I_V_AND: case I_V_LSHRREV: case I_V_LSHLREV: case I_V_SUBREV: case I_V_ADD: case I_V_MOV:
            case I_V_MAD_U24: case I_V_LSHL_OR: case I_V_PERM: case I_V_AND_OR: {
                for (int k = 1; k < in.nops; ++k) need_ready(in, o[k]);
                need_ready(in, o[0]);  // a load still on its way to the destination would overwrite the result
                if (o[0].k != K_V) {
                    violation("`%s`: destination is not a vector register", in.text.c_str());
                    break;
                }
                // sources as arrays of 64 (scalars and literals broadcast), then one plain loop per operation
                uint32_t bc[3][64];
                const uint32_t *src[3] = {bc[0], bc[1], bc[2]};
                for (int k = 1; k <= 3; ++k) {
                    if (k < in.nops && o[k].k == K_V) {
                        src[k - 1] = w.v[o[k].reg];
                    } else {
                        const uint32_t val = k < in.nops ? vsrc(o[k], 0) : 0u;
                        for (int l = 0; l < 64; ++l) bc[k - 1][l] = val;
                    }
                }
                const uint32_t *A = src[0], *B = src[1], *Cs = src[2];
                uint32_t r[64];
                switch (in.c) {
                    case I_V_AND: for (int l = 0; l < 64; ++l) r[l] = A[l] & B[l]; break;
                    case I_V_LSHRREV: for (int l = 0; l < 64; ++l) r[l] = B[l] >> (A[l] & 31); break;
                    case I_V_LSHLREV: for (int l = 0; l < 64; ++l) r[l] = B[l] << (A[l] & 31); break;
                    case I_V_SUBREV: for (int l = 0; l < 64; ++l) r[l] = B[l] - A[l]; break;
                    case I_V_ADD: for (int l = 0; l < 64; ++l) r[l] = A[l] + B[l]; break;
                    case I_V_MOV: for (int l = 0; l < 64; ++l) r[l] = A[l]; break;
                    case I_V_MAD_U24: for (int l = 0; l < 64; ++l) r[l] = (A[l] & 0xFFFFFFu) * (B[l] & 0xFFFFFFu) + Cs[l]; break;
                    case I_V_LSHL_OR: for (int l = 0; l < 64; ++l) r[l] = (A[l] << (B[l] & 31)) | Cs[l]; break;
                    case I_V_PERM: for (int l = 0; l < 64; ++l) r[l] = v_perm(A[l], B[l], Cs[l]); break;
                    case I_V_AND_OR: for (int l = 0; l < 64; ++l) r[l] = (A[l] & B[l]) | Cs[l]; break;
                    default: break;
                }
                uint32_t *D = w.v[o[0].reg];
                if (w.exec == ~0ull) {
                    memcpy(D, r, sizeof r);
                } else {
                    for (int l = 0; l < 64; ++l)
                        if (w.exec >> l & 1) D[l] = r[l];
                }
                break;
            }
            case I_V_CMP_GT_U32: case I_V_CMPX_GT_U32: {
                need_ready(in, o[1]);
                need_ready(in, o[2]);
                uint64_t m = 0;
                for (int l = 0; l < 64; ++l)
                    if ((w.exec >> l & 1) && vsrc(o[1], l) > vsrc(o[2], l)) m |= 1ull << l;
                w.vcc = m;
                if (in.c == I_V_CMPX_GT_U32) w.exec = m;
                break;
            }
            case I_S_AND_SAVEEXEC: {
                const uint64_t src = o[1].k == K_VCC ? w.vcc : s64(o[1]);
                w.s[o[0].reg] = (uint32_t)w.exec;
                w.s[o[0].reg + 1] = (uint32_t)(w.exec >> 32);
                w.exec &= src;
                w.scc = w.exec != 0;
                break;
            }
            case I_S_MOV64: {
                const uint64_t src = o[1].k == K_VCC ? w.vcc : o[1].k == K_EXEC ? w.exec : s64(o[1]);
                if (o[0].k == K_EXEC)
                    w.exec = src;
                else if (o[0].k == K_VCC)
                    w.vcc = src;
                else {
                    w.s[o[0].reg] = (uint32_t)src;
                    w.s[o[0].reg + 1] = (uint32_t)(src >> 32);
                }
                break;
            }
            case I_S_MOV32: w.s[o[0].reg] = sval(o[1]); break;
            case I_S_ADD: {
                const uint64_t r = (uint64_t)sval(o[1]) + sval(o[2]);
                w.s[o[0].reg] = (uint32_t)r;
                w.scc = (r >> 32) != 0;
                break;
            }
            case I_S_SUB: {
                const uint32_t a = sval(o[1]), b = sval(o[2]);
                w.s[o[0].reg] = a - b;
                w.scc = b > a;
                break;
            }
            case I_S_LSHR: {
                const uint32_t r = sval(o[1]) >> (sval(o[2]) & 31);
                w.s[o[0].reg] = r;
                w.scc = r != 0;
                break;
            }
            case I_S_CMP_EQ: w.scc = sval(o[0]) == sval(o[1]); break;
            case I_S_CMP_LG: w.scc = sval(o[0]) != sval(o[1]); break;
            case I_S_CSELECT: w.s[o[0].reg] = w.scc ? sval(o[1]) : sval(o[2]); break;
            case I_S_NOP: break;
            case I_S_WAITCNT:
                if (in.wait_lgkm >= 0 && w.issued[1] >= (uint64_t)in.wait_lgkm)
                    w.done[1] = w.done[1] > w.issued[1] - in.wait_lgkm ? w.done[1] : w.issued[1] - in.wait_lgkm;
                if (in.wait_vm >= 0 && w.issued[2] >= (uint64_t)in.wait_vm)
                    w.done[2] = w.done[2] > w.issued[2] - in.wait_vm ? w.done[2] : w.issued[2] - in.wait_vm;
                break;
            case I_S_BRANCH: next = in.target; break;
            case I_S_CBRANCH_SCC1: if (w.scc) next = in.target; break;
            case I_S_CBRANCH_SCC0: if (!w.scc) next = in.target; break;
            case I_S_CBRANCH_EXECNZ: if (w.exec) next = in.target; break;
            case I_DS_READ_U8: case I_DS_READ_B64: {
                need_ready(in, o[1]);
                const int nb = in.c == I_DS_READ_U8 ? 1 : 8, nr = in.c == I_DS_READ_U8 ? 1 : 2;
                for (int j = 0; j < nr; ++j) need_ready(in, Opd{K_V, (uint16_t)(o[0].reg + j), 1, 0, ""});
                const uint64_t seq = ++w.issued[1];
                for (int l = 0; l < 64; ++l) {
                    if (!(w.exec >> l & 1)) continue;
                    const uint64_t addr = (uint64_t)w.v[o[1].reg][l] + (uint32_t)in.offset;
                    if (addr + nb > g_lds_launch && g_lds_reads_clamped) {
                        for (int j = 0; j < nr; ++j) w.v[o[0].reg + j][l] = 0;
                        continue;
                    }
                    if (addr + nb > g_lds_launch) {
                        g_cur = lanes[l] ? lanes[l] : g_cur;
                        violation("`%s`: lane %d reads LDS address 0x%llx, the launch has %zu bytes", in.text.c_str(), l,
                                  (unsigned long long)addr, g_lds_launch);
                        for (int j = 0; j < nr; ++j) w.v[o[0].reg + j][l] = 0xBAD0BAD0u;
                        continue;
                    }
                    if (nb == 8 && (addr & 7)) violation("`%s`: lane %d reads 8 bytes at the unaligned LDS address 0x%llx", in.text.c_str(), l, (unsigned long long)addr);
                    order_access((uint64_t)g_lds + addr, nb, false, true);
                    if (nb == 1) {
                        w.v[o[0].reg][l] = g_lds[addr];
                    } else {
                        memcpy(&w.v[o[0].reg][l], g_lds + addr, 4);
                        memcpy(&w.v[o[0].reg + 1][l], g_lds + addr + 4, 4);
                    }
                }
                for (int j = 0; j < nr; ++j) {
                    w.pend_kind[o[0].reg + j] = 1;
                    w.pend_seq[o[0].reg + j] = seq;
                }
                break;
            }
            case I_GLOAD_DWORD: case I_GLOAD_X4: {
                // global_load vdst, voffset, s[base:base+1] offset:N
                need_ready(in, o[1]);
                const int nr = in.c == I_GLOAD_DWORD ? 1 : 4;
                for (int j = 0; j < nr; ++j) need_ready(in, Opd{K_V, (uint16_t)(o[0].reg + j), 1, 0, ""});
                const uint64_t seq = ++w.issued[2];
                const uint64_t base = s64(o[2]);
                for (int l = 0; l < 64; ++l) {
                    if (!(w.exec >> l & 1)) continue;
                    const uint64_t addr = base + w.v[o[1].reg][l] + (int64_t)in.offset;
                    if (!find_alloc(addr, 4 * nr)) {
                        g_cur = lanes[l] ? lanes[l] : g_cur;
                        violation("`%s`: lane %d loads %d bytes at 0x%llx, outside every allocation (%s)", in.text.c_str(), l, 4 * nr,
                                  (unsigned long long)addr, describe_address(addr).c_str());
                        for (int j = 0; j < nr; ++j) w.v[o[0].reg + j][l] = 0xBAD0BAD0u;
                        continue;
                    }
                    if (addr & (nr == 4 ? 15 : 3))
                        violation("`%s`: lane %d loads %d bytes at the unaligned address 0x%llx", in.text.c_str(), l, 4 * nr, (unsigned long long)addr);
                    order_access(addr, 4 * nr, false, true);
                    for (int j = 0; j < nr; ++j) memcpy(&w.v[o[0].reg + j][l], (const void *)(addr + 4 * j), 4);
                }
                for (int j = 0; j < nr; ++j) {
                    w.pend_kind[o[0].reg + j] = 2;
                    w.pend_seq[o[0].reg + j] = seq;
                }
                break;
            }
            case I_GSTORE_BYTE: {
                // global_store_byte voffset, vdata, s[base:base+1]
                need_ready(in, o[0]);
                need_ready(in, o[1]);
                ++w.issued[2];
                const uint64_t base = s64(o[2]);
                for (int l = 0; l < 64; ++l) {
                    if (!(w.exec >> l & 1)) continue;
                    const uint64_t addr = base + w.v[o[0].reg][l] + (int64_t)in.offset;
                    if (!find_alloc(addr, 1)) {
                        g_cur = lanes[l] ? lanes[l] : g_cur;
                        violation("`%s`: lane %d stores a byte at 0x%llx, outside every allocation (%s)", in.text.c_str(), l,
                                  (unsigned long long)addr, describe_address(addr).c_str());
                        continue;
                    }
                    order_access(addr, 1, true, true);
                    *(uint8_t *)addr = (uint8_t)w.v[o[1].reg][l];
                }
                break;
            }
            case I_MFMA: {
                // v_mfma vdst[16], a[4], b[4], c[16]; ignores the execution mask
                for (int k = 0; k < 4; ++k) need_ready(in, o[k]);
                if (o[0].n != 16 || o[1].n != 4 || o[2].n != 4 || o[3].n != 16) {
                    violation("`%s`: operand sizes", in.text.c_str());
                    break;
                }
                static uint16_t a[64][8], b[64][8];
                static float c[64][16];
                for (int l = 0; l < 64; ++l) {
                    for (int j = 0; j < 4; ++j) {
                        memcpy(&a[l][2 * j], &w.v[o[1].reg + j][l], 4);
                        memcpy(&b[l][2 * j], &w.v[o[2].reg + j][l], 4);
                    }
                    for (int j = 0; j < 16; ++j) memcpy(&c[l][j], &w.v[o[3].reg + j][l], 4);
                }
                mfma_compute(a, b, c);
                for (int l = 0; l < 64; ++l)
                    for (int j = 0; j < 16; ++j) memcpy(&w.v[o[0].reg + j][l], &c[l][j], 4);
                break;
            }
            case I_END: break;
        }
        pc = next;
        if (pc < 0 || pc >= (int)p.ins.size()) {
            violation("asm statement: control leaves the statement");
            g_abort_launch = true;
            return;
        }
    }
    if (w.exec != part) violation("asm statement ends with an execution mask other than the one it started with (%016llx, was %016llx)",
                                  (unsigned long long)w.exec, (unsigned long long)part);
    // loads must have been waited for: the compiler knows nothing of them
    for (int r = 0; r < 256; ++r)
        if (!reg_ready(r)) {
            violation("asm statement ends with the load into v%d still in flight", r);
            break;
        }
    // operands out
    for (size_t k = 0; k < p.bind.size(); ++k) {
        const Binding &b = p.bind[k];
        if (!b.written || !b.vector) continue;
        for (int l = 0; l < 64; ++l) {
            if (!(part >> l & 1)) continue;
            const AsmOperand &op = ((const AsmArgs *)lanes[l]->args)->ops[k];
            uint32_t tmp[16];
            for (int j = 0; j < b.nregs; ++j) tmp[j] = w.v[b.reg + j][l];
            memcpy(op.ptr, tmp, op.bytes);
        }
    }
}

// ---- carrying out a meeting ------------------------------------------------------------------------------------
static void exec_collective(Fiber *wave0, int n_lanes) {
    Fiber *lanes[64] = {nullptr};
    uint64_t part = 0;
    int op = 0;
    const void *site = nullptr;
    for (int l = 0; l < n_lanes; ++l) {
        Fiber &f = wave0[l];
        if (f.st != WAIT_WAVE) continue;
        if (!part) {
            op = f.op;
            site = f.site;
        } else if (f.op != op || f.site != site) {
            g_cur = &f;
            violation("lanes of one wavefront wait at different wavefront-wide operations (%d and %d): diverged control flow around one", op, f.op);
            g_abort_launch = true;
            return;
        }
        lanes[l] = &f;
        part |= 1ull << l;
    }
    g_cur = lanes[__builtin_ctzll(part)];
    const uint32_t wave_index = (uint32_t)(wave0 - g_fib) / 64;
    ++g_wave_epoch[wave_index];  // what the lanes did before this operation lies before it for all of them ...
    auto has = [&](int l) { return l >= 0 && l < 64 && (part >> l & 1); };
    switch (op) {
        case OP_SYNC: break;
        case OP_BALLOT: {
            uint64_t m = 0;
            for (int l = 0; l < 64; ++l)
                if (has(l) && ((BallotArgs *)lanes[l]->args)->pred) m |= 1ull << l;
            for (int l = 0; l < 64; ++l)
                if (has(l)) ((BallotArgs *)lanes[l]->args)->out = m;
            break;
        }
        case OP_READLANE: case OP_READFIRST: case OP_SHFL: case OP_SHFL_UP: {
            int vals[64];
            for (int l = 0; l < 64; ++l) vals[l] = has(l) ? ((LaneArgs *)lanes[l]->args)->v : 0;
            for (int l = 0; l < 64; ++l) {
                if (!has(l)) continue;
                LaneArgs *a = (LaneArgs *)lanes[l]->args;
                int src = l;
                if (op == OP_READLANE)
                    src = a->sel & 63;
                else if (op == OP_READFIRST)
                    src = __builtin_ctzll(part);
                else if (op == OP_SHFL)
                    src = (l & ~(a->width - 1)) | (a->sel & (a->width - 1));
                else if ((l & (a->width - 1)) >= a->sel)
                    src = l - a->sel;
                if (op == OP_READLANE && !has(src)) violation("readlane of lane %d, which is not active", src);
                a->out = has(src) ? vals[src] : vals[l];
            }
            break;
        }
        case OP_DPP: {
            int srcv[64];
            for (int l = 0; l < 64; ++l) srcv[l] = has(l) ? ((DppArgs *)lanes[l]->args)->src : 0;
            for (int l = 0; l < 64; ++l) {
                if (!has(l)) continue;
                DppArgs *a = (DppArgs *)lanes[l]->args;
                const int c = a->ctrl, row = l & ~15, i = l & 15;
                int src = -1;
                if (c >= 0 && c <= 0xFF)
                    src = (l & ~3) | ((c >> (2 * (l & 3))) & 3);
                else if (c >= 0x101 && c <= 0x10F)
                    src = i + (c & 15) < 16 ? l + (c & 15) : -1;
                else if (c >= 0x111 && c <= 0x11F)
                    src = i >= (c & 15) ? l - (c & 15) : -1;
                else if (c >= 0x121 && c <= 0x12F)
                    src = row | ((i - (c & 15)) & 15);
                else if (c == 0x140)
                    src = row | (15 - i);
                else if (c == 0x141)
                    src = (l & ~7) | (7 - (l & 7));
                else
                    violation("DPP control 0x%x is not modelled", c);
                const bool enabled = (a->row_mask >> (l / 16) & 1) && (a->bank_mask >> ((l % 16) / 4) & 1);
                if (!enabled)
                    a->out = a->old;
                else if (src >= 0 && has(src))
                    a->out = srcv[src];
                else
                    a->out = a->bound_ctrl ? 0 : a->old;
            }
            break;
        }
        case OP_PERMSWAP: {
            uint32_t av[64], bv[64];
            for (int l = 0; l < 64; ++l) {
                av[l] = has(l) ? ((SwapArgs *)lanes[l]->args)->a : 0;
                bv[l] = has(l) ? ((SwapArgs *)lanes[l]->args)->b : 0;
            }
            const int rows = lanes[__builtin_ctzll(part)] ? ((SwapArgs *)lanes[__builtin_ctzll(part)]->args)->rows : 16;
            uint32_t na[64], nb[64];
            memcpy(na, av, sizeof na);
            memcpy(nb, bv, sizeof nb);
            for (int l = 0; l < 64; ++l) {
                const bool upper = rows == 16 ? ((l / 16) & 1) : l >= 32;  // odd rows / rows 2 and 3 of the first operand ...
                if (!upper) continue;
                na[l] = bv[l - rows];  // ... change places with even rows / rows 0 and 1 of the second
                nb[l - rows] = av[l];
            }
            if (part != ~0ull) violation("lane swap with inactive lanes");
            for (int l = 0; l < 64; ++l)
                if (has(l)) {
                    ((SwapArgs *)lanes[l]->args)->out_a = na[l];
                    ((SwapArgs *)lanes[l]->args)->out_b = nb[l];
                }
            break;
        }
        case OP_MFMA: {
            static uint16_t a[64][8], b[64][8];
            static float c[64][16];
            memset(a, 0, sizeof a);
            memset(b, 0, sizeof b);
            memset(c, 0, sizeof c);
            if (part != ~0ull) violation("matrix instruction with inactive lanes (it reads every lane's registers)");
            for (int l = 0; l < 64; ++l) {
                if (!has(l)) continue;
                MfmaArgs *m = (MfmaArgs *)lanes[l]->args;
                memcpy(a[l], m->a, 16);
                memcpy(b[l], m->b, 16);
                memcpy(c[l], m->c, 64);
            }
            mfma_compute(a, b, c);
            for (int l = 0; l < 64; ++l)
                if (has(l)) memcpy(((MfmaArgs *)lanes[l]->args)->c, c[l], 64);
            break;
        }
        case OP_ASM: exec_asm(lanes, n_lanes, part); break;
        default: violation("unknown wavefront-wide operation %d", op); break;
    }
    ++g_wave_epoch[wave_index];  // ... and what they do next after it
    for (int l = 0; l < 64; ++l)
        if (has(l)) lanes[l]->st = RUN;
}

static bool run_workgroup(uint32_t nthreads, const LaneCtx &proto) {
    for (uint32_t t = 0; t < nthreads; ++t) {
        fiber_reset(g_fib[t], (int)t);
        g_fib[t].ctx = proto;
        g_fib[t].ctx.thread_idx = Dim3(t, 0, 0);
    }
    memset(g_lds, 0xCD, g_lds_open);
    const uint32_t n_waves = (nthreads + 63) / 64;
    g_wg_index = (proto.block_idx.z * proto.grid_dim.y + proto.block_idx.y) * proto.grid_dim.x + proto.block_idx.x;
    order_start_workgroup(n_waves, g_lds_open);
    uint32_t order[kMaxThreads / 64];
    for (uint32_t i = 0; i < n_waves; ++i) order[i] = i;
    for (;;) {
        bool progress = false;
        uint32_t live = 0, at_wg = 0;
        if (g_schedule)  // another order of the wavefronts every round: the kernels must not depend on it
            for (uint32_t i = n_waves; i > 1; --i) {
                g_schedule ^= g_schedule << 13;
                g_schedule ^= g_schedule >> 7;
                g_schedule ^= g_schedule << 17;
                const uint32_t j = (uint32_t)(g_schedule % i), t = order[i - 1];
                order[i - 1] = order[j];
                order[j] = t;
            }
        for (uint32_t wi = 0; wi < n_waves; ++wi) {
            const uint32_t wv = order[wi];
            const uint32_t lo = wv * 64, hi = lo + 64 < nthreads ? lo + 64 : nthreads;
            uint32_t live_w = 0, wait_wave = 0, wait_wg = 0, catching_up = 0, spinning = 0;
            for (uint32_t t = lo; t < hi; ++t) {
                Fiber &f = g_fib[t];
                if (f.st == RUN) {
                    f.yielded = false;
                    g_cur = &f;
                    sim_switch(&g_sched_sp, f.sp);
                    g_cur = nullptr;
                    if (!f.yielded) progress = true;
                    if (g_abort_launch) return false;
                }
                if (f.st != DONE) ++live_w;
                if (f.st == WAIT_WAVE && f.op == OP_CATCHUP)
                    ++catching_up;
                else if (f.st == WAIT_WAVE)
                    ++wait_wave;
                if (f.st == WAIT_WG) ++wait_wg;
                if (f.st == RUN && f.yielded) ++spinning;  // (in a wait loop: it has got as far as it can, too)
            }
            if (catching_up && catching_up + wait_wave + wait_wg + spinning == live_w) {
                // everybody else of the wavefront has got as far as it can: the lanes that waited for that go on
                for (uint32_t t = lo; t < hi; ++t)
                    if (g_fib[t].st == WAIT_WAVE && g_fib[t].op == OP_CATCHUP) g_fib[t].st = RUN;
                ++g_wave_epoch[wv];
                progress = true;
            } else if (wait_wave && wait_wave + wait_wg == live_w) {
                exec_collective(&g_fib[lo], (int)(hi - lo));
                g_cur = nullptr;
                if (g_abort_launch) return false;
                progress = true;
            }
            live += live_w;
            at_wg += wait_wg;
        }
        if (live == 0) return true;
        if (at_wg == live) {
            uint32_t at_barrier = 0;  // the wavefronts that wait at it (one that has ended takes no part)
            for (uint32_t t = 0; t < nthreads; ++t)
                if (g_fib[t].st == WAIT_WG) {
                    g_fib[t].st = RUN;
                    at_barrier |= 1u << (t / 64);
                }
            order_barrier(at_barrier);
            for (uint32_t w = 0; w < n_waves; ++w) ++g_wave_epoch[w];
            progress = true;
        }
        if (!progress) {
            // nothing moved in a whole round: whoever still runs is spinning on a value nobody will write
            uint32_t spinning = 0, first = 0;
            for (uint32_t t = nthreads; t-- > 0;)
                if (g_fib[t].st == RUN) {
                    ++spinning;
                    first = t;
                }
            g_cur = &g_fib[first];
            violation("the workgroup cannot go on: %u threads alive, %u at the workgroup barrier, %u spinning (first: thread %u)", live,
                      at_wg, spinning, first);
            g_cur = nullptr;
            return false;
        }
    }
}

static std::map<const void *, int> g_dynamic_lds_allowed;
void allow_dynamic_lds(const void *fn, int bytes) { g_dynamic_lds_allowed[fn] = bytes; }

void launch(const char *name, const void *fn, Dim3 grid, Dim3 block, size_t shmem, const std::function<void()> &body) {
    sim_init();
    g_launches.push_back(name);
    if (const char *log = getenv("CI_HOSTMODEL_LAUNCH_LOG")) {  // every launch of a test run, for a look at which kernels it reaches
        if (FILE *f = fopen(log, "a")) {
            fprintf(f, "%s\n", name);
            fclose(f);
        }
    }
    const uint32_t nthreads = block.x * block.y * block.z;
    g_kernel = name;
    if (shmem > 65536) {
        const auto it = g_dynamic_lds_allowed.find(fn);
        if (it == g_dynamic_lds_allowed.end() || (size_t)it->second < shmem) {
            violation("launch with %zu bytes of dynamic LDS, and hipFuncSetAttribute(MaxDynamicSharedMemorySize) allowed this kernel %d: "
                      "the GPU runtime refuses such a launch", shmem, it == g_dynamic_lds_allowed.end() ? 65536 : it->second);
            g_launch_error = 719;
            g_kernel = "(no kernel)";
            return;
        }
    }
    if (nthreads == 0 || nthreads > kMaxThreads || block.y != 1 || block.z != 1 || shmem > kLdsBytes ||
        (uint64_t)grid.x * grid.y * grid.z == 0) {
        violation("launch configuration: grid (%u,%u,%u) block (%u,%u,%u) LDS %zu", grid.x, grid.y, grid.z, block.x, block.y, block.z, shmem);
        return;
    }
    g_body = &body;
    // kernels with static LDS arrays get them as ordinary statics; only dynamic LDS is bounded for the interpreter
    g_lds_launch = shmem;
    // ... and for plain C++ accesses, to the page: what lies behind the launch's dynamic LDS is inaccessible while it runs
    g_lds_open = (shmem + 4095) & ~(size_t)4095;
    if (g_lds_open < kLdsBytes) mprotect(g_lds + g_lds_open, kLdsBytes - g_lds_open, PROT_NONE);
    g_abort_launch = false;
    ++g_launch_seq;
    g_order_reports = 0;
    LaneCtx proto;
    proto.block_dim = block;
    proto.grid_dim = grid;
    for (uint32_t z = 0; z < grid.z && !g_abort_launch; ++z)
        for (uint32_t y = 0; y < grid.y && !g_abort_launch; ++y)
            for (uint32_t x = 0; x < grid.x && !g_abort_launch; ++x) {
                proto.block_idx = Dim3(x, y, z);
                if (!run_workgroup(nthreads, proto)) g_abort_launch = true;
            }
    mprotect(g_lds, kLdsBytes, PROT_READ | PROT_WRITE);
    g_lds_open = kLdsBytes;
    g_cur = nullptr;
    g_body = nullptr;
    g_kernel = "(no kernel)";
}

int take_launch_error() {
    const int e = g_launch_error;
    g_launch_error = 0;
    return e;
}
int cu_count() { return g_cus; }

static void on_segv(int sig, siginfo_t *info, void *uc) {
    // (async-signal-unsafe calls: the process is about to end anyway)
    const uint64_t addr = (uint64_t)info->si_addr;
    if (sig == SIGILL) {
        // a build of the kernel sources with the compiler's undefined-behaviour checks in trap mode ends here
        Dl_info dl;
        const void *pc = (const void *)((ucontext_t *)uc)->uc_mcontext.gregs[REG_RIP];
        const bool known = dladdr(pc, &dl) != 0;
        fprintf(stderr, "host model: illegal instruction %s at %s+0x%llx (%s)\n", where().c_str(), known ? dl.dli_fname : "?",
                (unsigned long long)((uint64_t)pc - (known ? (uint64_t)dl.dli_fbase : 0)), known && dl.dli_sname ? dl.dli_sname : "?");
        fflush(stderr);
        _exit(71);
    }
    fprintf(stderr, "host model: memory fault at %p %s: %s\n", info->si_addr, where().c_str(),
            addr >= (uint64_t)g_lds && addr < (uint64_t)g_lds + kLdsBytes + 4096 ? "in the LDS area, past the end of this launch's dynamic LDS" : describe_address(addr).c_str());
    fflush(stderr);
    _exit(70);
}

}  // namespace sim

using namespace sim;

extern "C" void sim_init(void) {
    static bool done = false;
    if (done) return;
    done = true;
    map_lds();
    g_stacks = (uint8_t *)mmap(nullptr, (size_t)kMaxThreads * kStackBytes, PROT_READ | PROT_WRITE,
                               MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (g_stacks == MAP_FAILED) abort();
    static uint8_t alt[65536];
    stack_t ss;
    ss.ss_sp = alt;
    ss.ss_size = sizeof alt;
    ss.ss_flags = 0;
    sigaltstack(&ss, nullptr);
    struct sigaction sa;
    memset(&sa, 0, sizeof sa);
    sa.sa_sigaction = on_segv;
    sa.sa_flags = SA_SIGINFO | SA_ONSTACK;
    sigaction(SIGSEGV, &sa, nullptr);
    sigaction(SIGBUS, &sa, nullptr);
    sigaction(SIGILL, &sa, nullptr);
}

extern "C" void *sim_alloc(size_t bytes, int end_at_guard) {
    const size_t page = 4096, body = (bytes + 15) & ~(size_t)15, pages = (body + page - 1) / page + (body == 0);
    const size_t total = (pages + 2) * page;
    uint8_t *map = (uint8_t *)mmap(nullptr, total, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
    if (map == MAP_FAILED) return nullptr;
    mprotect(map + page, pages * page, PROT_READ | PROT_WRITE);
    memset(map + page, 0xA5, pages * page);
    uint8_t *ptr = end_at_guard ? map + page + pages * page - body : map + page;
    g_allocs.push_back(Alloc{map, total, ptr, bytes});
    return ptr;
}

extern "C" void sim_free_all(void) {
    for (Alloc &a : g_allocs) munmap(a.map, a.map_bytes);
    g_allocs.clear();
    g_global_shadow.clear();
}

extern "C" void sim_set_cus(int n) { g_cus = n > 0 ? n : 1; }
extern "C" void sim_set_schedule(uint64_t seed) { g_schedule = seed; }
extern "C" void sim_trust_foreign_memory(int on) { g_any_memory = on != 0; }
extern "C" void sim_lds_reads_out_of_range_give_zero(int on) { g_lds_reads_clamped = on != 0; }
extern "C" int sim_violation_count(void) { return (int)g_viol.size(); }
extern "C" const char *sim_violation(int i) { return i >= 0 && i < (int)g_viol.size() ? g_viol[i].c_str() : ""; }
extern "C" void sim_clear(void) {
    g_viol.clear();
    g_launches.clear();
    g_launch_error = 0;
    g_asm_instructions = 0;
}
extern "C" int sim_launch_count(void) { return (int)g_launches.size(); }
extern "C" const char *sim_launch_name(int i) { return i >= 0 && i < (int)g_launches.size() ? g_launches[i].c_str() : ""; }
extern "C" uint64_t sim_asm_instructions(void) { return g_asm_instructions; }

// ---- the compiler's hooks (thread-sanitizer instrumentation of the kernel sources; see "ordering" above) -----------
// Only the instrumented build calls these; __tsan_init, which every instrumented object calls when the library is
// loaded, is what switches the ordering check on.
extern "C" {
void __tsan_init(void) { g_order_on = true; }
void __tsan_func_entry(void *) {}
void __tsan_func_exit(void) {}
void __tsan_vptr_update(void **, void *) {}
void __tsan_vptr_read(void **) {}
#define CI_SIM_HOOK(n)                                                                          \
    void __tsan_read##n(void *p) { order_access((uint64_t)p, n, false); }                       \
    void __tsan_write##n(void *p) { order_access((uint64_t)p, n, true); }                       \
    void __tsan_unaligned_read##n(void *p) { order_access((uint64_t)p, n, false); }             \
    void __tsan_unaligned_write##n(void *p) { order_access((uint64_t)p, n, true); }             \
    void __tsan_volatile_read##n(void *p) { order_access((uint64_t)p, n, false); }              \
    void __tsan_volatile_write##n(void *p) { order_access((uint64_t)p, n, true); }              \
    void __tsan_unaligned_volatile_read##n(void *p) { order_access((uint64_t)p, n, false); }    \
    void __tsan_unaligned_volatile_write##n(void *p) { order_access((uint64_t)p, n, true); }    \
    void __tsan_read_write##n(void *p) { order_access((uint64_t)p, n, true); }                  \
    void __tsan_unaligned_read_write##n(void *p) { order_access((uint64_t)p, n, true); }
CI_SIM_HOOK(1)
CI_SIM_HOOK(2)
CI_SIM_HOOK(4)
CI_SIM_HOOK(8)
CI_SIM_HOOK(16)
#undef CI_SIM_HOOK
void __tsan_read_range(void *p, unsigned long n) { order_access((uint64_t)p, n, false); }
void __tsan_write_range(void *p, unsigned long n) { order_access((uint64_t)p, n, true); }
// (called by host code these are the stand-ins of hipMemsetAsync / hipMemcpyAsync: what they write is written)
void *__tsan_memcpy(void *d, const void *s, unsigned long n) {
    if (!g_cur && g_order_on && n) mark_written((uint64_t)d, n);
    order_access((uint64_t)s, n, false);
    order_access((uint64_t)d, n, true);
    return memcpy(d, s, n);
}
void *__tsan_memmove(void *d, const void *s, unsigned long n) {
    if (!g_cur && g_order_on && n) mark_written((uint64_t)d, n);
    order_access((uint64_t)s, n, false);
    order_access((uint64_t)d, n, true);
    return memmove(d, s, n);
}
void *__tsan_memset(void *d, int v, unsigned long n) {
    if (!g_cur && g_order_on && n) mark_written((uint64_t)d, n);
    order_access((uint64_t)d, n, true);
    return memset(d, v, n);
}
// std::atomic in the host code of the sources (process-wide switches): carried out, nothing to check
#define CI_SIM_ATOMIC(bits, T)                                                                                       \
    T __tsan_atomic##bits##_load(const volatile T *p, int) { return __atomic_load_n(p, __ATOMIC_SEQ_CST); }          \
    void __tsan_atomic##bits##_store(volatile T *p, T v, int) { __atomic_store_n(p, v, __ATOMIC_SEQ_CST); }          \
    T __tsan_atomic##bits##_exchange(volatile T *p, T v, int) { return __atomic_exchange_n(p, v, __ATOMIC_SEQ_CST); } \
    T __tsan_atomic##bits##_fetch_add(volatile T *p, T v, int) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); } \
    T __tsan_atomic##bits##_fetch_sub(volatile T *p, T v, int) { return __atomic_fetch_sub(p, v, __ATOMIC_SEQ_CST); } \
    T __tsan_atomic##bits##_fetch_and(volatile T *p, T v, int) { return __atomic_fetch_and(p, v, __ATOMIC_SEQ_CST); } \
    T __tsan_atomic##bits##_fetch_or(volatile T *p, T v, int) { return __atomic_fetch_or(p, v, __ATOMIC_SEQ_CST); }   \
    T __tsan_atomic##bits##_fetch_xor(volatile T *p, T v, int) { return __atomic_fetch_xor(p, v, __ATOMIC_SEQ_CST); } \
    int __tsan_atomic##bits##_compare_exchange_strong(volatile T *p, T *e, T v, int, int) {                          \
        return __atomic_compare_exchange_n(p, e, v, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST);                      \
    }                                                                                                                \
    int __tsan_atomic##bits##_compare_exchange_weak(volatile T *p, T *e, T v, int, int) {                            \
        return __atomic_compare_exchange_n(p, e, v, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST);                      \
    }
CI_SIM_ATOMIC(8, uint8_t)
CI_SIM_ATOMIC(16, uint16_t)
CI_SIM_ATOMIC(32, uint32_t)
CI_SIM_ATOMIC(64, uint64_t)
#undef CI_SIM_ATOMIC
void __tsan_atomic_thread_fence(int) {}
void __tsan_atomic_signal_fence(int) {}
int sim_checks_ordering(void) { return g_order_on ? 1 : 0; }
void sim_mark_written(const void *p, size_t n) {
    if (g_order_on && n) mark_written((uint64_t)p, n);
}
void sim_check_unwritten_reads(int on) { g_check_unwritten = on != 0; }
}

// ---- the compiler's undefined-behaviour checks (build.py, `undefined=True`) ----------------------------------------------
// That build compiles the kernel sources with -fsanitize=bounds,shift,alignment,... and no sanitizer runtime: the
// calls the checks make come here and become violations with the source position the compiler recorded.  One kind
// is let through: an offset added to a null pointer (`a.ckpt + ...` where a weight has no checkpoints and the pointer
// is never read).  It is undefined in C++ and harmless in these kernels: no null test follows that the compiler could
// drop on the strength of it.
extern "C" {
struct CiSimUbLocation {
    const char *file;
    uint32_t line, column;
};
static void ub_report(const char *kind, const void *data, uint64_t a, uint64_t b) {
    const CiSimUbLocation *l = (const CiSimUbLocation *)data;
    violation("undefined behaviour: %s at %s:%u:%u (values 0x%llx, 0x%llx)", kind, l && l->file ? l->file : "?", l ? l->line : 0,
              l ? l->column : 0, (unsigned long long)a, (unsigned long long)b);
}
#define CI_SIM_UB(name)                                                                                 \
    void __ubsan_handle_##name(void *d, uint64_t a, uint64_t b) { ub_report(#name, d, a, b); }         \
    void __ubsan_handle_##name##_abort(void *d, uint64_t a, uint64_t b) { ub_report(#name, d, a, b); }
CI_SIM_UB(type_mismatch_v1)  // (null pointers and misaligned accesses)
CI_SIM_UB(shift_out_of_bounds)
CI_SIM_UB(add_overflow)
CI_SIM_UB(sub_overflow)
CI_SIM_UB(mul_overflow)
CI_SIM_UB(negate_overflow)
CI_SIM_UB(divrem_overflow)
CI_SIM_UB(builtin_unreachable)
CI_SIM_UB(missing_return)
CI_SIM_UB(vla_bound_not_positive)
CI_SIM_UB(load_invalid_value)
CI_SIM_UB(invalid_builtin)
#undef CI_SIM_UB
// An index past an array of known size: the compiler treats what follows as unreachable, so the process cannot go on.
void __ubsan_handle_out_of_bounds(void *d, uint64_t index) {
    const CiSimUbLocation *l = (const CiSimUbLocation *)d;
    fprintf(stderr, "host model: %sundefined behaviour: out_of_bounds at %s:%u:%u (index %llu)\n", where().c_str(), l->file ? l->file : "?",
            l->line, l->column, (unsigned long long)index);
    fflush(stderr);
    _exit(72);
}
void __ubsan_handle_out_of_bounds_abort(void *d, uint64_t index) { __ubsan_handle_out_of_bounds(d, index); }
void __ubsan_handle_pointer_overflow(void *d, uint64_t base, uint64_t result) {
    // (base below 4 GB: null, or null plus an earlier offset of the same expression; no array of the model lives there)
    if (base >> 32) ub_report("pointer_overflow", d, base, result);
}
void __ubsan_handle_pointer_overflow_abort(void *d, uint64_t base, uint64_t result) { __ubsan_handle_pointer_overflow(d, base, result); }
}
