// Host model of a gfx950 workgroup, for running the library's kernels on the CPU with checked memory.
//
//   * every thread of a workgroup is a fibre; a wavefront-wide operation (ballot, readlane, DPP, lane swaps,
//     shuffles, the matrix instruction, an assembly statement) is carried out when all the lanes of the wavefront
//     that are still alive wait at it, a workgroup barrier when all threads wait at it;
//   * `asm volatile` statements are run by an interpreter of the instructions they are made of (tests/hostmodel/
//     sim.cpp), on the 64 lanes at once, with an execution mask, SCC, VCC, and the counters of outstanding loads
//     (a register read before the s_waitcnt that covers its load is reported);
//   * LDS is one 160 KB area at an address whose low 32 bits are zero, so that an LDS pointer's low half is its
//     LDS address as on the GPU; accesses of the interpreter are checked against the launch's LDS size;
//   * global memory comes from sim_alloc: each allocation ends (or starts) at an inaccessible page, and the
//     interpreter checks every address it forms against the exact extent of the allocations.
//   * two more builds of the same sources take the calls of compiler instrumentation instead of a sanitizer runtime
//     (build.py): with every plain memory access reported, the model checks that two wavefronts never touch the same
//     byte without a barrier or a release / acquire pair between them, and that no kernel reads a byte of an array that
//     nothing has written; with the undefined-behaviour checks compiled in, what they report is a violation.
//
// Test infrastructure only.
#pragma once
#include <stddef.h>
#include <stdint.h>

#include <functional>

namespace sim {

struct Dim3 {
    uint32_t x, y, z;
    Dim3(uint32_t x_ = 1, uint32_t y_ = 1, uint32_t z_ = 1) : x(x_), y(y_), z(z_) {}
};

struct LaneCtx {
    Dim3 thread_idx, block_idx, block_dim, grid_dim;
};
const LaneCtx &lane_ctx();

typedef uint32_t u32x2v __attribute__((ext_vector_type(2)));

// wavefront-wide operations (each is a meeting point of the wavefront's live lanes)
uint64_t ballot(int pred);
int readlane(int v, int lane);
int readfirstlane(int v);
int update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl);
u32x2v permlane_swap(uint32_t a, uint32_t b, int rows);
int shfl(int v, int src, int width);
int shfl_up(int v, unsigned delta, int width);
void wave_sync();
void wave_catch_up();  // this lane waits until the other lanes of its wavefront have reached their next meeting point
void syncthreads();
void yield();
void mfma_impl(const void *a, const void *b, void *c);
template <typename A, typename C>
inline C mfma_32x32x16_bf16(A a, A b, C c) {
    static_assert(sizeof(A) == 16 && sizeof(C) == 64, "operands of v_mfma_f32_32x32x16_bf16");
    mfma_impl(&a, &b, &c);
    return c;
}
uint32_t v_perm(uint32_t s0, uint32_t s1, uint32_t sel);  // v_perm_b32 (no meeting point)

// The ordering check of the instrumented build (sim.cpp, "ordering between wavefronts"): an atomic access of kernel
// code, and a `__shared__` array of a kernel (a static in this build) made known as shared memory of the workgroup.
void order_atomic(const void *p, bool acquire, bool release);
void shared_static(const void *p, size_t bytes);

// assembly statements
struct AsmOperand {
    const char *name;        // symbolic name, or "" for a positional operand
    const char *constraint;  // "+v", "=&v", "v", "s"
    void *ptr;               // this lane's value
    uint32_t bytes;
};
void run_asm(const char *tmpl, AsmOperand *ops, int n_ops);

// launches
// `fn` = the kernel's address, the key under which allow_dynamic_lds recorded what hipFuncSetAttribute was given: a launch
// that asks for more than 64 KB of dynamic LDS without it fails on the GPU, and is a violation here.
void launch(const char *name, const void *fn, Dim3 grid, Dim3 block, size_t shmem, const std::function<void()> &body);
void allow_dynamic_lds(const void *fn, int bytes);
int take_launch_error();
int cu_count();
uint8_t *lds_base();
void *register_symbol(void *p, size_t bytes);

}  // namespace sim

extern "C" {
void sim_init(void);
void *sim_alloc(size_t bytes, int end_at_guard);  // end_at_guard: 1 = the byte after the array is inaccessible, 0 = the byte before
void sim_free_all(void);
void sim_set_cus(int n);
void sim_set_schedule(uint64_t seed);  // 0: wavefronts of a workgroup run in index order; else the seed of a new order every round
void sim_trust_foreign_memory(int on);  // 1: the interpreter also accepts addresses outside sim_alloc's arrays (a caller's own memory)
// 1: an LDS read of an assembly statement beyond the launch's LDS gives 0 and is no violation.  That is what the hardware does
// (out-of-range LDS reads return zero, writes are dropped), and it is the wrong setting for every test but one: on inputs an
// encoder wrote no kernel forms such an address, and one that does has a defect.  For inputs that are damaged on purpose.
void sim_lds_reads_out_of_range_give_zero(int on);
int sim_violation_count(void);
const char *sim_violation(int i);
void sim_clear(void);  // violations and the launch log
int sim_launch_count(void);
const char *sim_launch_name(int i);
uint64_t sim_asm_instructions(void);  // instructions the interpreter has run since sim_clear
int sim_checks_ordering(void);  // 1 in the build with instrumented memory accesses: unordered accesses of two wavefronts are violations
// In that build a kernel's read of a byte of a sim_alloc array that nothing has written is a violation too: an upload
// says what it wrote with sim_mark_written; sim_check_unwritten_reads(0) switches the check off.
void sim_mark_written(const void *p, size_t n);
void sim_check_unwritten_reads(int on);
}
