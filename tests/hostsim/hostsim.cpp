// Runtime of the host simulation (see hip/hip_runtime.h in this directory): workgroups in order, lanes as fibers.
#include <sys/mman.h>

#include "hip/hip_runtime.h"

namespace hostsim {

Idx g_thread, g_block;
dim3 g_block_dim, g_grid_dim;
constexpr int MAX_LANES = 1024;
constexpr size_t STACK_BYTES = 256 * 1024;
uint64_t g_exchange[MAX_LANES];
unsigned char g_alive[MAX_LANES];
// The LDS lives below 4 GB: the kernels keep LDS addresses as 32-bit values (as the hardware does) and the
// stand-in for the LDS-DMA load turns them back into pointers.
constexpr size_t LDS_BYTES = 160 * 1024;
static unsigned char* map_lds() {
    for (uintptr_t at = 0x40000000u; at < 0xF0000000u; at += 0x10000000u) {
        void* p = mmap((void*)at, LDS_BYTES + 4096, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_FIXED_NOREPLACE, -1, 0);
        if (p == (void*)at) {
            mprotect((unsigned char*)p + LDS_BYTES, 4096, PROT_NONE);     // the page after the LDS
            return (unsigned char*)p;
        }
        if (p != MAP_FAILED) munmap(p, LDS_BYTES + 4096);
    }
    fprintf(stderr, "hostsim: no room below 4 GB for the LDS\n");
    abort();
}
static unsigned char* const g_lds_region = map_lds();
// The dynamic LDS of a launch ENDS where the region ends (16-byte aligned start, all the hardware promises),
// so an access past the size the launch asked for hits the protected page; it starts every workgroup with
// all bits set (NaN / -1), as unpredictable as what the previous workgroup left on the hardware.
unsigned char* g_dynamic_lds = g_lds_region;
static float g_wave_store[MAX_LANES / 64][64][16];
float (*g_wave_f32)[64][16] = g_wave_store;

// Fiber switch: the callee-saved registers go on the old stack, the stack pointers are exchanged
// (swapcontext would make a signal-mask system call per switch, and a GEMM tile makes millions).
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
    .size hostsim_switch, .-hostsim_switch
)");
static void* g_scheduler_sp = nullptr;
static void* g_lane_sp[MAX_LANES];
static char* g_stacks = nullptr;
static Idx g_lane_idx[MAX_LANES];
static int g_current = 0, g_lanes = 0;
static const std::function<void()>* g_body = nullptr;
static unsigned g_alive_block = 0, g_arrived_block = 0, g_generation_block = 0;
static unsigned g_alive_wave[MAX_LANES / 64], g_arrived_wave[MAX_LANES / 64], g_generation_wave[MAX_LANES / 64];
static unsigned long g_progress = 0;

unsigned flat_thread() { return (unsigned)g_current; }
PendingDma g_dma[MAX_LANES][kMaxPendingDma];
int g_dma_first[MAX_LANES], g_dma_count[MAX_LANES];
int g_dma_eager = 0;
static int g_reverse_schedule = 0;

static void yield() { hostsim_switch(&g_lane_sp[g_current], g_scheduler_sp); }

void sync_threads() {
    const unsigned gen = g_generation_block;
    if (++g_arrived_block >= g_alive_block) {
        g_arrived_block = 0;
        ++g_generation_block;
        ++g_progress;
        return;
    }
    while (g_generation_block == gen) yield();
}

void sync_wave() {
    const int w = g_current >> 6;
    const unsigned gen = g_generation_wave[w];
    if (++g_arrived_wave[w] >= g_alive_wave[w]) {
        g_arrived_wave[w] = 0;
        ++g_generation_wave[w];
        ++g_progress;
        return;
    }
    while (g_generation_wave[w] == gen) yield();
}

static void lane_main() {
    (*g_body)();
    // a lane that returns no longer takes part in barriers; one that was the last awaited releases them
    const int w = g_current >> 6;
    g_alive[g_current] = 0;
    ++g_progress;
    if (--g_alive_block > 0 && g_arrived_block >= g_alive_block) { g_arrived_block = 0; ++g_generation_block; }
    if (--g_alive_wave[w] > 0 && g_arrived_wave[w] >= g_alive_wave[w]) { g_arrived_wave[w] = 0; ++g_generation_wave[w]; }
    hostsim_switch(&g_lane_sp[g_current], g_scheduler_sp);
    abort();        // a finished lane is never resumed
}

void launch(dim3 grid, dim3 block, size_t lds_bytes, const std::function<void()>& body) {
    const int lanes = (int)(block.x * block.y * block.z);
    if (lanes <= 0 || lanes > MAX_LANES) { fprintf(stderr, "hostsim: workgroup of %d lanes\n", lanes); abort(); }
    if (lds_bytes > LDS_BYTES) { fprintf(stderr, "hostsim: %zu bytes of dynamic LDS\n", lds_bytes); abort(); }
    if ((uint64_t)grid.x * grid.y * grid.z == 0) { fprintf(stderr, "hostsim: empty grid\n"); abort(); }
    if (!g_stacks) {
        g_stacks = (char*)mmap(nullptr, STACK_BYTES * MAX_LANES, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
        if (g_stacks == (char*)MAP_FAILED) { perror("hostsim: mmap"); abort(); }
    }
    g_dynamic_lds = g_lds_region + LDS_BYTES - (lds_bytes + 15) / 16 * 16;
    g_body = &body;
    g_block_dim = block;
    g_grid_dim = grid;
    g_lanes = lanes;
    for (unsigned bz = 0; bz < grid.z; ++bz)
        for (unsigned by = 0; by < grid.y; ++by)
            for (unsigned bx = 0; bx < grid.x; ++bx) {
                g_block = Idx{bx, by, bz};
                if (lds_bytes) memset(g_dynamic_lds, 0xFF, lds_bytes);
                g_alive_block = (unsigned)lanes;
                g_arrived_block = 0;
                for (int w = 0; w < MAX_LANES / 64; ++w) { g_alive_wave[w] = 0; g_arrived_wave[w] = 0; }
                for (int i = 0; i < lanes; ++i) {
                    g_lane_idx[i] = Idx{(unsigned)i % block.x, ((unsigned)i / block.x) % block.y, (unsigned)i / (block.x * block.y)};
                    g_alive[i] = 1;
                    g_dma_first[i] = g_dma_count[i] = 0;
                    ++g_alive_wave[i >> 6];
                    // a fresh stack that hostsim_switch can "return" into: six saved registers, then lane_main as the
                    // return address, at the alignment a called function expects
                    void** top = reinterpret_cast<void**>(g_stacks + (size_t)(i + 1) * STACK_BYTES);
                    *--top = nullptr;
                    *--top = reinterpret_cast<void*>(&lane_main);
                    for (int r = 0; r < 6; ++r) *--top = nullptr;
                    g_lane_sp[i] = top;
                }
                unsigned left = (unsigned)lanes;
                while (left > 0) {
                    const unsigned long before = g_progress;
                    left = 0;
                    for (int slot = 0; slot < lanes; ++slot) {
                        const int i = g_reverse_schedule ? lanes - 1 - slot : slot;
                        if (!g_alive[i]) continue;
                        g_current = i;
                        g_thread = g_lane_idx[i];
                        hostsim_switch(&g_scheduler_sp, g_lane_sp[i]);
                        left += g_alive[i];
                    }
                    if (left > 0 && g_progress == before) {
                        fprintf(stderr, "hostsim: workgroup (%u,%u,%u) is stuck: %u lanes wait at a barrier that the others never reach\n",
                                bx, by, bz, left);
                        abort();
                    }
                }
            }
    g_body = nullptr;
}

}  // namespace hostsim

// 0 (default): LDS loads land as late as their counted waits allow; 1: at their issue.
extern "C" void hostsim_set_dma_eager(int eager) { hostsim::g_dma_eager = eager; }

// Between two barriers the lanes of a workgroup run one after another: in ascending order (0, default) or
// in descending order (1).  A value that one wave writes to LDS and another reads with no barrier in
// between is read before it is written in one of the two orders.
extern "C" void hostsim_set_reverse_schedule(int reverse) { hostsim::g_reverse_schedule = reverse; }
