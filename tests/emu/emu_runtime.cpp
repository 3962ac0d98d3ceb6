// Scheduler of the host stand-in for the HIP runtime (hip/hip_runtime.h beside this file): fibers for the threads of
// the resident work-groups, wave-wide execution of the operations that involve other lanes.  Test infrastructure.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <sys/mman.h>

#include <map>
#include <vector>

extern "C" void emu_switch(void** save_sp, void* load_sp);
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
.size emu_switch, .-emu_switch
)");

namespace emu {

constexpr size_t kStackBytes = 512u << 10;   // the lowest words hold a pattern that is checked when the lane ends
constexpr uint64_t kCanary = 0x5afe57ac5afe57acull;
constexpr size_t kLdsBytes = 160u << 10;

struct Block {
    std::vector<Lane> lanes;
    dim3 idx;
    uint8_t* lds;
    uint8_t* stacks;
    size_t lds_used;
    uint32_t held, hold_left;
    std::map<const void*, void*> sites;
    uint32_t live;
};

struct Config {
    int order = 0;        // 0 ascending, 1 descending, n > 1: shuffled with seed n
    int lazy_loads = 1;   // LDS-direct loads land at the wait (1) or when issued (0)
    int resident = 64;    // work-groups in flight at a time
    bool fixed = false;   // no further work-group is started for lanes that poll (a launch with more work-groups
                          // than the device keeps resident: what its bounded waits are for)
};

static Config g_config;
static bool g_polling;   // some lane sleeps in a polling loop: what it waits for may be a work-group not yet started
static uint64_t g_counts[OP_KINDS], g_partial[OP_KINDS];
static hipError_t g_error = hipSuccess;
static char g_message[256];

Lane* cur = nullptr;
static void* g_scheduler_sp;
static const std::function<void()>* g_body;
static dim3 g_grid, g_block_dim;

dim3 thread_idx() {
    const uint32_t t = cur->tid;
    return dim3(t % g_block_dim.x, t / g_block_dim.x % g_block_dim.y, t / (g_block_dim.x * g_block_dim.y));
}
dim3 block_idx() { return cur->block->idx; }
dim3 block_dim() { return g_block_dim; }
dim3 grid_dim() { return g_grid; }

hipError_t last_error() {
    const hipError_t e = g_error;
    g_error = hipSuccess;
    return e;
}

static void fail(const char* what) {
    if (g_error == hipSuccess) snprintf(g_message, sizeof g_message, "%s", what);
    g_error = hipErrorLaunchFailure;
}

void wait(int op) {
    Lane* l = cur;
    l->op = op;
    emu_switch(&l->sp, g_scheduler_sp);
}

void* lds_alloc(const void* site, size_t bytes, size_t align) {
    Block* b = cur->block;
    auto it = b->sites.find(site);
    if (it != b->sites.end()) return it->second;
    size_t at = (b->lds_used + align - 1) / align * align;
    if (at + bytes > kLdsBytes) {
        fail("work-group asks for more than 160 KiB of LDS");
        at = 0;
    }
    b->lds_used = at + bytes;
    void* p = b->lds + at;
    b->sites[site] = p;
    return p;
}

static void complete(const Pending& p) { memcpy(p.dst, p.src, 16); }

void global_load_lds_dwordx4(uint32_t m0, uint32_t voffset, uint64_t sbase, int inst_offset) {
    Lane* l = cur;
    Pending p;
    p.src = (const uint8_t*)(uintptr_t)(sbase + voffset + (int64_t)inst_offset);
    const uint32_t dst = m0 + (uint32_t)inst_offset + 16u * l->lane;
    p.dst = (uint8_t*)(uintptr_t)dst;
    Block* b = l->block;
    if (p.dst < b->lds || p.dst + 16 > b->lds + kLdsBytes) {
        fail("LDS-direct load outside the work-group's LDS");
        return;
    }
    if (!g_config.lazy_loads) {
        complete(p);
        return;
    }
    if (l->vm_count == 256) {   // more in flight than the model keeps: the oldest lands
        complete(l->vm[l->vm_head]);
        l->vm_head = (l->vm_head + 1) % 256;
        l->vm_count--;
    }
    l->vm[(l->vm_head + l->vm_count) % 256] = p;
    l->vm_count++;
}

void s_waitcnt_vmcnt(int in_flight) {
    Lane* l = cur;
    while ((int)l->vm_count > in_flight) {
        complete(l->vm[l->vm_head]);
        l->vm_head = (l->vm_head + 1) % 256;
        l->vm_count--;
    }
}

// ---------------------------------------------------------------------------------------------------------------
static void trampoline() {
    Lane* l = cur;
    (*g_body)();
    s_waitcnt_vmcnt(0);   // a wave ends only after its memory operations
    l->done = true;
    l->op = OP_NONE;
    emu_switch(&l->sp, g_scheduler_sp);
    abort();
}

static void start_lane(Lane& l) {
    uintptr_t top = ((uintptr_t)l.stack + kStackBytes) & ~(uintptr_t)15;
    void** slot = (void**)(top - 16);
    slot[0] = (void*)&trampoline;
    slot[1] = nullptr;
    void** sp = slot - 6;
    for (int i = 0; i < 6; ++i) sp[i] = nullptr;
    l.sp = sp;
}

static void run(Lane& l) {
    cur = &l;
    emu_switch(&g_scheduler_sp, l.sp);
    cur = nullptr;
}

static float bf16_value(uint16_t bits) { return __builtin_bit_cast(float, (uint32_t)bits << 16); }

// executes operation `op` for the lanes of one wave listed in `who` (all of them waiting at it)
static void execute(int op, Lane* wave_lanes, const std::vector<int>& who, bool whole) {
    g_counts[op]++;
    if (!whole) g_partial[op]++;
    switch (op) {
    case OP_WAVE_BARRIER:
        break;
    case OP_MFMA_BF16:
    case OP_MFMA_F32: {
        // D[m][n] = C[m][n] + sum_k A[m][k] B[k][n] in fp32, inactive lanes' operands read as zeros
        const int K = op == OP_MFMA_BF16 ? 16 : 2, per_lane = K / 2;
        static float A[32][16], B[16][32], D[32][32];
        memset(A, 0, sizeof A);
        memset(B, 0, sizeof B);
        memset(D, 0, sizeof D);
        for (int i : who) {
            const Lane& l = wave_lanes[i];
            const int r = l.lane % 32, h = l.lane / 32;
            for (int e = 0; e < per_lane; ++e) {
                A[r][per_lane * h + e] = op == OP_MFMA_BF16 ? bf16_value(l.a16[e]) : l.a32;
                B[per_lane * h + e][r] = op == OP_MFMA_BF16 ? bf16_value(l.b16[e]) : l.b32;
            }
        }
        for (int m = 0; m < 32; ++m)
            for (int k = 0; k < K; ++k) {
                const float a = A[m][k];
                for (int n = 0; n < 32; ++n) D[m][n] += a * B[k][n];
            }
        for (int i : who) {
            Lane& l = wave_lanes[i];
            const int n = l.lane % 32, h = l.lane / 32;
            for (int e = 0; e < 16; ++e) l.acc[e] += D[8 * (e / 4) + 4 * h + e % 4][n];
        }
        break;
    }
    case OP_READFIRSTLANE: {
        const uint32_t v = wave_lanes[who[0]].value;
        for (int i : who) wave_lanes[i].result = v;
        break;
    }
    case OP_READLANE: {
        const uint32_t from = wave_lanes[who[0]].index;
        for (int i : who)
            if (wave_lanes[i].index != from) fail("v_readlane with a lane index that differs across the wave");
        if (from >= 64) fail("v_readlane of a lane beyond the wave");
        const uint32_t v = wave_lanes[from % 64].value;   // an inactive lane's register is read as well
        for (int i : who) wave_lanes[i].result = v;
        break;
    }
    case OP_BALLOT: {
        uint64_t m = 0;
        for (int i : who)
            if (wave_lanes[i].pred) m |= 1ull << wave_lanes[i].lane;
        for (int i : who) wave_lanes[i].result64 = m;
        break;
    }
    case OP_SHFL_XOR: {
        uint32_t v[64];
        for (int i = 0; i < 64; ++i) v[i] = wave_lanes[i].value;
        for (int i : who) wave_lanes[i].result = v[(wave_lanes[i].lane ^ wave_lanes[i].index) & 63];
        break;
    }
    case OP_DS_READ_TR16: {
        // groups of 16 lanes: lane 4 j + q supplies columns 4 q .. 4 q + 3 of row j; lane i receives column i
        if (!whole) fail("transposing LDS read with inactive lanes");
        for (int g = 0; g < 4 && whole; ++g) {
            uint16_t rows[4][16];
            for (int s = 0; s < 16; ++s) {
                const Lane& l = wave_lanes[16 * g + s];
                const uint8_t* a = (const uint8_t*)(uintptr_t)(uint32_t)(uintptr_t)l.addr;
                if (((uintptr_t)a & 7u) || a < l.block->lds || a + 8 > l.block->lds + kLdsBytes) {
                    fail("transposing LDS read misaligned or outside the work-group's LDS");
                    return;
                }
                memcpy(&rows[s / 4][4 * (s % 4)], a, 8);
            }
            for (int i = 0; i < 16; ++i)
                for (int j = 0; j < 4; ++j) wave_lanes[16 * g + i].tr[j] = rows[j][i];
        }
        break;
    }
    case OP_DPP: {
        uint32_t v[64];
        for (int i = 0; i < 64; ++i) v[i] = wave_lanes[i].value;
        for (int i : who) {
            Lane& l = wave_lanes[i];
            const int c = l.ctrl;
            uint32_t from = l.lane;
            if (c < 0x100) from = (l.lane & ~3u) | ((c >> (2 * (l.lane & 3))) & 3);             // quad permute
            else if (c == 0x140) from = (l.lane & ~15u) | (15 - (l.lane & 15));                   // row mirror
            else if (c == 0x141) from = (l.lane & ~7u) | (7 - (l.lane & 7));                      // half-row mirror
            else fail("DPP control the model does not know");
            l.result = v[from];
        }
        break;
    }
    default:
        fail("operation the model does not know");
    }
}

// One pass over a work-group: runs every lane that can run, then executes what has gathered.  Returns whether
// anything moved.
static uint64_t g_rng;
static uint32_t draw() {
    g_rng = g_rng * 6364136223846793005ull + 1442695040888963407ull;
    return (uint32_t)(g_rng >> 33);
}

static bool advance(Block& b, const std::vector<uint32_t>& order, bool force) {
    bool moved = false;
    // shuffled orders also hold back waves at random, so that one wave can run several steps ahead of another
    uint32_t held = 0;
    if (g_config.order > 1 && !force) {
        if (b.hold_left == 0) {
            b.held = draw();   // half of the waves, on average, for one to four passes
            b.hold_left = 1 + draw() % 4;
        }
        b.hold_left--;
        held = b.held;
    }
    for (int pass = 0; pass < 2 && !moved; ++pass) {
        for (uint32_t t : order) {
            Lane& l = b.lanes[t];
            if (l.done || l.op != OP_NONE) continue;
            if (pass == 0 && ((held >> (l.wave & 31)) & 1)) continue;
            run(l);
            moved = true;
            if (l.done) b.live--;
        }
        if (held == 0) break;
    }
    const uint32_t nt = (uint32_t)b.lanes.size();
    // work-group barriers: every live lane has arrived
    uint32_t at_barrier = 0, live = 0;
    int all = 1;
    for (Lane& l : b.lanes) {
        if (l.done) continue;
        live++;
        if (l.op == OP_BLOCK_BARRIER || l.op == OP_BLOCK_AND) {
            at_barrier++;
            if (l.op == OP_BLOCK_AND) all &= l.pred != 0;
        }
    }
    if (live > 0 && at_barrier == live) {
        g_counts[OP_BLOCK_BARRIER]++;
        for (Lane& l : b.lanes) {
            if (l.done) continue;
            l.result = (uint32_t)all;
            l.op = OP_NONE;
        }
        return true;
    }
    for (uint32_t w0 = 0; w0 < nt; w0 += 64) {
        Lane* wl = &b.lanes[w0];
        const uint32_t n = std::min(64u, nt - w0);
        std::vector<int> who;
        int op = OP_NONE;
        bool same = true, any_running = false;
        for (uint32_t i = 0; i < n; ++i) {
            if (wl[i].done) continue;
            if (wl[i].op == OP_NONE) { any_running = true; continue; }
            if (wl[i].op == OP_YIELD) { wl[i].op = OP_NONE; moved = true; g_polling = true; continue; }
            if (wl[i].op == OP_BLOCK_BARRIER || wl[i].op == OP_BLOCK_AND) { same = false; continue; }
            if (op == OP_NONE) op = wl[i].op;
            if (wl[i].op != op) same = false;
            else who.push_back((int)i);
        }
        if (op == OP_NONE || any_running) continue;
        uint32_t live_in_wave = 0;
        for (uint32_t i = 0; i < n; ++i) live_in_wave += !wl[i].done;
        const bool whole = same && who.size() == live_in_wave;
        if (!whole && !force) continue;
        // (forced: the wave has diverged; the lanes gathered at the first operation go on with the others masked off)
        execute(op, wl, who, whole && live_in_wave == n);
        for (int i : who) wl[i].op = OP_NONE;
        moved = true;
        if (force) return true;
    }
    return moved;
}

static Block* make_block(uint32_t linear, uint32_t nt) {
    Block* b = new Block;
    b->idx = dim3(linear % g_grid.x, linear / g_grid.x % g_grid.y, linear / (g_grid.x * g_grid.y));
    b->lds = (uint8_t*)mmap(nullptr, kLdsBytes, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_32BIT, -1, 0);
    if (b->lds == (uint8_t*)MAP_FAILED) abort();
    memset(b->lds, 0xff, kLdsBytes);
    b->lds_used = 0;
    b->held = b->hold_left = 0;
    b->live = nt;
    b->lanes.resize(nt);
    // one mapping for all stacks of the work-group (the process may hold only so many mappings)
    b->stacks = (uint8_t*)mmap(nullptr, nt * kStackBytes, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (b->stacks == (uint8_t*)MAP_FAILED) abort();
    for (uint32_t t = 0; t < nt; ++t) {
        Lane& l = b->lanes[t];
        memset(&l, 0, offsetof(Lane, vm));
        l.vm_head = l.vm_count = 0;
        l.stack = b->stacks + (size_t)t * kStackBytes;
        for (int i = 0; i < 8; ++i) ((uint64_t*)l.stack)[i] = kCanary;
        l.block = b;
        l.tid = t;
        l.lane = t % 64;
        l.wave = t / 64;
        start_lane(l);
    }
    return b;
}

static void free_block(Block* b) {
    for (Lane& l : b->lanes)
        for (int i = 0; i < 8; ++i)
            if (((uint64_t*)l.stack)[i] != kCanary) fail("a lane's stack overflowed (the model's, not the kernel's)");
    munmap(b->stacks, b->lanes.size() * kStackBytes);
    munmap(b->lds, kLdsBytes);
    delete b;
}

void launch(dim3 grid, dim3 block, size_t, hipStream_t, const std::function<void()>& body) {
    const uint64_t total = (uint64_t)grid.x * grid.y * grid.z;
    const uint32_t nt = block.x * block.y * block.z;
    if (total == 0 || nt == 0 || nt > 1024 || nt % 64 != 0) {   // the model runs whole waves
        fail("launch configuration");
        return;
    }
    g_grid = grid;
    g_block_dim = block;
    g_body = &body;
    g_rng = (uint64_t)g_config.order * 0x9E3779B97F4A7C15ull + 12345;
    std::vector<uint32_t> order(nt);
    for (uint32_t t = 0; t < nt; ++t) order[t] = g_config.order == 1 ? nt - 1 - t : t;
    if (g_config.order > 1) {
        uint64_t s = (uint64_t)g_config.order * 0x9E3779B97F4A7C15ull;
        for (uint32_t t = nt - 1; t > 0; --t) {
            s = s * 6364136223846793005ull + 1442695040888963407ull;
            std::swap(order[t], order[(s >> 33) % (t + 1)]);
        }
    }
    std::vector<Block*> active;
    uint64_t next = 0;
    size_t room = (size_t)g_config.resident;
    while (true) {
        // a launch that polls for other work-groups' results is one whose work-groups are all resident on the device
        if (g_polling && room < 2048 && !g_config.fixed) room += 16;
        g_polling = false;
        while (active.size() < room && next < total) active.push_back(make_block((uint32_t)next++, nt));
        if (active.empty()) break;
        bool moved = false;
        for (size_t i = 0; i < active.size();) {
            Block* b = active[i];
            moved |= advance(*b, order, false);
            if (b->live == 0) {
                free_block(b);
                active.erase(active.begin() + i);
                moved = true;
            } else {
                ++i;
            }
        }
        if (!moved) {
            bool forced = false;
            for (Block* b : active)
                if (advance(*b, order, true)) { forced = true; break; }
            if (!forced) {
                fail("deadlock: lanes wait at operations that the rest of their wave or work-group never reaches");
                for (Block* b : active) free_block(b);   // the fibers are abandoned where they stand
                break;
            }
        }
    }
    g_body = nullptr;
}

}  // namespace emu

extern "C" {
void emu_configure(int order, int lazy_loads, int resident) {
    emu::g_config.order = order;
    emu::g_config.lazy_loads = lazy_loads;
    emu::g_config.fixed = resident < 0;   // a negative count: exactly that many, whatever the lanes do
    emu::g_config.resident = resident > 0 ? resident : resident < 0 ? -resident : 1;
}
void emu_reset_counts() {
    memset(emu::g_counts, 0, sizeof emu::g_counts);
    memset(emu::g_partial, 0, sizeof emu::g_partial);
}
uint64_t emu_count(int op) { return op >= 0 && op < emu::OP_KINDS ? emu::g_counts[op] : 0; }
uint64_t emu_partial_count(int op) { return op >= 0 && op < emu::OP_KINDS ? emu::g_partial[op] : 0; }
const char* emu_message() { return emu::g_message; }
// memory that ends (up to rounding to 256 bytes) where an inaccessible page begins, and begins after one
void* emu_guarded_alloc(size_t bytes) {
    const size_t page = 4096, body = (bytes + page - 1) / page * page, placed = (bytes + 255) / 256 * 256;
    uint8_t* base = (uint8_t*)mmap(nullptr, body + 2 * page, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
    if (base == (uint8_t*)MAP_FAILED) return nullptr;
    mprotect(base + page, body, PROT_READ | PROT_WRITE);
    memset(base + page, 0xff, body);
    return base + page + (body - placed);
}
void emu_guarded_free(void* p, size_t bytes) {
    const size_t page = 4096, body = (bytes + page - 1) / page * page, placed = (bytes + 255) / 256 * 256;
    munmap((uint8_t*)p - (body - placed) - page, body + 2 * page);
}
}
