// Fiber scheduler, rendezvous, LDS arena and deferred global -> LDS moves of the CPU emulator.
#include "emu_runtime.h"

#include <execinfo.h>
#include <signal.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <unistd.h>

#include <algorithm>
#include <random>
#include <memory>
#include <vector>

extern "C" char __start_emu_lds[];
extern "C" char __stop_emu_lds[];

// void emu_switch(void** save_sp, void* load_sp): x86-64 SysV context switch (callee-saved registers + stack)
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
.size emu_switch,.-emu_switch
)");
extern "C" void emu_switch(void** save_sp, void* load_sp);

namespace emu {

namespace {

constexpr size_t kStackBytes = 256 * 1024;
constexpr unsigned kMaxBlockThreads = 1024;

struct Fiber {
  Lane lane;
  void* sp = nullptr;
  char* stack = nullptr;
  bool done = false;
  // what the fiber is waiting for: runnable once *wait_gen differs from wait_val (null: runnable)
  const unsigned long long* wait_gen = nullptr;
  unsigned long long wait_val = 0;
  struct Pending { uint32_t lds_dst; int bytes; uint8_t data[16]; };
  std::vector<Pending> dma;
};

}  // namespace

struct Wave {
  int n_lanes = 0;                 // lanes that exist
  int live = 0;                    // lanes that have not left the kernel
  int arrived = 0;
  unsigned long long gen = 0;      // completed rendezvous
  uint32_t tag = 0;
  bool lane_live[kWave];
  // the lanes that took part in the last rendezvous of each parity: what a lane reads after a
  // rendezvous must not depend on which of the others have meanwhile run on and left the kernel
  unsigned long long took_part[2] = {0, 0};
  alignas(64) uint8_t slot[2][kWave][kSlotBytes];
  void complete() {
    unsigned long long m = 0;
    for (int l = 0; l < kWave; ++l) m |= (unsigned long long)lane_live[l] << l;
    took_part[gen & 1] = m;
    arrived = 0;
    gen++;
  }
};

namespace {

struct Block {
  std::vector<Fiber> fibers;
  std::vector<Wave> waves;
  int live = 0;
  int arrived = 0;
  unsigned long long gen = 0;
  unsigned long long polls = 0;    // times a lane gave way inside a polling loop (counts as progress)
  // for workgroups that share the machine (see launch): its id, its LDS while another one runs,
  // the stacks it uses, the state of its skewed schedule
  Dim3 idx;
  std::vector<uint8_t> lds;
  size_t stack_slot = 0;
  std::mt19937 rng;
  unsigned long long stuck_draws = 0, idle_rounds = 0;
};

Block g_solo;
Block* g_blk = &g_solo;
#define g_block (*g_blk)
Fiber* g_cur = nullptr;
void* g_sched_sp = nullptr;
Dim3 g_block_idx, g_block_dim, g_grid_dim;
const std::function<void()>* g_body = nullptr;
int g_dma_eager = 0;
unsigned g_order_seed = 0;
unsigned g_wave_skew = 0;
unsigned g_concurrent = 0;         // 0 / 1: workgroups run one after the other; n: up to n share the machine
unsigned g_concurrent_seed = 0;
unsigned long long g_launches = 0;
unsigned long long g_blocks = 0;
unsigned long long g_polls = 0;
int g_cu_count = 256;
std::vector<char*> g_stacks;

void yield() { emu_switch(&g_cur->sp, g_sched_sp); }

void leave_wave(Fiber* f) {
  Wave* w = f->lane.wave;
  w->lane_live[f->lane.lane] = false;
  w->live--;
  // a rendezvous the others are waiting in may now be complete
  if (w->live > 0 && w->arrived == w->live) w->complete();
  g_block.live--;
  if (g_block.live > 0 && g_block.arrived == g_block.live) { g_block.arrived = 0; g_block.gen++; }
}

void fiber_main() {
  Fiber* f = g_cur;
  (*g_body)();
  f->dma.clear();
  f->done = true;
  leave_wave(f);
  yield();
  fail("a finished fiber was resumed");
}

char* get_stack(size_t i) {
  while (g_stacks.size() <= i) {
    void* p = mmap(nullptr, kStackBytes, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (p == MAP_FAILED) fail("mmap of a fiber stack failed");
    g_stacks.push_back(static_cast<char*>(p));
  }
  return g_stacks[i];
}

void prepare(Fiber* f) {
  uintptr_t top = (reinterpret_cast<uintptr_t>(f->stack) + kStackBytes) & ~uintptr_t(15);
  void** s = reinterpret_cast<void**>(top);
  *--s = nullptr;                                   // return address of fiber_main (never used)
  *--s = reinterpret_cast<void*>(&fiber_main);      // `ret` of the first switch lands here
  for (int i = 0; i < 6; ++i) *--s = nullptr;       // rbp rbx r12 r13 r14 r15
  f->sp = s;
}

// One round over the lanes of wavefront `wv` only; true when any of them ran.
bool run_wave_once(size_t wv) {
  bool ran = false;
  const size_t f0 = wv * kWave, f1 = std::min(g_block.fibers.size(), f0 + kWave);
  for (size_t i = f0; i < f1; ++i) {
    Fiber& f = g_block.fibers[i];
    if (f.done) continue;
    if (f.wait_gen != nullptr && *f.wait_gen == f.wait_val) continue;
    f.wait_gen = nullptr;
    g_cur = &f;
    emu_switch(&g_sched_sp, f.sp);
    ran = true;
  }
  return ran;
}

// Skewed schedule: the wavefronts of a workgroup do not advance together.  A wavefront drawn at
// random runs alone for a random stretch, up to the point where it can only wait for the others
// (a workgroup barrier, the end of the kernel), then another is drawn.  On the hardware nothing
// but barriers keeps wavefronts in step; a kernel that relies on them advancing together (a ring
// slot refilled while a slower wavefront still reads it, a flag read before it is written)
// passes under the even schedule and fails under this one.
// One draw of it, on the current workgroup:
void step_block_skewed() {
  Block& b = g_block;
  const size_t n_waves = b.waves.size();
  // seeds from 1000 on: one wavefront (seed % wavefronts) is held back -- it only gets a turn, one
  // step at a time, when none of the others can move
  const bool hold_one = g_wave_skew >= 1000;
  const size_t held = g_wave_skew % n_waves;
  size_t wv = b.rng() % n_waves;
  unsigned stretch = 1u + b.rng() % ((b.rng() & 3) == 0 ? 4096u : 48u);          // mostly short, now and then as far as it gets
  if (hold_one) {
    if (b.stuck_draws >= 8 * n_waves) { wv = held; stretch = 1; }
    else if (wv == held) wv = (wv + 1) % n_waves;
  }
  bool any = false;
  for (unsigned r = 0; r < stretch && run_wave_once(wv); ++r) any = true;
  if (any) {
    b.stuck_draws = 0;
  } else if (++b.stuck_draws > 64 * n_waves) {                                   // every wavefront drawn many times, none could run
    fail("deadlock in block (%u,%u,%u): %d lanes wait at barriers that cannot complete", b.idx.x, b.idx.y, b.idx.z, b.live);
  }
}

// Even schedule, one round: every lane that can run does, up to its next rendezvous.  A full round
// without any lane finishing, any rendezvous completing or any polling loop giving way means the
// lanes are waiting for each other in different places.
void step_block_even() {
  Block& b = g_block;
  unsigned long long before = b.gen + b.polls;
  for (Wave& w : b.waves) before += w.gen;
  const int live_before = b.live;
  for (Fiber& f : b.fibers) {
    if (f.done) continue;
    if (f.wait_gen != nullptr && *f.wait_gen == f.wait_val) continue;
    f.wait_gen = nullptr;
    g_cur = &f;
    emu_switch(&g_sched_sp, f.sp);
  }
  unsigned long long after = b.gen + b.polls;
  for (Wave& w : b.waves) after += w.gen;
  if (after == before && b.live == live_before) {
    if (++b.idle_rounds > 4)
      fail("deadlock in block (%u,%u,%u): %d lanes wait at barriers that cannot complete", b.idx.x, b.idx.y, b.idx.z, b.live);
  } else {
    b.idle_rounds = 0;
  }
}

void step_block() {
  if (g_wave_skew != 0 && g_block.waves.size() > 1) step_block_skewed();
  else step_block_even();
  g_cur = nullptr;
}

// Makes `b` the current workgroup, with all its lanes at the start of the kernel.  Does not touch LDS.
void setup_block(Block& b, Dim3 bidx, size_t stack_slot) {
  const unsigned n = g_block_dim.x * g_block_dim.y * g_block_dim.z;
  const unsigned n_waves = (n + kWave - 1) / kWave;
  if (n > kMaxBlockThreads) fail("workgroup of %u lanes", n);
  g_blk = &b;
  g_block_idx = bidx;
  b.idx = bidx;
  b.stack_slot = stack_slot;
  b.rng.seed(g_wave_skew * 2654435761u + bidx.x * 40503u + bidx.y * 97u + bidx.z);
  b.stuck_draws = b.idle_rounds = b.polls = 0;
  b.fibers.assign(n, Fiber());
  b.waves.assign(n_waves, Wave());
  b.live = (int)n;
  b.arrived = 0;
  b.gen = 0;
  for (unsigned i = 0; i < n; ++i) {
    Fiber& f = b.fibers[i];
    Wave& w = b.waves[i / kWave];
    f.lane.flat = (int)i;
    f.lane.lane = (int)(i % kWave);
    f.lane.tid = Dim3(i % g_block_dim.x, (i / g_block_dim.x) % g_block_dim.y, i / (g_block_dim.x * g_block_dim.y));
    f.lane.wave = &w;
    w.n_lanes++;
    w.live++;
    w.lane_live[i % kWave] = true;
    f.stack = get_stack(stack_slot * kMaxBlockThreads + i);
    prepare(&f);
  }
  for (Wave& w : b.waves) {
    for (int l = w.n_lanes; l < kWave; ++l) w.lane_live[l] = false;
    w.took_part[0] = w.took_part[1] = w.n_lanes == kWave ? ~0ull : (1ull << w.n_lanes) - 1ull;
  }
}

// One workgroup from start to end, alone on the machine.
void run_block(Dim3 bidx) {
  setup_block(g_solo, bidx, 0);
  memset(__start_emu_lds, 0xFB, __stop_emu_lds - __start_emu_lds);   // LDS holds no defined values at workgroup start
  while (g_block.live > 0) step_block();
}

// Up to `g_concurrent` workgroups share the machine: one of them, drawn at random, advances by a
// few scheduling steps, then another.  The one LDS arena holds the running workgroup's contents;
// the others' are kept aside.  What this adds over one workgroup at a time: a workgroup that waits
// for another one (the last arrival of a split merge polling for the others' published bits)
// really waits, and the others really publish while it does.
void run_blocks_concurrently(const std::vector<size_t>& order, Dim3 grid) {
  const size_t lds_size = (size_t)(__stop_emu_lds - __start_emu_lds);
  std::mt19937 rng(g_concurrent_seed * 7919u + 13u);
  std::vector<std::unique_ptr<Block>> active;
  std::vector<size_t> free_slots;
  for (size_t k = g_concurrent; k-- > 0;) free_slots.push_back(k);
  size_t next = 0;
  Block* in_lds = nullptr;
  while (next < order.size() || !active.empty()) {
    while (active.size() < g_concurrent && next < order.size()) {
      const size_t i = order[next++];
      active.emplace_back(new Block());
      active.back()->lds.assign(lds_size, 0xFB);
      setup_block(*active.back(), Dim3((unsigned)(i % grid.x), (unsigned)((i / grid.x) % grid.y), (unsigned)(i / ((size_t)grid.x * grid.y))),
                  free_slots.back());
      free_slots.pop_back();
    }
    const size_t pick = rng() % active.size();
    Block* b = active[pick].get();
    if (in_lds != b) {
      if (in_lds != nullptr) memcpy(in_lds->lds.data(), __start_emu_lds, lds_size);
      memcpy(__start_emu_lds, b->lds.data(), lds_size);
      in_lds = b;
    }
    g_blk = b;
    g_block_idx = b->idx;
    const unsigned quanta = 1u + rng() % 8u;
    for (unsigned q = 0; q < quanta && b->live > 0; ++q) step_block();
    if (b->live == 0) {
      free_slots.push_back(b->stack_slot);
      in_lds = nullptr;
      active.erase(active.begin() + (long)pick);
    }
  }
  g_blk = &g_solo;
}

}  // namespace

void fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  fprintf(stderr, "[emu] ");
  vfprintf(stderr, fmt, ap);
  fprintf(stderr, "\n");
  va_end(ap);
  fflush(stderr);
  abort();
}

Lane* self() { return &g_cur->lane; }
Dim3 block_idx() { return g_block_idx; }
Dim3 block_dim() { return g_block_dim; }
Dim3 grid_dim() { return g_grid_dim; }
int cu_count() { return g_cu_count; }

int wave_rendezvous(const void* post, size_t bytes, uint32_t tag) {
  Fiber* f = g_cur;
  Wave* w = f->lane.wave;
  if (bytes > (size_t)kSlotBytes) fail("rendezvous operand of %zu bytes", bytes);
  const unsigned long long my_gen = w->gen;
  const int parity = (int)(my_gen & 1);
  if (bytes) memcpy(w->slot[parity][f->lane.lane], post, bytes);
  if (w->arrived == 0) w->tag = tag;
  else if (w->tag != tag)
    fail("block (%u,%u,%u) wave %d: lanes reached different wave-wide operations (tags %08x / %08x): "
         "a collective inside divergent control flow", g_block_idx.x, g_block_idx.y, g_block_idx.z,
         f->lane.flat / kWave, w->tag, tag);
  w->arrived++;
  f->lane.parity = parity;
  if (w->arrived == w->live) {
    w->complete();
  } else {
    f->wait_gen = &w->gen;
    f->wait_val = my_gen;
    yield();
  }
  return parity;
}

const uint8_t* wave_slot(int parity, int lane) { return g_cur->lane.wave->slot[parity][lane]; }
bool wave_lane_live(int lane) { return (g_cur->lane.wave->took_part[g_cur->lane.parity] >> lane) & 1; }

void poll_yield() {
  g_block.polls++;
  g_polls++;
  yield();
}

void block_barrier() {
  g_work.barriers_lane_calls++;
  const unsigned long long my_gen = g_block.gen;
  g_block.arrived++;
  if (g_block.arrived == g_block.live) {
    g_block.arrived = 0;
    g_block.gen++;
  } else {
    g_cur->wait_gen = &g_block.gen;
    g_cur->wait_val = my_gen;
    yield();
  }
}

uint32_t lds_addr(const void* p) {
  const char* c = static_cast<const char*>(p);
  if (c < __start_emu_lds || c > __stop_emu_lds) fail("lds_addr of an object outside LDS");
  return (uint32_t)(c - __start_emu_lds);
}

uint8_t* lds_ptr(uint32_t addr, size_t bytes) {
  const size_t size = (size_t)(__stop_emu_lds - __start_emu_lds);
  if ((size_t)addr + bytes > size)
    fail("LDS access out of bounds: address %u + %zu, arena %zu (block (%u,%u,%u), thread %d)", addr, bytes, size,
         g_block_idx.x, g_block_idx.y, g_block_idx.z, g_cur ? g_cur->lane.flat : -1);
  return reinterpret_cast<uint8_t*>(__start_emu_lds) + addr;
}

WorkCounts g_work = {0, 0, 0, 0, 0, 0, 0};
void count_mfma(int m, int k) {
  g_work.mfma_lane_calls++;
  g_work.mfma_flops += 2ull * m * m * k / kWave;          // a lane's share
}

bool g_lds_profile = false;
unsigned long long g_lds_stats[9] = {0};

void lds_account(uint32_t addr, int bytes, int kind) {
  (kind == 2 ? g_work.lds_write_bytes : g_work.lds_read_bytes) += (unsigned long long)bytes;
  if (!g_lds_profile) return;
  const int par = wave_rendezvous(&addr, sizeof(addr), 0x4c424b30u + (uint32_t)kind);
  Lane* me = self();
  int first_live = 0;
  while (first_live < kWave && !wave_lane_live(first_live)) ++first_live;
  if (me->lane != first_live) return;                     // one lane does the sums for the wavefront
  const int group = bytes >= 16 ? 16 : (bytes == 8 ? 32 : 64);
  unsigned long long passes = 0, ideal = 0;
  for (int g0 = 0; g0 < kWave; g0 += group) {
    uint32_t words[64][4];                                // distinct word addresses seen per bank (small sets)
    int n_words[64] = {0};
    bool any = false;
    for (int l = g0; l < g0 + group; ++l) {
      if (!wave_lane_live(l)) continue;
      any = true;
      uint32_t a;
      memcpy(&a, wave_slot(par, l), sizeof(a));
      for (int w = 0; w < bytes / 4; ++w) {
        const uint32_t word = a / 4 + w;
        const int bank = word % 64;
        bool seen = false;
        for (int k = 0; k < n_words[bank] && k < 4; ++k) seen |= words[bank][k] == word;
        if (!seen) {
          if (n_words[bank] < 4) words[bank][n_words[bank]] = word;
          n_words[bank]++;                                // (beyond four distinct words the count may overshoot: it is a conflict either way)
        }
      }
    }
    if (!any) continue;
    int worst = 1;
    for (int b = 0; b < 64; ++b) worst = std::max(worst, n_words[b]);
    passes += worst;
    ideal += 1;
  }
  g_lds_stats[3 * kind + 0] += 1;
  g_lds_stats[3 * kind + 1] += passes;
  g_lds_stats[3 * kind + 2] += ideal;
}

void dma_issue(const void* src, uint32_t lds_dst, int bytes) {
  if (bytes != 0 && bytes != 4 && bytes != 16) fail("dma of %d bytes per lane", bytes);
  g_work.dma_bytes += (unsigned long long)bytes;
  g_work.dma_lane_calls += bytes != 0;
  if (g_dma_eager) {
    if (bytes == 0) return;
    memcpy(lds_ptr(lds_dst, bytes), src, bytes);
    return;
  }
  Fiber::Pending p;
  p.lds_dst = lds_dst;
  p.bytes = bytes;
  if (bytes != 0) {                                  // 0: a lane that sits out a move of its wavefront (kept for the count)
    memcpy(p.data, src, bytes);
    lds_ptr(lds_dst, bytes);                         // bounds check at issue
  }
  g_cur->dma.push_back(p);
}

void dma_wait(int allowed_in_flight) {
  std::vector<Fiber::Pending>& q = g_cur->dma;
  const size_t keep = std::min(q.size(), (size_t)std::max(allowed_in_flight, 0));
  const size_t land = q.size() - keep;
  for (size_t i = 0; i < land; ++i)
    if (q[i].bytes != 0) memcpy(lds_ptr(q[i].lds_dst, q[i].bytes), q[i].data, q[i].bytes);
  q.erase(q.begin(), q.begin() + land);
}

namespace {
// A stray global access by an emulated kernel: say where it happened before the process dies.
void on_segv(int sig, siginfo_t* info, void*) {
  char buf[256];
  const int n = snprintf(buf, sizeof(buf),
                         "[emu] signal %d at address %p in block (%u,%u,%u), thread %d of the workgroup\n", sig,
                         info ? info->si_addr : nullptr, g_block_idx.x, g_block_idx.y, g_block_idx.z,
                         g_cur ? g_cur->lane.flat : -1);
  if (n > 0) (void)!write(2, buf, (size_t)n);
  void* frames[32];
  const int depth = backtrace(frames, 32);
  backtrace_symbols_fd(frames, depth, 2);
  signal(sig, SIG_DFL);
  raise(sig);
}
void install_handler() {
  static bool done = false;
  if (done) return;
  done = true;
  static char alt[1 << 16];
  stack_t ss;
  ss.ss_sp = alt;
  ss.ss_size = sizeof(alt);
  ss.ss_flags = 0;
  sigaltstack(&ss, nullptr);
  struct sigaction sa;
  memset(&sa, 0, sizeof(sa));
  sa.sa_sigaction = on_segv;
  sa.sa_flags = SA_SIGINFO | SA_ONSTACK | SA_RESETHAND;
  sigaction(SIGSEGV, &sa, nullptr);
  sigaction(SIGBUS, &sa, nullptr);
}
}  // namespace

void launch(Dim3 grid, Dim3 block, const std::function<void()>& body) {
  if (g_cur != nullptr) fail("launch from inside a kernel");
  install_handler();
  g_launches++;
  g_block_dim = block;
  g_grid_dim = grid;
  g_body = &body;
  const size_t n_blocks = (size_t)grid.x * grid.y * grid.z;
  g_blocks += n_blocks;
  std::vector<size_t> order(n_blocks);
  for (size_t i = 0; i < n_blocks; ++i) order[i] = i;
  if (g_order_seed) {
    std::mt19937 rng(g_order_seed);
    std::shuffle(order.begin(), order.end(), rng);
  }
  if (g_concurrent > 1 && n_blocks > 1) {
    run_blocks_concurrently(order, grid);
  } else {
    for (size_t i : order)
      run_block(Dim3((unsigned)(i % grid.x), (unsigned)((i / grid.x) % grid.y), (unsigned)(i / ((size_t)grid.x * grid.y))));
  }
  g_cur = nullptr;
  g_body = nullptr;
}

}  // namespace emu

extern "C" {
void emu_set_dma_mode(int eager) { emu::g_dma_eager = eager; }
void emu_set_block_order(unsigned seed) { emu::g_order_seed = seed; }
void emu_set_wave_skew(unsigned seed) { emu::g_wave_skew = seed; }
void emu_set_concurrent_blocks(unsigned n, unsigned seed) { emu::g_concurrent = n; emu::g_concurrent_seed = seed; }
unsigned long long emu_launch_count(void) { return emu::g_launches; }
unsigned long long emu_block_count(void) { return emu::g_blocks; }
unsigned long long emu_poll_count(void) { return emu::g_polls; }
void emu_set_cu_count(int n) { emu::g_cu_count = n; }
void emu_set_lds_profile(int on) {
  emu::g_lds_profile = on != 0;
  for (auto& v : emu::g_lds_stats) v = 0;
}
void emu_work_counts(double out[7], int reset) {
  const emu::WorkCounts& w = emu::g_work;
  out[0] = (double)w.mfma_lane_calls / emu::kWave;
  out[1] = (double)w.mfma_flops;
  out[2] = (double)w.lds_read_bytes;
  out[3] = (double)w.lds_write_bytes;
  out[4] = (double)w.dma_bytes;
  out[5] = (double)w.dma_lane_calls / emu::kWave;
  out[6] = (double)w.barriers_lane_calls / emu::kWave;
  if (reset) emu::g_work = emu::WorkCounts{0, 0, 0, 0, 0, 0, 0};
}
void emu_lds_profile(unsigned long long out[9]) {
  for (int i = 0; i < 9; ++i) out[i] = emu::g_lds_stats[i];
}
}
