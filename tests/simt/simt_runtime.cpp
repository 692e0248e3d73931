// The fiber scheduler, the guard-page allocator and the fault handler behind
// include/hip/hip_runtime.h (see there).  Built only by the tests, for the host.
#include <hip/hip_runtime.h>

#include <signal.h>
#include <stdlib.h>
#include <sys/mman.h>
#include <unistd.h>

#include <string>
#include <vector>

extern "C" void simt_switch(void** save_sp, void* load_sp);
asm(R"(
.text
.globl simt_switch
.type simt_switch,@function
simt_switch:
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
.size simt_switch,.-simt_switch
)");

extern "C" char __start_simt_lds[], __stop_simt_lds[];

namespace simt {

enum { READY = 0, WAITING = 1, DONE = 2 };
static const int MAX_THREADS = 1024, WAVE = 64;
static const size_t STACK_BYTES = 512 * 1024;

struct Gate {                 // a barrier of a wavefront or of the workgroup
  int alive = 0, arrived = 0, gen = 0;
};

struct Wave {
  Gate gate;
  uint32_t words[2][WAVE];
  alignas(16) unsigned char fa[2][WAVE][16], fb[2][WAVE][16];
};

struct Fiber {
  void* sp;
  char* stack;
  int state;
  Gate* wait_gate;
  int wait_gen;
  Idx tid;
  int flat, lane;
  Wave* wave;
  int xpar, fpar;
};

Fiber* g_cur = nullptr;
static Fiber g_fibers[MAX_THREADS];
static Wave g_waves[MAX_THREADS / WAVE];
static Gate g_block_gate;
static void* g_sched_sp;
static Idx g_block_idx, g_block_dim, g_grid_dim;
static Body g_body;
static void* g_body_arg;
static const char* g_kernel = "(none)";
static bool g_stacks_ready = false;
static long g_launches = 0;
static bool g_reverse = false;         // run a workgroup's threads from the last to the first

const Idx& thread_idx() { return g_cur->tid; }
const Idx& block_idx() { return g_block_idx; }
const Idx& block_dim() { return g_block_dim; }
const Idx& grid_dim() { return g_grid_dim; }
int lane_id() { return g_cur->lane; }

static void die(const char* what) {
  fprintf(stderr, "[simt] %s in kernel %s, workgroup (%u,%u,%u), thread %d\n", what, g_kernel, g_block_idx.x,
          g_block_idx.y, g_block_idx.z, g_cur ? g_cur->flat : -1);
  fflush(stderr);
  _exit(96);
}

static void yield_to_scheduler() { simt_switch(&g_cur->sp, g_sched_sp); }

static void arrive(Gate& g) {
  Fiber* f = g_cur;
  const int gen = g.gen;
  if (++g.arrived >= g.alive) {
    g.arrived = 0;
    ++g.gen;
    return;
  }
  f->state = WAITING;
  f->wait_gate = &g;
  f->wait_gen = gen;
  yield_to_scheduler();
}

void block_sync() { arrive(g_block_gate); }
void wave_sync() { arrive(g_cur->wave->gate); }

uint32_t lane_exchange(uint32_t v, int src, uint32_t fallback) {
  Fiber* f = g_cur;
  Wave* w = f->wave;
  const int par = f->xpar;
  f->xpar ^= 1;
  w->words[par][f->lane] = v;
  arrive(w->gate);
  return (src >= 0 && src < WAVE) ? w->words[par][src] : fallback;
}

void frag_publish(const void* a, const void* b, int bytes) {
  Fiber* f = g_cur;
  Wave* w = f->wave;
  f->fpar ^= 1;
  memcpy(w->fa[f->fpar][f->lane], a, bytes);
  memcpy(w->fb[f->fpar][f->lane], b, bytes);
  arrive(w->gate);
}
const void* frag_a(int lane) { return g_cur->wave->fa[g_cur->fpar][lane]; }
const void* frag_b(int lane) { return g_cur->wave->fb[g_cur->fpar][lane]; }

// ---- matrix-core instructions (lane layouts: see the header) ---------------------------------------
static inline float bf16_bits(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

// 32x32x16: lane l gives row (a) / column (b) l % 32 and k = 8 * (l / 32) .. +7; it receives, for
// r in 0..15, row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.
void mfma_32x32x16(const void* a, const void* b, float* c) {
  frag_publish(a, b, 16);
  const int l = lane_id(), col = l % 32;
  for (int r = 0; r < 16; ++r) {
    const int row = 8 * (r / 4) + 4 * (l / 32) + r % 4;
    float s = c[r];
    for (int k = 0; k < 16; ++k) {
      const uint16_t* av = (const uint16_t*)frag_a(row + 32 * (k / 8));
      const uint16_t* bv = (const uint16_t*)frag_b(col + 32 * (k / 8));
      s += bf16_bits(av[k % 8]) * bf16_bits(bv[k % 8]);
    }
    c[r] = s;
  }
}
// 16x16x32: lane l gives row / column l % 16 and k = 8 * (l / 16) .. +7; it receives rows
// 4 * (l / 16) + r, r in 0..3, column l % 16.
void mfma_16x16x32(const void* a, const void* b, float* c) {
  frag_publish(a, b, 16);
  const int l = lane_id(), col = l % 16;
  for (int r = 0; r < 4; ++r) {
    const int row = 4 * (l / 16) + r;
    float s = c[r];
    for (int k = 0; k < 32; ++k) {
      const uint16_t* av = (const uint16_t*)frag_a(row + 16 * (k / 8));
      const uint16_t* bv = (const uint16_t*)frag_b(col + 16 * (k / 8));
      s += bf16_bits(av[k % 8]) * bf16_bits(bv[k % 8]);
    }
    c[r] = s;
  }
}
// 4x4x4, 16 products: lane l gives row (a) / column (b) l % 4 of product l / 4 and 4 consecutive
// k; it receives column l % 4 of that product, rows 0..3.
void mfma_4x4x4(const void* a, const void* b, float* c) {
  frag_publish(a, b, 8);
  const int l = lane_id(), blk = l / 4;
  const uint16_t* bv = (const uint16_t*)frag_b(l);
  for (int r = 0; r < 4; ++r) {
    const uint16_t* av = (const uint16_t*)frag_a(blk * 4 + r);
    float s = c[r];
    for (int k = 0; k < 4; ++k) s += bf16_bits(av[k]) * bf16_bits(bv[k]);
    c[r] = s;
  }
}

int dpp_source(int lane, int ctrl) {
  const int row = lane & ~15, in_row = lane & 15;
  if (ctrl >= 0 && ctrl <= 0xFF) return (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3);     // quad_perm
  if (ctrl >= 0x101 && ctrl <= 0x10F) { const int s = in_row + (ctrl & 15); return s < 16 ? row + s : -1; }   // row_shl
  if (ctrl >= 0x111 && ctrl <= 0x11F) { const int s = in_row - (ctrl & 15); return s >= 0 ? row + s : -1; }   // row_shr
  if (ctrl >= 0x121 && ctrl <= 0x12F) return row + ((in_row - (ctrl & 15)) & 15);                              // row_ror
  if (ctrl == 0x140) return row + 15 - in_row;                      // row_mirror
  if (ctrl == 0x141) return (lane & ~7) + 7 - (lane & 7);           // row_half_mirror
  if (ctrl == 0x142) return lane >= 16 ? row - 1 : -1;              // row_bcast:15
  if (ctrl == 0x143) return lane >= 32 ? 31 : -1;                   // row_bcast:31
  die("unknown DPP control");
  return -1;
}

static void fiber_main() {
  g_body(g_body_arg);
  g_cur->state = DONE;
  yield_to_scheduler();
  die("a finished fiber was resumed");
}

static void prepare_fiber(Fiber& f) {
  uintptr_t top = ((uintptr_t)f.stack + STACK_BYTES) & ~(uintptr_t)15;
  void** s = (void**)top;
  s[-1] = nullptr;                     // where fiber_main would return to (it never does)
  s[-2] = (void*)&fiber_main;
  for (int i = 3; i <= 8; ++i) s[-i] = nullptr;
  f.sp = (void*)(s - 8);
}

// ---- guarded memory ----------------------------------------------------------------------------
struct Range { uintptr_t lo, hi, map_lo; size_t map_bytes; std::string name; };
static std::vector<Range> g_ranges;
static const size_t PAGE = 4096;

static struct sigaction g_old_actions[64];

static void on_fault(int sig, siginfo_t* info, void* uctx) {
  if (g_cur == nullptr) {
    // not inside a simulated kernel: whoever handled this signal before (Python's fault handler,
    // the default action) gets it
    const struct sigaction& old = g_old_actions[sig];
    if ((old.sa_flags & SA_SIGINFO) && old.sa_sigaction) { old.sa_sigaction(sig, info, uctx); return; }
    if (old.sa_handler != SIG_DFL && old.sa_handler != SIG_IGN && old.sa_handler) { old.sa_handler(sig); return; }
    signal(sig, SIG_DFL);
    return;
  }
  const uintptr_t a = (uintptr_t)info->si_addr;
  char where[256] = "no guarded tensor is near";
  for (const Range& r : g_ranges) {
    if (a >= r.map_lo && a < r.map_lo + r.map_bytes) {
      if (a >= r.hi) snprintf(where, sizeof(where), "%ld bytes past the end of '%s' (%ld bytes)", (long)(a - r.hi), r.name.c_str(), (long)(r.hi - r.lo));
      else if (a < r.lo) snprintf(where, sizeof(where), "%ld bytes before the start of '%s' (%ld bytes)", (long)(r.lo - a), r.name.c_str(), (long)(r.hi - r.lo));
      else snprintf(where, sizeof(where), "inside '%s'?", r.name.c_str());
      break;
    }
  }
  fprintf(stderr, "[simt] signal %d: access to %p, %s; kernel %s, workgroup (%u,%u,%u) of (%u,%u,%u), thread %d of %u\n", sig,
          info->si_addr, where, g_kernel, g_block_idx.x, g_block_idx.y, g_block_idx.z, g_grid_dim.x, g_grid_dim.y,
          g_grid_dim.z, g_cur ? g_cur->flat : -1, g_block_dim.x * g_block_dim.y * g_block_dim.z);
  fflush(stderr);
  _exit(97);
}

static void install_handler() {
  static bool done = false;
  if (done) return;
  done = true;
  static char alt[1 << 16];
  stack_t ss;
  ss.ss_sp = alt; ss.ss_size = sizeof(alt); ss.ss_flags = 0;
  sigaltstack(&ss, nullptr);
  struct sigaction sa;
  memset(&sa, 0, sizeof(sa));
  sa.sa_sigaction = on_fault;
  sa.sa_flags = SA_SIGINFO | SA_ONSTACK;
  sigaction(SIGSEGV, &sa, &g_old_actions[SIGSEGV]);
  sigaction(SIGBUS, &sa, &g_old_actions[SIGBUS]);
  sigaction(SIGILL, &sa, &g_old_actions[SIGILL]);      // a trap of a build with -fsanitize-trap: si_addr is the instruction
  sigaction(SIGFPE, &sa, &g_old_actions[SIGFPE]);
}

void launch(const char* name, dim3 grid, dim3 block, Body body, void* arg) {
  const int nthreads = (int)(block.x * block.y * block.z);
  if (nthreads <= 0 || nthreads > MAX_THREADS || nthreads % WAVE != 0) {
    fprintf(stderr, "[simt] kernel %s: %d threads a workgroup\n", name, nthreads);
    _exit(95);
  }
  install_handler();
  if (!g_stacks_ready) {
    char* all = (char*)mmap(nullptr, STACK_BYTES * MAX_THREADS, PROT_READ | PROT_WRITE,
                            MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (all == MAP_FAILED) { perror("mmap stacks"); _exit(95); }
    for (int i = 0; i < MAX_THREADS; ++i) g_fibers[i].stack = all + (size_t)i * STACK_BYTES;
    g_stacks_ready = true;
  }
  ++g_launches;
  g_kernel = name;
  g_body = body;
  g_body_arg = arg;
  g_block_dim = Idx{block.x, block.y, block.z};
  g_grid_dim = Idx{grid.x, grid.y, grid.z};
  const int nwaves = nthreads / WAVE;
  for (unsigned bz = 0; bz < grid.z; ++bz)
    for (unsigned by = 0; by < grid.y; ++by)
      for (unsigned bx = 0; bx < grid.x; ++bx) {
        g_block_idx = Idx{bx, by, bz};
        memset(__start_simt_lds, 0x7f, __stop_simt_lds - __start_simt_lds);
        g_block_gate = Gate();
        g_block_gate.alive = nthreads;
        for (int w = 0; w < nwaves; ++w) { g_waves[w].gate = Gate(); g_waves[w].gate.alive = WAVE; }
        for (int t = 0; t < nthreads; ++t) {
          Fiber& f = g_fibers[t];
          f.state = READY;
          f.flat = t;
          f.lane = t % WAVE;
          f.tid = Idx{(unsigned)t % block.x, ((unsigned)t / block.x) % block.y, (unsigned)t / (block.x * block.y)};
          f.wave = &g_waves[t / WAVE];
          f.xpar = f.fpar = 0;
          prepare_fiber(f);
        }
        int remaining = nthreads;
        while (remaining > 0) {
          bool progressed = false;
          for (int t0 = 0; t0 < nthreads; ++t0) {
            const int t = g_reverse ? nthreads - 1 - t0 : t0;
            Fiber& f = g_fibers[t];
            if (f.state == DONE) continue;
            if (f.state == WAITING) {
              if (f.wait_gate->gen == f.wait_gen) continue;
              f.state = READY;
            }
            g_cur = &f;
            simt_switch(&g_sched_sp, f.sp);
            progressed = true;
            if (f.state == DONE) {
              --remaining;
              // a thread that has ended no longer counts at the barriers
              Gate* gates[2] = {&f.wave->gate, &g_block_gate};
              for (Gate* g : gates) {
                --g->alive;
                if (g->alive > 0 && g->arrived >= g->alive) { g->arrived = 0; ++g->gen; }
              }
            }
          }
          if (!progressed) {
            g_cur = nullptr;
            for (int t = 0; t < nthreads; ++t)
              if (g_fibers[t].state == WAITING) { g_cur = &g_fibers[t]; break; }
            die("deadlock: threads wait at a barrier or cross-lane operation that the others never reach");
          }
        }
        g_cur = nullptr;
      }
  g_kernel = "(none)";
}

}  // namespace simt

// A tensor's memory with a protected page on both sides.  at_start = 0: the tensor ends right at
// the protected page behind it (rounded up to 16 bytes); 1: it starts right after the page in front.
extern "C" void* sim_alloc(size_t nbytes, int at_start, const char* name) {
  using namespace simt;
  install_handler();
  const size_t body = ((nbytes ? nbytes : 1) + PAGE - 1) / PAGE * PAGE;
  const size_t total = body + 2 * PAGE;
  char* m = (char*)mmap(nullptr, total, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
  if (m == MAP_FAILED) return nullptr;
  mprotect(m, PAGE, PROT_NONE);
  mprotect(m + PAGE + body, PAGE, PROT_NONE);
  const size_t padded = (nbytes + 15) / 16 * 16;
  char* p = at_start ? m + PAGE : m + PAGE + body - padded;
  memset(m + PAGE, 0x7f, body);        // what nobody wrote is a large number, a far address, a NaN-free float
  g_ranges.push_back(Range{(uintptr_t)p, (uintptr_t)p + nbytes, (uintptr_t)m, total, name ? name : "?"});
  return p;
}

extern "C" int sim_free(void* p) {
  using namespace simt;
  for (size_t i = 0; i < g_ranges.size(); ++i)
    if (g_ranges[i].lo == (uintptr_t)p) {
      munmap((void*)g_ranges[i].map_lo, g_ranges[i].map_bytes);
      g_ranges[i] = g_ranges.back();
      g_ranges.pop_back();
      return 0;
    }
  return 1;
}

// 0: a workgroup's threads run in ascending order between barriers, 1: in descending order.  A kernel
// that lacks a barrier between a write and a read of workgroup memory shows in at least one of them.
extern "C" void sim_set_order(int reverse) { simt::g_reverse = reverse != 0; }

extern "C" long sim_launch_count() { return simt::g_launches; }
