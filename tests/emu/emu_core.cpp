// Lockstep-wave emulation behind the host stand-in for <hip/hip_runtime.h> (include/hip/hip_runtime.h in this
// folder). Test infrastructure only.
//
// A launch runs workgroup after workgroup on the calling thread. Each thread of a workgroup is a fiber with its own
// stack; a fiber runs until it reaches a barrier or a wave-wide operation, then the scheduler resumes the next one.
// A wave-wide operation completes when every live lane of the wave has arrived at one; if the whole workgroup is
// stuck (lanes of a wave took different branches), the lanes that did arrive complete theirs among themselves, which
// is what the execution mask does on the GPU.
//
// Environment: EMU_CUS   number of compute units hipGetDeviceProperties reports (default 8)
//              EMU_XCDS  number of XCDs hipDeviceGetAttribute reports (default 8)
//              EMU_LDS_POISON  set: every workgroup starts with LDS full of 0xFF bytes (NaN patterns)
//              EMU_DMA   "late" (default): a global->LDS load writes LDS when its wave's counter wait retires it,
//                        the latest moment the hardware allows; "early": at issue, the earliest
//              EMU_SEED  non-zero: fibers are resumed in a shuffled order (changes which wave runs ahead)
#include <hip/hip_runtime.h>

#include <dlfcn.h>
#include <execinfo.h>
#include <signal.h>
#include <unistd.h>
#include <sys/mman.h>
#include <vector>

dim3 threadIdx, blockIdx, blockDim, gridDim;

// EMU_TSAN: the kernels are compiled with ThreadSanitizer (this file is not) and every wave is one of its fibers, so
// that it reports accesses of two waves of a workgroup to the same bytes (LDS or global memory) that no barrier
// orders, whatever the order they happen to run in here. Lanes of one wave share a fiber: within a wave the
// instruction order is the order. Workgroups and launches are ordered one after the other.
#ifdef EMU_TSAN
extern "C" {
void* __tsan_get_current_fiber(void);
void* __tsan_create_fiber(unsigned flags);
void __tsan_destroy_fiber(void* fiber);
void __tsan_switch_to_fiber(void* fiber, unsigned flags);
void __tsan_acquire(void* addr);
void __tsan_release(void* addr);
}
#define TSAN(x) x
#else
#define TSAN(x)
#endif

extern "C" char __start_emu_lds[];
extern "C" char __stop_emu_lds[];

namespace emu {
namespace {

struct Ctx { void* rsp; };
extern "C" void emu_switch(Ctx* from, Ctx* to);
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
  movq (%rsi), %rsp
  popq %r15
  popq %r14
  popq %r13
  popq %r12
  popq %rbx
  popq %rbp
  ret
.size emu_switch, .-emu_switch
)");

constexpr size_t STACK = 1 << 20;
constexpr int MAX_THREADS = 1024;
enum State { READY, WAVE_WAIT, BAR_WAIT, DONE };

struct Pending { const char* src; char* dst; int bytes; };
struct Fiber {
  Ctx ctx;
  int tid;
  State state;
  uint64_t wait_gen;
  std::vector<Pending> dmaq;
};
struct Wave {
  int alive, waiting;
  bool wait[64];
  bool join[64];                 // the lane waits at a join point (wave_join): for every live lane of the wave
  const void* site[64];          // where the lane waits (the call that started the exchange, or its end)
  uint64_t epoch[64];            // how often the lane has moved backwards in the code (loop iterations, roughly)
  unsigned long long mask[64];   // lanes of the exchange the lane was released from last
  alignas(16) unsigned char slot[64][64];
};

char* g_stacks = nullptr;
Fiber g_f[MAX_THREADS];
Wave g_w[MAX_THREADS / 64];
Ctx g_sched;
Fiber* g_cur = nullptr;
int g_nt = 0, g_alive = 0, g_bar_arrived = 0;
uint64_t g_bar_gen = 0;
const std::function<void()>* g_body = nullptr;
alignas(1024) __attribute__((section("emu_lds"))) char g_dyn_lds[160 * 1024];
bool g_dma_early = false;
unsigned g_seed = 0;
uint64_t g_nonuniform = 0;

#ifdef EMU_TSAN
void* g_tsan_main = nullptr;
void* g_tsan_wave[MAX_THREADS / 64];
// Sync objects: one per barrier generation (mod 64), launch start, workgroup end. The sanitizer keys them by address
// in 8-byte cells, so each gets a cache line of its own.
struct alignas(64) SyncCell { char c[64]; };
SyncCell g_tsan_bar_cells[64], g_tsan_launch_cell, g_tsan_done_cell;
#define g_tsan_launch g_tsan_launch_cell.c[0]
#define g_tsan_done g_tsan_done_cell.c[0]
#endif

void yield() {
  TSAN(__tsan_switch_to_fiber(g_tsan_main, 1));  // 1 = no synchronisation implied by the switch
  emu_switch(&g_cur->ctx, &g_sched);
}

uint64_t g_divergent = 0;
// Lanes of a wave that wait at the same place are released together once no lane of the wave can still join them:
// all live lanes wait at exchanges (force = false), or nothing in the workgroup can run (force = true). When they wait
// at different places (lanes took different branches, or left a loop at different times), the lanes that are behind
// in the program go first and meet the others further down, as the hardware runs a branch to its join point.
// "Behind" is judged by (epoch, code address): a lane's epoch goes up whenever its next exchange lies at a lower
// address than its last one (a loop's back edge); lanes released together continue with the same epoch.
// That guess fails where a divergent region ends a loop body (the lanes that skipped it wait at the top of the next
// iteration, at a lower address and the same epoch as the lanes inside it). A kernel marks such a place with
// __builtin_amdgcn_wave_barrier() (wave_join below): lanes that wait there are released only when every live lane of
// the wave has arrived, so lanes still inside a divergent region always go first.
void try_release(Wave& w, bool force) {
  if (w.waiting == 0 || (!force && w.waiting < w.alive)) return;
  bool other = false;  // some lane waits at an ordinary exchange
  for (int l = 0; l < 64; ++l) other |= w.wait[l] && !w.join[l];
  int pick = -1;
  for (int l = 0; l < 64; ++l)
    if (w.wait[l] && !(other && w.join[l]) &&
        (pick < 0 || w.epoch[l] < w.epoch[pick] || (w.epoch[l] == w.epoch[pick] && w.site[l] < w.site[pick]))) pick = l;
  unsigned long long m = 0;
  uint64_t top = 0;
  for (int l = 0; l < 64; ++l)
    if (w.wait[l] && w.site[l] == w.site[pick]) { m |= 1ull << l; top = std::max(top, w.epoch[l]); }
  for (int l = 0; l < 64; ++l)
    if ((m >> l) & 1) { w.wait[l] = false; w.mask[l] = m; w.epoch[l] = top; --w.waiting; }
  if (__builtin_popcountll(m) != w.alive && g_divergent++ < 8 && getenv("EMU_TRACE")) {
    Dl_info info;
    dladdr(w.site[pick], &info);
    fprintf(stderr, "emu: exchange among part of a wave: lanes %016llx of %d live ones, caller +0x%zx (block %u wave %d)\n", m, w.alive,
            (size_t)((const char*)w.site[pick] - (const char*)info.dli_fbase), blockIdx.x, (int)(&w - g_w));
  }
}
void release_barrier() {
  g_bar_arrived = 0;
  ++g_bar_gen;
}

void drain(Fiber& f, size_t keep) {
  size_t n = f.dmaq.size();
  if (n <= keep) return;
  for (size_t i = 0; i < n - keep; ++i) memcpy(f.dmaq[i].dst, f.dmaq[i].src, f.dmaq[i].bytes);
  f.dmaq.erase(f.dmaq.begin(), f.dmaq.begin() + (n - keep));
}

void fiber_main() {
  Fiber* f = g_cur;
  TSAN(__tsan_acquire(&g_tsan_launch));
  (*g_body)();
  drain(*f, 0);
  TSAN(__tsan_release(&g_tsan_done));
  f->state = DONE;
  Wave& w = g_w[f->tid >> 6];
  --w.alive;
  --g_alive;
  try_release(w, false);
  if (g_bar_arrived > 0 && g_bar_arrived == g_alive) release_barrier();
  yield();
  fail("a finished fiber was resumed");
}

void wave_sync(const void* site, bool join = false) {
  Fiber* f = g_cur;
  Wave& w = g_w[f->tid >> 6];
  const int l = f->tid & 63;
  w.wait[l] = true;
  w.join[l] = join;
  if (site < w.site[l]) ++w.epoch[l];
  w.site[l] = site;
  ++w.waiting;
  try_release(w, false);
  if (!w.wait[l]) return;
  f->state = WAVE_WAIT;
  while (w.wait[l]) yield();
  f->state = READY;
}

bool runnable(const Fiber& f) {
  switch (f.state) {
    case READY: return true;
    case WAVE_WAIT: return !g_w[f.tid >> 6].wait[f.tid & 63];
    case BAR_WAIT: return g_bar_gen != f.wait_gen;
    default: return false;
  }
}

void run_workgroup(unsigned order_seed) {
  const int nt = g_nt;
  static std::vector<int> order;
  order.resize(nt);
  for (int i = 0; i < nt; ++i) order[i] = i;
  if (order_seed) {
    // Shuffle whole waves and the lanes inside them (a wave's lanes still meet at their exchanges).
    uint32_t s = order_seed;
    auto rnd = [&]() { s = s * 1664525u + 1013904223u; return s >> 8; };
    for (int i = nt - 1; i > 0; --i) std::swap(order[i], order[rnd() % (i + 1)]);
  }
  for (int i = 0; i < nt; ++i) {
    Fiber& f = g_f[i];
    f.tid = i;
    f.state = READY;
    f.dmaq.clear();
    char* top = g_stacks + (size_t)(i + 1) * STACK;
    void** sp = (void**)(top - 16);
    *sp = (void*)&fiber_main;  // return address of the first switch
    sp -= 6;                   // rbp rbx r12 r13 r14 r15
    for (int k = 0; k < 6; ++k) sp[k] = nullptr;
    f.ctx.rsp = sp;
  }
  for (int w = 0; w < (nt + 63) / 64; ++w) {
    g_w[w].alive = std::min(64, nt - 64 * w);
    g_w[w].waiting = 0;
    memset(g_w[w].wait, 0, sizeof(g_w[w].wait));
    memset(g_w[w].join, 0, sizeof(g_w[w].join));
    memset(g_w[w].site, 0, sizeof(g_w[w].site));
    memset(g_w[w].epoch, 0, sizeof(g_w[w].epoch));
  }
  g_alive = nt;
  g_bar_arrived = 0;
#ifdef EMU_TSAN
  // A workgroup's fibers start knowing everything the main fiber knows, which includes the workgroups before it
  // (LDS and the lanes' stacks are reused from one workgroup to the next): the check is for waves of one workgroup.
  for (int w = 0; w < (nt + 63) / 64; ++w) g_tsan_wave[w] = __tsan_create_fiber(0);
#endif
  while (g_alive > 0) {
    bool progress = false;
    for (int k = 0; k < nt; ++k) {
      Fiber& f = g_f[order[k]];
      if (!runnable(f)) continue;
      progress = true;
      g_cur = &f;
      threadIdx = dim3(f.tid % blockDim.x, (f.tid / blockDim.x) % blockDim.y, f.tid / (blockDim.x * blockDim.y));
      TSAN(__tsan_switch_to_fiber(g_tsan_wave[f.tid >> 6], 1));
      emu_switch(&g_sched, &f.ctx);
    }
    if (progress) continue;
    // Stuck: lanes of a wave are at different places. Let the lanes that wait at an exchange finish it without the others.
    bool released = false;
    for (int w = 0; w < (nt + 63) / 64; ++w)
      if (g_w[w].waiting > 0) { try_release(g_w[w], true); released = true; }
    if (!released) fail("deadlock: every thread of the workgroup waits at a barrier that cannot complete");
  }
#ifdef EMU_TSAN
  __tsan_acquire(&g_tsan_done);
  for (int w = 0; w < (nt + 63) / 64; ++w) __tsan_destroy_fiber(g_tsan_wave[w]);
#endif
}

}  // namespace

void fail(const char* what) {
  fprintf(stderr, "emu: %s (block %u,%u thread %d)\n", what, blockIdx.x, blockIdx.y, g_cur ? g_cur->tid : -1);
  fflush(stderr);
  abort();
}

// EMU_TRACE: a memory fault inside a kernel prints where it happened (addresses relative to the library's load
// address, for llvm-symbolizer) before the process dies.
static void on_segv(int, siginfo_t* si, void*) {
  Dl_info info;
  dladdr((void*)&on_segv, &info);
  fprintf(stderr, "emu: memory fault at address %p in block %u,%u thread %d; library base %p; frames:\n", si->si_addr, blockIdx.x,
          blockIdx.y, g_cur ? g_cur->tid : -1, info.dli_fbase);
  void* frames[24];
  const int n = backtrace(frames, 24);
  for (int i = 0; i < n; ++i) fprintf(stderr, "  +0x%zx\n", (size_t)((char*)frames[i] - (char*)info.dli_fbase));
  fflush(stderr);
  _exit(139);
}

void launch(dim3 grid, dim3 block, size_t dyn, const std::function<void()>& body) {
  static bool handler = false;
  if (!handler && getenv("EMU_TRACE")) {
    handler = true;
    static char alt[1 << 16];
    stack_t ss{alt, 0, sizeof(alt)};
    sigaltstack(&ss, nullptr);
    struct sigaction sa;
    memset(&sa, 0, sizeof(sa));
    sa.sa_sigaction = on_segv;
    sa.sa_flags = SA_SIGINFO | SA_ONSTACK;
    sigaction(SIGSEGV, &sa, nullptr);
  }
  const int nt = (int)(block.x * block.y * block.z);
  if (nt <= 0 || nt > MAX_THREADS) fail("block size");
  if (dyn > sizeof(g_dyn_lds)) fail("dynamic LDS size");
  if ((size_t)(__stop_emu_lds - __start_emu_lds) >= (1ull << 32)) fail("LDS range does not fit 32-bit addresses");
  if (!g_stacks) {
    g_stacks = (char*)mmap(nullptr, STACK * MAX_THREADS, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (g_stacks == (char*)MAP_FAILED) fail("mmap of the fiber stacks");
  }
  const char* d = getenv("EMU_DMA");
  g_dma_early = d && d[0] == 'e';
  const char* s = getenv("EMU_SEED");
  g_seed = s ? (unsigned)atoi(s) : 0;
  g_nt = nt;
  g_body = &body;
  blockDim = block;
  gridDim = grid;
  TSAN(g_tsan_main = __tsan_get_current_fiber());
  TSAN(__tsan_release(&g_tsan_launch));
  unsigned wg = 0;
  const bool poison = getenv("EMU_LDS_POISON") != nullptr;
  for (unsigned z = 0; z < grid.z; ++z)
    for (unsigned y = 0; y < grid.y; ++y)
      for (unsigned x = 0; x < grid.x; ++x, ++wg) {
        blockIdx = dim3(x, y, z);
        // EMU_LDS_POISON: a workgroup starts with all of LDS holding 0xFF bytes (NaN as bf16, fp16 and fp32), as
        // far from a previous workgroup's leftovers as it gets: an output that depends on LDS bytes its own
        // workgroup never wrote comes out as NaN.
        if (poison) memset(__start_emu_lds, 0xFF, (size_t)(__stop_emu_lds - __start_emu_lds));
        run_workgroup(g_seed ? g_seed * 2654435761u + wg * 40503u + 1u : 0u);
        // ... and nothing may have been written behind the launch's dynamic LDS size (the GPU drops such writes)
        if (poison)
          for (size_t b = dyn; b < sizeof(g_dyn_lds); ++b)
            if ((unsigned char)g_dyn_lds[b] != 0xFF) fail("write beyond the dynamic LDS size of the launch");
      }
  g_cur = nullptr;
}

void* dyn_lds() { return g_dyn_lds; }

void syncthreads() {
  Fiber* f = g_cur;
  TSAN(char* sync = &g_tsan_bar_cells[g_bar_gen & 63].c[0]);
  TSAN(__tsan_release(sync));
  if (++g_bar_arrived == g_alive) {
    release_barrier();
  } else {
    f->wait_gen = g_bar_gen;
    f->state = BAR_WAIT;
    while (g_bar_gen == f->wait_gen) yield();
    f->state = READY;
  }
  TSAN(__tsan_acquire(sync));
}

int lane() { return g_cur->tid & 63; }

__attribute__((noinline)) const unsigned char* exchange(const void* mine, int bytes, const void* site) {
  if (!site) site = __builtin_return_address(0);
  Wave& w = g_w[g_cur->tid >> 6];
  memcpy(w.slot[g_cur->tid & 63], mine, bytes);
  wave_sync(site);
  return &w.slot[0][0];
}
unsigned long long exchange_mask() { return g_w[g_cur->tid >> 6].mask[g_cur->tid & 63]; }
__attribute__((noinline)) void exchange_done(const void* site) {
  if (!site) site = __builtin_return_address(0);
  wave_sync((const char*)site + 1);
}

// A place where the whole wave is together again (the top of a loop whose body ends in a divergent region).
__attribute__((noinline)) void wave_join() { wave_sync(__builtin_return_address(0), true); }

__attribute__((noinline)) int readfirstlane(int v) {
  const void* site = __builtin_return_address(0);
  const unsigned char* t = exchange(&v, 4, site);
  const unsigned long long m = exchange_mask();
  int r;
  memcpy(&r, t + 64 * (__builtin_ffsll((long long)m) - 1), 4);
  if (r != v) {
    // Not an error by itself (the GPU also takes the first active lane's value), but rarely what a kernel means.
    if (g_nonuniform++ < 8 && getenv("EMU_TRACE")) {
      Dl_info info;
      void* ra = __builtin_return_address(0);
      dladdr(ra, &info);
      fprintf(stderr, "emu: readfirstlane of a value that differs between lanes: lane %d has %d, first lane %d; caller +0x%zx (block %u thread %d)\n",
              lane(), v, r, (size_t)((char*)ra - (char*)info.dli_fbase), blockIdx.x, g_cur->tid);
    }
  }
  exchange_done(site);
  return r;
}

__attribute__((noinline)) unsigned long long ballot(int pred) {
  const void* site = __builtin_return_address(0);
  const unsigned char* t = exchange(&pred, 4, site);
  const unsigned long long m = exchange_mask();
  unsigned long long r = 0;
  for (int l = 0; l < 64; ++l) {
    int p;
    memcpy(&p, t + 64 * l, 4);
    if (((m >> l) & 1) && p) r |= 1ull << l;
  }
  exchange_done(site);
  return r;
}

char* lds_ptr(uint32_t addr, int bytes) {
  const uintptr_t base = (uintptr_t)__start_emu_lds, end = (uintptr_t)__stop_emu_lds;
  uintptr_t p = (base & ~0xFFFFFFFFull) | addr;
  if (p < base) p += 1ull << 32;
  if (p < base || p + bytes > end) fail("LDS address out of range");
  return (char*)p;
}

void dma(int bytes, const void* sbase, uint32_t voff, uint32_t lds_addr) {
  Fiber* f = g_cur;
  Pending q{(const char*)sbase + voff, lds_ptr(lds_addr + (uint32_t)bytes * (uint32_t)(f->tid & 63), bytes), bytes};
  if (g_dma_early) memcpy(q.dst, q.src, bytes);
  else f->dmaq.push_back(q);
}
// s_waitcnt is a wave-wide instruction: when a lane passes it, every lane of the wave has issued the loads before it
// and (all but the newest n of) them have landed, for all lanes.
__attribute__((noinline)) void wait_vm(int n) {
  const char* site = (const char*)__builtin_return_address(0);
  wave_sync(site);
  drain(*g_cur, (size_t)n);
  wave_sync(site + 1);
}
// s_waitcnt lgkmcnt(0): the wave's LDS accesses so far are complete, for all lanes.
__attribute__((noinline)) void wait_lds() {
  const char* site = (const char*)__builtin_return_address(0);
  wave_sync(site);
}

// ---- matrix instructions: lane l holds row / column l % 16 and the k chunk l / 16 of its operand; of the result,
// rows 4 (l / 16) .. + 3 of column l % 16 (A = first operand: rows; B = second: columns).
template <class V, int KL>
static f32x4 mfma_generic(V a, V b, f32x4 c, float (*cvt)(const unsigned char*, int), const void* site) {
  struct { V a, b; } mine{a, b};
  static_assert(sizeof(mine) <= 64, "");
  const unsigned char* t = exchange(&mine, sizeof(mine), site);
  const int l = lane(), col = l & 15, rq = l >> 4;
  f32x4 d = c;
  for (int r = 0; r < 4; ++r) {
    const int row = 4 * rq + r;
    float acc = 0.f;
    for (int kc = 0; kc < 4; ++kc) {
      const unsigned char* pa = t + 64 * (row + 16 * kc);
      const unsigned char* pb = t + 64 * (col + 16 * kc) + sizeof(V);
      for (int k = 0; k < KL; ++k) acc += cvt(pa, k) * cvt(pb, k);
    }
    d[r] = c[r] + acc;
  }
  exchange_done(site);
  return d;
}
static float cvt_bf16(const unsigned char* p, int k) {
  uint16_t h;
  memcpy(&h, p + 2 * k, 2);
  return __builtin_bit_cast(float, (uint32_t)h << 16);
}
static float cvt_f16(const unsigned char* p, int k) {
  _Float16 h;
  memcpy(&h, p + 2 * k, 2);
  return (float)h;
}
static float fp8_e4m3fn(unsigned char v) {
  const int s = v >> 7, e = (v >> 3) & 15, m = v & 7;
  float r;
  if (e == 15 && m == 7) r = NAN;
  else if (e == 0) r = ldexpf((float)m, -9);
  else r = ldexpf((float)(8 + m), e - 10);
  return s ? -r : r;
}
static float cvt_fp8(const unsigned char* p, int k) { return fp8_e4m3fn(p[k]); }

__attribute__((noinline)) f32x4 mfma_16x16x32_bf16(bf16x8 a, bf16x8 b, f32x4 c) {
  return mfma_generic<bf16x8, 8>(a, b, c, cvt_bf16, __builtin_return_address(0));
}
__attribute__((noinline)) f32x4 mfma_16x16x32_f16(f16x8 a, f16x8 b, f32x4 c) {
  return mfma_generic<f16x8, 8>(a, b, c, cvt_f16, __builtin_return_address(0));
}
__attribute__((noinline)) f32x4 mfma_16x16x128_fp8(i32x8v a, i32x8v b, f32x4 c) {
  const char* site = (const char*)__builtin_return_address(0);
  // 64 bytes per lane do not fit one deposit: two halves of 16 k values each (k chunk l / 16 holds 32 values).
  typedef __attribute__((__vector_size__(16))) int i32x4v;
  f32x4 d = c;
  for (int h = 0; h < 2; ++h) {
    i32x4v ah{a[4 * h], a[4 * h + 1], a[4 * h + 2], a[4 * h + 3]}, bh{b[4 * h], b[4 * h + 1], b[4 * h + 2], b[4 * h + 3]};
    d = mfma_generic<i32x4v, 16>(ah, bh, d, cvt_fp8, site + 2 * h);
  }
  return d;
}

// Transposing LDS read of 16-bit elements: in every group of 16 lanes, lane j supplies the address of 4
// consecutive elements M[j][0..3]; lane i receives R[i][e] = M[4 e + i / 4][i % 4].
__attribute__((noinline)) i16x4 ds_read_tr16_b64(uint32_t lds_addr) {
  const void* site = __builtin_return_address(0);
  uint64_t mine;
  memcpy(&mine, lds_ptr(lds_addr, 8), 8);
  const unsigned char* t = exchange(&mine, 8, site);
  const int l = lane(), g0 = l & ~15, i = l & 15;
  i16x4 r;
  for (int e = 0; e < 4; ++e) {
    short v;
    memcpy(&v, t + 64 * (g0 + 4 * e + i / 4) + 2 * (i % 4), 2);
    r[e] = v;
  }
  exchange_done(site);
  return r;
}

uint32_t perm(uint32_t s0, uint32_t s1, uint32_t sel) {
  const uint64_t src = ((uint64_t)s0 << 32) | s1;
  uint32_t r = 0;
  for (int i = 0; i < 4; ++i) {
    const uint32_t c = (sel >> (8 * i)) & 0xFF;
    uint32_t b;
    if (c <= 7) b = (uint32_t)(src >> (8 * c)) & 0xFF;
    else if (c == 12) b = 0;
    else if (c >= 13) b = 0xFF;
    else { fail("v_perm_b32 selector 8..11 is not modelled"); b = 0; }
    r |= b << (8 * i);
  }
  return r;
}

__attribute__((noinline)) int ds_swizzle(int v, int pattern) {
  const void* site = __builtin_return_address(0);
  const int l = lane();
  int src;
  if (pattern & 0x8000) {
    src = (l & ~3) | ((pattern >> (2 * (l & 3))) & 3);
  } else {
    const int and_m = pattern & 31, or_m = (pattern >> 5) & 31, xor_m = (pattern >> 10) & 31;
    src = (l & 32) | ((((l & 31) & and_m) | or_m) ^ xor_m);
  }
  return get_lane(v, src, site);
}

// fp32 -> e4m3fn, round to nearest even, saturating at +-448 (the kernels scale or clamp into range first).
static unsigned char to_e4m3fn(float x) {
  if (x != x) return 0x7F;
  const uint32_t bits = __builtin_bit_cast(uint32_t, x);
  const unsigned char s = (unsigned char)((bits >> 31) << 7);
  const float a = fabsf(x);
  if (a >= 464.0f) return s | 0x7E;  // beyond the midpoint above 448
  if (a < ldexpf(1.0f, -10)) return s;  // below half of the smallest subnormal 2^-9 (ties to even -> 0)
  int e;
  (void)frexpf(a, &e);  // a = f * 2^e, f in [0.5, 1)
  int exp = e - 1;      // a = 1.xxx * 2^exp
  if (exp < -6) exp = -6;
  const float q = ldexpf(a, 3 - exp);  // in units of the mantissa step
  float rq = nearbyintf(q);            // ties to even in the default rounding mode
  int m = (int)rq;
  int be = exp + 7;
  if (exp == -6 && m < 8) return s | (unsigned char)m;  // subnormal (m in 0..7)
  if (m == 16) { m = 8; ++be; }
  if (be > 15 || (be == 15 && m - 8 > 6)) return s | 0x7E;
  return s | (unsigned char)((be << 3) | (m - 8));
}
int cvt_pk_fp8_f32(float a, float b, int old, bool hi) {
  const uint32_t pair = (uint32_t)to_e4m3fn(a) | ((uint32_t)to_e4m3fn(b) << 8);
  const uint32_t o = (uint32_t)old;
  return (int)(hi ? ((o & 0x0000FFFFu) | (pair << 16)) : ((o & 0xFFFF0000u) | pair));
}

}  // namespace emu

hipError_t hipGetDeviceProperties(hipDeviceProp_t* p, int) {
  const char* c = getenv("EMU_CUS");
  p->multiProcessorCount = c ? atoi(c) : 8;
  return hipSuccess;
}

hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t, int) {
  const char* c = getenv("EMU_XCDS");
  *value = c ? atoi(c) : 8;
  return hipSuccess;
}

extern "C" unsigned long long emu_nonuniform_readfirstlane() { return emu::g_nonuniform; }
extern "C" unsigned long long emu_divergent_exchanges() { return emu::g_divergent; }
