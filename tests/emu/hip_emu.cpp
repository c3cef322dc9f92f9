// TEST INFRASTRUCTURE -- runtime of the host-side HIP emulation (see hip_emu.h): fibers, the
// rendezvous of cross-lane operations and barriers, guarded allocations, error reports.
#include "hip_emu.h"

#include <sys/mman.h>
#include <unistd.h>

#include <cstdio>
#include <cstdlib>
#include <map>
#include <string>
#include <vector>

// ---- context switch (x86-64 System V): saves the callee-saved registers on the old stack -----------
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
.size emu_switch,.-emu_switch
)");

namespace emu {

Ctx* cur = nullptr;
void* dynamic_shared = nullptr;

namespace {

constexpr size_t kStackBytes = 256 * 1024;
constexpr int kMaxThreads = 1024;

struct Wave {
  uint64_t vals[2][64];
  uint64_t live_at[2];
  uint64_t live = 0;        // lanes still inside the kernel
  uint64_t arrived = 0;
  uint64_t gen = 0;
  const char* what = nullptr;
};

struct Fiber {
  Ctx ctx;
  void* sp = nullptr;
  char* stack = nullptr;
  bool done = true;
  const uint64_t* wait_on = nullptr;   // resumes when *wait_on != wait_val
  uint64_t wait_val = 0;
  const char* wait_what = nullptr;
};

Fiber fibers[kMaxThreads];
Wave waves[kMaxThreads / 64];
void* scheduler_sp = nullptr;
Fiber* running = nullptr;
const std::function<void()>* body_of_launch = nullptr;
const char* kernel_name = "";
uint64_t progress = 0;

// workgroup barrier
uint64_t barrier_gen = 0;
int barrier_arrived = 0;
int threads_live = 0;
int threads_total = 0;

hipError_t g_last_error = hipSuccess;
std::map<uintptr_t, size_t> g_blocks;      // guarded allocations: start -> bytes
struct Mapping { void* base; size_t bytes; };
std::map<uintptr_t, Mapping> g_mappings;
std::vector<std::pair<uintptr_t, size_t>> g_registered;   // memory the tests own (numpy arrays)
bool g_check_allocations = true;

void yield_to_scheduler() { emu_switch(&running->sp, scheduler_sp); }

void wait_for(const uint64_t* word, uint64_t old, const char* what) {
  Fiber* f = running;
  f->wait_on = word;
  f->wait_val = old;
  f->wait_what = what;
  while (*word == old) yield_to_scheduler();
  f->wait_on = nullptr;
}

void complete_wave(Wave& w) {
  w.live_at[w.gen & 1] = w.arrived;
  w.arrived = 0;
  ++w.gen;
  ++progress;
  // the buffer of the rendezvous after this one starts clean
  std::memset(w.vals[w.gen & 1], 0, sizeof(w.vals[0]));
}

void complete_barrier() {
  barrier_arrived = 0;
  ++barrier_gen;
  ++progress;
}

void fiber_exit() {
  Fiber* f = running;
  f->done = true;
  ++progress;
  Wave& w = waves[f->ctx.wave];
  w.live &= ~(1ull << f->ctx.lane);
  if (w.arrived != 0 && w.arrived == w.live) complete_wave(w);
  --threads_live;
  if (barrier_arrived > 0 && barrier_arrived == threads_live) complete_barrier();
  yield_to_scheduler();
  std::fprintf(stderr, "emu: a finished fiber was resumed\n");
  std::abort();
}

extern "C" void emu_fiber_entry() {
  (*body_of_launch)();
  fiber_exit();
}

void start_fiber(Fiber& f) {
  if (f.stack == nullptr) {
    f.stack = static_cast<char*>(mmap(nullptr, kStackBytes, PROT_READ | PROT_WRITE,
                                      MAP_PRIVATE | MAP_ANONYMOUS | MAP_STACK, -1, 0));
    if (f.stack == MAP_FAILED) fail("cannot map a fiber stack");
    mprotect(f.stack, 4096, PROT_NONE);              // overflow faults instead of corrupting
  }
  uintptr_t top = (reinterpret_cast<uintptr_t>(f.stack) + kStackBytes) & ~(uintptr_t)15;
  void** sp = reinterpret_cast<void**>(top);
  *--sp = nullptr;                                   // where the entry would return to
  *--sp = reinterpret_cast<void*>(&emu_fiber_entry); // popped by emu_switch's ret
  for (int i = 0; i < 6; ++i) *--sp = nullptr;       // rbp rbx r12 r13 r14 r15
  f.sp = sp;
  f.done = false;
  f.wait_on = nullptr;
}

void describe_and_abort(const char* what) {
  std::fprintf(stderr, "emu: %s\n  kernel %s", what, kernel_name);
  if (cur != nullptr)
    std::fprintf(stderr, ", block (%u,%u,%u) of (%u,%u,%u), thread %d (wave %d lane %d)", cur->bid.x,
                 cur->bid.y, cur->bid.z, cur->gdim.x, cur->gdim.y, cur->gdim.z, cur->linear,
                 cur->wave, cur->lane);
  std::fprintf(stderr, "\n");
  std::fflush(stderr);
  _exit(86);
}

}  // namespace
}  // namespace emu
// bounds of the section that holds every __shared__ array (hip_emu.h), provided by the linker
extern "C" char __start_emu_lds[] __attribute__((weak));
extern "C" char __stop_emu_lds[] __attribute__((weak));
namespace emu {
namespace {

// EMU_ORDER=reverse: threads (hence waves) and workgroups are run last to first.  Between two
// meeting points a thread runs alone, so the results may not depend on who goes first: if they do,
// a barrier is missing, or a workgroup relies on another.
bool reverse_order() {
  static const bool on = [] {
    const char* m = std::getenv("EMU_ORDER");
    return m != nullptr && !std::strcmp(m, "reverse");
  }();
  return on;
}

void run_block(int nthreads) {
  if (__start_emu_lds != nullptr && __stop_emu_lds > __start_emu_lds)
    std::memset(__start_emu_lds, 0xCB, (size_t)(__stop_emu_lds - __start_emu_lds));
  threads_total = threads_live = nthreads;
  barrier_arrived = 0;
  const int nwaves = (nthreads + 63) / 64;
  for (int w = 0; w < nwaves; ++w) {
    const int lanes = std::min(64, nthreads - w * 64);
    waves[w].live = lanes == 64 ? ~0ull : ((1ull << lanes) - 1ull);
    waves[w].arrived = 0;
    waves[w].gen = 0;
    std::memset(waves[w].vals, 0, sizeof(waves[w].vals));
  }
  for (int t = 0; t < nthreads; ++t) start_fiber(fibers[t]);
  uint64_t seen = progress;
  int idle_passes = 0;
  while (threads_live > 0) {
    for (int i = 0; i < nthreads; ++i) {
      Fiber& f = fibers[reverse_order() ? nthreads - 1 - i : i];
      if (f.done) continue;
      if (f.wait_on != nullptr && *f.wait_on == f.wait_val) continue;
      running = &f;
      cur = &f.ctx;
      emu_switch(&scheduler_sp, f.sp);
    }
    if (progress == seen) {
      if (++idle_passes >= 2) {
        std::fprintf(stderr, "emu: deadlock in kernel %s, block (%u,%u,%u): every live thread waits\n",
                     kernel_name, fibers[0].ctx.bid.x, fibers[0].ctx.bid.y, fibers[0].ctx.bid.z);
        for (int t = 0; t < nthreads; ++t)
          if (!fibers[t].done && (t % 64 == 0 || fibers[t].wait_what != fibers[t - 1].wait_what))
            std::fprintf(stderr, "  thread %d waits in %s\n", t,
                         fibers[t].wait_what ? fibers[t].wait_what : "?");
        std::fflush(stderr);
        _exit(87);
      }
    } else {
      idle_passes = 0;
      seen = progress;
    }
  }
  running = nullptr;
  cur = nullptr;
}

}  // namespace

[[noreturn]] void fail(const char* what) {
  describe_and_abort(what);
  std::abort();
}

hipError_t last_error() {
  const hipError_t e = g_last_error;
  g_last_error = hipSuccess;
  return e;
}

void launch(dim3 grid, dim3 block, size_t shared_bytes, const std::function<void()>& body,
            const char* name) {
  const size_t nthreads = (size_t)block.x * block.y * block.z;
  if (nthreads == 0 || nthreads > (size_t)kMaxThreads || shared_bytes > 160 * 1024 ||
      grid.x == 0 || grid.y == 0 || grid.z == 0 || grid.y > 65535 || grid.z > 65535) {
    g_last_error = hipErrorInvalidValue;
    return;
  }
  if (running != nullptr) fail("launch from inside a kernel");
  kernel_name = name;
  body_of_launch = &body;
  std::vector<char> shared(shared_bytes + 64);
  dynamic_shared = shared.data();
  const bool backwards = reverse_order();
  for (unsigned iz = 0; iz < grid.z; ++iz)
    for (unsigned iy = 0; iy < grid.y; ++iy)
      for (unsigned ix = 0; ix < grid.x; ++ix) {
        const unsigned bx = backwards ? grid.x - 1 - ix : ix, by = backwards ? grid.y - 1 - iy : iy,
                       bz = backwards ? grid.z - 1 - iz : iz;
        std::memset(shared.data(), 0xCB, shared.size());     // dynamic LDS starts as garbage too
        for (size_t t = 0; t < nthreads; ++t) {
          Ctx& c = fibers[t].ctx;
          c.tid = make_uint3((unsigned)(t % block.x), (unsigned)((t / block.x) % block.y),
                             (unsigned)(t / ((size_t)block.x * block.y)));
          c.bid = make_uint3(bx, by, bz);
          c.bdim = block;
          c.gdim = grid;
          c.linear = (int)t;
          c.lane = (int)(t & 63);
          c.wave = (int)(t >> 6);
        }
        run_block((int)nthreads);
      }
  body_of_launch = nullptr;
  dynamic_shared = nullptr;
}

const uint64_t* gather(uint64_t mine, uint64_t* live_mask, const char* what) {
  if (running == nullptr) fail("cross-lane operation outside a kernel");
  Wave& w = waves[cur->wave];
  const uint64_t gen = w.gen;
  const int buf = (int)(gen & 1);
  const uint64_t bit = 1ull << cur->lane;
  if (w.arrived & bit) fail("a lane arrived twice at one rendezvous");
  if (w.arrived != 0 && w.what != what && std::strcmp(w.what, what) != 0) {
    std::string msg = std::string("lanes of a wave met in different operations: ") + w.what +
                      " and " + what;
    fail(msg.c_str());
  }
  w.what = what;
  w.vals[buf][cur->lane] = mine;
  w.arrived |= bit;
  if (w.arrived == w.live) complete_wave(w);
  else wait_for(&w.gen, gen, what);
  *live_mask = w.live_at[buf];
  return w.vals[buf];
}

void barrier() {
  if (running == nullptr) fail("barrier outside a kernel");
  const uint64_t gen = barrier_gen;
  ++barrier_arrived;
  if (barrier_arrived == threads_live) complete_barrier();
  else wait_for(&barrier_gen, gen, "__syncthreads");
}

// ---- memory ---------------------------------------------------------------------------------------
void* allocate(size_t bytes, size_t align) {
  const size_t page = 4096;
  const size_t rounded = (std::max<size_t>(bytes, 1) + align - 1) & ~(align - 1);
  const size_t body = (rounded + page - 1) / page * page;
  char* base = static_cast<char*>(mmap(nullptr, body + 2 * page, PROT_READ | PROT_WRITE,
                                       MAP_PRIVATE | MAP_ANONYMOUS, -1, 0));
  if (base == MAP_FAILED) return nullptr;
  mprotect(base, page, PROT_NONE);
  mprotect(base + page + body, page, PROT_NONE);
  char* p = base + page + body - rounded;            // the block ends where the guard page begins
  std::memset(p, 0xCB, rounded);                     // not zero: nothing may rely on fresh memory
  g_blocks[reinterpret_cast<uintptr_t>(p)] = rounded;
  g_mappings[reinterpret_cast<uintptr_t>(p)] = Mapping{base, body + 2 * page};
  return p;
}

void release(void* p) {
  if (p == nullptr) return;
  auto it = g_mappings.find(reinterpret_cast<uintptr_t>(p));
  if (it == g_mappings.end()) fail("free of a pointer that was not allocated here");
  munmap(it->second.base, it->second.bytes);
  g_mappings.erase(it);
  g_blocks.erase(reinterpret_cast<uintptr_t>(p));
}

bool known(const void* p, size_t bytes) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  auto it = g_blocks.upper_bound(a);
  if (it != g_blocks.begin()) {
    --it;
    if (a >= it->first && a + bytes <= it->first + it->second) return true;
  }
  for (const auto& r : g_registered)
    if (a >= r.first && a + bytes <= r.first + r.second) return true;
  return false;
}

const void* remember(const void* p, size_t bytes) {
  if (!known(p, bytes)) g_registered.emplace_back(reinterpret_cast<uintptr_t>(p), bytes);
  return p;
}

bool buffer_ok(const Rsrc& r, uint32_t offset, uint32_t size, bool store) {
  (void)store;
  if ((uint64_t)offset + size > r.bytes) return false;       // out of range: zero / dropped
  if (g_check_allocations && !known(r.base + offset, size)) {
    std::fprintf(stderr, "emu: buffer %s at offset %u (+%u) is inside its descriptor (%u bytes) but "
                 "outside every allocation\n", store ? "store" : "load", offset, size, r.bytes);
    fail("buffer descriptor larger than the memory behind it");
  }
  return true;
}

}  // namespace emu

// ---- what the tests call ---------------------------------------------------------------------------
namespace emu {
// see hip_emu.h: the exact result, or its neighbour one unit in the last place away
float approx(float exact) {
  static const int mode = [] {
    const char* m = std::getenv("EMU_APPROX");
    if (m == nullptr) return 0;
    return !std::strcmp(m, "up") ? 1 : !std::strcmp(m, "down") ? 2 : !std::strcmp(m, "hash") ? 3 : 0;
  }();
  if (mode == 0 || exact == 0.0f || !std::isfinite(exact)) return exact;
  int step = mode == 1 ? 1 : -1;
  if (mode == 3) {
    // like the hardware: the same result for the same value every time, off either way or not at all
    uint32_t h;
    std::memcpy(&h, &exact, 4);
    h *= 0x9e3779b1u;
    h ^= h >> 15;
    h *= 0x85ebca77u;
    h ^= h >> 13;
    step = (int)(h % 3u) - 1;
    if (step == 0) return exact;
  }
  return std::nextafter(exact, step > 0 ? INFINITY : -INFINITY);
}
}  // namespace emu

extern "C" {
void* emu_alloc(size_t bytes) { return emu::allocate(bytes, 256); }
// the block ends within 15 bytes of an inaccessible page: an overrun faults
void* emu_alloc_tight(size_t bytes) { return emu::allocate(bytes, 16); }
void emu_free(void* p) { emu::release(p); }
// memory owned by the caller (a numpy array) that buffer descriptors may cover
void emu_register(const void* p, size_t bytes) {
  emu::g_registered.emplace_back(reinterpret_cast<uintptr_t>(p), bytes);
}
void emu_unregister_all(void) { emu::g_registered.clear(); }
// 0: buffer descriptors may cover memory the emulator did not allocate (arrays of another allocator)
void emu_check_allocations(int on) { emu::g_check_allocations = on != 0; }
}
