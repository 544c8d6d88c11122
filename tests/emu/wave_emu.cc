// Scheduler, cross-lane operations and guarded memory of the host execution of the HIP kernels
// (wave_emu.h).  Test infrastructure: nothing on the GPU path links this file.
#include "wave_emu.h"

#include <signal.h>
#include <sys/mman.h>
#include <ucontext.h>
#include <unistd.h>

#include <cstdio>
#include <map>
#include <string>
#include <vector>

namespace fa_emu {

dim3 g_thread_idx, g_block_idx, g_block_dim, g_grid_dim;
hipError_t g_last_error = hipSuccess;

namespace {

constexpr size_t kStackBytes = 256 * 1024;
constexpr int kWave = 64;

struct Fiber {
  ucontext_t ctx;
  char *stack = nullptr;
  bool done = false;
  unsigned tid = 0;
};

struct Wave {
  int n_alive = 0, arrived = 0;
  uint64_t gen = 0;
  const char *op = nullptr;
  void (*fn)(const void *const *, void *const *, int, void *) = nullptr;
  void *ctx = nullptr;
  const void *in[kWave];
  void *out[kWave];
};

struct Block {
  std::vector<Fiber> fibers;
  std::vector<Wave> waves;
  ucontext_t main;
  int cur = -1, n_alive = 0;
  int bar_arrived = 0;
  uint64_t bar_gen = 0;
  uint64_t progress = 0;
  const std::function<void()> *body = nullptr;
};

Block *g_blk = nullptr;
bool g_in_fiber = false;   // a lane is running (as opposed to the scheduler)
bool g_abort = false;      // a lane gave up: the scheduler unwinds the launch
std::string g_error;
bool g_faulted = false;
long long g_sel_stride = 1, g_sel_phase = 0, g_blocks_run = 0;
int g_burst = 1;            // > 1: random wave order, up to this many passes in a row for the picked wave
uint64_t g_rng = 1;
std::vector<long long> g_sel_list;

std::vector<char *> g_stacks;                   // lane stacks, indexed by thread id, reused by every workgroup
std::map<uintptr_t, size_t> g_ranges;           // registered [begin, begin + bytes)
int g_caller_ranges = 0;                        // how many of them the caller registered (the rest is library scratch)
struct Guarded { void *map; size_t map_bytes; };
std::map<uintptr_t, Guarded> g_guarded;         // user pointer -> mapping

std::string where() {
  char buf[160];
  std::snprintf(buf, sizeof buf, " [workgroup (%u, %u, %u) of (%u, %u, %u), thread %u]", g_block_idx.x, g_block_idx.y, g_block_idx.z,
                g_grid_dim.x, g_grid_dim.y, g_grid_dim.z, g_thread_idx.x);
  return buf;
}

void yield() {
  Fiber &f = g_blk->fibers[(size_t)g_blk->cur];
  swapcontext(&f.ctx, &g_blk->main);
}

void complete(Wave &w) {
  w.fn(w.in, w.out, w.arrived, w.ctx);
  w.arrived = 0;
  w.op = nullptr;
  ++w.gen;
  ++g_blk->progress;
}

void fiber_entry() {
  Block &b = *g_blk;
  (*b.body)();
  Fiber &f = b.fibers[(size_t)b.cur];
  f.done = true;
  --b.n_alive;
  ++b.progress;
  Wave &w = b.waves[f.tid / kWave];
  --w.n_alive;
  // lanes that have left no longer take part: release who waits for them
  if (w.n_alive > 0 && w.arrived == w.n_alive) complete(w);
  if (b.n_alive > 0 && b.bar_arrived == b.n_alive) { b.bar_arrived = 0; ++b.bar_gen; ++b.progress; }
  swapcontext(&f.ctx, &b.main);
}

// A stray access of a lane: note where, leave the lane for good and go back to the scheduler.
void on_segv(int sig, siginfo_t *si, void *) {
  if (!g_in_fiber || !g_blk) { signal(sig, SIG_DFL); raise(sig); return; }
  char buf[96];
  std::snprintf(buf, sizeof buf, "memory access outside every tensor at %p", si->si_addr);
  g_error = std::string(buf) + where();
  g_abort = true;
  g_in_fiber = false;
  setcontext(&g_blk->main);
}

bool run_block() {
  Block &b = *g_blk;
  const unsigned n = g_block_dim.x * g_block_dim.y * g_block_dim.z;
  b.fibers.assign(n, Fiber{});
  b.waves.assign((n + kWave - 1) / kWave, Wave{});
  b.n_alive = (int)n;
  b.bar_arrived = 0;
  for (unsigned t = 0; t < n; ++t) {
    Fiber &f = b.fibers[t];
    f.tid = t;
    if (t < g_stacks.size()) {
      f.stack = g_stacks[t];  // stacks are kept from one workgroup to the next
    } else {
      f.stack = static_cast<char *>(mmap(nullptr, kStackBytes, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0));
      if (f.stack == MAP_FAILED) { f.stack = nullptr; g_error = "no memory for a lane's stack"; return false; }
      g_stacks.push_back(f.stack);
    }
    getcontext(&f.ctx);
    f.ctx.uc_stack.ss_sp = f.stack;
    f.ctx.uc_stack.ss_size = kStackBytes;
    f.ctx.uc_link = &b.main;
    makecontext(&f.ctx, fiber_entry, 0);
    ++b.waves[t / kWave].n_alive;
  }
  // One pass over a wave resumes each of its lanes once (a lane runs until it blocks at a
  // cross-lane operation or a barrier, or ends).  Order of the waves: round robin, one pass each
  // (the default), or -- to look for missing barriers -- a wave picked at random that is given up
  // to `g_burst` passes in a row, so that it runs as far ahead of the others as the kernel's
  // synchronisation lets it.
  const unsigned n_waves = (unsigned)b.waves.size();
  unsigned w = 0;
  unsigned idle_waves = 0;  // consecutive waves that made no progress
  while (b.n_alive > 0) {
    if (g_burst > 1) {
      g_rng = g_rng * 6364136223846793005ull + 1442695040888963407ull;
      w = (unsigned)((g_rng >> 33) % n_waves);
    }
    const int passes = g_burst > 1 ? 1 + (int)((g_rng >> 20) % (uint64_t)g_burst) : 1;
    bool moved = false;
    for (int pass = 0; pass < passes; ++pass) {
      const uint64_t before = b.progress;
      for (unsigned t = w * kWave; t < std::min(n, (w + 1) * kWave); ++t) {
        Fiber &f = b.fibers[t];
        if (f.done) continue;
        b.cur = (int)t;
        g_thread_idx = dim3(t % g_block_dim.x, (t / g_block_dim.x) % g_block_dim.y, t / (g_block_dim.x * g_block_dim.y));
        g_in_fiber = true;
        swapcontext(&b.main, &f.ctx);
        g_in_fiber = false;
        if (g_abort) return false;
      }
      if (b.progress == before) break;  // the wave waits for the others
      moved = true;
    }
    idle_waves = moved ? 0 : idle_waves + 1;
    if (idle_waves > 64 * n_waves) {  // every wave has been tried many times over (random picks included)
      g_error = "deadlock: the lanes of a workgroup wait at different cross-lane operations or barriers" + where();
      return false;
    }
    if (g_burst <= 1) w = (w + 1) % n_waves;
  }
  return true;
}

void free_stacks() {
  if (g_blk) g_blk->fibers.clear();  // the stacks themselves stay in g_stacks for the next workgroup
}

bool selected(long long id) {
  if (!g_sel_list.empty()) return std::find(g_sel_list.begin(), g_sel_list.end(), id) != g_sel_list.end();
  return id % g_sel_stride == g_sel_phase;
}

}  // namespace

const char *last_error() { return g_error.c_str(); }

[[noreturn]] void fail(const char *what, const void *addr) {
  char buf[64] = "";
  if (addr) std::snprintf(buf, sizeof buf, " (address %p)", addr);
  g_error = std::string(what) + buf + where();
  if (!g_in_fiber || !g_blk) { std::fprintf(stderr, "fa_emu: %s\n", g_error.c_str()); std::abort(); }
  g_abort = true;
  g_in_fiber = false;
  setcontext(&g_blk->main);
  std::abort();  // not reached
}

int launch(dim3 grid, dim3 block, const std::function<void()> &body) {
  if (g_faulted) return -1;
  static bool handler_set = false;
  if (!handler_set) {
    struct sigaction sa;
    std::memset(&sa, 0, sizeof sa);
    sa.sa_sigaction = on_segv;
    sa.sa_flags = SA_SIGINFO | SA_NODEFER;
    sigaction(SIGSEGV, &sa, nullptr);
    sigaction(SIGBUS, &sa, nullptr);
    handler_set = true;
  }
  Block blk;
  blk.body = &body;
  g_blk = &blk;
  g_grid_dim = grid;
  g_block_dim = block;
  g_abort = false;
  long long id = 0;
  for (unsigned z = 0; z < grid.z; ++z)
    for (unsigned y = 0; y < grid.y; ++y)
      for (unsigned x = 0; x < grid.x; ++x, ++id) {
        if (!selected(id)) continue;
        g_block_idx = dim3(x, y, z);
        const bool ok = run_block();
        free_stacks();
        if (!ok) {  // a lane faulted or the workgroup hung: give up the launch, keep the message
          g_faulted = true;
          g_blk = nullptr;
          return -1;
        }
        ++g_blocks_run;
      }
  g_blk = nullptr;
  return 0;
}

void wave_rendezvous(const char *op, const void *in, void *out,
                     void (*fn)(const void *const *, void *const *, int, void *), void *ctx) {
  Block &b = *g_blk;
  const unsigned t = b.fibers[(size_t)b.cur].tid;
  Wave &w = b.waves[t / kWave];
  if (w.arrived == 0) { w.op = op; w.fn = fn; w.ctx = ctx; }
  else if (w.op != op && std::strcmp(w.op, op) != 0) {
    std::string m = std::string("lanes of one wave reached different cross-lane operations: ") + w.op + " and " + op;
    fail(m.c_str(), nullptr);
  }
  w.in[t % kWave] = in;
  w.out[t % kWave] = out;
  ++w.arrived;
  ++b.progress;
  if (w.arrived == w.n_alive) { complete(w); return; }
  const uint64_t gen = w.gen;
  while (w.gen == gen) yield();
}

void block_barrier() {
  Block &b = *g_blk;
  ++b.bar_arrived;
  ++b.progress;
  if (b.bar_arrived == b.n_alive) { b.bar_arrived = 0; ++b.bar_gen; return; }
  const uint64_t gen = b.bar_gen;
  while (b.bar_gen == gen) yield();
}

// ---- cross-lane operations ------------------------------------------------------------------
// `in` / `out` are indexed by arrival slot = lane id within the wave (slots of lanes that have
// exited hold stale pointers and are never read: these operations are only reached by full waves
// in the kernels at hand, and n < 64 is refused).
namespace {
struct MfmaIn { const void *a, *b; const f32x16_t *c; };

template <typename V> void mfma_fn(const void *const *in, void *const *out, int n, void *) {
  if (n != kWave) fail("MFMA with exited lanes", nullptr);
  static thread_local double A[32][16], B[16][32];
  for (int l = 0; l < kWave; ++l) {
    const MfmaIn *x = static_cast<const MfmaIn *>(in[l]);
    const V &a = *static_cast<const V *>(x->a), &b = *static_cast<const V *>(x->b);
    const int r = l % 32, g = l / 32;
    for (int j = 0; j < 8; ++j) { A[r][8 * g + j] = (double)(float)a[j]; B[8 * g + j][r] = (double)(float)b[j]; }
  }
  for (int l = 0; l < kWave; ++l) {
    const MfmaIn *x = static_cast<const MfmaIn *>(in[l]);
    f32x16_t d;
    const int nn = l % 32, g = l / 32;
    for (int i = 0; i < 16; ++i) {
      const int m = 8 * (i / 4) + 4 * g + i % 4;
      double acc = (double)(*x->c)[i];
      for (int k = 0; k < 16; ++k) acc += A[m][k] * B[k][nn];
      d[i] = (float)acc;
    }
    *static_cast<f32x16_t *>(out[l]) = d;
  }
}

void tr_fn(const void *const *in, void *const *out, int n, void *) {
  if (n != kWave) fail("transposing LDS read with exited lanes", nullptr);
  for (int l = 0; l < kWave; ++l) {
    const int base = l & ~15, i = l & 15;
    s16x4_t v;
    for (int j = 0; j < 4; ++j) {
      const short *row = *static_cast<const short *const *>(in[base + 4 * j + i / 4]);
      v[j] = row[i % 4];
    }
    *static_cast<s16x4_t *>(out[l]) = v;
  }
}

// (ballot and readfirstlane clear the slots before they meet, so a lane that has exited has a null
// slot: its bit stays clear, and the first live lane is the first non-null one)
void ballot_fn(const void *const *in, void *const *out, int, void *) {
  uint64_t m = 0;
  for (int l = 0; l < kWave; ++l)
    if (in[l] && *static_cast<const bool *>(in[l])) m |= uint64_t(1) << l;
  for (int l = 0; l < kWave; ++l)
    if (out[l]) *static_cast<uint64_t *>(out[l]) = m;
}

void first_fn(const void *const *in, void *const *out, int, void *) {
  unsigned v = 0;
  for (int l = 0; l < kWave; ++l)
    if (in[l]) { v = *static_cast<const unsigned *>(in[l]); break; }
  for (int l = 0; l < kWave; ++l)
    if (out[l]) *static_cast<unsigned *>(out[l]) = v;
}

struct Swap { unsigned a, b; };
void swap_fn(const void *const *in, void *const *out, int n, void *) {
  if (n != kWave) fail("permlane32_swap with exited lanes", nullptr);
  for (int l = 0; l < kWave; ++l) {
    const Swap &own = *static_cast<const Swap *>(in[l]);
    const Swap &other = *static_cast<const Swap *>(in[l ^ 32]);
    // the upper half of the first operand changes places with the lower half of the second
    u32x2_t r;
    r[0] = l < 32 ? own.a : other.b;
    r[1] = l < 32 ? other.a : own.b;
    *static_cast<u32x2_t *>(out[l]) = r;
  }
}

struct Perm { int index, value; };
void bperm_fn(const void *const *in, void *const *out, int n, void *) {
  if (n != kWave) fail("ds_bpermute with exited lanes", nullptr);
  for (int l = 0; l < kWave; ++l) {
    const int src = (static_cast<const Perm *>(in[l])->index >> 2) & 63;
    *static_cast<int *>(out[l]) = static_cast<const Perm *>(in[src])->value;
  }
}

struct Shfl { unsigned v; int mask, width; };
void shfl_fn(const void *const *in, void *const *out, int n, void *) {
  if (n != kWave) fail("__shfl_xor with exited lanes", nullptr);
  for (int l = 0; l < kWave; ++l) {
    const Shfl &s = *static_cast<const Shfl *>(in[l]);
    int src = l ^ s.mask;
    if (src / s.width != l / s.width) src = l;  // outside the lane's segment: own value
    *static_cast<unsigned *>(out[l]) = static_cast<const Shfl *>(in[src])->v;
  }
}

void clear_slots() {
  Wave &w = g_blk->waves[g_blk->fibers[(size_t)g_blk->cur].tid / kWave];
  if (w.arrived == 0) for (int l = 0; l < kWave; ++l) { w.in[l] = nullptr; w.out[l] = nullptr; }
}
}  // namespace

void wave_sync() {
  wave_rendezvous("wave_sync", nullptr, nullptr, [](const void *const *, void *const *, int, void *) {});
}

f32x16_t mfma_32x32x16_f16(f16x8_t a, f16x8_t b, f32x16_t c, int, int, int) {
  MfmaIn in{&a, &b, &c};
  f32x16_t d;
  wave_rendezvous("mfma_f16", &in, &d, mfma_fn<f16x8_t>);
  return d;
}
f32x16_t mfma_32x32x16_bf16(bf16x8_t a, bf16x8_t b, f32x16_t c, int, int, int) {
  MfmaIn in{&a, &b, &c};
  f32x16_t d;
  wave_rendezvous("mfma_bf16", &in, &d, mfma_fn<bf16x8_t>);
  return d;
}
s16x4_t ds_read_tr16_b64(const void *p) {
  s16x4_t v;
  wave_rendezvous("ds_read_tr16_b64", &p, &v, tr_fn);
  return v;
}
uint64_t ballot_w64(bool pred) {
  uint64_t m = 0;
  clear_slots();
  wave_rendezvous("ballot", &pred, &m, ballot_fn);
  return m;
}
unsigned readfirstlane(unsigned v) {
  unsigned r = 0;
  clear_slots();
  wave_rendezvous("readfirstlane", &v, &r, first_fn);
  return r;
}
u32x2_t permlane32_swap(unsigned a, unsigned b, bool, bool) {
  Swap in{a, b};
  u32x2_t r;
  wave_rendezvous("permlane32_swap", &in, &r, swap_fn);
  return r;
}
int ds_bpermute(int byte_index, int v) {
  Perm in{byte_index, v};
  int r = 0;
  wave_rendezvous("ds_bpermute", &in, &r, bperm_fn);
  return r;
}
unsigned shfl_xor_u32(unsigned v, int mask, int width) {
  Shfl in{v, mask, width};
  unsigned r = 0;
  wave_rendezvous("shfl_xor", &in, &r, shfl_fn);
  return r;
}

// ---- memory ------------------------------------------------------------------------------------
void register_range(const void *p, size_t bytes) { g_ranges[reinterpret_cast<uintptr_t>(p)] = bytes; }
void unregister_range(const void *p) { g_ranges.erase(reinterpret_cast<uintptr_t>(p)); }
// The table is only consulted when the caller has entered its tensors; scratch that the library
// itself takes (hipMallocAsync) is in it too, but on its own says nothing about the caller's memory.
bool range_ok(const void *p, size_t bytes) {
  if (g_caller_ranges == 0) return true;
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  auto it = g_ranges.upper_bound(a);
  if (it == g_ranges.begin()) return false;
  --it;
  return a >= it->first && a + bytes <= it->first + it->second;
}

void *guarded_alloc(size_t bytes, bool at_end) {
  const size_t page = (size_t)sysconf(_SC_PAGESIZE);
  const size_t body = (std::max<size_t>(bytes, 1) + page - 1) / page * page;
  const size_t total = body + 2 * page;
  char *m = static_cast<char *>(mmap(nullptr, total, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0));
  if (m == MAP_FAILED) return nullptr;
  if (mprotect(m + page, body, PROT_READ | PROT_WRITE) != 0) { munmap(m, total); return nullptr; }
  // at_end: the last byte of the tensor is the last byte before the protected page (sizes are
  // multiples of 16 bytes or the start is rounded down to one)
  char *p = at_end ? m + page + body - (bytes + 15) / 16 * 16 : m + page;
  g_guarded[reinterpret_cast<uintptr_t>(p)] = Guarded{m, total};
  register_range(p, bytes);
  return p;
}
void guarded_free(void *p) {
  auto it = g_guarded.find(reinterpret_cast<uintptr_t>(p));
  if (it == g_guarded.end()) return;
  unregister_range(p);
  munmap(it->second.map, it->second.map_bytes);
  g_guarded.erase(it);
}

// scratch the launchers take with hipMallocAsync: guarded like the caller's tensors
hipError_t hipMallocAsync(void **p, size_t bytes, hipStream_t) {
  *p = guarded_alloc(bytes, true);
  return *p ? hipSuccess : hipErrorOutOfMemory;
}
hipError_t hipFreeAsync(void *p, hipStream_t) {
  guarded_free(p);
  return hipSuccess;
}

}  // namespace fa_emu

extern "C" {
void *fa_emu_alloc(size_t bytes, int at_end) { return fa_emu::guarded_alloc(bytes, at_end != 0); }
void fa_emu_free(void *p) { fa_emu::guarded_free(p); }
void fa_emu_register(const void *p, size_t bytes) { fa_emu::register_range(p, bytes); ++fa_emu::g_caller_ranges; }
void fa_emu_unregister(const void *p) { fa_emu::unregister_range(p); if (fa_emu::g_caller_ranges > 0) --fa_emu::g_caller_ranges; }
// run only the workgroups whose linear id (x fastest) is phase modulo stride; (1, 0): all
void fa_emu_select(long long stride, long long phase) {
  fa_emu::g_sel_list.clear();
  fa_emu::g_sel_stride = stride > 0 ? stride : 1;
  fa_emu::g_sel_phase = phase;
}
void fa_emu_select_list(const long long *ids, int n) { fa_emu::g_sel_list.assign(ids, ids + n); }
// burst <= 1: waves round robin; burst > 1: a wave picked at random (seeded) runs up to `burst`
// passes in a row before the next pick
void fa_emu_schedule(int burst, unsigned long long seed) { fa_emu::g_burst = burst; fa_emu::g_rng = seed * 2 + 1; }
const char *fa_emu_last_error(void) { return fa_emu::last_error(); }
int fa_emu_faulted(void) { return fa_emu::g_faulted ? 1 : 0; }
void fa_emu_reset(void) { fa_emu::g_faulted = false; fa_emu::g_error.clear(); fa_emu::g_blocks_run = 0; fa_emu::g_last_error = 0; }
long long fa_emu_blocks_run(void) { return fa_emu::g_blocks_run; }
}
