// Runtime of the CPU test build of the kernels: runs a grid workgroup by workgroup, each lane a
// ucontext fiber scheduled round-robin (see hip/hip_runtime.h in this folder).  Test-only.
#include <hip/hip_runtime.h>
#include <sys/mman.h>
#include <unistd.h>

#include <mutex>

// dynamic LDS of the kernels (declared `extern __shared__` in gdn_common.h)
thread_local __attribute__((aligned(16))) unsigned char gdn_smem[emu::kLds + 4096];

namespace emu {

thread_local Block* g_blk = nullptr;

static void fiber_main() {
  Block* b = g_blk;
  (*b->body)();
  b->fibers[b->cur].done = true;
  b->alive--;
  if (b->alive > 0 && b->bar_count == b->alive) {  // last straggler left while others wait
    b->bar_count = 0;
    b->bar_gen++;
  }
  swapcontext(&b->fibers[b->cur].ctx, &b->sched);
}

static void run_block(Block& b, size_t smem) {
  g_blk = &b;
  const int n = b.nthreads;
  b.alive = n;
  b.bar_count = 0;
  memset(gdn_smem, 0xFF, smem);                       // uninitialised LDS reads as NaN
  memset(gdn_smem + smem, 0xA5, sizeof(gdn_smem) - smem);
  for (auto& w : b.waves) { w.gen = 0; w.count = 0; }
  for (int i = 0; i < n; ++i) {
    Fiber& f = b.fibers[i];
    f.done = false;
    getcontext(&f.ctx);
    f.ctx.uc_stack.ss_sp = b.stacks.data() + (size_t)i * kStack;
    f.ctx.uc_stack.ss_size = kStack;
    f.ctx.uc_link = &b.sched;
    makecontext(&f.ctx, fiber_main, 0);
  }
  long spins = 0;
  while (b.alive > 0) {
    for (int i = 0; i < n; ++i) {
      if (b.fibers[i].done) continue;
      b.cur = i;
      swapcontext(&b.sched, &b.fibers[i].ctx);
    }
    if (++spins > 50000000L) {
      fprintf(stderr, "emu: workgroup (%u,%u,%u) does not finish (divergent barrier or collective?)\n",
              b.bidx.x, b.bidx.y, b.bidx.z);
      abort();
    }
  }
  for (size_t i = smem; i < sizeof(gdn_smem); ++i)
    if (gdn_smem[i] != 0xA5) {
      fprintf(stderr, "emu: LDS overrun at byte %zu (requested %zu) in workgroup (%u,%u,%u)\n", i, smem,
              b.bidx.x, b.bidx.y, b.bidx.z);
      abort();
    }
  g_blk = nullptr;
}

void run_grid(dim3 grid, dim3 block, size_t smem, const std::function<void()>& body) {
  const int nthreads = block.x * block.y * block.z;
  if (nthreads > kMaxThreads || smem > kLds) {
    fprintf(stderr, "emu: bad launch config (%d threads, %zu B LDS)\n", nthreads, smem);
    abort();
  }
  const long nblocks = (long)grid.x * grid.y * grid.z;
  if (nblocks == 0) return;
  const char* env = getenv("GDN_EMU_THREADS");
  int nworkers = env ? atoi(env) : (int)std::thread::hardware_concurrency();
  nworkers = (int)std::max(1L, std::min<long>(nworkers, nblocks));
  std::atomic<long> next{0};
  auto worker = [&]() {
    Block b;
    b.nthreads = nthreads;
    b.bdim = {block.x, block.y, block.z};
    b.gdim = {grid.x, grid.y, grid.z};
    b.fibers.resize(nthreads);
    b.waves.resize((nthreads + kWave - 1) / kWave);
    b.stacks.resize((size_t)nthreads * kStack);
    b.body = &body;
    for (;;) {
      long i = next.fetch_add(1);
      if (i >= nblocks) break;
      b.bidx.x = (unsigned)(i % grid.x);
      b.bidx.y = (unsigned)((i / grid.x) % grid.y);
      b.bidx.z = (unsigned)(i / ((long)grid.x * grid.y));
      run_block(b, smem);
    }
  };
  if (nworkers == 1) {
    worker();
  } else {
    std::vector<std::thread> ts;
    for (int t = 0; t < nworkers; ++t) ts.emplace_back(worker);
    for (auto& t : ts) t.join();
  }
}

}  // namespace emu

// ---- guard-page allocator for test buffers: [PROT_NONE | data ... end-of-page | PROT_NONE] ----
extern "C" void* emu_guard_alloc(size_t nbytes, int at_end) {
  const size_t pg = (size_t)sysconf(_SC_PAGESIZE);
  const size_t body = (std::max<size_t>(nbytes, 1) + pg - 1) / pg * pg;
  unsigned char* base = (unsigned char*)mmap(nullptr, body + 2 * pg, PROT_READ | PROT_WRITE,
                                             MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
  if (base == MAP_FAILED) return nullptr;
  mprotect(base, pg, PROT_NONE);
  mprotect(base + pg + body, pg, PROT_NONE);
  memset(base + pg, 0xFF, body);
  if (!at_end) return base + pg;
  size_t off = body - ((nbytes + 15) / 16 * 16);  // keep 16-byte alignment, end flush with the guard
  return base + pg + off;
}
