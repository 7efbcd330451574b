// CPU execution of HIP kernels compiled as plain C++ (see shim/hip/hip_runtime.h): blocks run one after the other,
// every thread of a block is a fiber (ucontext), and fibers meet at wavefront shuffles and block barriers exactly as
// 64-lane wavefronts do. One OS thread runs everything, so runs are deterministic. Checks that hardware does not make:
//   - a shuffle reached by only part of a wavefront, or with different lane masks, aborts with a message;
//   - a block barrier that some live wavefront never reaches while others wait aborts with a message.
// Test infrastructure only.
#include <hip/hip_runtime.h>

#include <sys/mman.h>
#include <ucontext.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

hostsim::Index threadIdx, blockIdx;
dim3 blockDim, gridDim;

namespace hostsim {

unsigned char* dynamic_lds = nullptr;

namespace {
constexpr int MAX_THREADS = 1024;
constexpr int WAVE = 64;
constexpr size_t STACK_BYTES = 256 << 10;
constexpr size_t LDS_BYTES = 160 << 10;

enum State { RUNNABLE, AT_SHUFFLE, AT_BARRIER, DONE };

struct Fiber {
  ucontext_t ctx;
  State state;
  uint64_t bits;
  int mask;
};

Fiber fibers[MAX_THREADS];
unsigned char* stacks = nullptr;
ucontext_t scheduler;
int current = -1;
const std::function<void()>* kernel_body = nullptr;
dim3 cur_block_dim;

[[noreturn]] void die(const char* what) {
  std::fprintf(stderr, "hostsim: %s (block %u,%u,%u thread %d)\n", what, blockIdx.x, blockIdx.y, blockIdx.z, current);
  std::abort();
}

void fiber_main() {
  (*kernel_body)();
  fibers[current].state = DONE;
  swapcontext(&fibers[current].ctx, &scheduler);
  die("resumed a finished fiber");
}

void yield() { swapcontext(&fibers[current].ctx, &scheduler); }

void resume(int t) {
  current = t;
  threadIdx.x = t % cur_block_dim.x;
  threadIdx.y = (t / cur_block_dim.x) % cur_block_dim.y;
  threadIdx.z = t / (cur_block_dim.x * cur_block_dim.y);
  swapcontext(&scheduler, &fibers[t].ctx);
}

void run_block(int nthreads) {
  for (int t = 0; t < nthreads; ++t) {
    Fiber& f = fibers[t];
    getcontext(&f.ctx);
    f.ctx.uc_stack.ss_sp = stacks + static_cast<size_t>(t) * STACK_BYTES;
    f.ctx.uc_stack.ss_size = STACK_BYTES;
    f.ctx.uc_link = nullptr;
    makecontext(&f.ctx, fiber_main, 0);
    f.state = RUNNABLE;
  }
  const int waves = (nthreads + WAVE - 1) / WAVE;
  for (;;) {
    for (int w = 0; w < waves; ++w) {
      const int lo = w * WAVE, hi = std::min(nthreads, lo + WAVE);
      for (;;) {
        for (int t = lo; t < hi; ++t)
          if (fibers[t].state == RUNNABLE) resume(t);
        int at_shuffle = 0, live = 0;
        for (int t = lo; t < hi; ++t) {
          live += fibers[t].state != DONE;
          at_shuffle += fibers[t].state == AT_SHUFFLE;
        }
        if (at_shuffle == 0) break;             // wavefront finished or waits at the block barrier
        current = lo;
        if (at_shuffle != hi - lo) die("wavefront shuffle reached by only some of the lanes");
        uint64_t in[WAVE];
        const int mask = fibers[lo].mask;
        for (int t = lo; t < hi; ++t) {
          if (fibers[t].mask != mask) die("lanes of one wavefront shuffle with different masks");
          in[t - lo] = fibers[t].bits;
        }
        for (int t = lo; t < hi; ++t) {
          const int src = (t - lo) ^ mask;
          fibers[t].bits = src < hi - lo ? in[src] : in[t - lo];
          fibers[t].state = RUNNABLE;
        }
        (void)live;
      }
    }
    int done = 0, waiting = 0;
    for (int t = 0; t < nthreads; ++t) {
      done += fibers[t].state == DONE;
      waiting += fibers[t].state == AT_BARRIER;
    }
    if (done == nthreads) return;
    if (waiting == 0) die("scheduler stalled with no thread at a barrier");
    // hardware counts the wavefronts that are still alive; a wavefront with some lanes finished and others at the
    // barrier is fine (the finished lanes are simply masked off)
    for (int t = 0; t < nthreads; ++t)
      if (fibers[t].state == AT_BARRIER) fibers[t].state = RUNNABLE;
  }
}
}  // namespace

uint64_t shfl_xor_bits(uint64_t bits, int mask) {
  Fiber& f = fibers[current];
  f.bits = bits;
  f.mask = mask;
  f.state = AT_SHUFFLE;
  yield();
  return fibers[current].bits;
}

void sync_block() {
  fibers[current].state = AT_BARRIER;
  yield();
}

int compute_units() {
  const char* e = std::getenv("HOSTSIM_CUS");
  const int n = e ? std::atoi(e) : 4;
  return n > 0 ? n : 4;
}

void launch(dim3 grid, dim3 block, size_t dynamic_lds_bytes, const std::function<void()>& body) {
  const uint64_t nthreads = static_cast<uint64_t>(block.x) * block.y * block.z;
  if (nthreads == 0 || nthreads > MAX_THREADS) { std::fprintf(stderr, "hostsim: block of %llu threads\n", (unsigned long long)nthreads); std::abort(); }
  if (dynamic_lds_bytes > LDS_BYTES) { std::fprintf(stderr, "hostsim: %zu bytes of dynamic LDS\n", dynamic_lds_bytes); std::abort(); }
  if (static_cast<uint64_t>(grid.x) * grid.y * grid.z == 0) { std::fprintf(stderr, "hostsim: empty grid\n"); std::abort(); }
  if (stacks == nullptr) {
    void* p = mmap(nullptr, MAX_THREADS * STACK_BYTES + LDS_BYTES, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (p == MAP_FAILED) { std::perror("hostsim: mmap"); std::abort(); }
    stacks = static_cast<unsigned char*>(p);
    dynamic_lds = stacks + MAX_THREADS * STACK_BYTES;
  }
  kernel_body = &body;
  cur_block_dim = block;
  blockDim = block;
  gridDim = grid;
  for (unsigned z = 0; z < grid.z; ++z)
    for (unsigned y = 0; y < grid.y; ++y)
      for (unsigned x = 0; x < grid.x; ++x) {
        blockIdx = Index{x, y, z};
        run_block(static_cast<int>(nthreads));
      }
  kernel_body = nullptr;
  current = -1;
}

}  // namespace hostsim
