// CPU execution of HIP kernels compiled as plain C++ (see shim/hip/hip_runtime.h): blocks run one after the other,
// every thread of a block is a fiber (ucontext), and fibers meet at wavefront-wide operations (shuffles, MFMA, LDS
// transpose reads) and block barriers exactly as 64-lane wavefronts do. One OS thread runs everything, so runs are
// deterministic. Checks that hardware does not make:
//   - a wavefront-wide operation reached by only part of a wavefront, or by lanes that disagree on the operation,
//     aborts with a message;
//   - a block barrier that some live wavefront never reaches while others wait aborts with a message.
// Direct global -> LDS transfers are asynchronous on the hardware. HOSTSIM_DMA picks one of the two extreme timings:
//   late  (default)  a transfer lands only when its lane executes the vmcnt wait that covers it: a missing or too
//                    weak wait leaves stale (poisoned) LDS behind the reads that needed it;
//   early            a transfer lands the moment it is issued: a slot that is refilled before every wavefront has
//                    finished reading it corrupts those reads.
// Between two block barriers the wavefronts of a block run in an order HOSTSIM_ORDER picks; a kernel whose wavefronts
// exchange data through LDS or global memory without a barrier gives different results under different orders:
//   forward (default)   wavefront 0 as far as it can go, then wavefront 1, ... (later wavefronts are the slow ones)
//   reverse             the last wavefront first
//   random              a new random order after every barrier (HOSTSIM_SEED)
//   interleave          the wavefronts advance side by side, one wavefront-wide operation (MFMA, shuffle, LDS transpose
//                       read) at a time
//   interleave_random   the same, in a new random order every turn
// Dynamic LDS is filled with 0xFF bytes (NaN in every float format used) at the start of every block.
// Test infrastructure only.
#include <hip/hip_runtime.h>

#include <sys/mman.h>
#include <ucontext.h>

// Switching fibers with swapcontext costs two system calls (the signal mask). The plain x86-64 build switches with
// a dozen instructions instead; the AddressSanitizer build keeps swapcontext, which the sanitizer knows how to follow.
#if defined(__x86_64__) && !defined(__SANITIZE_ADDRESS__) && !(defined(__has_feature) && __has_feature(address_sanitizer))
#define HOSTSIM_FAST_SWITCH 1
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
    .size hostsim_switch,.-hostsim_switch
)");
#else
#define HOSTSIM_FAST_SWITCH 0
#endif

#include <cstdio>
#include <cstdlib>
#include <cstring>
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

enum State { RUNNABLE, AT_COLLECTIVE, AT_BARRIER, DONE };

struct Transfer {
  const void* src;
  uint32_t lds_offset;
  int bytes;
};

struct Fiber {
  ucontext_t ctx;
  void* sp;      // saved stack pointer (fast switch)
  State state;
  Resolver resolver;
  void* payload;
  std::vector<Transfer> pending;   // issued, not yet landed, oldest first
};

bool dma_early = false;
size_t lds_in_use = 0;
enum WaveOrder { ORDER_FORWARD, ORDER_REVERSE, ORDER_RANDOM, ORDER_INTERLEAVE, ORDER_INTERLEAVE_RANDOM };
WaveOrder wave_order = ORDER_FORWARD;
uint64_t random_state = 1;
uint32_t next_random() {   // xorshift64*
  random_state ^= random_state >> 12;
  random_state ^= random_state << 25;
  random_state ^= random_state >> 27;
  return static_cast<uint32_t>((random_state * 0x2545F4914F6CDD1DULL) >> 33);
}

Fiber fibers[MAX_THREADS];
unsigned char* stacks = nullptr;
ucontext_t scheduler;
void* scheduler_sp = nullptr;
int current = -1;
const std::function<void()>* kernel_body = nullptr;
dim3 cur_block_dim;

[[noreturn]] void die(const char* what) {
  std::fprintf(stderr, "hostsim: %s (block %u,%u,%u thread %d)\n", what, blockIdx.x, blockIdx.y, blockIdx.z, current);
  std::abort();
}

void yield() {
#if HOSTSIM_FAST_SWITCH
  hostsim_switch(&fibers[current].sp, scheduler_sp);
#else
  swapcontext(&fibers[current].ctx, &scheduler);
#endif
}

void fiber_main() {
  (*kernel_body)();
  fibers[current].state = DONE;
  yield();
  die("resumed a finished fiber");
}

void resume(int t) {
  current = t;
  threadIdx.x = t % cur_block_dim.x;
  threadIdx.y = (t / cur_block_dim.x) % cur_block_dim.y;
  threadIdx.z = t / (cur_block_dim.x * cur_block_dim.y);
#if HOSTSIM_FAST_SWITCH
  hostsim_switch(&scheduler_sp, fibers[t].sp);
#else
  swapcontext(&scheduler, &fibers[t].ctx);
#endif
}

void run_block(int nthreads) {
  for (int t = 0; t < nthreads; ++t) {
    Fiber& f = fibers[t];
#if HOSTSIM_FAST_SWITCH
    // initial frame: six callee-saved registers, then the address `ret` jumps to; fiber_main must find the stack as
    // after a call (16-byte aligned before the return address was pushed)
    void** top = reinterpret_cast<void**>(stacks + static_cast<size_t>(t + 1) * STACK_BYTES);
    top -= 2;                                            // keeps (top of frame + 8) 16-byte aligned
    *--top = nullptr;                                    // slot a caller's return address would occupy
    *--top = reinterpret_cast<void*>(&fiber_main);
    for (int r = 0; r < 6; ++r) *--top = nullptr;
    f.sp = top;
#else
    getcontext(&f.ctx);
    f.ctx.uc_stack.ss_sp = stacks + static_cast<size_t>(t) * STACK_BYTES;
    f.ctx.uc_stack.ss_size = STACK_BYTES;
    f.ctx.uc_link = nullptr;
    makecontext(&f.ctx, fiber_main, 0);
#endif
    f.state = RUNNABLE;
    f.pending.clear();
  }
  std::memset(dynamic_lds, 0xff, lds_in_use);
  const int waves = (nthreads + WAVE - 1) / WAVE;
  // Runs wavefront w until it has no runnable lane and no pending wavefront-wide operation (it is done or waits at
  // the block barrier), or, with `one_step`, until it has resolved one wavefront-wide operation. Returns whether it
  // made progress.
  auto run_wave = [&](int w, bool one_step) -> bool {
    const int lo = w * WAVE, hi = std::min(nthreads, lo + WAVE);
    bool progressed = false;
    for (;;) {
      for (int t = lo; t < hi; ++t)
        if (fibers[t].state == RUNNABLE) { resume(t); progressed = true; }
      int arrived = 0;
      for (int t = lo; t < hi; ++t) arrived += fibers[t].state == AT_COLLECTIVE;
      if (arrived == 0) return progressed;      // wavefront finished or waits at the block barrier
      current = lo;
      if (arrived != hi - lo) die("wavefront-wide operation reached by only some of the lanes");
      void* payloads[WAVE];
      for (int t = lo; t < hi; ++t) {
        if (fibers[t].resolver != fibers[lo].resolver) die("lanes of one wavefront are at different wavefront-wide operations");
        payloads[t - lo] = fibers[t].payload;
      }
      fibers[lo].resolver(payloads, hi - lo);
      for (int t = lo; t < hi; ++t) fibers[t].state = RUNNABLE;
      progressed = true;
      if (one_step) return true;
    }
  };
  int order[MAX_THREADS / WAVE];
  for (;;) {
    // the order in which the wavefronts run between two block barriers (see the header comment)
    for (int w = 0; w < waves; ++w) order[w] = wave_order == ORDER_REVERSE ? waves - 1 - w : w;
    if (wave_order == ORDER_RANDOM || wave_order == ORDER_INTERLEAVE_RANDOM)
      for (int w = waves - 1; w > 0; --w) std::swap(order[w], order[next_random() % (w + 1)]);
    if (wave_order == ORDER_INTERLEAVE || wave_order == ORDER_INTERLEAVE_RANDOM) {
      // one wavefront-wide operation per wavefront and turn: the wavefronts advance side by side
      for (bool any = true; any;) {
        any = false;
        for (int i = 0; i < waves; ++i) any |= run_wave(order[i], true);
        if (wave_order == ORDER_INTERLEAVE_RANDOM)
          for (int w = waves - 1; w > 0; --w) std::swap(order[w], order[next_random() % (w + 1)]);
      }
    } else {
      for (int i = 0; i < waves; ++i) run_wave(order[i], false);
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

void wave_collective(Resolver resolver, void* payload) {
  Fiber& f = fibers[current];
  f.resolver = resolver;
  f.payload = payload;
  f.state = AT_COLLECTIVE;
  yield();
}

void fail(const char* what) { die(what); }

unsigned lane_id() { return static_cast<unsigned>(current) & (WAVE - 1); }

namespace {
struct Shuffle { uint64_t bits; int mask; };
void resolve_shuffle(void** payloads, int lanes) {
  uint64_t in[WAVE];
  const int mask = static_cast<Shuffle*>(payloads[0])->mask;
  for (int l = 0; l < lanes; ++l) {
    if (static_cast<Shuffle*>(payloads[l])->mask != mask) die("lanes of one wavefront shuffle with different masks");
    in[l] = static_cast<Shuffle*>(payloads[l])->bits;
  }
  for (int l = 0; l < lanes; ++l) static_cast<Shuffle*>(payloads[l])->bits = (l ^ mask) < lanes ? in[l ^ mask] : in[l];
}

void land(const Transfer& t) {
  if (static_cast<size_t>(t.lds_offset) + t.bytes > lds_in_use) die("global -> LDS transfer outside the block's LDS allocation");
  std::memcpy(dynamic_lds + t.lds_offset, t.src, t.bytes);
}
}  // namespace

namespace {
void resolve_gather(void** payloads, int lanes) {
  uint64_t in[WAVE];
  for (int l = 0; l < lanes; ++l) in[l] = static_cast<Shuffle*>(payloads[l])->bits;
  for (int l = 0; l < lanes; ++l) {
    const int from = static_cast<Shuffle*>(payloads[l])->mask;
    if (from < 0 || from >= lanes) die("lane exchange reads a lane that is not part of the wavefront");
    static_cast<Shuffle*>(payloads[l])->bits = in[from];
  }
}
}  // namespace

uint64_t gather_bits(uint64_t bits, int source_lane) {
  Shuffle s{bits, source_lane};
  wave_collective(resolve_gather, &s);
  return s.bits;
}

uint64_t shfl_xor_bits(uint64_t bits, int mask) {
  Shuffle s{bits, mask};
  wave_collective(resolve_shuffle, &s);
  return s.bits;
}

void dma_issue(const void* src, uint32_t lds_offset, int bytes) {
  const Transfer t{src, lds_offset, bytes};
  if (dma_early) land(t);
  else fibers[current].pending.push_back(t);
}

void dma_wait(int may_stay_outstanding) {
  std::vector<Transfer>& q = fibers[current].pending;
  const int n = static_cast<int>(q.size()) - may_stay_outstanding;
  if (n <= 0) return;
  for (int i = 0; i < n; ++i) land(q[i]);
  q.erase(q.begin(), q.begin() + n);
}

uint32_t lds_offset_of(uint32_t low_address_bits) {
  return low_address_bits - static_cast<uint32_t>(reinterpret_cast<uintptr_t>(dynamic_lds));
}

void sync_block() {
  fibers[current].state = AT_BARRIER;
  yield();
}


// ---- wavefront-wide instructions (declared in the stand-in header; here so that they are compiled with optimisation
// while the kernel sources themselves are not) ----
void resolve_tr_read(void** payloads, int lanes) {
  if (lanes != 64) fail("LDS transpose read in a partial wavefront");
  short raw[64][4];
  for (int l = 0; l < 64; ++l) std::memcpy(raw[l], static_cast<TrRead*>(payloads[l])->addr, 8);
  for (int l = 0; l < 64; ++l) {
    const int blk = l & ~15, i = l & 15;
    for (int e = 0; e < 4; ++e) static_cast<TrRead*>(payloads[l])->out[e] = raw[blk + 4 * e + (i >> 2)][i & 3];
  }
}

template <bool BF16>
static inline float widen(uint16_t bits) {
  if (BF16) { const uint32_t u = static_cast<uint32_t>(bits) << 16; float f; std::memcpy(&f, &u, 4); return f; }
  return __half2float(__ushort_as_half(bits));
}
template <bool BF16>
static void resolve_mfma(void** payloads, int lanes) {
  if (lanes != 64) fail("MFMA in a partial wavefront");
  float A[32][16], B[16][32];
  for (int l = 0; l < 64; ++l) {
    const Mfma* m = static_cast<const Mfma*>(payloads[l]);
    for (int t = 0; t < 8; ++t) {
      A[l & 31][8 * (l >> 5) + t] = widen<BF16>(m->a[t]);
      B[8 * (l >> 5) + t][l & 31] = widen<BF16>(m->b[t]);
    }
  }
  for (int l = 0; l < 64; ++l) {
    float* c = static_cast<Mfma*>(payloads[l])->c;
    const int j = l & 31;
    for (int r = 0; r < 16; ++r) {
      const int i = 8 * (r / 4) + 4 * (l >> 5) + r % 4;
      float s = c[r];
      for (int k = 0; k < 16; ++k) s += A[i][k] * B[k][j];
      c[r] = s;
    }
  }
}
// v_mfma_f32_32x32x2_f32: lane l holds A[l & 31][l >> 5] and B[l >> 5][l & 31]
void resolve_mfma_f32(void** payloads, int lanes) {
  if (lanes != 64) fail("MFMA in a partial wavefront");
  float A[32][2], B[2][32];
  for (int l = 0; l < 64; ++l) {
    const MfmaF32* m = static_cast<const MfmaF32*>(payloads[l]);
    A[l & 31][l >> 5] = m->a;
    B[l >> 5][l & 31] = m->b;
  }
  for (int l = 0; l < 64; ++l) {
    float* c = static_cast<MfmaF32*>(payloads[l])->c;
    const int j = l & 31;
    for (int r = 0; r < 16; ++r) {
      const int i = 8 * (r / 4) + 4 * (l >> 5) + r % 4;
      c[r] = std::fmaf(A[i][1], B[1][j], std::fmaf(A[i][0], B[0][j], c[r]));
    }
  }
}
void resolve_mfma_f16(void** payloads, int lanes) { resolve_mfma<false>(payloads, lanes); }
void resolve_mfma_bf16(void** payloads, int lanes) { resolve_mfma<true>(payloads, lanes); }

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
  const char* mode = std::getenv("HOSTSIM_DMA");
  dma_early = mode != nullptr && std::strcmp(mode, "early") == 0;
  const char* ord = std::getenv("HOSTSIM_ORDER");
  wave_order = ord == nullptr ? ORDER_FORWARD
               : std::strcmp(ord, "reverse") == 0 ? ORDER_REVERSE
               : std::strcmp(ord, "random") == 0 ? ORDER_RANDOM
               : std::strcmp(ord, "interleave") == 0 ? ORDER_INTERLEAVE
               : std::strcmp(ord, "interleave_random") == 0 ? ORDER_INTERLEAVE_RANDOM : ORDER_FORWARD;
  if (const char* seed = std::getenv("HOSTSIM_SEED")) random_state = std::strtoull(seed, nullptr, 10) * 2654435761ULL + 1;
  lds_in_use = dynamic_lds_bytes;
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
