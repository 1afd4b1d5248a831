// Runner of the host build of the kernels (see hip/hip_runtime.h in this
// directory): tensors between canary pages and inaccessible guard regions, one
// child process per launch so that a trap ends the child and not the test, and
// inside it one cooperative fiber per thread of the block that is running.
// Test infrastructure only.
#include "hip/hip_runtime.h"
#include "kernel_table.h"
#include <csignal>
#include <ctime>
#include <string>
#include <sys/mman.h>
#include <sys/wait.h>
#include <ucontext.h>
#include <unistd.h>
#include <vector>

HmDim threadIdx, blockIdx, blockDim, gridDim;

namespace {
constexpr size_t kPage = 4096, kGuard = 1 << 20;
struct Range {
  char *lo, *hi;
  std::string name;
};
std::vector<Range> ranges;
const char *cur_kernel = "";
// what the child reports to the parent: shared between the two
struct Report {
  long violations;
  char first[512];
};
Report *report = nullptr;

void describe(char *buf, size_t n, const void *p) {
  const char *c = (const char *)p;
  const Range *best = nullptr;
  long dist = 0;
  for (auto &r : ranges) {
    const long d = c < r.lo ? r.lo - c : c >= r.hi ? c - r.hi + 1 : 0;
    if (!best || d < dist) {
      best = &r;
      dist = d;
    }
  }
  if (best)
    snprintf(buf, n, "%s%+ld (the tensor holds %ld bytes)", best->name.c_str(), (long)(c - best->lo),
             (long)(best->hi - best->lo));
  else
    snprintf(buf, n, "%p", p);
}
void note(const char *text) {
  if (report->violations++ == 0)
    snprintf(report->first, sizeof report->first, "%s", text);
}
void on_trap(int sig, siginfo_t *si, void *) {
  char at[200], text[480];
  describe(at, sizeof at, si->si_addr);
  // (a general-protection trap, which is what a misaligned 16-byte access raises, reports no address)
  snprintf(text, sizeof text, "%s in %s, block %u thread %u: %s", si->si_addr ? "access outside the tensors" :
           "misaligned 16-byte access (or a wild pointer)", cur_kernel, blockIdx.x, threadIdx.x, si->si_addr ? at : "");
  note(text);
  (void)sig;
  _exit(0);
}

// ---- who wrote what: no byte of a tensor may be changed by two blocks of one launch ------------
bool check_owners = false;
struct Shadow {
  std::vector<char> before;          // the tensor as the last block left it
  std::vector<unsigned char> owned;  // 1: some block of this launch has changed the byte
};
std::vector<Shadow> shadows;
void owners_begin() {
  shadows.assign(ranges.size(), Shadow());
  for (size_t i = 0; i < ranges.size(); ++i) {
    shadows[i].before.assign(ranges[i].lo, ranges[i].hi);
    shadows[i].owned.assign(ranges[i].hi - ranges[i].lo, 0);
  }
}
void owners_after_block() {
  for (size_t i = 0; i < ranges.size(); ++i) {
    Shadow &sh = shadows[i];
    const char *now = ranges[i].lo;
    const size_t n = sh.before.size();
    if (!std::memcmp(now, sh.before.data(), n))
      continue;
    for (size_t b = 0; b < n; ++b)
      if (now[b] != sh.before[b]) {
        if (sh.owned[b]) {
          char text[300];
          snprintf(text, sizeof text, "%s, block %u changed byte %zu of %s, which an earlier block of the launch had written",
                   cur_kernel, blockIdx.x, b, ranges[i].name.c_str());
          note(text);
        }
        sh.owned[b] = 1;
        sh.before[b] = now[b];
      }
  }
}

// ---- one block as cooperative fibers ---------------------------------------------
enum State { kRun, kWaitWave, kWaitBlock, kDone };
struct PendingLoad { // a load into LDS that has been issued and has not landed
  char *dst;
  int size;
  char data[16];
};
struct Fiber {
  ucontext_t ctx;
  State state;
  unsigned ops; // cross-lane operations begun: picks the half of the exchange area
  std::vector<PendingLoad> pending;
};
bool late_loads = false;
int thread_order = 0;
unsigned first_block = 0, block_limit = ~0u; // the blocks of a launch that run
unsigned pass_seed = 12345;
constexpr size_t kStack = 512 * 1024;
constexpr unsigned kMaxThreads = 1024;
Fiber *fibers = nullptr;
char *stacks = nullptr;
char (*slots)[2][64][128] = nullptr; // per wave: two halves, used in turn
ucontext_t scheduler;
unsigned current = 0, threads = 0;
void (*kernel_fn)(void **, const void *) = nullptr;
void **kernel_pointers = nullptr;
const void *kernel_params = nullptr;

void fiber_main() {
  kernel_fn(kernel_pointers, kernel_params);
  fibers[current].state = kDone;
}
void wait_as(State s) {
  fibers[current].state = s;
  swapcontext(&fibers[current].ctx, &scheduler);
}
// false: the block's threads wait for each other at different places (noted in the report)
bool run_block() {
  if (!fibers) {
    fibers = new Fiber[kMaxThreads];
    stacks = (char *)mmap(nullptr, kStack * kMaxThreads, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE,
                          -1, 0);
    slots = (char(*)[2][64][128])calloc(kMaxThreads / 64, sizeof *slots);
    for (unsigned t = 0; t < kMaxThreads; ++t) // a stack that overflows traps instead of running into its neighbour
      mprotect(stacks + (size_t)t * kStack, kPage, PROT_NONE);
  }
  for (unsigned t = 0; t < threads; ++t) {
    getcontext(&fibers[t].ctx);
    fibers[t].ctx.uc_stack.ss_sp = stacks + (size_t)t * kStack;
    fibers[t].ctx.uc_stack.ss_size = kStack;
    fibers[t].ctx.uc_link = &scheduler;
    makecontext(&fibers[t].ctx, fiber_main, 0);
    fibers[t].state = kRun;
    fibers[t].ops = 0;
    fibers[t].pending.clear();
  }
  for (;;) {
    bool ran = false;
    const unsigned waves = (threads + 63) / 64;
    const unsigned shift = thread_order == 2 ? (pass_seed = pass_seed * 1664525u + 1013904223u) >> 16 : 0;
    for (unsigned i = 0; i < threads; ++i) {
      // the order in which the threads get their turn: ascending, descending, or the waves rotated by a
      // different amount in every pass (no result may depend on it)
      unsigned t = thread_order == 1 ? threads - 1 - i : i;
      if (thread_order == 2)
        t = ((i / 64 + shift) % waves) * 64 + i % 64;
      if (t >= threads)
        continue;
      if (fibers[t].state == kRun) {
        current = t;
        threadIdx = {t, 0, 0};
        swapcontext(&scheduler, &fibers[t].ctx);
        ran = true;
      }
    }
    // a wave goes on when all its live lanes wait for each other, the block when all its live threads do
    bool released = false;
    unsigned done = 0, at_barrier = 0;
    for (unsigned w = 0; w * 64 < threads; ++w) {
      unsigned waiting = 0, live = 0;
      for (unsigned t = w * 64; t < std::min(threads, w * 64 + 64); ++t) {
        waiting += fibers[t].state == kWaitWave;
        live += fibers[t].state != kDone;
        done += fibers[t].state == kDone;
        at_barrier += fibers[t].state == kWaitBlock;
      }
      if (waiting && waiting == live) {
        for (unsigned t = w * 64; t < std::min(threads, w * 64 + 64); ++t)
          if (fibers[t].state == kWaitWave)
            fibers[t].state = kRun;
        released = true;
      }
    }
    if (done == threads)
      return true;
    if (at_barrier && at_barrier + done == threads) {
      for (unsigned t = 0; t < threads; ++t)
        if (fibers[t].state == kWaitBlock)
          fibers[t].state = kRun;
      released = true;
    }
    if (!ran && !released) {
      char text[200];
      snprintf(text, sizeof text, "%s, block %u: the threads wait for each other at different places (%u of %u at "
               "the barrier, %u done)", cur_kernel, blockIdx.x, at_barrier, threads, done);
      note(text);
      return false;
    }
  }
}
} // namespace

void hm_wave_sync() { wait_as(kWaitWave); }
void hm_block_sync() { wait_as(kWaitBlock); }

void hm_check_global(const void *p, size_t n, const char *what) {
  if (ranges.empty()) // (a caller that runs in its own memory: hm_run_direct)
    return;
  const char *c = (const char *)p;
  for (auto &r : ranges)
    if (c >= r.lo && c + n <= r.hi)
      return;
  char at[200], text[480];
  describe(at, sizeof at, p);
  snprintf(text, sizeof text, "%s outside the tensors in %s, block %u thread %u: %zu bytes at %s", what, cur_kernel,
           blockIdx.x, threadIdx.x, n, at);
  note(text);
}

// ---- cross-lane operations: every lane puts its operands into its slot of the wave's exchange area, the wave
// meets, every lane computes its result from the slots.  The area has two halves used in turn, so that a lane
// that has gone on to the next operation does not overwrite what a slower lane still reads.
namespace {
inline int lane_id() { return (int)(current & 63); }
char *my_slot() {
  Fiber &f = fibers[current];
  ++f.ops;
  return slots[current / 64][f.ops & 1][current & 63];
}
const char *slot_of(int lane) { return slots[current / 64][fibers[current].ops & 1][lane & 63]; }
double widen(int type, const char *p, int k) {
  switch (type) {
  case HM_F32: {
    float f;
    std::memcpy(&f, p + 4 * k, 4);
    return f;
  }
  case HM_F16: {
    _Float16 h;
    std::memcpy(&h, p + 2 * k, 2);
    return (double)(float)h;
  }
  case HM_BF16: {
    uint16_t h;
    std::memcpy(&h, p + 2 * k, 2);
    const uint32_t w = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &w, 4);
    return f;
  }
  case HM_I8: return (double)(int8_t)p[k];
  case HM_E4M3: return hm_f8_to_f32((unsigned char)p[k], 4);
  default: return hm_f8_to_f32((unsigned char)p[k], 5);
  }
}
int elem_bytes(int type) { return type == HM_F32 ? 4 : (type == HM_F16 || type == HM_BF16) ? 2 : 1; }
} // namespace

void hm_load_lds(HmRsrc r, void *lds, int size, int voff, int soff, int ioff, int) {
  PendingLoad load;
  load.dst = (char *)lds + lane_id() * size; // the wave's lanes land back to back
  load.size = size;
  std::memset(load.data, 0, sizeof load.data);
  const uint64_t off = (uint64_t)(unsigned)voff + (unsigned)ioff;
  if (off < r.num_records && off + (unsigned)soff < r.num_records) {
    const char *src = r.base + off + (unsigned)soff;
    hm_check_global(src, size, "buffer load into LDS");
    std::memcpy(load.data, src, size);
  }
  if (late_loads)
    fibers[current].pending.push_back(load);
  else
    std::memcpy(load.dst, load.data, size);
}
void hm_waitcnt(int immediate) {
  // gfx9 encoding: vmcnt[3:0] in bits 3:0, vmcnt[5:4] in bits 15:14
  const size_t allowed = (size_t)((immediate & 0xF) | (((immediate >> 14) & 3) << 4));
  auto &q = fibers[current].pending;
  size_t land = q.size() > allowed ? q.size() - allowed : 0;
  for (size_t i = 0; i < land; ++i)
    std::memcpy(q[i].dst, q[i].data, q[i].size);
  q.erase(q.begin(), q.begin() + land);
  wait_as(kWaitWave);
}
hm_v4i hm_load_b128(HmRsrc r, int voff, int soff, int) {
  hm_v4i v = {0, 0, 0, 0};
  const uint64_t off = (uint64_t)(unsigned)voff;
  if (off >= r.num_records || off + (unsigned)soff >= r.num_records)
    return v;
  const char *src = r.base + off + (unsigned)soff;
  hm_check_global(src, 16, "buffer load");
  std::memcpy(&v, src, 16);
  return v;
}
void hm_first_lane(void *value, size_t bytes) {
  std::memcpy(my_slot(), value, bytes);
  wait_as(kWaitWave);
  std::memcpy(value, slot_of(0), bytes);
}
uint64_t hm_ballot(bool p) {
  *my_slot() = p ? 1 : 0;
  wait_as(kWaitWave);
  uint64_t m = 0;
  for (int l = 0; l < 64; ++l)
    m |= (uint64_t)(*slot_of(l) & 1) << l;
  return m;
}
int hm_bpermute(int byte_index, int v) {
  std::memcpy(my_slot(), &v, 4);
  wait_as(kWaitWave);
  int out;
  std::memcpy(&out, slot_of((byte_index >> 2) & 63), 4);
  return out;
}
void hm_shuffle_xor(void *value, size_t bytes, int mask, int width) {
  std::memcpy(my_slot(), value, bytes);
  wait_as(kWaitWave);
  const int l = lane_id(), from = (l & ~(width - 1)) | ((l ^ mask) & (width - 1));
  std::memcpy(value, slot_of(from), bytes);
}
void hm_read_transposed(const void *p, int eb, void *out8) {
  std::memcpy(my_slot(), p, 8);
  wait_as(kWaitWave);
  const int l = lane_id(), group = l & ~15, i = l & 15;
  const int per_row = 8 / eb; // elements a lane names, and rows of the block: 4 of 16-bit, 8 of 8-bit elements
  char *out = (char *)out8;
  const int lanes_per_row = 16 / per_row; // lanes that together name one row of 16 elements
  for (int e = 0; e < per_row; ++e)       // column i of rows 0 .. per_row - 1
    std::memcpy(out + e * eb, slot_of(group + lanes_per_row * e + i / per_row) + (i % per_row) * eb, eb);
}
float hm_f8_to_f32(unsigned code, int ebits) {
  const int mbits = 7 - ebits, bias = (1 << (ebits - 1)) - 1;
  const int s = (code >> 7) & 1, e = (code >> mbits) & ((1 << ebits) - 1), m = code & ((1 << mbits) - 1);
  float v;
  if (ebits == 5 && e == 31)
    v = m ? NAN : INFINITY;
  else if (ebits == 4 && e == 15 && m == 7)
    v = NAN;
  else if (e == 0)
    v = std::ldexp((float)m, 1 - bias - mbits);
  else
    v = std::ldexp((float)((1 << mbits) + m), e - bias - mbits);
  return s ? -v : v;
}
static unsigned f32_to_f8(float f, int ebits) {
  if (f != f)
    return ebits == 4 ? 0x7f : 0x7e;
  unsigned best = 0;
  double best_err = INFINITY;
  const double a = std::fabs((double)f);
  for (unsigned c = 0; c < 128; ++c) {
    const float v = hm_f8_to_f32(c, ebits);
    if (v != v || std::isinf(v))
      continue;
    const double err = std::fabs((double)v - a);
    if (err < best_err || (err == best_err && (c & 1) == 0 && (best & 1) == 1)) {
      best = c;
      best_err = err;
    }
  }
  return best | (std::signbit(f) ? 0x80u : 0u);
}
int hm_cvt_pk_f8(float a, float b, int old, bool hi, int ebits) {
  const unsigned pair = f32_to_f8(a, ebits) | (f32_to_f8(b, ebits) << 8);
  return hi ? (int)(((unsigned)old & 0xffffu) | (pair << 16)) : (int)(((unsigned)old & 0xffff0000u) | pair);
}
// The products are formed in double precision and added to the accumulator once per instruction: exact, like
// the hardware's result, on the integer-valued data the tests use.
void hm_mfma_32x32(int type_a, int type_b, const void *a, const void *b, int lane_bytes, void *acc16) {
  char *mine = my_slot();
  std::memcpy(mine, a, lane_bytes);
  std::memcpy(mine + 64, b, lane_bytes);
  wait_as(kWaitWave);
  const int l = lane_id(), j = l & 31, per_lane = lane_bytes / elem_bytes(type_a);
  const bool int_acc = type_a == HM_I8;
  for (int v = 0; v < 16; ++v) {
    const int i = 8 * (v / 4) + 4 * (l / 32) + v % 4;
    double sum = 0.0;
    for (int half = 0; half < 2; ++half) {
      const char *ra = slot_of(i + 32 * half), *cb = slot_of(j + 32 * half) + 64;
      for (int k = 0; k < per_lane; ++k)
        sum += widen(type_a, ra, k) * widen(type_b, cb, k);
    }
    if (int_acc)
      ((int *)acc16)[v] = (int)((double)((int *)acc16)[v] + sum);
    else
      ((float *)acc16)[v] = (float)((double)((float *)acc16)[v] + sum);
  }
}

extern "C" {
// 0: loads into LDS land when issued; 1: not before the wait that covers them
void hm_set_late_loads(int on) { late_loads = on != 0; }
// the order in which a block's threads take their turns: 0 ascending, 1 descending, 2 waves rotated per pass
void hm_set_thread_order(int order) { thread_order = order; }
// 1: after every block the tensors are compared with what they were before it, and a byte that two blocks of one
// launch change is reported (every output element belongs to one block; costs a pass over the tensors per block)
void hm_set_owner_check(int on) { check_owners = on != 0; }
// only blocks [first, first + count) of every launch run (a problem too large to run whole: its last tiles)
void hm_set_blocks(unsigned first, unsigned count) {
  first_block = first;
  block_limit = count;
}
void hm_clear() {
  for (auto &r : ranges) {
    const size_t body = ((size_t)(r.hi - r.lo) + kPage - 1) / kPage * kPage + 2 * kPage;
    munmap(r.lo - kPage - kGuard, body + 2 * kGuard);
  }
  ranges.clear();
}
// A tensor of `bytes` bytes, 256-byte aligned like a device allocation, a page of canary bytes in front of it and
// canary bytes up to the end of its last page plus one more page behind it, all between two inaccessible regions.
void *hm_alloc(size_t bytes, const char *name) {
  const size_t body = (bytes + kPage - 1) / kPage * kPage + 2 * kPage;
  char *m = (char *)mmap(nullptr, body + 2 * kGuard, PROT_READ | PROT_WRITE, MAP_SHARED | MAP_ANONYMOUS, -1, 0);
  if (m == MAP_FAILED)
    return nullptr;
  mprotect(m, kGuard, PROT_NONE);
  mprotect(m + kGuard + body, kGuard, PROT_NONE);
  std::memset(m + kGuard, 0xA5, body);
  char *data = m + kGuard + kPage;
  ranges.push_back({data, data + bytes, name});
  return data;
}
// canary bytes around the tensor that no longer hold their value
long hm_canaries(void *data, size_t bytes) {
  char *d = (char *)data;
  long bad = 0;
  const size_t end = (bytes + kPage - 1) / kPage * kPage + kPage;
  for (char *p = d - kPage; p < d; ++p)
    bad += (unsigned char)*p != 0xA5;
  for (char *p = d + bytes; p < d + end; ++p)
    bad += (unsigned char)*p != 0xA5;
  return bad;
}
int hm_knows(const char *name) {
  for (const HmEntry *e = hm_kernel_table(); e->name; ++e)
    if (!std::strcmp(e->name, name))
      return 1;
  return 0;
}
// The same in the calling process, for a caller whose tensors are its own memory (nothing is registered then, and
// buffer loads are not range-checked; a trap ends the caller).  Returns -3 when the launch has not finished
// after `seconds` of wall time (0: no limit).
long hm_run_direct(const char *name, const void *params, void **pointers, unsigned grid, unsigned block, int seconds) {
  void (*fn)(void **, const void *) = nullptr;
  for (const HmEntry *e = hm_kernel_table(); e->name; ++e)
    if (!std::strcmp(e->name, name))
      fn = e->fn;
  if (!fn)
    return -1;
  static Report local;
  report = &local;
  std::memset(report, 0, sizeof *report);
  cur_kernel = name;
  gridDim = {grid, 1, 1};
  blockDim = {block, 1, 1};
  kernel_fn = fn;
  kernel_pointers = pointers;
  kernel_params = params;
  threads = block;
  const time_t start = time(nullptr);
  for (unsigned b = first_block; b < grid && b - first_block < block_limit; ++b) {
    blockIdx = {b, 0, 0};
    if (!run_block())
      break;
    if (seconds > 0 && time(nullptr) - start > seconds)
      return -3;
  }
  return report->violations;
}
// Runs every block of the launch, one after the other.  Returns the number of accesses outside the tensors (-1: no such
// kernel in this build, -2: the child could not be started); `first` receives a description of the first one.
long hm_run(const char *name, const void *params, void **pointers, unsigned grid, unsigned block, char *first,
            size_t first_bytes) {
  void (*fn)(void **, const void *) = nullptr;
  for (const HmEntry *e = hm_kernel_table(); e->name; ++e)
    if (!std::strcmp(e->name, name))
      fn = e->fn;
  if (!fn)
    return -1;
  if (!report)
    report = (Report *)mmap(nullptr, sizeof(Report), PROT_READ | PROT_WRITE, MAP_SHARED | MAP_ANONYMOUS, -1, 0);
  std::memset(report, 0, sizeof *report);
  fflush(nullptr);
  const pid_t child = fork();
  if (child < 0)
    return -2;
  if (child == 0) {
    static char trap_stack[64 * 1024];
    stack_t alt;
    alt.ss_sp = trap_stack;
    alt.ss_size = sizeof trap_stack;
    alt.ss_flags = 0;
    sigaltstack(&alt, nullptr);
    struct sigaction sa;
    std::memset(&sa, 0, sizeof sa);
    sa.sa_sigaction = on_trap;
    sa.sa_flags = SA_SIGINFO | SA_ONSTACK;
    sigaction(SIGSEGV, &sa, nullptr);
    sigaction(SIGBUS, &sa, nullptr);
    cur_kernel = name;
    gridDim = {grid, 1, 1};
    blockDim = {block, 1, 1};
    kernel_fn = fn;
    kernel_pointers = pointers;
    kernel_params = params;
    threads = block;
    if (check_owners)
      owners_begin();
    for (unsigned b = first_block; b < grid && b - first_block < block_limit; ++b) {
      blockIdx = {b, 0, 0};
      if (!run_block())
        break;
      if (check_owners)
        owners_after_block();
    }
    _exit(0);
  }
  int status = 0;
  waitpid(child, &status, 0);
  if (!WIFEXITED(status) || WEXITSTATUS(status) != 0) {
    report->violations += 1;
    if (!report->first[0])
      snprintf(report->first, sizeof report->first, "the run of %s ended with status %d", name, status);
  }
  if (first && first_bytes)
    snprintf(first, first_bytes, "%s", report->first);
  return report->violations;
}
}
