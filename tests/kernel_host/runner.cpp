// Runner of the host build of the contraction kernels (see hip/hip_runtime.h in
// this directory): tensors between canary pages and inaccessible guard regions,
// one child process per launch so that a trap ends the child and not the test.
// Test infrastructure only.
#include "hip/hip_runtime.h"
#include "kernel_table.h"
#include <csignal>
#include <string>
#include <sys/mman.h>
#include <sys/wait.h>
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
} // namespace

void hm_check_global(const void *p, size_t n, const char *what) {
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

extern "C" {
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
// Runs every block and thread of the launch.  Returns the number of accesses outside the tensors (-1: no such
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
    struct sigaction sa;
    std::memset(&sa, 0, sizeof sa);
    sa.sa_sigaction = on_trap;
    sa.sa_flags = SA_SIGINFO;
    sigaction(SIGSEGV, &sa, nullptr);
    sigaction(SIGBUS, &sa, nullptr);
    cur_kernel = name;
    gridDim = {grid, 1, 1};
    blockDim = {block, 1, 1};
    for (unsigned b = 0; b < grid; ++b) {
      blockIdx = {b, 0, 0};
      for (unsigned t = 0; t < block; ++t) {
        threadIdx = {t, 0, 0};
        fn(pointers, params);
      }
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
