// Runtime shared by the emulated kernel libraries (see hip_emu.h): memory that ends or begins at an
// inaccessible page, the handler that turns an access to such a page into a message that names the
// kernel, the block, the thread and the buffer, and the settings of a run.
#include <signal.h>
#include <sys/mman.h>
#include <unistd.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>

namespace {

struct Region {
  char* mapping;
  size_t mapped;
  char* data;
  size_t bytes;
  std::string label;
};

std::map<uintptr_t, Region> regions;      // by data start
size_t page_bytes = 4096;
const char* current_kernel = "";
char current_call[128] = "";
unsigned where[4] = {0, 0, 0, 0};
int schedule_mode = 0, lds_mode = 0;
unsigned schedule_seed = 0;
bool handler_installed = false;
char alt_stack[1 << 16];

void describe(char* out, size_t size, const char* what, const void* address) {
  int n = snprintf(out, size,
                   "\n[emu] %s\n[emu]   call %s, kernel %s, block (%u, %u, %u), thread %u\n", what,
                   current_call[0] ? current_call : "?", current_kernel[0] ? current_kernel : "?", where[0],
                   where[1], where[2], where[3]);
  if (address && n > 0 && static_cast<size_t>(n) < size) {
    const char* a = static_cast<const char*>(address);
    for (const auto& entry : regions) {
      const Region& r = entry.second;
      if (a >= r.mapping && a < r.mapping + r.mapped) {
        if (a >= r.data + r.bytes)
          snprintf(out + n, size - n, "[emu]   address %p lies %zd bytes past the end of %s (%zu bytes)\n", address,
                   static_cast<ssize_t>(a - (r.data + r.bytes)), r.label.c_str(), r.bytes);
        else
          snprintf(out + n, size - n, "[emu]   address %p lies %zd bytes before the start of %s (%zu bytes)\n", address,
                   static_cast<ssize_t>(r.data - a), r.label.c_str(), r.bytes);
        return;
      }
    }
    snprintf(out + n, size - n, "[emu]   address %p belongs to no buffer of this call\n", address);
  }
}

void on_fault(int sig, siginfo_t* info, void*) {
  static char message[1024];
  describe(message, sizeof message,
           sig == SIGSEGV ? "memory fault in an emulated kernel (out of bounds, or a misaligned 16-byte access)"
                          : "bus error in an emulated kernel",
           info ? info->si_addr : nullptr);
  ssize_t ignored = write(2, message, strlen(message));
  (void)ignored;
  _exit(97);
}

void install_handler() {
  if (handler_installed) return;
  handler_installed = true;
  page_bytes = static_cast<size_t>(sysconf(_SC_PAGESIZE));
  stack_t ss;
  ss.ss_sp = alt_stack;
  ss.ss_size = sizeof alt_stack;
  ss.ss_flags = 0;
  sigaltstack(&ss, nullptr);
  struct sigaction sa;
  memset(&sa, 0, sizeof sa);
  sa.sa_sigaction = on_fault;
  sa.sa_flags = SA_SIGINFO | SA_ONSTACK;
  sigemptyset(&sa.sa_mask);
  sigaction(SIGSEGV, &sa, nullptr);
  sigaction(SIGBUS, &sa, nullptr);
}

}  // namespace

extern "C" {

void emu_rt_enter(const char* kernel) {
  install_handler();
  current_kernel = kernel;
}
void emu_rt_leave() { current_kernel = ""; }
void emu_rt_where(unsigned bx, unsigned by, unsigned bz, unsigned tx) {
  where[0] = bx;
  where[1] = by;
  where[2] = bz;
  where[3] = tx;
}
void emu_rt_call(const char* name) {
  snprintf(current_call, sizeof current_call, "%s", name ? name : "");
}
int emu_rt_schedule_mode() { return schedule_mode; }
unsigned emu_rt_schedule_seed() { return schedule_seed; }
void emu_rt_schedule(int mode, unsigned seed) {
  schedule_mode = mode;
  schedule_seed = seed;
}
int emu_rt_lds_mode() { return lds_mode; }
void emu_rt_set_lds_mode(int mode) { lds_mode = mode; }

void emu_rt_fail(const char* message) {
  static char text[1024];
  describe(text, sizeof text, message, nullptr);
  ssize_t ignored = write(2, text, strlen(text));
  (void)ignored;
  _exit(98);
}

// `bytes` of memory that end right before an inaccessible page (guard_before == 0: an overrun
// faults) or begin right after one (guard_before != 0: an underrun faults).  The start has the
// same remainder modulo 16 as `keep_alignment_of`, so code that asks whether a pointer is aligned
// gets the answer it gets for the original; what lies between the data and the other end of the
// mapping is filled with 0xff.  The block never straddles a multiple of 4 GiB.
void* emu_rt_guarded(size_t bytes, int guard_before, size_t keep_alignment_of) {
  install_handler();
  const size_t rem = keep_alignment_of % 16;
  const size_t body = ((bytes + 32 + page_bytes - 1) / page_bytes) * page_bytes;
  for (int attempt = 0; attempt < 8; ++attempt) {
    char* mapping = static_cast<char*>(mmap(nullptr, body + 2 * page_bytes, PROT_READ | PROT_WRITE,
                                            MAP_PRIVATE | MAP_ANONYMOUS, -1, 0));
    if (mapping == MAP_FAILED) return nullptr;
    const uintptr_t first = reinterpret_cast<uintptr_t>(mapping), last = first + body + 2 * page_bytes - 1;
    if ((first >> 32) != (last >> 32)) continue;     // leak the straddling mapping; the next one lies elsewhere
    memset(mapping, 0xff, body + 2 * page_bytes);
    mprotect(mapping, page_bytes, PROT_NONE);
    mprotect(mapping + page_bytes + body, page_bytes, PROT_NONE);
    char* data;
    if (guard_before) {
      data = mapping + page_bytes + rem;
    } else {
      uintptr_t end = reinterpret_cast<uintptr_t>(mapping + page_bytes + body);
      uintptr_t start = end - bytes;
      start -= (start - rem) % 16;     // largest start <= end - bytes with start % 16 == rem
      data = reinterpret_cast<char*>(start);
    }
    regions[reinterpret_cast<uintptr_t>(data)] = Region{mapping, body + 2 * page_bytes, data, bytes, "a buffer"};
    return data;
  }
  return nullptr;
}

void emu_rt_label(void* data, const char* label) {
  auto it = regions.find(reinterpret_cast<uintptr_t>(data));
  if (it != regions.end()) it->second.label = label ? label : "";
}

void emu_rt_release(void* data) {
  auto it = regions.find(reinterpret_cast<uintptr_t>(data));
  if (it == regions.end()) return;
  munmap(it->second.mapping, it->second.mapped);
  regions.erase(it);
}

}  // extern "C"
