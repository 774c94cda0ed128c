// Error reporting and version of the C ABI declared in include/mega_hip.h.
#include "common.h"

namespace mega {
namespace {
thread_local char g_err[512] = "";
}
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
}  // namespace mega

extern "C" const char* mega_last_error(void) { return mega::g_err; }
extern "C" int mega_abi_version(void) { return 3; }

// ------------------------------------------------------------------------------------------------
// Status of the bounded waits.  One word of pinned, device-mapped host memory per device: a kernel that
// gives up stores 1 into it (system scope); the entry points that launch such kernels look at it first and
// refuse the call once, the way a sticky launch error surfaces on the next call
// (C10_CUDA_KERNEL_LAUNCH_CHECK(), fairseq/csrc/ops/timestep_norm_kernel.cu:641).
#include <stdlib.h>

#include <atomic>
#include <mutex>

namespace mega {
namespace {
constexpr int kMaxDevices = 64;
constexpr uint32_t kDefaultSpinLimit = 1u << 22;
struct StatusSlot {
  volatile uint32_t* host = nullptr;   // what the host reads
  uint32_t* dev = nullptr;             // the same word as the kernels address it
  bool tried = false;
};
StatusSlot g_status[kMaxDevices];
volatile uint32_t g_plain[kMaxDevices];   // stands in where no pinned word exists (no device, allocation refused)
std::mutex g_status_mu;
std::atomic<uint32_t> g_spin_limit{kDefaultSpinLimit};
std::atomic<int> g_withhold_first{0};
std::atomic<int> g_checked{-1};             // -1: not decided yet (the environment decides at the first question)

int current_slot() {
  int d = 0;
  if (hipGetDevice(&d) != hipSuccess) {
    (void)hipGetLastError();
    d = 0;
  }
  return d >= 0 && d < kMaxDevices ? d : 0;
}

StatusSlot& slot_of(int d, bool may_allocate) {
  std::lock_guard<std::mutex> lock(g_status_mu);
  StatusSlot& s = g_status[d];
  if (!s.host) s.host = &g_plain[d];
  if (!s.dev && !s.tried && may_allocate) {
    s.tried = true;
    void* h = nullptr;
    void* dv = nullptr;
    if (hipHostMalloc(&h, 64, hipHostMallocMapped) == hipSuccess && h &&
        hipHostGetDevicePointer(&dv, h, 0) == hipSuccess && dv) {
      *(volatile uint32_t*)h = g_plain[d];
      s.host = (volatile uint32_t*)h;
      s.dev = (uint32_t*)dv;
    } else {
      (void)hipGetLastError();
    }
  }
  return s;
}
}  // namespace

LookbackLaunch lookback_launch(bool may_allocate) {
  StatusSlot& s = slot_of(current_slot(), may_allocate);
  LookbackLaunch l;
  l.status = s.dev;
  l.spin_limit = g_spin_limit.load();
  l.withhold_first = g_withhold_first.load();
  return l;
}

bool lookback_checked() {
  int v = g_checked.load();
  if (v < 0) {
    const char* e = getenv("MEGA_LOOKBACK_CHECKED");
    v = (e && e[0] && e[0] != '0') ? 1 : 0;
    g_checked.store(v);
  }
  return v != 0;
}

int lookback_verify(const char* entry, hipStream_t stream) {
  if (!lookback_checked()) return MEGA_OK;
  const hipError_t e = hipStreamSynchronize(stream);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    set_error("%s: checked mode could not wait for the launch (%s); it cannot be used under stream capture", entry,
              hipGetErrorString(e));
    return MEGA_ERR_LAUNCH;
  }
  StatusSlot& s = slot_of(current_slot(), false);
  if (*s.host == 0u) return MEGA_OK;
  *s.host = 0u;
  set_error("%s: this launch gave up waiting for the words of an earlier tile (workgroups not dispatched in id "
            "order, or a workspace shared by launches that overlap); it has written NaN into the outputs and "
            "statistics that depended on them.  The status is now clear", entry);
  return MEGA_ERR_LAUNCH;
}

int lookback_pending(const char* entry) {
  StatusSlot& s = slot_of(current_slot(), false);
  if (*s.host == 0u) return MEGA_OK;
  *s.host = 0u;
  set_error("%s: an earlier launch on this device gave up waiting for the words of an earlier tile (workgroups "
            "not dispatched in id order, or a workspace shared by launches that overlap); it has written NaN into "
            "the outputs and statistics that depended on them.  This call was not launched; the status is now clear",
            entry);
  return MEGA_ERR_LAUNCH;
}
}  // namespace mega

extern "C" int mega_lookback_init(void) {
  auto& s = mega::slot_of(mega::current_slot(), true);
  if (!s.dev) {
    mega::set_error("lookback_init: the status word of device %d could not be created (pinned, device-mapped host "
                    "memory refused)", mega::current_slot());
    return MEGA_ERR_LAUNCH;
  }
  return MEGA_OK;
}

extern "C" void mega_lookback_checked(int on) { mega::g_checked.store(on ? 1 : 0); }

extern "C" int mega_lookback_status(int clear) {
  auto& s = mega::slot_of(mega::current_slot(), false);
  const int v = (int)*s.host;
  if (clear) *s.host = 0u;
  return v;
}

extern "C" void mega_test_lookback(unsigned spin_limit, int withhold_first, int raise) {
  mega::g_spin_limit.store(spin_limit ? spin_limit : mega::kDefaultSpinLimit);
  mega::g_withhold_first.store(withhold_first ? 1 : 0);
  if (raise) *mega::slot_of(mega::current_slot(), false).host = 1u;
}

// ------------------------------------------------------------------------------------------------
// Address audit: see common.h.  Thread-local, like the error text.
namespace mega {
namespace {
struct AuditRange {
  uintptr_t lo, hi;
};
struct AuditState {
  bool on = false;
  int nranges = 0, nviolations = 0, nchecks = 0;
  AuditRange ranges[32];
};
thread_local AuditState g_audit;
}  // namespace

bool audit_on() { return g_audit.on; }

bool audit_use(const void* p, size_t bytes, const char* what) {
  AuditState& a = g_audit;
  ++a.nchecks;
  const uintptr_t lo = (uintptr_t)p, hi = lo + bytes;
  for (int i = 0; i < a.nranges; ++i)
    if (lo >= a.ranges[i].lo && hi <= a.ranges[i].hi) return true;
  if (a.nviolations++ == 0)
    set_error("audit: %s addresses [%p, %p), %zu bytes, outside every registered range", what, p, (const void*)hi,
              bytes);
  return false;
}
}  // namespace mega

extern "C" void mega_audit_begin(void) {
  mega::g_audit = mega::AuditState();
  mega::g_audit.on = true;
}

extern "C" int mega_audit_add(const void* base, size_t bytes) {
  mega::AuditState& a = mega::g_audit;
  if (!a.on || a.nranges >= 32) return MEGA_ERR_ARG;
  a.ranges[a.nranges++] = {(uintptr_t)base, (uintptr_t)base + bytes};
  return MEGA_OK;
}

extern "C" int mega_audit_end(int* checks) {
  mega::AuditState& a = mega::g_audit;
  const int v = a.nviolations;
  if (checks) *checks = a.nchecks;
  a.on = false;
  return v;
}
