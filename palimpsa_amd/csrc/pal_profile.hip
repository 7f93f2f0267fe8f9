// Per-kernel timing aid: when enabled, every kernel launch made through the library (from any thread:
// autograd runs the backward entry points on a thread of its own) is bracketed by two HIP events on the
// launch stream.  Meant for benchmarks.  This is the only state of the library that calls share; the
// switch is an atomic flag and the event list and counters are guarded by a mutex, so concurrent callers
// are safe whether it is on or off, and when it is off (the default) a launch only reads the flag.
#include <atomic>
#include <mutex>
#include <vector>

#include "pal_common.h"
#include "pal_profile.h"

namespace pal {

struct Pair { int id; hipEvent_t a, b; };
static std::atomic<bool> g_on{false};
static std::mutex g_mu;                 // guards everything below
static std::vector<Pair> g_pending;
static double g_ms[kKernCount];
static long long g_n[kKernCount];

ProfScope::ProfScope(int id_, hipStream_t s_) : id(id_), s(s_), e0(nullptr), on(g_on.load(std::memory_order_relaxed)) {
  if (!on) return;
  if (hipEventCreate(&e0) != hipSuccess) { on = false; return; }
  (void)hipEventRecord(e0, s);
}
ProfScope::~ProfScope() {
  if (!on) return;
  hipEvent_t e1;
  if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return; }
  (void)hipEventRecord(e1, s);
  std::lock_guard<std::mutex> lk(g_mu);
  g_pending.push_back({id, e0, e1});
}

// caller holds g_mu
static void drain() {
  for (auto& p : g_pending) {
    float ms = 0.f;
    if (hipEventSynchronize(p.b) == hipSuccess && hipEventElapsedTime(&ms, p.a, p.b) == hipSuccess) {
      g_ms[p.id] += ms;
      g_n[p.id] += 1;
    }
    (void)hipEventDestroy(p.a);
    (void)hipEventDestroy(p.b);
  }
  g_pending.clear();
}

static const char* kNames[kKernCount] = {
    "recurrent_fwd_kernel", "chunk_delta_kernel", "chunk_scan_kernel", "chunk_out_kernel", "chunk_bwd_local_kernel",
    "chunk_bwd_carry_scan_kernel", "chunk_bwd_carry_apply_kernel", "chunk_bwd_gate_kernel",
    "chunk_bwd_head_reduce_kernel", "recurrent_bwd_state_kernel", "recurrent_bwd_kernel", "gla_out_kernel",
    "gla_dq_kernel", "gla_dv_kernel", "gla_dk_kernel", "gla_bwd_scan_kernel", "gla_bwd_gate_kernel",
    "prologue_fwd_kernel", "prologue_bwd_kernel", "epilogue_fwd_kernel", "epilogue_bwd_kernel",
    "gla_recurrent_fwd_kernel", "chunk_states_kernel", "gla_bwd_states_kernel", "gla_bwd_tile_kernel"};

}  // namespace pal

extern "C" {

int pal_profile_enable(int on) {
  std::lock_guard<std::mutex> lk(pal::g_mu);
  pal::drain();
  for (int i = 0; i < pal::kKernCount; ++i) { pal::g_ms[i] = 0.0; pal::g_n[i] = 0; }
  pal::g_on.store(on != 0, std::memory_order_relaxed);
  return PAL_OK;
}

int pal_profile_kernel_count(void) { return pal::kKernCount; }

const char* pal_profile_kernel_name(int id) {
  return (id >= 0 && id < pal::kKernCount) ? pal::kNames[id] : "";
}

int pal_profile_read(int id, double* total_ms, int64_t* launches) {
  if (id < 0 || id >= pal::kKernCount || !total_ms || !launches) return PAL_E_DIM;
  std::lock_guard<std::mutex> lk(pal::g_mu);
  pal::drain();
  *total_ms = pal::g_ms[id];
  *launches = pal::g_n[id];
  return PAL_OK;
}

}  // extern "C"
