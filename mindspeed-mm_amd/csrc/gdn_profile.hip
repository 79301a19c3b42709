// Per-kernel event timing behind gdn_profile_* (see gdn_profile.h).  Host code only.
#include "gdn_profile.h"

#include <stdint.h>

#include <mutex>
#include <vector>

namespace gdn {

static const char* const kNames[kKernCount] = {
    "chunk_table_kernel", "chunk_prep_kernel", "chunk_state_kernel", "chunk_out_kernel",
    "chunk_state_bwd_kernel", "chunk_bwd_local_kernel",
    "recurrent_kernel", "conv1d_fwd_kernel", "conv1d_final_state_kernel",
    "conv1d_bwd_kernel", "conv1d_reduce_kernel", "conv1d_dh0_kernel", "conv1d_update_kernel",
    "rmsnorm_gated_fwd_kernel", "rmsnorm_gated_bwd_kernel", "rmsnorm_gated_dw_reduce_kernel",
    "gate_fwd_kernel", "gate_bwd_kernel", "gate_reduce_kernel", "kda_prep_kernel", "kda_bwd_finish_kernel", "kda_bwd_reduce_kernel"};

struct Pending { int id; hipEvent_t a, b; };
static bool g_on = false;
static std::mutex g_mu;
static std::vector<Pending> g_pending;
static hipEvent_t g_open[kKernCount];

bool profile_on() { return g_on; }

void profile_before(int id, hipStream_t st) {
  hipEvent_t e;
  if (hipEventCreate(&e) != hipSuccess) return;
  (void)hipEventRecord(e, st);
  std::lock_guard<std::mutex> lk(g_mu);
  g_open[id] = e;
}

void profile_after(int id, hipStream_t st) {
  hipEvent_t e;
  if (hipEventCreate(&e) != hipSuccess) return;
  (void)hipEventRecord(e, st);
  std::lock_guard<std::mutex> lk(g_mu);
  g_pending.push_back(Pending{id, g_open[id], e});
}

}  // namespace gdn

extern "C" int gdn_profile_enable(int on) {
  gdn::g_on = on != 0;
  return 0;
}

extern "C" int gdn_profile_kernel_count(void) { return gdn::kKernCount; }

extern "C" const char* gdn_profile_kernel_name(int id) {
  return (id >= 0 && id < gdn::kKernCount) ? gdn::kNames[id] : "";
}

// Waits for every recorded launch, adds its duration to total_ms[id] and 1 to launches[id], forgets it.
extern "C" int gdn_profile_collect(double* total_ms, int64_t* launches) {
  std::vector<gdn::Pending> todo;
  {
    std::lock_guard<std::mutex> lk(gdn::g_mu);
    todo.swap(gdn::g_pending);
  }
  int rc = 0;
  for (const gdn::Pending& p : todo) {
    float ms = 0.f;
    if (hipEventSynchronize(p.b) != hipSuccess || hipEventElapsedTime(&ms, p.a, p.b) != hipSuccess) rc = 1;
    else if (total_ms && launches) { total_ms[p.id] += ms; launches[p.id] += 1; }
    (void)hipEventDestroy(p.a);
    (void)hipEventDestroy(p.b);
  }
  return rc;
}
