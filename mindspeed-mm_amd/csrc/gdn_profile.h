// Optional per-kernel timing with HIP events on the launch stream (off by default; when off a launch is a
// plain hipLaunchKernelGGL).  Used by the benchmark to attribute step time to kernels.
#pragma once
#include <hip/hip_runtime.h>

namespace gdn {

enum KernelId {
  kKernChunkTable = 0, kKernPrep, kKernStateFwd, kKernOut, kKernStateBwd, kKernBwdLocal,
  kKernRecurrent, kKernConvFwd, kKernConvState, kKernConvBwd, kKernConvReduce,
  kKernConvDh0, kKernConvUpdate, kKernRmsNormFwd, kKernRmsNormBwd, kKernRmsNormReduce,
  kKernGateFwd, kKernGateBwd, kKernGateReduce, kKernKdaPrep, kKernKdaBwdFinish, kKernKdaBwdReduce, kKernCount
};

bool profile_on();
void profile_before(int id, hipStream_t st);
void profile_after(int id, hipStream_t st);

}  // namespace gdn

#define GDN_LAUNCH(id, st, ...)                               \
  do {                                                        \
    if (gdn::profile_on()) gdn::profile_before((id), (st));   \
    hipLaunchKernelGGL(__VA_ARGS__);                          \
    if (gdn::profile_on()) gdn::profile_after((id), (st));    \
  } while (0)
