// Optional per-kernel timing with HIP events on the launch stream (off by default).
#pragma once
#include <hip/hip_runtime.h>

namespace pal {

enum KernelId {
  kKernRecurrentFwd = 0,
  kKernChunkState,
  kKernChunkScan,
  kKernChunkOut,
  kKernBwdLocal,
  kKernBwdCarryScan,
  kKernBwdCarryApply,
  kKernBwdGate,   // unused since the gate gradients moved into the carry apply kernel (kept: ids are positional)
  kKernBwdHeadReduce,
  kKernRecurrentBwdFwdPass,
  kKernRecurrentBwd,
  kKernGlaOut,
  kKernGlaDq,
  kKernGlaDv,
  kKernGlaDk,
  kKernGlaBwdScan,
  kKernGlaBwdGate,
  kKernPrologueFwd,
  kKernPrologueBwd,
  kKernEpilogueFwd,
  kKernEpilogueBwd,
  kKernGlaRecurrentFwd,
  kKernChunkStates,
  kKernGlaBwdStates,
  kKernGlaBwdTile,
  kKernCount
};

// Records an event before and after the launch it brackets when timing is enabled.
struct ProfScope {
  int id;
  hipStream_t s;
  hipEvent_t e0;
  bool on;
  ProfScope(int id_, hipStream_t s_);
  ~ProfScope();
};

}  // namespace pal

#define PAL_TIMED_LAUNCH(id, stream, ...)      \
  do {                                         \
    pal::ProfScope ps__(id, stream);           \
    hipLaunchKernelGGL(__VA_ARGS__);           \
  } while (0)
