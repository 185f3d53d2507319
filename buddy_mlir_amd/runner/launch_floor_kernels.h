// launch_floor_kernels.h -- probe kernels of launch_floor_probe (two builds of
// launch_floor_kernels.hip: namespaces `plain` and `preload`).
#pragma once

#include <hip/hip_runtime.h>

struct Args30 {
  int v[30];
};

enum ProbeKernel {
  kEmpty, kArgs30, kArgs14, kTouch, kTouchStore, kTouchMeetStore, kStartTime, kCodeStraight, kCodeLoop
};

#define PROBE_DECLARE(ns)                                                      \
  namespace ns {                                                               \
  void launch(int which, int blocks, int threads, hipStream_t st,              \
              const Args30 &a, const void *w, unsigned tiles, int *sink);      \
  }
PROBE_DECLARE(plain)
PROBE_DECLARE(preload)
