// launch_floor_probe -- what one kernel of a dependent chain costs on this GPU
// before it has moved a byte, and how the decode GEMV's time splits into that
// fixed part and a bandwidth part.
//
// A decode step is ~143 kernels, each depending on the one before it.  This
// program replays chains of probe kernels from a hipGraph (the way the decode
// step runs) and prints the time per kernel:
//   (i)   a kernel that does nothing, at the grids the decode step uses;
//   (ii)  the same with ~30 kernel arguments read at wave start, with the
//         arguments preloaded into SGPRs by the command processor, with one
//         cold 1 KiB load per wavefront, with a store behind that load, with
//         the wavefronts of a workgroup meeting in LDS before the store (a
//         GEMV's tail), and with 16 KiB of straight-line code
//         against the same instruction count in a loop (cold instruction fetch);
//   (iii) the M = 1 int8 GEMV of libbuddy_hip over a ladder of matrix sizes,
//         weights rotated through 1 GiB so that every launch streams from HBM,
//         with the least-squares fit  time = a + bytes / b.
// Run it under `rocprofv3 --kernel-trace --stats` to see the same chains as
// per-kernel durations.
//
//   launch_floor_probe [--chain 128] [--replays 20] [--no-graph] [--layer]
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <vector>

#include "buddy_hip/buddy_hip.h"

#define CK(x)                                                                  \
  do {                                                                         \
    hipError_t e_ = (x);                                                       \
    if (e_ != hipSuccess) {                                                    \
      fprintf(stderr, "%s failed: %s (line %d)\n", #x, hipGetErrorString(e_),  \
              __LINE__);                                                       \
      exit(1);                                                                 \
    }                                                                          \
  } while (0)

#include "launch_floor_kernels.h"

namespace {

int g_chain = 128, g_replays = 20;
bool g_graph = true;
bool g_layer_only = false; // --layer: only the GEMV ladder and the fused launches
hipStream_t g_stream;

// Captures `chain` launches made by `enqueue(i)` into a graph, replays it and
// returns microseconds per launch.
template <typename F> double time_chain(F &&enqueue) {
  if (!g_graph) { // plain stream launches (for a profiler that traces each one)
    for (int i = 0; i < g_chain; ++i)
      enqueue(i);
    CK(hipStreamSynchronize(g_stream));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    CK(hipEventRecord(e0, g_stream));
    for (int r = 0; r < g_replays; ++r)
      for (int i = 0; i < g_chain; ++i)
        enqueue(i);
    CK(hipEventRecord(e1, g_stream));
    CK(hipEventSynchronize(e1));
    float ms = 0.f;
    CK(hipEventElapsedTime(&ms, e0, e1));
    CK(hipEventDestroy(e0));
    CK(hipEventDestroy(e1));
    return (double)ms * 1e3 / ((double)g_chain * g_replays);
  }
  hipGraph_t graph;
  hipGraphExec_t exec;
  CK(hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal));
  for (int i = 0; i < g_chain; ++i)
    enqueue(i);
  CK(hipStreamEndCapture(g_stream, &graph));
  CK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
  for (int i = 0; i < 3; ++i)
    CK(hipGraphLaunch(exec, g_stream));
  CK(hipStreamSynchronize(g_stream));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  CK(hipEventRecord(e0, g_stream));
  for (int i = 0; i < g_replays; ++i)
    CK(hipGraphLaunch(exec, g_stream));
  CK(hipEventRecord(e1, g_stream));
  CK(hipEventSynchronize(e1));
  float ms = 0.f;
  CK(hipEventElapsedTime(&ms, e0, e1));
  CK(hipEventDestroy(e0));
  CK(hipEventDestroy(e1));
  CK(hipGraphExecDestroy(exec));
  CK(hipGraphDestroy(graph));
  return (double)ms * 1e3 / ((double)g_chain * g_replays);
}

} // namespace

int main(int argc, char **argv) {
  for (int i = 1; i < argc; ++i) {
    if (!strcmp(argv[i], "--chain") && i + 1 < argc)
      g_chain = atoi(argv[++i]);
    else if (!strcmp(argv[i], "--replays") && i + 1 < argc)
      g_replays = atoi(argv[++i]);
    else if (!strcmp(argv[i], "--no-graph"))
      g_graph = false;
    else if (!strcmp(argv[i], "--layer"))
      g_layer_only = true;
  }
  CK(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
  int *sink; // 16 ints per wavefront of the largest grid
  CK(hipMalloc(&sink, sizeof(int) * 16 * 2374 * 4));
  const size_t pool_bytes = (size_t)1 << 30;
  int8_t *pool;
  CK(hipMalloc(&pool, pool_bytes));
  CK(hipMemset(pool, 1, pool_bytes));
  CK(hipDeviceSynchronize());

  struct Grid {
    int blocks, threads;
  };
  const Grid grids[] = {{1, 64}, {256, 256}, {560, 512}, {2374, 256}};
  Args30 a30;
  for (int i = 0; i < 30; ++i)
    a30.v[i] = i;
  printf("chains of %d dependent kernels %s, us per kernel\n", g_chain,
         g_graph ? "replayed from a hipGraph" : "launched on one stream");
  printf("(p) = built with kernel-argument preload into SGPRs\n");
  printf("%-10s %7s %7s %7s %9s %8s %10s %9s %9s %8s %8s\n", "grid", "empty", "args30",
         "args14", "args14(p)", "touch1K", "touch1K(p)", "touch+st", "+meet+st", "code16K",
         "codeloop");
  const unsigned window = 16u << 20; // a fresh 16 MiB per launch: tiles come from HBM
  for (const Grid &g : grids) {
    if (g_layer_only)
      break;
    auto run = [&](bool pre, int which) {
      return time_chain([&](int i) {
        const int8_t *w = pool + ((size_t)i * window) % (pool_bytes - window);
        (pre ? preload::launch : plain::launch)(which, g.blocks, g.threads, g_stream, a30, w,
                                                window / 1024, sink);
      });
    };
    char name[32];
    snprintf(name, sizeof name, "%dx%d", g.blocks, g.threads);
    printf("%-10s %7.2f %7.2f %7.2f %9.2f %8.2f %10.2f %9.2f %9.2f %8.2f %8.2f\n", name,
           run(false, kEmpty), run(false, kArgs30), run(false, kArgs14), run(true, kArgs14),
           run(false, kTouch), run(true, kTouch), run(false, kTouchStore),
           run(false, kTouchMeetStore), run(false, kCodeStraight), run(false, kCodeLoop));
    fflush(stdout);
  }

  // ---- how long the dispatcher takes to start every wavefront of a grid -----
  if (!g_layer_only) {
    printf("\ndispatch spread: first to last wavefront start of one launch, us "
           "(median of 20 launches)\n");
    printf("%-12s %8s %10s %12s %14s\n", "grid", "waves", "no LDS", "1 KiB LDS", "14 args in SGPRs");
    const Grid dg[] = {{960, 64},  {240, 256}, {120, 512}, {60, 1024}, {128, 512},
                       {4480, 64}, {1120, 256}, {560, 512}, {280, 1024}, {96, 1024}};
    unsigned long long *ts;
    const int max_waves = 8192;
    CK(hipMalloc(&ts, sizeof(unsigned long long) * max_waves));
    std::vector<unsigned long long> h(max_waves);
    for (const Grid &g : dg) {
      const int waves = g.blocks * (g.threads / 64);
      double res[3];
      for (int mode = 0; mode < 3; ++mode) {
        std::vector<double> spreads;
        for (int rep = 0; rep < 20; ++rep) {
          (mode == 2 ? preload::launch : plain::launch)(
              kStartTime, g.blocks, g.threads, g_stream, a30, nullptr, mode == 1 ? 1024u : 0u,
              reinterpret_cast<int *>(ts));
          CK(hipStreamSynchronize(g_stream));
          CK(hipMemcpy(h.data(), ts, sizeof(unsigned long long) * waves, hipMemcpyDeviceToHost));
          unsigned long long lo = ~0ull, hi = 0;
          for (int i = 0; i < waves; ++i) {
            lo = h[i] < lo ? h[i] : lo;
            hi = h[i] > hi ? h[i] : hi;
          }
          spreads.push_back((double)(hi - lo) / 100.0);
        }
        std::sort(spreads.begin(), spreads.end());
        res[mode] = spreads[spreads.size() / 2];
      }
      char name[32];
      snprintf(name, sizeof name, "%dx%d", g.blocks, g.threads);
      printf("%-12s %8d %10.2f %12.2f %14.2f\n", name, waves, res[0], res[1], res[2]);
    }
    CK(hipFree(ts));
  }

  // ---- the M = 1 int8 GEMV over a size ladder ------------------------------
  const int64_t K = 1536;
  float *x, *scale, *y;
  const int64_t n_max = ((int64_t)256 << 20) / K;
  CK(hipMalloc(&x, sizeof(float) * K));
  CK(hipMalloc(&scale, sizeof(float) * n_max));
  CK(hipMalloc(&y, sizeof(float) * n_max));
  CK(hipMemset(x, 0, sizeof(float) * K));
  CK(hipMemset(scale, 0, sizeof(float) * n_max));
  printf("\nM = 1 int8 GEMV, K = %lld, weights rotated through %zu MiB (HBM-cold)\n",
         (long long)K, pool_bytes >> 20);
  printf("%10s %10s %10s %10s\n", "MB", "N", "us", "GB/s");
  std::vector<double> xs, ys;
  for (int mb = 1; mb <= (g_layer_only ? 32 : 256); mb *= 2) {
    const int64_t N = ((int64_t)mb << 20) / K / 16 * 16;
    const size_t bytes = (size_t)K * N;
    const size_t slots = pool_bytes / bytes;
    const double us = time_chain([&](int i) {
      buddy_hip_linear_desc d;
      memset(&d, 0, sizeof d);
      d.A = x;
      d.lda = K;
      d.W0 = pool + (size_t)(i % slots) * bytes;
      d.scale0 = scale;
      d.C = y;
      d.ldc = N;
      d.M = 1;
      d.K = K;
      d.N = N;
      d.epilogue = BUDDY_HIP_EPI_STORE;
      if (buddy_hip_linear_w8a32(&d, g_stream)) {
        fprintf(stderr, "gemv failed: %s\n", buddy_hip_last_error());
        exit(1);
      }
    });
    const double b = (double)bytes + 4.0 * (K + 2 * N);
    printf("%10.1f %10lld %10.2f %10.0f\n", b / 1e6, (long long)N, us, b / us / 1e3);
    xs.push_back(b);
    ys.push_back(us);
  }
  // ---- the fused GEMV launches of one decoder layer (Qwen2-1.5B shapes) ----
  // against the line fitted below: what the fusions cost on top of streaming
  struct Fused {
    const char *name;
    int64_t K, N;
    bool norm, dual;
    int epi;
  };
  const Fused fused[] = {
      {"RMSNorm + q|k|v (1536 -> 2048)", 1536, 2048, true, false, BUDDY_HIP_EPI_STORE},
      {"o_proj + residual (1536 -> 1536)", 1536, 1536, false, false, BUDDY_HIP_EPI_ACCUM},
      {"RMSNorm + gate|up + SiLU*mul (1536 -> 2 x 8960)", 1536, 8960, true, true,
       BUDDY_HIP_EPI_SILU_MUL},
      {"gate|up + SiLU*mul, no norm", 1536, 8960, false, true, BUDDY_HIP_EPI_SILU_MUL},
      {"one matrix of the same bytes (1536 -> 17920)", 1536, 17920, false, false,
       BUDDY_HIP_EPI_STORE},
      {"the same with RMSNorm", 1536, 17920, true, false, BUDDY_HIP_EPI_STORE},
      {"down + residual (8960 -> 1536)", 8960, 1536, false, false, BUDDY_HIP_EPI_ACCUM},
      {"the same K, twice the channels (8960 -> 3072)", 8960, 3072, false, false,
       BUDDY_HIP_EPI_ACCUM},
      {"the same K, 8960 -> 4096", 8960, 4096, false, false, BUDDY_HIP_EPI_ACCUM},
  };
  float *xin, *nw;
  CK(hipMalloc(&xin, sizeof(float) * 8960));
  CK(hipMalloc(&nw, sizeof(float) * 8960));
  CK(hipMemset(xin, 0, sizeof(float) * 8960));
  CK(hipMemset(nw, 0, sizeof(float) * 8960));
  // The small operands (activation row, norm weight, scales, output row) either
  // stay where they are from launch to launch (they sit in every L2) or rotate
  // through their own 512 MiB like the weights: in a decoder every layer has its
  // own, read once per step.
  const size_t small_bytes = (size_t)512 << 20;
  char *small_pool;
  CK(hipMalloc(&small_pool, small_bytes));
  CK(hipMemset(small_pool, 0, small_bytes));
  const size_t small_slot = (size_t)256 << 10; // 4 vectors of up to 64 KiB
  std::vector<std::pair<double, double>> fused_res;
  for (int cold = 0; cold < 2; ++cold) {
    printf("\nfused launches of a decoder layer, same rotation of the weights; small operands %s\n",
           cold ? "rotated too (cold)" : "in place (cache-warm)");
    for (const Fused &f : fused) {
      const size_t bytes = (size_t)f.K * f.N;
      const size_t per = bytes * (f.dual ? 2 : 1);
      const size_t slots = pool_bytes / per;
      const double us = time_chain([&](int i) {
        buddy_hip_linear_desc d;
        memset(&d, 0, sizeof d);
        float *sm = reinterpret_cast<float *>(
            small_pool + ((size_t)i * 7919 % (small_bytes / small_slot)) * small_slot);
        d.A = cold ? sm : xin;
        d.lda = f.K;
        d.W0 = pool + (size_t)(i % slots) * per;
        d.scale0 = cold ? sm + 16384 : scale;
        if (f.dual) {
          d.W1 = d.W0 + bytes;
          d.scale1 = d.scale0 + f.N;
        }
        if (f.norm) {
          d.norm_w = cold ? sm + 49152 : nw;
          d.norm_eps = 1e-6f;
        }
        d.C = cold ? sm + 32768 : y;
        d.ldc = f.N;
        d.M = 1;
        d.K = f.K;
        d.N = f.N;
        d.epilogue = f.epi;
        if (buddy_hip_linear_w8a32(&d, g_stream)) {
          fprintf(stderr, "gemv failed: %s\n", buddy_hip_last_error());
          exit(1);
        }
      });
      const double b = (double)per + 4.0 * (f.K * (f.norm ? 2 : 1) + f.N * (f.dual ? 3 : 2) +
                                            (f.epi == BUDDY_HIP_EPI_ACCUM ? f.N : 0));
      fused_res.push_back({b, us});
      printf("  %-50s %8.2f MB %7.2f us %6.0f GB/s\n", f.name, b / 1e6, us, b / us / 1e3);
    }
  }

  // least squares  us = a + bytes / b
  double sx = 0, sy = 0, sxx = 0, sxy = 0;
  const double n = (double)xs.size();
  for (size_t i = 0; i < xs.size(); ++i) {
    sx += xs[i];
    sy += ys[i];
    sxx += xs[i] * xs[i];
    sxy += xs[i] * ys[i];
  }
  const double slope = (n * sxy - sx * sy) / (n * sxx - sx * sx);
  const double a = (sy - slope * sx) / n;
  printf("fit over the ladder: us = %.2f + bytes / %.0f GB/s\n", a, 1.0 / slope / 1e3);
  // the same over the sizes a 1.5B decoder layer uses (up to 32 MB)
  sx = sy = sxx = sxy = 0;
  int cnt = 0;
  for (size_t i = 0; i < xs.size() && xs[i] < 40e6; ++i, ++cnt) {
    sx += xs[i];
    sy += ys[i];
    sxx += xs[i] * xs[i];
    sxy += xs[i] * ys[i];
  }
  const double slope2 = (cnt * sxy - sx * sy) / (cnt * sxx - sx * sx);
  printf("fit up to 32 MB:     us = %.2f + bytes / %.0f GB/s\n", (sy - slope2 * sx) / cnt,
         1.0 / slope2 / 1e3);
  return 0;
}
