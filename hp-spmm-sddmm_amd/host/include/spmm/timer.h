// Timers of the SpMM drivers (include/spmm/utils/timer_cuda.h:3-40,
// include/spmm/utils/timer_cpu.h:4-28), on HIP events / the wall clock.
#pragma once

#include <hip/hip_runtime_api.h>
#include <sys/time.h>

#define WARMUP_NUM_CUDA 20
#define EXE_NUM_CUDA 200
#define WARMUP_NUM_CPU 2
#define EXE_NUM_CPU 2

struct GpuTimer {
  hipEvent_t start, stop;
  hipStream_t stream;
  explicit GpuTimer(hipStream_t s = nullptr) : stream(s) {
    (void)hipEventCreate(&start);
    (void)hipEventCreate(&stop);
  }
  ~GpuTimer() {
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
  }
  GpuTimer(const GpuTimer&) = delete;
  GpuTimer& operator=(const GpuTimer&) = delete;
  void Start() { (void)hipEventRecord(start, stream); }
  void Stop() { (void)hipEventRecord(stop, stream); }
  // milliseconds between Start() and Stop(); waits for Stop()
  float Elapsed() {
    float ms = 0.f;
    (void)hipEventSynchronize(stop);
    (void)hipEventElapsedTime(&ms, start, stop);
    return ms;
  }
};

struct CpuTimer {
  timeval start, stop;
  void Start() { gettimeofday(&start, nullptr); }
  void Stop() { gettimeofday(&stop, nullptr); }
  float Elapsed() {
    return (float)(((double)(stop.tv_sec - start.tv_sec) + (double)(stop.tv_usec - start.tv_usec) * 1e-6) * 1e3);
  }
};
