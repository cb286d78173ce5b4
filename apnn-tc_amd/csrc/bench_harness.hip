// Timing loops for the benchmark driver: the counterpart of the timing section of the reference's
// benchmark mains (APNN-TC-lib/bmmaTensorCoreGemm/src/71_bmmaTensorCoreGemm.cu:526-549), which
// launch the kernel NUM_PROFILES times between CUDA events.  Built into libapnn_bench.so, which
// links libapnn_tc.so and calls it only through the C ABI.
#include <hip/hip_runtime.h>

#include <chrono>

#include "../../include/apnn_tc.h"

namespace {

template <class F>
int timed_loop(F &&launch, int warmup, int iters, hipStream_t stream, float *event_ms, double *wall_ms) {
  hipEvent_t e0, e1;
  hipError_t err;
  if ((err = hipEventCreate(&e0)) != hipSuccess) return (int)err;
  if ((err = hipEventCreate(&e1)) != hipSuccess) return (int)err;
  int rc = 0;
  for (int i = 0; i < warmup && rc == 0; ++i) rc = launch();
  if (rc == 0 && (err = hipStreamSynchronize(stream)) != hipSuccess) rc = (int)err;
  if (rc == 0) {
    const auto t0 = std::chrono::steady_clock::now();
    (void)hipEventRecord(e0, stream);
    for (int i = 0; i < iters && rc == 0; ++i) rc = launch();
    (void)hipEventRecord(e1, stream);
    err = hipStreamSynchronize(stream);
    const auto t1 = std::chrono::steady_clock::now();
    if (rc == 0 && err != hipSuccess) rc = (int)err;
    if (rc == 0) {
      float ms = 0.f;
      (void)hipEventElapsedTime(&ms, e0, e1);
      *event_ms = ms;
      *wall_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    }
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return rc;
}

// Same measurement with the launches replayed from a HIP graph: `batch` launches are captured once
// (on a stream of its own, default priority) and the graph is launched ceil(n / batch) times, the last
// time through a second graph holding the remainder, so exactly `iters` kernels run in the timed region.
// The host then issues one graph launch per `batch` kernels instead of one call per kernel.  Every
// executable graph the timed region uses is launched once, untimed, beforehand (the first launch of a
// graph pays for its upload to the device: a timed region of one or two graph launches would otherwise
// measure that), so at least `warmup` untimed kernels run, rounded up to whole graphs.
template <class F>
int timed_graph_loop(F &&launch_on, int warmup, int iters, int batch, float *event_ms, double *wall_ms) {
  if (batch < 1) batch = 1;
  hipStream_t cs = nullptr;
  hipError_t err = hipStreamCreateWithFlags(&cs, hipStreamNonBlocking);
  if (err != hipSuccess) return (int)err;
  hipGraphExec_t full = nullptr, rest_w = nullptr, rest_i = nullptr;
  int rc = 0;
  auto capture = [&](int n, hipGraphExec_t *exec) -> int {
    if (n <= 0) return 0;
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamBeginCapture(cs, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return (int)e;
    int r = 0;
    for (int i = 0; i < n && r == 0; ++i) r = launch_on(cs);
    e = hipStreamEndCapture(cs, &g);
    if (r != 0) return r;
    if (e != hipSuccess) return (int)e;
    e = hipGraphInstantiate(exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    return (int)e;
  };
  const int nfull_needed = (warmup >= batch || iters >= batch) ? batch : 0;
  if ((rc = capture(nfull_needed, &full)) == 0 && (rc = capture(warmup % batch, &rest_w)) == 0)
    rc = capture(iters % batch, &rest_i);
  auto replay = [&](int n, hipGraphExec_t rest) -> int {
    for (int i = 0; i < n / batch; ++i) {
      const hipError_t e = hipGraphLaunch(full, cs);
      if (e != hipSuccess) return (int)e;
    }
    if (n % batch) {
      const hipError_t e = hipGraphLaunch(rest, cs);
      if (e != hipSuccess) return (int)e;
    }
    return 0;
  };
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (rc == 0 && (err = hipEventCreate(&e0)) != hipSuccess) rc = (int)err;
  if (rc == 0 && (err = hipEventCreate(&e1)) != hipSuccess) rc = (int)err;
  if (rc == 0) rc = replay(warmup, rest_w);
  if (rc == 0 && warmup < batch && iters >= batch && (err = hipGraphLaunch(full, cs)) != hipSuccess) rc = (int)err;
  if (rc == 0 && rest_i != nullptr && (err = hipGraphLaunch(rest_i, cs)) != hipSuccess) rc = (int)err;
  if (rc == 0 && (err = hipStreamSynchronize(cs)) != hipSuccess) rc = (int)err;
  if (rc == 0) {
    const auto t0 = std::chrono::steady_clock::now();
    (void)hipEventRecord(e0, cs);
    rc = replay(iters, rest_i);
    (void)hipEventRecord(e1, cs);
    err = hipStreamSynchronize(cs);
    const auto t1 = std::chrono::steady_clock::now();
    if (rc == 0 && err != hipSuccess) rc = (int)err;
    if (rc == 0) {
      float ms = 0.f;
      (void)hipEventElapsedTime(&ms, e0, e1);
      *event_ms = ms;
      *wall_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    }
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (full) (void)hipGraphExecDestroy(full);
  if (rest_w) (void)hipGraphExecDestroy(rest_w);
  if (rest_i) (void)hipGraphExecDestroy(rest_i);
  (void)hipStreamDestroy(cs);
  return rc;
}

}  // namespace

extern "C" {

// apnn_bench_gemm with the launches replayed from HIP graphs of `batch` launches each.
int apnn_bench_gemm_graph(const apnn_gemm_desc *d, int warmup, int iters, int batch, float *event_ms,
                          double *wall_ms) {
  return timed_graph_loop([&](hipStream_t cs) { return apnn_gemm(d, cs); }, warmup, iters, batch, event_ms, wall_ms);
}

// Cold-cache variant: launch i works on descriptor descs[i % nsets], every descriptor naming buffers of
// its own.  With graphs of `batch` = nsets launches and nsets x (bytes of one buffer set) larger than the
// last-level cache, a buffer set is revisited only after every other set went through the caches.
int apnn_bench_gemm_graph_rotate(const apnn_gemm_desc *descs, int nsets, int warmup, int iters, int batch,
                                 float *event_ms, double *wall_ms) {
  if (descs == nullptr || nsets < 1) return APNN_EINVAL;
  long long next = 0;
  return timed_graph_loop([&](hipStream_t cs) { return apnn_gemm(&descs[next++ % nsets], cs); }, warmup, iters, batch,
                          event_ms, wall_ms);
}

// Runs `iters` back-to-back apnn_gemm launches of the same descriptor on `stream` after `warmup`
// untimed ones.  event_ms: HIP-event time over the timed launches; wall_ms: host wall clock from
// first launch to stream idle.
int apnn_bench_gemm(const apnn_gemm_desc *d, int warmup, int iters, apnn_stream_t s, float *event_ms,
                    double *wall_ms) {
  hipStream_t stream = static_cast<hipStream_t>(s);
  return timed_loop([&]() { return apnn_gemm(d, s); }, warmup, iters, stream, event_ms, wall_ms);
}

int apnn_bench_conv_graph(const apnn_conv_desc *d, int warmup, int iters, int batch, float *event_ms,
                          double *wall_ms) {
  return timed_graph_loop([&](hipStream_t cs) { return apnn_conv(d, cs); }, warmup, iters, batch, event_ms, wall_ms);
}

int apnn_bench_conv(const apnn_conv_desc *d, int warmup, int iters, apnn_stream_t s, float *event_ms,
                    double *wall_ms) {
  hipStream_t stream = static_cast<hipStream_t>(s);
  return timed_loop([&]() { return apnn_conv(d, s); }, warmup, iters, stream, event_ms, wall_ms);
}

__global__ void apnn_bench_empty_kernel() {}

// Launch floor of the machine: the same loop around an empty kernel.
int apnn_bench_empty(int warmup, int iters, apnn_stream_t s, float *event_ms, double *wall_ms) {
  hipStream_t stream = static_cast<hipStream_t>(s);
  return timed_loop(
      [&]() {
        hipLaunchKernelGGL(apnn_bench_empty_kernel, dim3(1), dim3(64), 0, stream);
        return (int)hipGetLastError();
      },
      warmup, iters, stream, event_ms, wall_ms);
}

__global__ __launch_bounds__(256) void apnn_bench_copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                              long long n16) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n16;
       i += (long long)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

// Plain device-to-device copy of `bytes` (multiple of 16): reads `bytes`, writes `bytes`.  Used to
// calibrate the HBM traffic counters (FETCH_SIZE / WRITE_SIZE) against a kernel of known traffic.
int apnn_bench_copy(const void *src, void *dst, long long bytes, apnn_stream_t s) {
  if (src == nullptr || dst == nullptr || bytes <= 0 || (bytes % 16) != 0) return APNN_EINVAL;
  hipLaunchKernelGGL(apnn_bench_copy_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(s),
                     static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), bytes / 16);
  return (int)hipGetLastError();
}

// The int32 store of the matrix-core kernels, alone: a wave owns a 32-row x 32-column block and every
// store instruction writes two 128-byte row segments (lane half g, register j -> row 8q + 4g + j,
// lane%32 -> column), the segments of one instruction being four rows apart.  Writes rows x cols x 4
// bytes exactly once; calibrates WRITE_SIZE for this store pattern.
__global__ __launch_bounds__(256) void apnn_bench_store_blocks_kernel(int *__restrict__ dst, int rows, int cols) {
  const int lane = threadIdx.x & 63, li = lane & 31, g = lane >> 5;
  const int blocks_per_row = cols / 32;
  const long long nblocks = (long long)(rows / 32) * blocks_per_row;
  const long long wave0 = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  for (long long b = wave0; b < nblocks; b += (long long)gridDim.x * 4) {
    const int r0 = (int)(b / blocks_per_row) * 32, c0 = (int)(b % blocks_per_row) * 32;
    int *base = dst + (long long)(r0 + 4 * g) * cols + c0 + li;
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) base[(long long)(8 * q + j) * cols] = (int)b + q + j;
  }
}

int apnn_bench_store_blocks(int *dst, int rows, int cols, apnn_stream_t s) {
  if (dst == nullptr || rows <= 0 || cols <= 0 || (rows % 32) != 0 || (cols % 32) != 0) return APNN_EINVAL;
  hipLaunchKernelGGL(apnn_bench_store_blocks_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(s), dst, rows,
                     cols);
  return (int)hipGetLastError();
}

}  // extern "C"
