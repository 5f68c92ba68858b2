// bikv_link_probe — what the host link of this box does for hipMemcpyAsync, and what a release of device
// memory does to it. A deployment diagnostic of the staging pipeline (it helps choose between the staging
// modes: the pipelined mode moves bytes with hipMemcpyAsync, the direct and pipelined_kernel modes with the
// library's own kernels); the reference has no counterpart.
//
//   bikv_link_probe [GiB ...]      default: 8 32
//
// For every size X: streams created up front (and one created after the release) take turns copying
// 16 MiB device -> host and host -> device with hipMemcpyAsync, then X GiB of device memory is allocated,
// written and freed again (hipFree returns at once), and the copies go on. Reported: the rates before, how
// long copies stay below 80 % of that after the free and at what rate, per direction; and, next to them,
// the rate of a kernel that stores the same bytes through the device mapping of the pinned buffer.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define CK(x)                                                                        \
  do {                                                                               \
    hipError_t e_ = (x);                                                             \
    if (e_ != hipSuccess) {                                                          \
      fprintf(stderr, "%s failed: %s (line %d)\n", #x, hipGetErrorString(e_), __LINE__); \
      exit(1);                                                                       \
    }                                                                                \
  } while (0)

// one 16-byte vector per lane, 64-lane workgroups: the shape of the library's movers
__global__ __launch_bounds__(64) void store_to_host(const char* src, char* dst, size_t bytes) {
  const size_t lo = (size_t)blockIdx.x * 1024 + threadIdx.x * 16;
  if (lo < bytes) __builtin_nontemporal_store(__builtin_nontemporal_load((const u32x4*)(src + lo)), (u32x4*)(dst + lo));
}

int main(int argc, char** argv) {
  std::vector<int> sizes;
  for (int i = 1; i < argc; ++i) sizes.push_back(atoi(argv[i]));
  if (sizes.empty()) sizes = {8, 32};
  const size_t n = (size_t)16 << 20;
  char *dev, *host, *host_dev;
  CK(hipMalloc(&dev, n));
  CK(hipHostMalloc(&host, n, hipHostMallocMapped | hipHostMallocPortable));
  CK(hipHostGetDevicePointer((void**)&host_dev, host, 0));
  CK(hipMemset(dev, 0x5a, n));
  const int kStreams = 3;
  hipStream_t s[kStreams + 1];
  for (int i = 0; i < kStreams; ++i) CK(hipStreamCreateWithFlags(&s[i], hipStreamNonBlocking));
  CK(hipDeviceSynchronize());
  const auto T0 = std::chrono::steady_clock::now();
  auto now = [&] { return std::chrono::duration<double>(std::chrono::steady_clock::now() - T0).count(); };
  struct Sample { double t, d2h, h2d, kernel; };
  auto sample = [&](hipStream_t st) {
    Sample x;
    x.t = now();
    double a = now();
    CK(hipMemcpyAsync(host, dev, n, hipMemcpyDeviceToHost, st));
    CK(hipStreamSynchronize(st));
    x.d2h = (double)n / (now() - a) / 1e9;
    a = now();
    CK(hipMemcpyAsync(dev, host, n, hipMemcpyHostToDevice, st));
    CK(hipStreamSynchronize(st));
    x.h2d = (double)n / (now() - a) / 1e9;
    a = now();
    hipLaunchKernelGGL(store_to_host, dim3((unsigned)(n / 1024)), dim3(64), 0, st, dev, host_dev, n);
    CK(hipStreamSynchronize(st));
    x.kernel = (double)n / (now() - a) / 1e9;
    return x;
  };
  for (int i = 0; i < 8; ++i) (void)sample(s[0]);       // first touches
  for (int gib : sizes) {
    std::vector<Sample> before, after;
    const double t_b = now();
    while (now() - t_b < 0.5)
      for (int i = 0; i < kStreams; ++i) before.push_back(sample(s[i]));
    void* big = nullptr;
    if (hipMalloc(&big, (size_t)gib << 30) != hipSuccess) {
      (void)hipGetLastError();
      printf("%3d GiB: hipMalloc failed, skipped\n", gib);
      continue;
    }
    CK(hipMemset(big, 1, (size_t)gib << 30));
    CK(hipDeviceSynchronize());
    const double t_f0 = now();
    CK(hipFree(big));
    const double t_free = now();
    CK(hipStreamCreateWithFlags(&s[kStreams], hipStreamNonBlocking));     // a stream that did not exist before the free
    const double budget = 2.0 + gib / 8.0;
    while (now() - t_free < budget)
      for (int i = 0; i <= kStreams; ++i) after.push_back(sample(s[i]));
    CK(hipStreamDestroy(s[kStreams]));
    double b_d = 0, b_h = 0, b_k = 0;
    for (const Sample& x : before) { b_d += x.d2h; b_h += x.h2d; b_k += x.kernel; }
    b_d /= before.size(); b_h /= before.size(); b_k /= before.size();
    // the slow period of a direction ends with the last slow copy that is followed by 20 fast ones in a row
    // (a single late outlier does not extend it)
    double last_d = -1, last_h = -1, sum_d = 0, sum_h = 0, sum_k = 0;
    int n_d = 0, n_h = 0, n_k = 0;
    auto period = [&](bool d2h, double* last, double* sum, int* cnt) {
      int fast_run = 0;
      for (const Sample& x : after) {
        const bool slow = d2h ? x.d2h < 0.8 * b_d : x.h2d < 0.8 * b_h;
        if (slow && fast_run < 20) { *last = x.t - t_free; *sum += d2h ? x.d2h : x.h2d; ++*cnt; fast_run = 0; }
        else if (!slow) ++fast_run;
      }
    };
    period(true, &last_d, &sum_d, &n_d);
    period(false, &last_h, &sum_h, &n_h);
    const double slow_until = last_d > last_h ? last_d : last_h;
    for (const Sample& x : after)
      if (x.t - t_free <= slow_until) { sum_k += x.kernel; ++n_k; }
    printf("%3d GiB written and freed (hipFree took %.1f ms):\n", gib, (t_free - t_f0) * 1e3);
    printf("    hipMemcpyAsync device -> host: %5.1f GB/s before; below 80 %% of that for %.2f s after the free (%d copies, mean %.1f GB/s)\n",
           b_d, last_d < 0 ? 0.0 : last_d, n_d, n_d ? sum_d / n_d : 0.0);
    printf("    hipMemcpyAsync host -> device: %5.1f GB/s before; below 80 %% of that for %.2f s after the free (%d copies, mean %.1f GB/s)\n",
           b_h, last_h < 0 ? 0.0 : last_h, n_h, n_h ? sum_h / n_h : 0.0);
    printf("    kernel storing to the mapped pinned buffer: %5.1f GB/s before, %5.1f GB/s during that time\n", b_k,
           n_k ? sum_k / n_k : b_k);
    if (slow_until > 0) printf("    => %.1f GiB of freed memory per second of slow copies\n", gib / slow_until);
    fflush(stdout);
  }
  return 0;
}
