// Cold-data HBM bandwidth ceilings of this device: plain read / copy / add kernels over a ring of buffers whose total
// size exceeds the 256 MB memory-side cache, so that no launch finds its operands cached.  The fused elementwise and
// reduction kernels the plugin generates are compared with these figures (same sizes, same timing method: HIP events
// around 64 back-to-back launches on one stream).
//   mi355x-bw [megabytes per stream ...]      (default: the sizes of the fused-op benchmark shapes)
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "%s (line %d)\n", hipGetErrorString(e_), __LINE__); return 1; } } while (0)
typedef float __attribute__((ext_vector_type(4))) f4;

__global__ void __launch_bounds__(256) copy_once(const f4* __restrict__ a, f4* __restrict__ o, size_t n) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) o[i] = a[i];
}
__global__ void __launch_bounds__(256) add_once(const f4* __restrict__ a, const f4* __restrict__ b, f4* __restrict__ o, size_t n) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) o[i] = a[i] + b[i];
}
template <int U, bool NT>
__global__ void __launch_bounds__(256) copy_strided(const f4* __restrict__ a, f4* __restrict__ o, size_t n) {
  size_t stride = (size_t)gridDim.x * 256, i = (size_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + (U - 1) * stride < n; i += U * stride) {
    f4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = NT ? __builtin_nontemporal_load(&a[i + u * stride]) : a[i + u * stride];
#pragma unroll
    for (int u = 0; u < U; ++u) { if (NT) __builtin_nontemporal_store(v[u], &o[i + u * stride]); else o[i + u * stride] = v[u]; }
  }
  for (; i < n; i += stride) o[i] = a[i];
}
template <int U>
__global__ void __launch_bounds__(256) read_strided(const f4* __restrict__ a, float* __restrict__ o, size_t n) {
  size_t stride = (size_t)gridDim.x * 256, i = (size_t)blockIdx.x * 256 + threadIdx.x;
  f4 acc = {0, 0, 0, 0};
  for (; i + (U - 1) * stride < n; i += U * stride) {
    f4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = a[i + u * stride];
#pragma unroll
    for (int u = 0; u < U; ++u) acc += v[u];
  }
  for (; i < n; i += stride) acc += a[i];
  float s = acc.x + acc.y + acc.z + acc.w;
  if (s == 12345.678f) o[blockIdx.x] = s;   // never true for the zero-filled buffers: keeps the loads alive
}

int main(int argc, char** argv) {
  std::vector<double> sizes;
  for (int i = 1; i < argc; ++i) sizes.push_back(atof(argv[i]));
  if (sizes.empty()) sizes = {6.3, 25.2, 33.6, 40.0, 67.1};
  const int R = 64;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  hipStream_t st;
  CK(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
  printf("%-10s %-26s %9s %10s\n", "MB/stream", "kernel", "us", "GB/s");
  for (double mb : sizes) {
    size_t bytes = (size_t)(mb * 1e6) / 16 * 16, n = bytes / 16;
    int sets = (int)((700000000ull + 3 * bytes - 1) / (3 * bytes));
    if (sets < 3) sets = 3;
    std::vector<f4*> A(sets), B(sets), O(sets);
    for (int s = 0; s < sets; ++s) {
      CK(hipMalloc(&A[s], bytes)); CK(hipMalloc(&B[s], bytes)); CK(hipMalloc(&O[s], bytes));
      CK(hipMemsetAsync(A[s], 0, bytes, st)); CK(hipMemsetAsync(B[s], 0, bytes, st));
    }
    float* sink;
    CK(hipMalloc(&sink, 1 << 20));
    auto run = [&](const char* name, double algoBytes, auto launch) -> int {
      for (int r = 0; r < 8; ++r) launch(r % sets);
      CK(hipStreamSynchronize(st));
      float best = 1e9f;
      for (int rep = 0; rep < 3; ++rep) {
        CK(hipEventRecord(e0, st));
        for (int r = 0; r < R; ++r) launch(r % sets);
        CK(hipEventRecord(e1, st));
        CK(hipStreamSynchronize(st));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        if (ms < best) best = ms;
      }
      double us = best * 1e3 / R;
      printf("%-10.1f %-26s %9.2f %10.1f\n", mb, name, us, algoBytes / us / 1e3);
      return 0;
    };
    unsigned one = (unsigned)((n + 255) / 256);
    if (run("read (16 vectors/lane)", 1.0 * bytes, [&](int s) { read_strided<16><<<2048, 256, 0, st>>>(A[s], sink, n); })) return 1;
    if (run("copy (one vector/lane)", 2.0 * bytes, [&](int s) { copy_once<<<one, 256, 0, st>>>(A[s], O[s], n); })) return 1;
    if (run("copy (nontemporal, 4/lane)", 2.0 * bytes, [&](int s) { copy_strided<4, true><<<2048, 256, 0, st>>>(A[s], O[s], n); })) return 1;
    if (run("add (one vector/lane)", 3.0 * bytes, [&](int s) { add_once<<<one, 256, 0, st>>>(A[s], B[s], O[s], n); })) return 1;
    for (int s = 0; s < sets; ++s) { CK(hipFree(A[s])); CK(hipFree(B[s])); CK(hipFree(O[s])); }
    CK(hipFree(sink));
  }
  return 0;
}
