// Device code that is compiled into libkeops_hip.so itself (everything else is JIT-compiled per formula):
//   * the static scratch buffer of the entry point that allocates nothing (keops_hip_launch_noalloc),
//   * half <-> float conversion kernels (use_half launches compute in float32),
//   * a fill kernel (zero formulas: a kernel instead of hipMemsetAsync, which must stay out of captured graphs),
//   * the kernels that build the lookup table of a block-sparse launch from the caller's ranges on the device.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <mutex>
#include <type_traits>

#include "keops_static.h"

// ---- static scratch ---------------------------------------------------------------------------------------------

static __device__ __align__(256) unsigned char scratch[KEOPS_STATIC_SCRATCH_BYTES];

namespace {
std::mutex g_scratch_mutex;
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
}  // namespace

// Address of this device's copy of the scratch array (every GPU holds its own copy at its own address); looked up
// once per device with that device current.  Returns a hipError_t.
int keops_static_scratch(int device, void** ptr, size_t* bytes) {
  if (device < 0 || device >= kMaxDevices) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return (int)e;
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[device] = p;
  }
  *ptr = g_scratch_ptr[device];
  *bytes = (size_t)KEOPS_STATIC_SCRATCH_BYTES;
  return 0;
}

// ---- fill -----------------------------------------------------------------------------------------------------------

static __global__ void __launch_bounds__(256) keops_fill_zero_u32(uint32_t* dst, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = 0u;
}

// zero `bytes` bytes (a multiple of 4) at dst on `stream`
int keops_static_fill_zero(void* dst, size_t bytes, void* stream) {
  const long long n = (long long)(bytes / 4);
  if (n == 0) return 0;
  hipLaunchKernelGGL(keops_fill_zero_u32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (uint32_t*)dst, n);
  return (int)hipGetLastError();
}

// ---- half precision <-> float -------------------------------------------------------------------------------------

static __global__ void __launch_bounds__(256) keops_half_to_float(float* dst, const _Float16* src, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = (float)src[i];
}
static __global__ void __launch_bounds__(256) keops_float_to_half(_Float16* dst, const float* src, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = (_Float16)src[i];
}

int keops_static_convert_half(void* dst, const void* src, long long n, int to_float, void* stream) {
  if (n <= 0) return 0;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (to_float)
    hipLaunchKernelGGL(keops_half_to_float, grid, dim3(256), 0, (hipStream_t)stream, (float*)dst, (const _Float16*)src, n);
  else
    hipLaunchKernelGGL(keops_float_to_half, grid, dim3(256), 0, (hipStream_t)stream, (_Float16*)dst, (const float*)src, n);
  return (int)hipGetLastError();
}

// ---- lookup table of block-sparse launches, built on the device --------------------------------------------------
//
// Counterpart of range_preprocess_from_device (keopscore/keopscore/binders/nvrtc/keops_nvrtc.cpp:152-248), which
// copies the row ranges to the host at every call, builds the table there and copies it back.  Here the table is
// built by a few small kernels on the launch stream: no read-back, no synchronisation, and the launch can be
// recorded in a HIP graph.  The number of workgroups is not known on the host, so the grid has nblocks_max =
// nranges + rows_total / rows_per_block workgroups (enough for disjoint row ranges) and the surplus ones find an
// empty entry and return.  Every index is clamped to its axis (the map-reduce kernels sweep the ranges unchecked);
// two sticky status words in pinned host memory record
// that something had to be clamped or dropped (plain stores of 1: every writer stores the same value).  Row ranges are ordered by the reduced rows they sweep, longest
// first, as the host path does (stable: ties keep their order), up to 16384 ranges; beyond, in table order.

static __global__ void __launch_bounds__(256) keops_ranges_clean_y(const KeopsRangeBuild B) {
  const long long k = (long long)blockIdx.x * 256 + threadIdx.x;
  if (k >= B.nred) return;
  const long long a = B.ry[2 * k], b = B.ry[2 * k + 1];
  const long long a2 = a < 0 ? 0 : (a > B.cols_total ? B.cols_total : a);
  const long long b2 = b < a2 ? a2 : (b > B.cols_total ? B.cols_total : b);
  B.ry_clean[2 * k] = a2;
  B.ry_clean[2 * k + 1] = b2;
  if (a2 != a || b2 != b) B.status[0] = 1u;
}

static __global__ void __launch_bounds__(256) keops_ranges_rows(const KeopsRangeBuild B) {
  const long long r = (long long)blockIdx.x * 256 + threadIdx.x;
  if (r >= B.nranges) return;
  const long long s = B.rx[2 * r], e = B.rx[2 * r + 1];
  const long long s2 = s < 0 ? 0 : (s > B.rows_total ? B.rows_total : s);
  const long long e2 = e < s2 ? s2 : (e > B.rows_total ? B.rows_total : e);
  auto clamp_slice = [&](long long v) { return v < 0 ? 0 : (v > B.nred ? B.nred : v); };
  const long long a = r == 0 ? 0 : clamp_slice(B.sl[r - 1]), b = clamp_slice(B.sl[r]);
  if (s2 != s || e2 != e || b != B.sl[r]) B.status[0] = 1u;
  B.sl_clean[r] = b;
  B.nb[r] = (e2 - s2 + B.rows_per_block - 1) / B.rows_per_block;
  long long w = 0;
  for (long long k = a; k < b; k++) w += B.ry_clean[2 * k + 1] - B.ry_clean[2 * k];
  B.work[r] = w;
}

// order[rank] = r with rank = number of ranges that come before r in a stable sort by decreasing work
static __global__ void __launch_bounds__(256) keops_ranges_rank(const KeopsRangeBuild B, int sorted) {
  __shared__ long long ws[256];
  const long long r = (long long)blockIdx.x * 256 + threadIdx.x;
  if (!sorted) {
    if (r < B.nranges) B.order[r] = r;
    return;
  }
  const long long w = r < B.nranges ? B.work[r] : 0;
  long long rank = 0;
  for (long long q0 = 0; q0 < B.nranges; q0 += 256) {
    __syncthreads();
    ws[threadIdx.x] = q0 + threadIdx.x < B.nranges ? B.work[q0 + threadIdx.x] : -1;
    __syncthreads();
    const int n = (int)(B.nranges - q0 < 256 ? B.nranges - q0 : 256);
    for (int t = 0; t < n; t++) {
      const long long wq = ws[t];
      rank += (wq > w || (wq == w && q0 + t < r)) ? 1 : 0;
    }
  }
  if (r < B.nranges) B.order[rank] = r;
}

// offs[i] = first workgroup of the i-th range in issue order (one workgroup of 1024 threads scans everything)
static __global__ void __launch_bounds__(1024) keops_ranges_scan(const KeopsRangeBuild B) {
  __shared__ long long part[1024];
  const int t = threadIdx.x;
  const long long per = (B.nranges + 1023) / 1024, lo = t * per, hi = lo + per < B.nranges ? lo + per : B.nranges;
  long long s = 0;
  for (long long i = lo; i < hi; i++) s += B.nb[B.order[i]];
  part[t] = s;
  __syncthreads();
  for (int o = 1; o < 1024; o <<= 1) {
    const long long v = t >= o ? part[t - o] : 0;
    __syncthreads();
    part[t] += v;
    __syncthreads();
  }
  long long run = part[t] - s;  // exclusive
  for (long long i = lo; i < hi; i++) {
    B.offs[i] = run;
    run += B.nb[B.order[i]];
  }
  if (t == 1023 && part[1023] > B.nblocks_max) B.status[1] = 1u;
}

// every entry starts empty (range 0, no rows)
static __global__ void __launch_bounds__(256) keops_ranges_clear(const KeopsRangeBuild B) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  if (e < 3 * B.nblocks_max) B.lookup[e] = 0;
}

static __global__ void __launch_bounds__(256) keops_ranges_fill(const KeopsRangeBuild B) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= B.nranges) return;
  const long long r = B.order[i];
  const long long s = B.rx[2 * r], e = B.rx[2 * r + 1];
  const long long s2 = s < 0 ? 0 : (s > B.rows_total ? B.rows_total : s);
  const long long e2 = e < s2 ? s2 : (e > B.rows_total ? B.rows_total : e);
  long long idx = B.offs[i];
  for (long long j = s2; j < e2 && idx < B.nblocks_max; j += B.rows_per_block, idx++) {
    B.lookup[3 * idx] = r;
    B.lookup[3 * idx + 1] = j;
    B.lookup[3 * idx + 2] = j + B.rows_per_block < e2 ? j + B.rows_per_block : e2;
  }
}

size_t keops_static_range_build_words(long long nranges, long long nred, long long nblocks_max) {
  return (size_t)(3 * nblocks_max + nranges + 2 * nred + 4 * nranges + 2);
}

int keops_static_build_ranges(const KeopsRangeBuild* b, void* stream) {
  const KeopsRangeBuild B = *b;
  hipStream_t st = (hipStream_t)stream;
  auto grid = [](long long n) { return dim3((unsigned)((n + 255) / 256 > 0 ? (n + 255) / 256 : 1)); };
  hipLaunchKernelGGL(keops_ranges_clear, grid(3 * B.nblocks_max), dim3(256), 0, st, B);
  if (B.nred > 0) hipLaunchKernelGGL(keops_ranges_clean_y, grid(B.nred), dim3(256), 0, st, B);
  if (B.nranges > 0) {
    hipLaunchKernelGGL(keops_ranges_rows, grid(B.nranges), dim3(256), 0, st, B);
    hipLaunchKernelGGL(keops_ranges_rank, grid(B.nranges), dim3(256), 0, st, B, B.nranges <= 16384 ? 1 : 0);
    hipLaunchKernelGGL(keops_ranges_scan, dim3(1), dim3(1024), 0, st, B);
    hipLaunchKernelGGL(keops_ranges_fill, grid(B.nranges), dim3(256), 0, st, B);
  }
  return (int)hipGetLastError();
}
