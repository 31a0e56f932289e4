// Device code that is compiled into libkeops_hip.so itself (everything else is JIT-compiled per formula):
//   * the static scratch buffer of the entry point that allocates nothing (keops_hip_launch_noalloc),
//   * a fill kernel (zero formulas: a kernel instead of hipMemsetAsync, which must stay out of captured graphs),
//   * loop-only calibration kernels for the vector ALU and the matrix cores (keops_hip_calibrate): they measure
//     what an instruction stream without memory traffic sustains, the ceiling the map-reduce kernels are held to.
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

// ---- calibration loops ----------------------------------------------------------------------------------------------

// Every lane runs `iters` rounds of CHAINS independent dependency chains.  MIX 0: v_fmac_f32 only; MIX 1: the
// instruction mix of a Gaussian pair (3 subtractions, 1 multiplication, 2 fused multiply-adds, 1 multiplication,
// v_exp_f32, 1 fused multiply-add = 9 instructions per chain and round); MIX 2: the same mix without v_exp_f32
// (8 instructions).  The asm statements are empty: they only keep the compiler from hoisting or folding the rounds.
template <int CHAINS, int MIX>
static __global__ void __launch_bounds__(256) keops_valu_loop(float* out, int iters, float c0, float c1) {
  float a[CHAINS], acc[CHAINS];
#pragma unroll
  for (int k = 0; k < CHAINS; k++) {
    a[k] = 1.0f + 1e-3f * (float)(threadIdx.x + k);
    acc[k] = 0.f;
  }
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int k = 0; k < CHAINS; k++) {
      if (MIX == 0) {
#pragma unroll
        for (int u = 0; u < 8; u++) a[k] = __builtin_fmaf(a[k], c0, c1);
      } else {
        const float d0 = a[k] - c0, d1 = a[k] - c1, d2 = c0 - a[k];
        float s = d0 * d0;
        s = __builtin_fmaf(d1, d1, s);
        s = __builtin_fmaf(d2, d2, s);
        float t = s * c1;
        if (MIX == 1) t = __builtin_amdgcn_exp2f(-t);
        acc[k] = __builtin_fmaf(t, c0, acc[k]);
      }
      asm volatile("" : "+v"(a[k]), "+v"(acc[k]));
    }
  }
  float r = 0.f;
#pragma unroll
  for (int k = 0; k < CHAINS; k++) r += a[k] + acc[k];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = r;
}

typedef float keops_f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 keops_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 keops_f16x8 __attribute__((ext_vector_type(8)));

// `iters` rounds of CHAINS independent v_mfma_f32_32x32x16_bf16 (HALF = 0) or _f16 (HALF = 1) accumulation chains per
// wavefront; the operands carry full-width random significands (the power drawn, hence the sustained clock,
// depends on the data)
template <int CHAINS, int HALF>
static __global__ void __launch_bounds__(256) keops_mfma_loop(float* out, int iters) {
  keops_f32x16 acc[CHAINS];
  typedef typename std::conditional<HALF == 1, keops_f16x8, keops_bf16x8>::type vec8;
  typedef typename std::conditional<HALF == 1, _Float16, __bf16>::type elem;
  vec8 a, b;
  unsigned h = 0x9e3779b9u * (threadIdx.x + 1u);
#pragma unroll
  for (int e = 0; e < 8; e++) {
    h = h * 1664525u + 1013904223u;
    a[e] = (elem)(1.0f + (float)(h >> 8) * (1.0f / 16777216.0f));
    h = h * 1664525u + 1013904223u;
    b[e] = (elem)(((h & 1u) ? -1.0f : 1.0f) * (0.5f + (float)(h >> 8) * (0.5f / 16777216.0f)));
  }
#pragma unroll
  for (int k = 0; k < CHAINS; k++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[k][e] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 4; u++)
#pragma unroll
      for (int k = 0; k < CHAINS; k++) {
        if constexpr (HALF == 1) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[k], 0, 0, 0);
        else acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[k], 0, 0, 0);
      }
  }
  float r = 0.f;
#pragma unroll
  for (int k = 0; k < CHAINS; k++)
#pragma unroll
    for (int e = 0; e < 16; e++) r += acc[k][e];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = r;
}

// Runs one calibration loop on `stream`: grid of `blocks` workgroups of 256 lanes (4 wavefronts), `iters` rounds.
// kind 0/1/2: vector loop with MIX = kind; kind 3 / 4: matrix loop on bf16 / f16 operands.  chains: 1, 2, 4 or 8 (vector), 1, 2 or 4 (matrix).
// instr_per_lane receives the number of counted instructions one wavefront issues (vector: per lane = per wavefront
// instruction count; matrix: v_mfma instructions).  out must hold blocks * 256 floats.
int keops_static_calibrate(int kind, int chains, int blocks, int iters, float* out, void* stream, double* instr_per_wave) {
  hipStream_t s = (hipStream_t)stream;
  const dim3 g((unsigned)blocks), b(256);
#define VALU_CASE(C, M) hipLaunchKernelGGL((keops_valu_loop<C, M>), g, b, 0, s, out, iters, 1.0009765625f, 0.99951171875f)
  if (kind >= 0 && kind <= 2) {
    const double per_round = kind == 0 ? 8.0 : (kind == 1 ? 9.0 : 8.0);
    *instr_per_wave = per_round * chains * (double)iters;
    if (kind == 0) {
      if (chains == 1) VALU_CASE(1, 0); else if (chains == 2) VALU_CASE(2, 0); else if (chains == 4) VALU_CASE(4, 0);
      else if (chains == 8) VALU_CASE(8, 0); else return (int)hipErrorInvalidValue;
    } else if (kind == 1) {
      if (chains == 1) VALU_CASE(1, 1); else if (chains == 2) VALU_CASE(2, 1); else if (chains == 4) VALU_CASE(4, 1);
      else if (chains == 8) VALU_CASE(8, 1); else return (int)hipErrorInvalidValue;
    } else {
      if (chains == 1) VALU_CASE(1, 2); else if (chains == 2) VALU_CASE(2, 2); else if (chains == 4) VALU_CASE(4, 2);
      else if (chains == 8) VALU_CASE(8, 2); else return (int)hipErrorInvalidValue;
    }
  } else if (kind == 3 || kind == 4) {
    *instr_per_wave = 4.0 * chains * (double)iters;
#define MFMA_CASE(C) do { if (kind == 3) hipLaunchKernelGGL((keops_mfma_loop<C, 0>), g, b, 0, s, out, iters); \
                          else hipLaunchKernelGGL((keops_mfma_loop<C, 1>), g, b, 0, s, out, iters); } while (0)
    if (chains == 1) MFMA_CASE(1);
    else if (chains == 2) MFMA_CASE(2);
    else if (chains == 4) MFMA_CASE(4);
    else return (int)hipErrorInvalidValue;
#undef MFMA_CASE
  } else {
    return (int)hipErrorInvalidValue;
  }
#undef VALU_CASE
  return (int)hipGetLastError();
}
