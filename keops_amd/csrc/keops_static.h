// Interface between the host library (keops_hip.cpp, host compiler) and the device code that is compiled into
// libkeops_hip.so itself (keops_static.hip, hipcc).
#pragma once
#include <stddef.h>

// Size of the static device scratch buffer behind keops_hip_launch_noalloc: 128 MiB per GPU, held from the first
// use of the library's device code on that GPU until the process ends.
#define KEOPS_STATIC_SCRATCH_BYTES (128u << 20)

int keops_static_scratch(int device, void** ptr, size_t* bytes);
int keops_static_fill_zero(void* dst, size_t bytes, void* stream);
int keops_static_calibrate(int kind, int chains, int blocks, int iters, float* out, void* stream, double* instr_per_wave);
