// Interface between the host library (keops_hip.cpp, host compiler) and the device code that is compiled into
// libkeops_hip.so itself (keops_static.hip, hipcc).
#pragma once
#include <stddef.h>

int keops_static_fill_zero(void* dst, size_t bytes, void* stream);
int keops_static_calibrate(int kind, int chains, int blocks, int iters, float* out, void* stream, double* instr_per_wave);
