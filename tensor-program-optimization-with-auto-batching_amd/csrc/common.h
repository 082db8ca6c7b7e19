// Shared device helpers and host-side error plumbing for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/mlora.h"

typedef _Float16 f16;
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

#define WAVE 64

// ---------------------------------------------------------------------------------------------
// host side: error reporting
// ---------------------------------------------------------------------------------------------
int mlora_set_error(int code, const char* fmt, ...);

#define MLORA_CHECK(cond, code, ...)                         \
  do {                                                       \
    if (!(cond)) return mlora_set_error((code), __VA_ARGS__); \
  } while (0)

static inline int mlora_launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return mlora_set_error(MLORA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return MLORA_OK;
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// 16-token tiles of the fragment-ordered activation layout: the tile count the decode GEMV is compiled
// for (1, 2 or 4), so that producer and consumer agree on the stride between k-steps.
static inline int mlora_frag_tiles(int T) { return T <= 16 ? 1 : (T <= 32 ? 2 : (T <= 64 ? 4 : (T + 15) / 16)); }

// ---------------------------------------------------------------------------------------------
// device side
// ---------------------------------------------------------------------------------------------
// Element offset of x[t, k] in the fragment-ordered activation layout with TT 16-token tiles:
//   Xf[k/32][t/16][(k%32)/8][t%16][k%8]
__device__ __forceinline__ size_t frag_offset(int t, int k, int TT) {
  return ((((size_t)(k >> 5) * TT + (t >> 4)) * 4 + ((k >> 3) & 3)) * 16 + (t & 15)) * 8 + (k & 7);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// 16-byte global load of 8 fp16 values
__device__ __forceinline__ f16x8 ld8(const f16* p) { return *reinterpret_cast<const f16x8*>(p); }
__device__ __forceinline__ void st8(f16* p, f16x8 v) { *reinterpret_cast<f16x8*>(p) = v; }

// a.x*b.x + a.y*b.y + c with fp32 accumulation (v_dot2_f32_f16)
__device__ __forceinline__ float dot2(f16x2 a, f16x2 b, float c) {
  return __builtin_amdgcn_fdot2(a, b, c, false);
}

__device__ __forceinline__ float dot8(f16x8 a, f16x8 b, float c) {
  c = dot2(f16x2{a[0], a[1]}, f16x2{b[0], b[1]}, c);
  c = dot2(f16x2{a[2], a[3]}, f16x2{b[2], b[3]}, c);
  c = dot2(f16x2{a[4], a[5]}, f16x2{b[4], b[5]}, c);
  c = dot2(f16x2{a[6], a[7]}, f16x2{b[6], b[7]}, c);
  return c;
}

// A workgroup barrier and nothing else.  __syncthreads() is a fence and then the barrier, and for the fence the compiler
// waits for EVERY memory request of the wave (s_waitcnt vmcnt(0)) - also for the direct-to-LDS loads of later stages,
// which a software pipeline means to keep in flight across the barrier: with __syncthreads() a ring of several stages
// runs as if it had one.  The caller first waits for exactly what the barrier must publish (its own s_waitcnt: the
// loads of the stage that is read next, and its LDS accesses).
__device__ __forceinline__ void bare_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
