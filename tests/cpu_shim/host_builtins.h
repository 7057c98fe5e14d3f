// TEST INFRASTRUCTURE ONLY: nothing in the product includes this file or runs kernels on the CPU.
// Pre-included in front of the real device prelude when a generated translation unit is built for the host (bounds
// checks on the CPU, tests/cpu_bounds.py): HIP keywords, thread coordinates and the handful of GPU builtins the
// prelude uses.  One thread runs at a time, so values that cross lanes or waves are not reproduced (a shuffle returns
// the caller's own value, the MFMA stub only consumes its operands) and a spin on another workgroup's barrier flag
// ends at once: only the addresses a thread touches are meaningful.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>

#define __device__
#define __global__
#define __shared__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __hip_atomic_store(p, v, order, scope) (*(p) = (v))
#define __hip_atomic_load(p, order, scope) (*(p))
#define __builtin_amdgcn_s_sleep(x) break /* the only use is the body of a spin on a flag */
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(mask, size, sync) ((void)0)
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#define __hip_atomic_compare_exchange_strong(p, expected, v, ok, fail, scope) (*(p) == *(expected) ? (*(p) = (v), true) : false)
#define __builtin_amdgcn_s_barrier() ((void)0)
#define __builtin_amdgcn_readfirstlane(x) (x)
#define MONONN_PIN_ACC(v) ((void)0) /* register placement only */
#define MONONN_LOAD_THROUGH_L2(v, p) ((v) = *(p)) /* a GPU load instruction written in assembly */
#define __HIP_MEMORY_SCOPE_WORKGROUP 1
#define __builtin_amdgcn_s_getreg(reg) (blockIdx.x & 7u) /* the only register read is the XCD number */
#define MONONN_OPAQUE_VALUE(v) ((void)0) /* an empty asm with a GPU register constraint */
/* buffer descriptor + 16-byte load at descriptor base + lane offset + wave offset */
typedef const char* __amdgpu_buffer_rsrc_t;
#define __builtin_amdgcn_make_buffer_rsrc(p, stride, records, flags) ((const char*)(p))
typedef unsigned host_uint4 __attribute__((ext_vector_type(4)));
inline host_uint4 __builtin_amdgcn_raw_buffer_load_b128(const char* rsrc, unsigned voffset, unsigned soffset, int) {
  host_uint4 v;
  std::memcpy(&v, rsrc + (size_t)voffset + (size_t)soffset, 16);
  return v;
}
inline void __builtin_amdgcn_raw_buffer_store_b128(host_uint4 v, const char* rsrc, unsigned voffset, unsigned soffset, int) {
  std::memcpy(const_cast<char*>(rsrc) + (size_t)voffset + (size_t)soffset, &v, 16);
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, row_mask, bank_mask, bound) (src)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __shfl_xor(v, ...) (v)
#define __syncthreads() ((void)0)
#define __expf expf
#define __logf logf

struct Dim3 {
  unsigned x = 0, y = 0, z = 0;
};
extern Dim3 threadIdx, blockIdx, gridDim, blockDim;
using std::max;
using std::min;
inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }
inline unsigned long long wall_clock64() { return 1; }
typedef _Float16 host_half2 __attribute__((ext_vector_type(2)));
inline float __builtin_amdgcn_fdot2(host_half2 a, host_half2 b, float c, bool) { return (float)a[0] * (float)b[0] + (float)a[1] * (float)b[1] + c; }
typedef _Float16 host_half8 __attribute__((ext_vector_type(8)));
typedef float host_float4 __attribute__((ext_vector_type(4)));
typedef float host_float16 __attribute__((ext_vector_type(16)));
inline host_float16 __builtin_amdgcn_mfma_f32_32x32x16_f16(host_half8 a, host_half8 b, host_float16 c, int, int, int) {
  c[0] += (float)a[0] * (float)b[0] + (float)a[7] * (float)b[7];   // keeps the operand loads alive
  return c;
}
inline host_float4 __builtin_amdgcn_mfma_f32_16x16x4f32(float a, float b, host_float4 c, int, int, int) {
  c[0] += a * b;
  return c;
}
inline host_float4 __builtin_amdgcn_mfma_f32_16x16x32_f16(host_half8 a, host_half8 b, host_float4 c, int, int, int) {
  c[0] += (float)a[0] * (float)b[0] + (float)a[7] * (float)b[7];   // keeps the operand loads alive
  return c;
}
typedef __bf16 host_bf16x8 __attribute__((ext_vector_type(8)));
inline host_float16 __builtin_amdgcn_mfma_f32_32x32x16_bf16(host_bf16x8 a, host_bf16x8 b, host_float16 c, int, int, int) {
  c[0] += (float)a[0] * (float)b[0] + (float)a[7] * (float)b[7];   // keeps the operand loads alive
  return c;
}
inline host_float4 __builtin_amdgcn_mfma_f32_16x16x32_bf16(host_bf16x8 a, host_bf16x8 b, host_float4 c, int, int, int) {
  c[0] += (float)a[0] * (float)b[0] + (float)a[7] * (float)b[7];
  return c;
}
#define __builtin_amdgcn_fence(order, scope) ((void)0)
#define __builtin_amdgcn_wave_barrier() ((void)0)
