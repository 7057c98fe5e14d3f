// Host stand-in for the device prelude of generated kernels, for bounds checks on the CPU: a generated
// translation unit made of element-wise / row-program stages (no MFMA tiles) compiles against this header with a
// host compiler and runs one thread at a time, every buffer placed against inaccessible guard pages.  Values that
// cross threads (reductions, lane exchanges) are not reproduced - only the addresses a thread touches matter here,
// and in these stages no address depends on such a value.
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
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __expf expf
#define __logf logf
#define __syncthreads() ((void)0)

struct Dim3 {
  unsigned x = 0, y = 0, z = 0;
};
extern Dim3 threadIdx, blockIdx, gridDim, blockDim;
using std::max;
using std::min;
inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }
inline unsigned long long wall_clock64() { return 1; }

namespace mononn_dev {
constexpr int kWaveSize = 64;
constexpr int kFlagStride = 64;
inline int lane_id() { return threadIdx.x & (kWaveSize - 1); }
inline int wave_id() { return threadIdx.x / kWaveSize; }
struct GridBarrier {
  void init(unsigned*) {}
  void arrive() {}
  void wait() {}
  void sync() {}
};
template <class T>
inline void st1(T* p, T v) { *p = v; }
template <class T>
inline void st1_plain(T* p, T v) { *p = v; }
template <class T, int N>
inline void stN(T* p, const T (&v)[N]) { std::memcpy(p, v, sizeof(v)); }
template <class T, int N>
inline void stN_plain(T* p, const T (&v)[N]) { std::memcpy(p, v, sizeof(v)); }
template <class T, class Op>
inline T wave_all_reduce(T v, Op) { return v; }
template <class T, class Op>
inline T block_all_reduce(T v, Op, T* scratch) {
  scratch[wave_id()] = v;   // the LDS slot a wave really writes
  return scratch[0];
}
template <class T>
inline T lane_xor(T v, int) { return v; }
inline float fast_tanh(float x) { return tanhf(x); }
template <class T>
inline T sign_of(T x) { return x > T(0) ? T(1) : (x < T(0) ? T(-1) : T(0)); }
}  // namespace mononn_dev
