// Device-side runtime of the generated monolithic kernel (gfx950 / CDNA4, wave64).
//
// This text is embedded into the host compiler and prepended to every generated program before it
// goes to hipRTC.  It is the counterpart of the string prelude the reference assembles from
// mononn_engine/core/gpu/{synchronization,reduction,memory,headers}.cc, re-designed for 64-wide
// wavefronts, MFMA and a 256-CU / 8-XCD part:
//   * grid_sync         <- synchronization.cc:45-82 (flag array; block 0 as master).  Here every
//                          workgroup publishes a monotonically increasing epoch and polls all
//                          flags itself, so there is no master round trip and nothing to clear.
//   * wave/block reduce <- reduce_impl.cc:480-680 (32-lane shuffles) -> 64-lane butterflies.
//   * gemm              <- gemm_impl.cc:42-141 (CUTLASS device GEMM, persistent tile swizzle)
//                          -> register-resident MFMA 16x16x32 f16 tiles fed straight from
//                          global memory, K split across the waves of a workgroup.
#pragma once

// hipRTC provides no <cstdint>; generated code uses these names for HLO integer types
#if defined(__HIPCC_RTC__)
typedef signed char int8_t;
typedef unsigned char uint8_t;
typedef short int16_t;
typedef unsigned short uint16_t;
typedef int int32_t;
typedef unsigned int uint32_t;
typedef long long int64_t;
typedef unsigned long long uint64_t;
#else
#include <cstdint>
#endif

typedef _Float16 half_t;
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef int int4_t __attribute__((ext_vector_type(4)));

#ifndef MONONN_BARRIER_FENCE
#define MONONN_BARRIER_FENCE 0
#endif
#ifndef MONONN_COHERENT_STORES
#define MONONN_COHERENT_STORES 0
#endif
// waves that share a SIMD when the whole grid is resident: the kernel is compiled for 512 / this many VGPRs per wave
#ifndef MONONN_WAVES_PER_SIMD
#define MONONN_WAVES_PER_SIMD 1
#endif

// an empty statement after which the compiler knows nothing about the value of `v` (a vector register)
#ifndef MONONN_OPAQUE_VALUE
#define MONONN_OPAQUE_VALUE(v) asm volatile("" : "+v"(v))
#endif
// an empty statement that requires `v` in accumulation registers at this point of the program
#ifndef MONONN_PIN_ACC
#define MONONN_PIN_ACC(v) asm volatile("" : "+a"(v))
#endif

namespace mononn_dev {

constexpr int kWaveSize = 64;
constexpr int kFlagStride = 64;   // 256 bytes between workgroup flags: measured fastest among 64 B .. 4 KiB

// The thread's index in its workgroup, opaque to the compiler (MONONN_OPAQUE_THREAD_ID: the host compiler turns it on in
// kernels that hold an LDS-staged GEMM tile or whose specification asks for it, off otherwise): the kernel is
// one function holding every stage, and whatever the compiler can derive from threadIdx.x once -- lane and wave
// numbers, address parts of every stage -- it computes ahead of the stage loop and keeps in registers through all
// stages.  A stage with a large register tile then pushes those values out to scratch, and the stages that use
// them reload them in their inner loops (measured on a 12-layer decoder: one 256-register GEMM tile in the kernel
// made the attention stages 29 -> 65 us and the row programs 14 -> 24 us; with the index re-read per use the same
// kernel runs faster than without the tile).
#ifndef MONONN_OPAQUE_THREAD_ID
#define MONONN_OPAQUE_THREAD_ID 1
#endif
__device__ __forceinline__ int thread_id() {
  int t = threadIdx.x;
#if MONONN_OPAQUE_THREAD_ID
  MONONN_OPAQUE_VALUE(t);
#endif
  return t;
}
__device__ __forceinline__ int lane_id() { return thread_id() & (kWaveSize - 1); }
__device__ __forceinline__ int wave_id() { return thread_id() / kWaveSize; }

// ---------------------------------------------------------------------------------------------
// grid-wide barrier
// ---------------------------------------------------------------------------------------------
// Waits are bounded: the kernel notes the wall clock (100 MHz) when it starts, and a wait that is still polling
// MONONN_BARRIER_BUDGET_TICKS later gives up, records the barrier's ordinal in the error word and returns.  From
// then on every wait of every workgroup that finds a flag missing returns after one look at the clock, so the
// workgroups run through their remaining stages (on incomplete data, but every address they form is in range
// whatever the data: run-time indices are clamped) and the kernel ends normally.  The host reads the error word
// after synchronising.  What this guards against: a grid that is not resident as a whole (an ordinary launch next
// to another kernel), where the resident workgroups would otherwise poll for ever.
#ifndef MONONN_BARRIER_BUDGET_TICKS
#define MONONN_BARRIER_BUDGET_TICKS 1000000000ull   // 10 s
#endif

// Regional tier (MONONN_REGIONAL_SYNC): the 8 XCDs of the part have an L2 each, and a launch of one workgroup per
// compute unit deals the workgroups to them round-robin: workgroup b runs on XCD (b + s) % 8, where the start s is the
// same for every workgroup of a launch and depends on the hardware queue the launch went through (0 in a process with
// one stream; measured 7 and 5 on the null stream once a second and a fourth stream existed).  So the 32 workgroups
// with equal b % 8 share an XCD whatever s is, which is all the regional tier relies on; every workgroup leaves its
// XCC_ID beside its flag, and the first regional wait of a workgroup compares the 32 it polls with its own (a mismatch
// is reported through the error word).  Where every value that crosses a stage
// boundary is produced and consumed on the same XCD, the hand-over stays inside that L2: ordinary stores (acknowledged
// by the L2), a flag array of its own published with a store that stops at the L2, and a wait that looks at the 32
// flags of the workgroup's XCD only, with loads that miss the compute unit's L1 (nt) and hit the L2.  Measured in
// isolation, store -> flag -> poll -> dependent load: 0.84 us against 3.1 us through the memory side.
// Counterpart of the reference's regional synchronisation (regional_synchronization_assignment_pass.cc:35-72).
#ifndef MONONN_REGIONAL_SYNC
#define MONONN_REGIONAL_SYNC 0
#endif
constexpr int kXcds = 8;
constexpr unsigned kErrorRegional = 0x40000000u;    // error word: a wait of the regional tier gave up
constexpr unsigned kErrorPlacement = 0x80000000u;   // error word: two workgroups with equal blockIdx.x % 8 run on different XCDs

// a load that is served by the L2 (the compute unit's L1 does not keep what it returns); an asm statement because no
// builtin combines this cache policy with the ordering a spin loop needs (a load instruction reads no data register
// that an earlier instruction writes, so there are no wait states for the compiler to place around it)
#ifndef MONONN_LOAD_THROUGH_L2
#define MONONN_LOAD_THROUGH_L2(v, p) asm volatile("global_load_dword %0, %1, off nt\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory")
#endif
__device__ __forceinline__ unsigned load_through_l2(const unsigned* p) {
  unsigned v;
  MONONN_LOAD_THROUGH_L2(v, p);
  return v;
}

struct GridBarrier {
  unsigned* flags;   // [gridDim.x * kFlagStride]
  unsigned* error;   // [0]: 0, or 1 + ordinal of the first barrier a wait gave up on
  unsigned epoch;    // last epoch this workgroup has published
  unsigned first;    // epoch at kernel start (for the ordinal in the error word)
  unsigned long long deadline;
#if MONONN_REGIONAL_SYNC
  unsigned* rflags;  // [gridDim.x * kFlagStride]: flags of the regional tier
  unsigned repoch, rfirst;
  unsigned xcc;          // the XCD this workgroup runs on
  bool placement_seen;   // this workgroup has compared its XCD with that of the workgroups it polls

  __device__ __forceinline__ void init_regional(unsigned* f) {
    rflags = f;
    repoch = load_through_l2(&rflags[blockIdx.x * kFlagStride]);
    rfirst = repoch;
    xcc = __builtin_amdgcn_s_getreg(6164) & (kXcds - 1);   // hwreg(HW_REG_XCC_ID, 0, 4)
    placement_seen = false;
    // beside the flag, in its line: in the L2 before the first flag of this launch is (arrive_regional waits for it)
    if (threadIdx.x == 0) __hip_atomic_store(&rflags[blockIdx.x * kFlagStride + 1], xcc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  // the workgroup's part of the stage is in the XCD's L2 (every wave has its stores acknowledged), then the flag
  __device__ __forceinline__ void arrive_regional() {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    repoch += 1;
    if (threadIdx.x == 0) __hip_atomic_store(&rflags[blockIdx.x * kFlagStride], repoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  __device__ __forceinline__ void wait_regional() {
    for (int b = (blockIdx.x & (kXcds - 1)) + kXcds * threadIdx.x; b < (int)gridDim.x; b += kXcds * blockDim.x) {
      unsigned spins = 0;
      while ((int)(load_through_l2(&rflags[b * kFlagStride]) - repoch) < 0) {
        __builtin_amdgcn_s_sleep(1);
        if ((++spins & 63u) == 0u && wall_clock64() > deadline) {
          unsigned expected = 0;
          __hip_atomic_compare_exchange_strong(error, &expected, kErrorRegional | (repoch - rfirst), __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
      }
      if (!placement_seen) {
        const unsigned theirs = load_through_l2(&rflags[b * kFlagStride + 1]) & (kXcds - 1);
        if (theirs != xcc) {
          unsigned expected = 0;
          __hip_atomic_compare_exchange_strong(error, &expected, kErrorPlacement | (theirs << 24) | (xcc << 20) | ((unsigned)b & 0xfffffu), __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    placement_seen = true;
    __syncthreads();
  }
#endif

  __device__ __forceinline__ void init(unsigned* f, unsigned* err) {
    flags = f;
    error = err;
    // all workgroups left the previous launch at the same epoch; pick it up from our own flag
    epoch = __hip_atomic_load(&flags[blockIdx.x * kFlagStride], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    first = epoch;
    deadline = wall_clock64() + MONONN_BARRIER_BUDGET_TICKS;
  }

  // A workgroup announces that its part of the stage is written (arrive) and, before it reads anything another
  // workgroup wrote in that stage, makes sure that every workgroup has announced (wait).  Between the two it may
  // do whatever does not depend on the stage: requesting constant operands of its next unit, for instance.  A
  // workgroup without work in a stage need not wait for it at all: flags only grow, so it may announce the next
  // stage right away and wait, when it has work again, for the latest one.
  __device__ __forceinline__ void arrive() {
#if MONONN_BARRIER_FENCE == 2
    // The flag is a relaxed store, and the workgroup barrier below waits for LDS traffic only: every wave first
    // waits until its own write-through stores are acknowledged (vmcnt(0); expcnt / lgkmcnt fields left at their
    // maxima), so that no byte of the stage is still on its way when thread 0 publishes the flag.
    __builtin_amdgcn_s_waitcnt(0x0F70);
#endif
    __syncthreads();
    epoch += 1;
    if (threadIdx.x == 0) {
#if MONONN_BARRIER_FENCE == 2
      __hip_atomic_store(&flags[blockIdx.x * kFlagStride], epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#else
      __hip_atomic_store(&flags[blockIdx.x * kFlagStride], epoch, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
#endif
    }
  }

  // polls flag b until it reaches this workgroup's epoch or the kernel's time budget is spent
  __device__ __forceinline__ void poll(int b) {
    unsigned spins = 0;
    while ((int)(__hip_atomic_load(&flags[b * kFlagStride], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - epoch) < 0) {
      __builtin_amdgcn_s_sleep(1);
      if ((++spins & 63u) == 0u && wall_clock64() > deadline) {
        unsigned expected = 0;
        __hip_atomic_compare_exchange_strong(error, &expected, epoch - first, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
    }
  }

  __device__ __forceinline__ void wait() {
#if MONONN_BARRIER_FENCE == 0
    if (threadIdx.x < kWaveSize) {
      for (int b = threadIdx.x; b < (int)gridDim.x; b += kWaveSize) poll(b);
      __atomic_thread_fence(__ATOMIC_ACQUIRE);   // agent scope: drop stale lines before the next stage reads
    }
#else
    for (int b = threadIdx.x; b < (int)gridDim.x; b += blockDim.x) poll(b);
#if MONONN_BARRIER_FENCE == 1
    __atomic_thread_fence(__ATOMIC_ACQUIRE);
#endif
#endif
    __syncthreads();
  }

  // MONONN_BARRIER_FENCE: 0 = one thread per workgroup performs the release / acquire cache
  // maintenance (an agent-scope acquire invalidates the XCD's whole L2, so issuing it from every
  // wave multiplies that cost by the number of resident waves); 1 = every thread fences;
  // 2 = no cache maintenance at all (valid with MONONN_COHERENT_STORES and a write-once temp arena).
  __device__ __forceinline__ void sync() {
    arrive();
    wait();
  }
};

// ---------------------------------------------------------------------------------------------
// stores of data that another workgroup reads in a later stage
// ---------------------------------------------------------------------------------------------
// The XCDs of one GPU do not keep their L2s coherent with each other.  Instead of flushing and
// invalidating caches at every grid barrier, stage outputs are written with agent-scope (write-
// through) stores: the data is at the memory side when the store retires, no L2 keeps a dirty copy.
// Together with the rule that an address of the temp arena is written at most once per launch, a
// reader can never find a stale line: nothing can have cached the line before its only write, and
// the launch boundary invalidates what earlier launches left behind.  Readers use plain cached loads.
#if MONONN_COHERENT_STORES
template <class T>
__device__ __forceinline__ void st1(T* p, T v) {
  if constexpr (sizeof(T) == 1) {
    unsigned char b;
    __builtin_memcpy(&b, &v, 1);
    __hip_atomic_store(reinterpret_cast<unsigned char*>(p), b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else if constexpr (sizeof(T) == 2) {
    unsigned short b;
    __builtin_memcpy(&b, &v, 2);
    __hip_atomic_store(reinterpret_cast<unsigned short*>(p), b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else if constexpr (sizeof(T) == 4) {
    unsigned b;
    __builtin_memcpy(&b, &v, 4);
    __hip_atomic_store(reinterpret_cast<unsigned*>(p), b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else {
    unsigned long long b;
    __builtin_memcpy(&b, &v, 8);
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}
#else
template <class T>
__device__ __forceinline__ void st1(T* p, T v) { *p = v; }
#endif
#if MONONN_COHERENT_STORES
// 16 bytes written through to the memory side with one instruction.  Agent-scope atomic stores stop at 8 bytes (two
// instructions, two requests per lane); the cache policy they carry (sc1) is also available on a buffer store, which
// the compiler knows as an ordinary store instruction: it places the wait states between whatever produced the data
// registers (an MFMA, a conversion) and the store, and counts it in vmcnt, which is what the grid barrier's arrive()
// waits on.  The descriptor spans the 2 GiB window that holds the address: its base, the upper bits of the address,
// must be wave-uniform, so the lanes of a wave that straddle a window boundary take their turns in the loop.
typedef unsigned store16_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store16_agent(void* p, store16_t v) {
  const unsigned long long a = reinterpret_cast<unsigned long long>(p);
  const unsigned window = static_cast<unsigned>(a >> 31), offset = static_cast<unsigned>(a) & 0x7fffffffu;
  for (;;) {
    const unsigned w0 = __builtin_amdgcn_readfirstlane(window);
    if (window == w0) {
      __builtin_amdgcn_raw_buffer_store_b128(v, __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(static_cast<unsigned long long>(w0) << 31), 0, -1, 0x00020000),
                                             offset, 0, 16 /* sc1 */);
      break;
    }
  }
}
#endif
// N consecutive elements starting at an address aligned to N * sizeof(T) (N * sizeof(T) in {4, 8, 16})
template <class T, int N>
__device__ __forceinline__ void stN(T* p, const T (&v)[N]) {
  constexpr int BYTES = N * (int)sizeof(T);
  static_assert(BYTES == 4 || BYTES == 8 || BYTES == 16, "unsupported packed store");
  if constexpr (BYTES == 4) {
    unsigned b;
    __builtin_memcpy(&b, v, 4);
    st1(reinterpret_cast<unsigned*>(p), b);
  } else if constexpr (BYTES == 8) {
    unsigned long long b;
    __builtin_memcpy(&b, v, 8);
    st1(reinterpret_cast<unsigned long long*>(p), b);
  } else {
#if MONONN_COHERENT_STORES
    store16_t b;
    __builtin_memcpy(&b, v, 16);
    store16_agent(p, b);
#else
    unsigned long long b[2];
    __builtin_memcpy(b, v, 16);
    st1(reinterpret_cast<unsigned long long*>(p), b[0]);
    st1(reinterpret_cast<unsigned long long*>(p) + 1, b[1]);
#endif
  }
}

// Stores of results that nothing inside the kernel reads back: ordinary cached stores (the L2 merges them into
// whole lines and writes them out by the end of the kernel at the latest).
template <class T>
__device__ __forceinline__ void st1_plain(T* p, T v) { *p = v; }
template <class T, int N>
__device__ __forceinline__ void stN_plain(T* p, const T (&v)[N]) {
  constexpr int BYTES = N * (int)sizeof(T);
  static_assert(BYTES == 4 || BYTES == 8 || BYTES == 16, "unsupported packed store");
  if constexpr (BYTES == 4) {
    unsigned b;
    __builtin_memcpy(&b, v, 4);
    *reinterpret_cast<unsigned*>(p) = b;
  } else if constexpr (BYTES == 8) {
    unsigned long long b;
    __builtin_memcpy(&b, v, 8);
    *reinterpret_cast<unsigned long long*>(p) = b;
  } else {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    v4u b;
    __builtin_memcpy(&b, v, 16);
    *reinterpret_cast<v4u*>(p) = b;
  }
}

// N consecutive elements at an address that is only known to be aligned to one element: a copy without an alignment
// promise, for which the compiler picks whatever store width the target's unaligned-access rules allow
template <class T, int N>
__device__ __forceinline__ void stN_plain_unaligned(T* p, const T (&v)[N]) {
  __builtin_memcpy(p, v, N * sizeof(T));
}

// ---------------------------------------------------------------------------------------------
// reductions (all lanes / all threads receive the result)
// ---------------------------------------------------------------------------------------------
// value of `v` in the lane that the DPP control word names (rows of 16 lanes)
template <int CTRL, class T>
__device__ __forceinline__ T dpp_move(T v) {
  static_assert(sizeof(T) == 4, "DPP moves one dword");
  int b;
  __builtin_memcpy(&b, &v, 4);
  b = __builtin_amdgcn_update_dpp(b, b, CTRL, 0xf, 0xf, false);
  T r;
  __builtin_memcpy(&r, &b, 4);
  return r;
}

template <class T, class Op>
__device__ __forceinline__ T wave_all_reduce(T v, Op op) {
  if constexpr (sizeof(T) == 4) {
    // inside a row of 16 lanes: data-parallel-primitive moves on the vector ALU (neighbour in the quad, other
    // pair of the quad, mirrored half row, mirrored row); across the four rows: two LDS-crossbar permutes
    v = op(v, dpp_move<0xB1>(v));    // quad_perm [1,0,3,2]
    v = op(v, dpp_move<0x4E>(v));    // quad_perm [2,3,0,1]
    v = op(v, dpp_move<0x141>(v));   // row_half_mirror
    v = op(v, dpp_move<0x140>(v));   // row_mirror
    v = op(v, __shfl_xor(v, 16, kWaveSize));
    v = op(v, __shfl_xor(v, 32, kWaveSize));
    return v;
  } else {
#pragma unroll
    for (int off = kWaveSize / 2; off > 0; off >>= 1) v = op(v, __shfl_xor(v, off, kWaveSize));
    return v;
  }
}

// Reduction over the 64 / G lanes that share (lane % G), G = 8, 4 or 2: a wave that works on G rows at once keeps row r
// in lanes r, r + G, ..., r + 64 - G.  Rotations by G .. 8 inside the row of 16 lanes on the vector ALU (a rotation by
// half the distance already covered doubles the set of lanes a value stands for, like the butterfly does), then two
// LDS-crossbar permutes.
template <int G, class T, class Op>
__device__ __forceinline__ T lane_group_all_reduce(T v, Op op) {
  static_assert(G == 8 || G == 4 || G == 2, "8, 4 or 2 rows per wave");
  if constexpr (sizeof(T) == 4) {
    v = op(v, dpp_move<0x128>(v));                          // row_ror:8
    if constexpr (G <= 4) v = op(v, dpp_move<0x124>(v));    // row_ror:4
    if constexpr (G <= 2) v = op(v, dpp_move<0x122>(v));    // row_ror:2
  } else {
#pragma unroll
    for (int off = 8; off >= G; off >>= 1) v = op(v, __shfl_xor(v, off, kWaveSize));
  }
  v = op(v, __shfl_xor(v, 16, kWaveSize));
  v = op(v, __shfl_xor(v, 32, kWaveSize));
  return v;
}

// value of `v` in lane (own lane ^ mask), for any type of up to 8 bytes (tuple reductions exchange every member)
template <class T>
__device__ __forceinline__ T lane_xor(T v, int mask) {
  static_assert(sizeof(T) <= 8, "lane exchange of at most 8 bytes");
  if constexpr (sizeof(T) <= 4) {
    int b = 0;
    __builtin_memcpy(&b, &v, sizeof(T));
    b = __shfl_xor(b, mask, kWaveSize);
    T r;
    __builtin_memcpy(&r, &b, sizeof(T));
    return r;
  } else {
    long long b;
    __builtin_memcpy(&b, &v, 8);
    b = __shfl_xor(b, mask, kWaveSize);
    T r;
    __builtin_memcpy(&r, &b, 8);
    return r;
  }
}

// `scratch` holds at least blockDim.x / 64 elements of T in LDS
template <class T, class Op>
__device__ __forceinline__ T block_all_reduce(T v, Op op, T* scratch) {
  v = wave_all_reduce(v, op);
#if defined(MONONN_BLOCK_SIZE)
  constexpr int nw = MONONN_BLOCK_SIZE / kWaveSize;   // the kernel is generated for one workgroup size
#else
  const int nw = blockDim.x / kWaveSize;
#endif
  if (lane_id() == 0) scratch[wave_id()] = v;
  __syncthreads();
  T r = scratch[0];
  for (int w = 1; w < nw; ++w) r = op(r, scratch[w]);
  __syncthreads();
  return r;
}

// ---------------------------------------------------------------------------------------------
// math helpers used by generated element-wise code
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float fast_tanh(float x) {
  // tanh(x) = 1 - 2 / (exp(2x) + 1); exact enough in fp32 and safe for large |x|
  float e = __expf(2.0f * x);
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}
// A run-time index (gather row, dynamic-slice start) clamped to [0, hi] in the index's own type, then narrowed:
// a 64-bit index far out of range must land on the nearest end, not on whatever its low 32 bits say.
template <class T>
__device__ __forceinline__ int clamp_index(T v, int hi) {
  return v < (T)0 ? 0 : (v > (T)hi ? hi : (int)v);
}
template <class T>
__device__ __forceinline__ T sign_of(T x) {
  return (T)((x > (T)0) - (x < (T)0));
}

// The right operand of P.V in the fused attention when the key count n is off the MFMA step: elements k .. k + 3 and
// k + 16 .. k + 19 of a row of V^T, without an alignment promise; positions past the end read the last element.
__device__ __forceinline__ half8_t load_key_run(const half_t* row, int k, int n) {
  half8_t v;
  if (k + 20 <= n) {
    __builtin_memcpy(&v, row + k, 8);
    __builtin_memcpy(reinterpret_cast<char*>(&v) + 8, row + k + 16, 8);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int lo = k + e, hi = k + 16 + e;
      v[e] = row[lo < n ? lo : n - 1];
      v[4 + e] = row[hi < n ? hi : n - 1];
    }
  }
  return v;
}

// ---------------------------------------------------------------------------------------------
// GEMM:  D[m][n] = sum_k A[m][k] * B[k][n]      A contiguous along k
// ---------------------------------------------------------------------------------------------
// One workgroup owns a BM x BN output tile.  Its waves are arranged WM x WN x WK: WM*WN waves split
// the tile, WK waves split the k range of each sub-tile (k steps interleaved).  Every wave feeds
// One 16x16x32 MFMA step on operands held as 16-byte pieces: the f16 form, or the bf16 form on the same bits (the
// tiles move operands without looking at them, so bf16 GEMMs share every layout and every load with f16 ones).
template <bool BF16>
__device__ __forceinline__ float4_t mfma_16x16x32(half8_t a, half8_t b, float4_t c) {
  if constexpr (BF16) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// v_mfma_f32_16x16x32_f16 directly from global memory: a lane's operand is 8 consecutive halves
// along k, i.e. one 16-byte load, and because a weight element is only ever needed by the waves that
// own its columns there is nothing to share through LDS in the main loop.  Partial sums of the WK
// waves meet in LDS once, after the loop.
//
// At batch 1 a stage is bound by memory latency, not by bandwidth or MFMA rate, so the loop is
// organised around round trips: the k steps of a wave are cut into chunks of CH steps, all loads of
// a chunk are issued back to back (and the next chunk's before the current chunk's MFMAs), which
// leaves one exposed memory latency per tile instead of one per k step.
//
// A is row-major [M, lda] or, when the producing stage of this kernel stores it so (PACKED_A), in the same
// fragment order as packed weights: a lane's 16 rows x 16 bytes of a row-major operand touch 16 cache lines per
// quarter wave, a fragment-order operand is one contiguous KiB per MFMA step.
// B comes in one of two layouts:
//   PACKED_B = false : Bt[n][k], k contiguous (activation operands such as K in Q.K^T)
//   PACKED_B = true  : fragment order [n/16][k/32][lane][8] written by the host at upload for
//                      constant weights: one MFMA operand = one contiguous 1 KiB block, a wave
//                      walks its k range through consecutive memory.
//
// The MFMA is issued with the B fragment as first operand so that a lane ends up with four
// consecutive n of one row m (n = n0 + 4*(lane/16) + r, m = m0 + lane%16): the epilogue then
// stores 8 contiguous bytes per lane.  D_ALONG_M swaps the operands: four consecutive m of one
// column n (m = m0 + 4*(lane/16) + r, n = n0 + lane%16), for results that are stored transposed.
//
// Epilogue functor:  struct Pre;  void preload(int batch, int m, int n, Pre&) const   (loads what operator() will read)
//                    void operator()(int batch, int m, int n, const float (&v)[4])   (n % 4 == 0)
// Rows/cols beyond M / N are clamped on load and skipped on store, so M and N need not divide.
//
// Prologue functor (optional): a row program over the rows of A (LayerNorm) applied to the A
// fragments in registers before they reach the MFMAs.  It needs a wave's whole k range resident
// (one chunk).  Interface:  static constexpr bool enabled;
//   void operator()(half8_t (&a)[CH][TM], int m_base, int wk, int mn_wave, bool store, char* smem)
// `store` is true for the one wave column (wn == 0 of tile_n == 0) that also writes the transformed
// rows to memory for later consumers.
struct NoPrologue {
  static constexpr bool enabled = false;
  static constexpr bool after_mfma = false;
};

// Where row m, column k of the left operand lives.  The default is a row-major [M, lda] matrix; an implicit-GEMM
// convolution supplies a map that gathers the row from the input image.  k is a multiple of 8 and the 8 elements
// from there on are contiguous and 16-byte aligned.
struct RowMajorA {
  static constexpr bool kRowMajor = true;
  __device__ __forceinline__ const half_t* operator()(const half_t* A, int m, int k, int lda) const { return A + (long)m * lda + k; }
};

// k steps of one wave that are loaded together: (TM + TN) * 4 * CH * 2 (double buffer) stays within ~256 VGPRs.
// With the right operand requested ahead of the tile (pre_b) a wave whose whole k range fits into 224 VGPRs takes
// it as one chunk: there is nothing left to double-buffer.
__device__ constexpr int gemm_chunk_steps(int TM, int TN, int my_steps, bool pre_b = false) {
  constexpr int whole = MONONN_WAVES_PER_SIMD >= 2 ? 24 : 56, chunk0 = MONONN_WAVES_PER_SIMD >= 2 ? 16 : 32;   // half the registers: half the fragments
  if (pre_b && my_steps * (TM + TN) <= whole) return my_steps;
  const int chunk = TM * TN > 32 ? chunk0 / 2 : chunk0;   // more than 128 accumulator registers: smaller operand chunks
  const int ch_max = chunk / (TM + TN) > 0 ? chunk / (TM + TN) : 1;
  return my_steps < ch_max ? my_steps : ch_max;
}

// Right-operand fragments of a wave's first chunk, requested before the tile's left operand exists.  Packed weights
// are constants of the module: a workgroup asks for them between announcing the end of its previous stage and
// waiting for the other workgroups, so their way from memory overlaps the barrier instead of following it.
template <int REGS>
struct PreB {
  half8_t v[REGS];
};
struct NoPreB {
  half8_t v[1];
};

template <int BM, int BN, int WM, int WN, int WK, int K, int KTOTAL, class Pre>
__device__ __forceinline__ void gemm_b_preload(const half_t* B, int N, int tile_n, Pre& pb) {
  constexpr int TM = BM / WM / 16;
  constexpr int TN = BN / WN / 16;
  constexpr bool RAGGED_K = K % 32 != 0;   // the last k step is partly past the end: its missing elements are zeros
  constexpr int KSTEPS = (K + 31) / 32;
  constexpr int MY_STEPS = (KSTEPS + WK - 1) / WK;
  constexpr int CH = gemm_chunk_steps(TM, TN, MY_STEPS, true);
  static_assert(CH * TN * sizeof(half8_t) <= sizeof(pb.v), "preload buffer too small for this tile");
  const int lane = lane_id();
  const int wave = wave_id();
  const int wk = wave % WK;
  const int wn = (wave / WK) % WN;
  const int n_base = tile_n * BN + wn * (TN * 16);
  const int nt_max = (N + 15) / 16 - 1;
#pragma unroll
  for (int s = 0; s < CH; ++s) {
    int ks = s * WK + wk;
    ks = ks < KSTEPS ? ks : KSTEPS - 1;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int nt = (n_base >> 4) + j;
      nt = nt < nt_max ? nt : nt_max;
      pb.v[s * TN + j] = *reinterpret_cast<const half8_t*>(B + (((long)nt * (KTOTAL / 32) + ks) * 64 + lane) * 8);
    }
  }
}

// K is the k extent this call contracts over; KTOTAL the k extent of the operands in memory (they differ
// when the k range is split over workgroups: the caller then offsets A and B to the start of its slice).
// PRE_B: the right operand's first chunk was requested by gemm_b_preload with the same parameters and comes in `pb`.
// B_ALONG_N: the right operand is stored [K, ldb] with n contiguous (a run-time [K, N] matrix, weights passed as
// kernel parameters): a lane gathers its eight k values of one column with eight 2-byte loads.  Slower per byte
// than the k-contiguous layouts, but the contraction stays on the MFMAs.
// A_ALONG_M: likewise the left operand stored [K, lda] with m contiguous (gemm_impl.cc:408-469 takes either operand
// in either order): a lane gathers the eight k values of its row.
template <int BM, int BN, int WM, int WN, int WK, int K, bool PACKED_B, int KTOTAL, class Epi, class Pro = NoPrologue, class AMap = RowMajorA,
          bool PRE_B = false, class Pre = NoPreB, bool PACKED_A = false, bool D_ALONG_M = false, bool B_ALONG_N = false, bool BF16 = false,
          bool A_ALONG_M = false>
__device__ __forceinline__ void gemm_tile(const half_t* A, const half_t* B, int M, int N, int lda, int ldb,
                                          int batch, int tile_m, int tile_n, Epi& epi, char* smem, const Pro& pro = Pro(),
                                          const AMap& amap = AMap(), const Pre* pb = nullptr) {
  constexpr int TM = BM / WM / 16;
  constexpr int TN = BN / WN / 16;
  constexpr bool RAGGED_K = K % 32 != 0;   // the last k step is partly past the end: its missing elements are zeros
  constexpr int KSTEPS = (K + 31) / 32;
  constexpr int MY_STEPS = (KSTEPS + WK - 1) / WK;
  constexpr int CH = gemm_chunk_steps(TM, TN, MY_STEPS, PRE_B);
  constexpr int NCHUNK = (MY_STEPS + CH - 1) / CH;
  static_assert(!PRE_B || PACKED_B, "only packed weights can be requested ahead of the tile");
  static_assert(!PACKED_A || AMap::kRowMajor, "a fragment-order left operand takes no row map");
  static_assert(BM % (WM * 16) == 0 && BN % (WN * 16) == 0, "tile/wave mismatch");
  static_assert(!RAGGED_K || (!PACKED_A && !PACKED_B && !PRE_B && AMap::kRowMajor && K == KTOTAL && !Pro::enabled),
                "a k extent that is not a multiple of 32 is taken from plain k-contiguous operands only");
  static_assert(!B_ALONG_N || (!PACKED_B && !PRE_B), "an n-contiguous right operand is neither packed nor requested ahead");
  static_assert(!A_ALONG_M || (!PACKED_A && AMap::kRowMajor && !Pro::enabled), "an m-contiguous left operand is plain memory: no fragment order, row map or row program");
  const int lane = lane_id();
  const int wave = wave_id();
  const int wk = wave % WK;
  const int wn = (wave / WK) % WN;
  const int wm = wave / (WK * WN);
  const int m_base = tile_m * BM + wm * (TM * 16);
  const int n_base = tile_n * BN + wn * (TN * 16);
  const int r16 = lane & 15;
  const int kq = (lane >> 4) * 8;

  const half_t* a_ptr[TM];
  const half_t* b_ptr[TN];
  int a_row[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    int m = m_base + i * 16 + r16;
    m = m < M ? m : M - 1;
    a_row[i] = m;
    if constexpr (PACKED_A) {
      // fragment order [m/16][k/32][lane][8], written that way by the producing stage (M is a multiple of 16)
      int mt = (m_base >> 4) + i;
      const int mt_max = M / 16 - 1;
      mt = mt < mt_max ? mt : mt_max;
      a_ptr[i] = A + ((long)mt * (KTOTAL / 32) * 64 + lane) * 8;
    } else if constexpr (A_ALONG_M) {
      a_ptr[i] = A + m + (long)kq * lda;
    } else {
      a_ptr[i] = A + (long)m * lda + kq;
    }
  }
  constexpr int A_STEP = PACKED_A ? 64 * 8 : 32;   // halves between consecutive k steps
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    if (PACKED_B) {
      int nt = (n_base >> 4) + j;
      const int nt_max = (N + 15) / 16 - 1;
      nt = nt < nt_max ? nt : nt_max;
      b_ptr[j] = B + ((long)nt * (KTOTAL / 32) * 64 + lane) * 8;
    } else {
      int n = n_base + j * 16 + r16;
      n = n < N ? n : N - 1;
      b_ptr[j] = B_ALONG_N ? B + n + (long)kq * ldb : B + (long)n * ldb + kq;
    }
  }
  constexpr int B_STEP = PACKED_B ? 64 * 8 : 32;   // halves between consecutive k steps (k-contiguous layouts)
  // eight k values of one column of an n-contiguous operand, zero past the end of k
  auto load_along_n = [&](const half_t* p, int k0, int ld) {
    half8_t v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (!RAGGED_K || k0 + e < K) ? p[(long)e * ld] : half_t(0);
    return v;
  };

  half8_t a[2][CH][TM], b[2][CH][TN];
  // Rows whose k extent is not a multiple of 32 start at odd element offsets, so their fragments are read
  // without an alignment promise, and the lanes whose 8 elements cross the end read them one by one.
  auto load_ragged = [&](const half_t* p, int k0) {
    half8_t v;
    if (k0 + 8 <= K) {
      __builtin_memcpy(&v, p, sizeof(v));
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = k0 + e < K ? p[e] : half_t(0);
    }
    return v;
  };
  auto load_chunk = [&](int c, int buf) {
#pragma unroll
    for (int s = 0; s < CH; ++s) {
      int ks = (c * CH + s) * WK + wk;
      ks = ks < KSTEPS ? ks : KSTEPS - 1;   // surplus steps re-read a valid block and are not accumulated
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if (PRE_B && c == 0) b[buf][s][j] = pb->v[s * TN + j];
        else if constexpr (B_ALONG_N) b[buf][s][j] = load_along_n(b_ptr[j] + (long)ks * 32 * ldb, ks * 32 + kq, ldb);
        else if constexpr (RAGGED_K) b[buf][s][j] = load_ragged(b_ptr[j] + (long)ks * B_STEP, ks * 32 + kq);
        else b[buf][s][j] = *reinterpret_cast<const half8_t*>(b_ptr[j] + (long)ks * B_STEP);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        if constexpr (A_ALONG_M) a[buf][s][i] = load_along_n(a_ptr[i] + (long)ks * 32 * lda, ks * 32 + kq, lda);
        else if constexpr (RAGGED_K) a[buf][s][i] = load_ragged(a_ptr[i] + (long)ks * A_STEP, ks * 32 + kq);
        else if constexpr (AMap::kRowMajor) a[buf][s][i] = *reinterpret_cast<const half8_t*>(a_ptr[i] + (long)ks * A_STEP);
        else a[buf][s][i] = *reinterpret_cast<const half8_t*>(amap(A, a_row[i], ks * 32 + kq, lda));
      }
    }
  };

  float4_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

  load_chunk(0, 0);
  // The epilogue's operands (bias, residual) of the fragments this wave finalises are requested now and used
  // after the main loop, so that their latency overlaps it.  Slot q belongs to fragment q * WK + wk; the
  // addresses are clamped instead of guarded so that the loads stay in this basic block (a load under a
  // branch gets its wait inside the branch, which would stall on every operand load issued above).
  constexpr int NSLOT = (TM * TN + WK - 1) / WK;
  typename Epi::Pre pre[NSLOT];
#pragma unroll
  for (int q = 0; q < NSLOT; ++q) {
    int f = q * WK + wk;
    f = f < TM * TN ? f : TM * TN - 1;
    int m = m_base + (f / TN) * 16 + (D_ALONG_M ? (lane >> 4) * 4 : r16);
    int n = n_base + (f % TN) * 16 + (D_ALONG_M ? r16 : (lane >> 4) * 4);
    if (D_ALONG_M) {
      m = m < M ? m : (M >= 4 ? M - 4 : 0);
      n = n < N ? n : N - 1;
    } else {
      m = m < M ? m : M - 1;
      n = n < N ? n : (N >= 4 ? N - 4 : 0);
    }
    epi.preload(batch, m, n, pre[q]);
  }
  // (a row program in front of the MFMAs runs after those requests: it waits for the left operand and, with the
  // k range split over waves, at a workgroup barrier)
  if constexpr (Pro::enabled && !Pro::after_mfma) {
    static_assert(NCHUNK == 1, "a GEMM prologue needs the whole k range of a wave in registers");
    pro(a[0], m_base, wk, wave / WK, tile_n == 0 && wn == 0, wn == 0 ? tile_n : -1, smem);
  }
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (c + 1 < NCHUNK) load_chunk(c + 1, (c + 1) & 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < CH; ++s) {
      const int ks = (c * CH + s) * WK + wk;
      if (ks < KSTEPS) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = D_ALONG_M ? mfma_16x16x32<BF16>(a[c & 1][s][i], b[c & 1][s][j], acc[i][j])
                                  : mfma_16x16x32<BF16>(b[c & 1][s][j], a[c & 1][s][i], acc[i][j]);
      }
    }
  }

  // A functor that only derives something from the left operand's fragments for the epilogue (row statistics of a
  // folded LayerNorm) runs here, behind the issued MFMAs: its vector-ALU work passes while the matrix pipe drains.
  if constexpr (Pro::enabled && Pro::after_mfma) {
    static_assert(NCHUNK == 1, "a GEMM prologue needs the whole k range of a wave in registers");
    pro(a[0], m_base, wk, wave / WK, tile_n == 0 && wn == 0, wn == 0 ? tile_n : -1, smem);
  }
  if (WK > 1) {
    // [wk][wm*wn][frag][lane] float4 : each wave writes its own slab, then every wave finalises the
    // fragments f with f % WK == wk from all WK slabs.
    float4_t* red = reinterpret_cast<float4_t*>(smem);
    const int mn = wave / WK;
    __syncthreads();   // smem may still be in use by the previous tile's readers
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        red[((wk * (WM * WN) + mn) * (TM * TN) + (i * TN + j)) * kWaveSize + lane] = acc[i][j];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int f = i * TN + j;
        if (f % WK != wk) continue;
        // every slab is read, the wave's own included: no branch on the wave index, so the LDS reads are
        // issued together, and the k slices are added in one order whatever wave finalises the fragment
        float4_t part[WK];
#pragma unroll
        for (int w = 0; w < WK; ++w) part[w] = red[((w * (WM * WN) + mn) * (TM * TN) + f) * kWaveSize + lane];
        float4_t s = part[0];
#pragma unroll
        for (int w = 1; w < WK; ++w) s += part[w];
        const int m = m_base + i * 16 + (D_ALONG_M ? (lane >> 4) * 4 : r16);
        const int n = n_base + j * 16 + (D_ALONG_M ? r16 : (lane >> 4) * 4);
        if (m < M && n < N) {
          float v[4] = {s[0], s[1], s[2], s[3]};
          epi(batch, m, n, v, pre[f / WK]);
        }
      }
  } else {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int m = m_base + i * 16 + (D_ALONG_M ? (lane >> 4) * 4 : r16);
        const int n = n_base + j * 16 + (D_ALONG_M ? r16 : (lane >> 4) * 4);
        if (m < M && n < N) {
          float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
          epi(batch, m, n, v, pre[i * TN + j]);
        }
      }
  }
}

// ---------------------------------------------------------------------------------------------
// f32 GEMM:  D[m][n] = sum_k A[m][k] * B[k][n], all f32, on v_mfma_f32_16x16x4_f32
// ---------------------------------------------------------------------------------------------
// A workgroup of WM x WN waves owns a BM x BN tile; each wave keeps (BM / WM / 16) x (BN / WN / 16) accumulator
// fragments and walks the whole k range in chunks of 16: a lane loads four consecutive k of its row (one 16-byte
// load when the operand is k-contiguous) and the chunk is four MFMAs, the s-th of which contracts the s-th
// element of every lane (k = 4 * (lane / 16) + s within the chunk: any split of the 16 k over the four MFMAs is
// as good as any other, as long as both operands use the same one).  A is row-major [M, lda]; B is [N, ldb]
// (k-contiguous) or, with B_ALONG_N, [K, ldb].  The last chunk of a k extent that is not a multiple of 16 is
// zero-filled.  Rows / columns beyond M / N are clamped on load and skipped on store.  Epilogue functor and lane
// layout of the result as in gemm_tile.
template <int BM, int BN, int WM, int WN, int K, bool B_ALONG_N, bool D_ALONG_M, class Epi>
__device__ __forceinline__ void gemm_tile_f32(const float* A, const float* B, int M, int N, int lda, int ldb, int batch, int tile_m, int tile_n,
                                              Epi& epi) {
  constexpr int TM = BM / WM / 16, TN = BN / WN / 16;
  constexpr int CHUNKS = (K + 15) / 16;
  static_assert(BM % (WM * 16) == 0 && BN % (WN * 16) == 0, "tile/wave mismatch");
  const int lane = lane_id();
  const int wave = wave_id();
  const int wn = wave % WN, wm = wave / WN;
  const int m_base = tile_m * BM + wm * (TM * 16);
  const int n_base = tile_n * BN + wn * (TN * 16);
  const int r16 = lane & 15;
  const int kq = (lane >> 4) * 4;
  const float* a_ptr[TM];
  const float* b_ptr[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    int m = m_base + i * 16 + r16;
    m = m < M ? m : M - 1;
    a_ptr[i] = A + (long)m * lda + kq;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    int n = n_base + j * 16 + r16;
    n = n < N ? n : N - 1;
    b_ptr[j] = B_ALONG_N ? B + n + (long)kq * ldb : B + (long)n * ldb + kq;
  }
  // four consecutive k from a k-contiguous row (no alignment promise: rows of an odd length start anywhere)
  auto load_k4 = [&](const float* p, int k0) {
    float4_t v;
    if ((K % 16 == 0) || k0 + 4 <= K) {
      __builtin_memcpy(&v, p, 16);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = k0 + e < K ? p[e] : 0.f;
    }
    return v;
  };
  auto load_n4 = [&](const float* p, int k0) {
    float4_t v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = ((K % 16 == 0) || k0 + e < K) ? p[(long)e * ldb] : 0.f;
    return v;
  };
  float4_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
  typename Epi::Pre pre[TM * TN];
#pragma unroll
  for (int f = 0; f < TM * TN; ++f) {
    int m = m_base + (f / TN) * 16 + (D_ALONG_M ? (lane >> 4) * 4 : r16);
    int n = n_base + (f % TN) * 16 + (D_ALONG_M ? r16 : (lane >> 4) * 4);
    if (D_ALONG_M) {
      m = m < M ? m : (M >= 4 ? M - 4 : 0);
      n = n < N ? n : N - 1;
    } else {
      m = m < M ? m : M - 1;
      n = n < N ? n : (N >= 4 ? N - 4 : 0);
    }
    epi.preload(batch, m, n, pre[f]);
  }
  float4_t a[2][TM], b[2][TN];
  auto load_chunk = [&](int c, int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i) a[buf][i] = load_k4(a_ptr[i] + c * 16, c * 16 + kq);
#pragma unroll
    for (int j = 0; j < TN; ++j) b[buf][j] = B_ALONG_N ? load_n4(b_ptr[j] + (long)c * 16 * ldb, c * 16 + kq) : load_k4(b_ptr[j] + c * 16, c * 16 + kq);
  };
  load_chunk(0, 0);
  for (int c = 0; c < CHUNKS; c += 2) {
    // two chunks per trip so that the register set a chunk is loaded into is known at compile time
    if (c + 1 < CHUNKS) load_chunk(c + 1, 1);
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = D_ALONG_M ? __builtin_amdgcn_mfma_f32_16x16x4f32(a[0][i][s], b[0][j][s], acc[i][j], 0, 0, 0)
                                : __builtin_amdgcn_mfma_f32_16x16x4f32(b[0][j][s], a[0][i][s], acc[i][j], 0, 0, 0);
    if (c + 1 < CHUNKS) {
      if (c + 2 < CHUNKS) load_chunk(c + 2, 0);
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = D_ALONG_M ? __builtin_amdgcn_mfma_f32_16x16x4f32(a[1][i][s], b[1][j][s], acc[i][j], 0, 0, 0)
                                  : __builtin_amdgcn_mfma_f32_16x16x4f32(b[1][j][s], a[1][i][s], acc[i][j], 0, 0, 0);
    }
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int m = m_base + i * 16 + (D_ALONG_M ? (lane >> 4) * 4 : r16);
      const int n = n_base + j * 16 + (D_ALONG_M ? r16 : (lane >> 4) * 4);
      if (m < M && n < N) {
        float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
        epi(batch, m, n, v, pre[i * TN + j]);
      }
    }
}

// ---------------------------------------------------------------------------------------------
// GEMM for large problems: operand tiles staged through LDS, once per workgroup
// ---------------------------------------------------------------------------------------------
// gemm_tile above has every wave fetch its own fragments from global memory; with many rows the same fragment is
// wanted by all waves (and all workgroups) of a tile row / column and the vector L1 becomes the limit.  Here a
// workgroup of WM x WN waves owns a BM x BN tile, every k tile of BK is brought into LDS once, by all waves
// together, and each wave reads the fragments of its (BM / WM) x (BN / WN) block from there.
//
// The MFMA is v_mfma_f32_32x32x16_f16: measured on this part it retires 32 clocks apart at twice the work of the
// 16x16x32 form, which retires 27 clocks apart (2.2 against 1.4 PFLOP/s with every SIMD busy).  An operand fragment
// is 32 rows x 16 k: lane l holds row l % 32, k piece l / 32 (8 halves).  LDS holds fragments in exactly that
// order, block (row block of 32, k step of 16) = 1 KiB with lane l's piece at byte 16 * l, so that a fragment
// read is ds_read_b128 at 16 * lane and a copy is ds_write_b128 at 16 * lane (no bank conflicts).  Memory keeps
// the layouts of the rest of the kernel (row-major k-contiguous, or the 16-row x 32-k fragment order of packed
// weights and in-kernel operands): each lane simply loads the 16 bytes that belong in its slot; from
// fragment-order memory the 64 pieces of a block are four runs of 256 contiguous bytes.
//
// Pipeline, in k tiles: tile t is multiplied out of LDS buffer t % 2 while tile t + 1 is written from registers into
// the other buffer and tile t + 3 is requested from memory into the registers that this frees; tile t + 2 is on
// its way in a second set of registers.  A wave alone on its SIMD has nobody to hide its memory instructions
// behind, and it issues in order: fragment reads, LDS writes and global loads are placed between the MFMAs by
// hand, one MFMA at a time, each slot fenced from the instruction scheduler.  (The direct global-to-LDS load was
// tried first: on this part one such load keeps the memory pipeline busy for hundreds of clocks, copies alone took
// as long as the MFMAs alone, and in-order issue adds the two up.)
//
// One workgroup barrier per k tile, before its last step: "every wave has written its share of tile t + 1" and
// "every wave has the last fragments of tile t in registers", so buffer t % 2 may be written during tile t + 1.

// A buffer descriptor over `base` (byte offsets of up to 4 GiB): loads address memory as descriptor + 32-bit lane
// offset + wave-uniform offset, which keeps one register per copy alive across the k loop.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t whole_buffer(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, -1, 0x00020000);
}
__device__ __forceinline__ half8_t buffer_load_16(__amdgpu_buffer_rsrc_t buffer, unsigned lane_offset, unsigned wave_offset) {
  typedef unsigned uint4_t __attribute__((ext_vector_type(4)));
  // the wave-uniform offset is named as such: where the compiler cannot prove it, it wraps the load into a loop
  // over the distinct values
  const uint4_t v = __builtin_amdgcn_raw_buffer_load_b128(buffer, lane_offset, __builtin_amdgcn_readfirstlane(wave_offset), 0);
  half8_t h;
  __builtin_memcpy(&h, &v, 16);
  return h;
}

template <bool B>
struct BoolConstant {
  static constexpr bool value = B;
};

constexpr int gemm_lds_bytes(int BM, int BN, int BK) { return 2 * (BM + BN) * BK * 2; }

typedef float float16_t __attribute__((ext_vector_type(16)));

template <bool BF16>
__device__ __forceinline__ float16_t mfma_32x32x16(half8_t a, half8_t b, float16_t c) {
  if constexpr (BF16) return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// No rows to store behind a folded LayerNorm (the default of gemm_tile_lds' last template argument).
struct NoRowStore {
  static constexpr bool enabled = false;
};

// BK: k extent of one LDS buffer (a multiple of 32); K a multiple of 32.
// LN_STATS: the left operand's rows are the input of a LayerNorm that has been folded into weights and epilogue: while
// a wave multiplies, it also adds up x and x * x of the fragments it reads (v_dot2_f32_f16 between the MFMAs: a
// lane holds 8 values of one row), and in front of the epilogue leaves (mean, rsqrt(var + ln_eps)) of its rows in
// ln_stats[row of the tile][2] (LDS) for the epilogue's rank-1 correction.  The waves that share rows write the same
// values; a wave reads only rows it has written itself.
// Rows (with LN_STATS): other stages read the normalised rows, so this GEMM also stores them: the column tiles of a
// row block share the k range (tile_n of tiles_n takes a block of 16-byte runs), the waves that share rows split
// them, and rows(m, k, x[m][k .. k + 7], mean, rsqrt) normalises and stores one run.
template <int BM, int BN, int WM, int WN, int K, int KTOTAL, bool PACKED_A, bool PACKED_B, bool D_ALONG_M, int BK, class Epi,
          class AMap = RowMajorA, bool BF16 = false, bool ROWS_LDS = false, bool LN_STATS = false, class Rows = NoRowStore>
__device__ __forceinline__ void gemm_tile_lds(const half_t* A, const half_t* B, int M, int N, int lda, int ldb, int batch, int tile_m,
                                              int tile_n, Epi& epi, char* smem, const AMap& amap = AMap(), float ln_eps = 0.f, float* ln_stats = nullptr,
                                              const Rows& rows = Rows(), int tiles_n = 1) {
  constexpr int NW = WM * WN;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;             // 32 x 32 fragments per wave
  constexpr int KSTP = BK / 16;                                    // MFMA steps per k tile
  constexpr int ABLK = BM / 32 * KSTP, BBLK = BN / 32 * KSTP;      // 1 KiB blocks of one k tile
  constexpr int STAGE_BYTES = (ABLK + BBLK) * 1024;
  constexpr int KSTEPS = K / 16;
  constexpr int KT = (KSTEPS + KSTP - 1) / KSTP;                   // k tiles; the last one may hold fewer steps
  constexpr bool SHORT_LAST = KSTEPS % KSTP != 0;
  static_assert(K % 32 == 0 && BK % 32 == 0, "the LDS-staged tile takes k extents that are multiples of 32");
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "tile/wave mismatch");
  static_assert(ABLK % NW == 0 && BBLK % NW == 0, "the waves share the copy of a k tile evenly");
  static_assert(!PACKED_A || AMap::kRowMajor, "a fragment-order left operand takes no row map");
  constexpr int ACPY = ABLK / NW, BCPY = BBLK / NW;                // copies per lane and k tile
  constexpr int CPY = ACPY + BCPY;
  const int lane = lane_id();
  const int wave = wave_id();
  const int wn = wave % WN;
  const int wm = wave / WN;
  const int r32 = lane & 31;
  const int kq = (lane >> 5) * 8;   // this lane's k piece inside a step of 16

  // Byte offset from the operand's base of the piece this lane copies for block (row block, step 0 of k tile 0).
  // Fragment-order memory: [row / 16][k / 32][(k % 32 / 8) * 16 + row % 16][8 halves]; a step of 16 k is half such
  // a block, 512 bytes on.
  auto piece_offset = [&](bool packed, int row, int ld) -> unsigned {
    if (packed) return (((unsigned)(row >> 4) * (KTOTAL / 32)) * 512u + ((kq >> 3) * 16 + (row & 15)) * 8) * 2u;
    return ((unsigned)row * (unsigned)ld + kq) * 2u;
  };
  constexpr unsigned A_STEP = PACKED_A ? 512u : 32u;   // bytes between consecutive steps of 16 k
  constexpr unsigned B_STEP = PACKED_B ? 512u : 32u;
  const __amdgpu_buffer_rsrc_t a_buf = whole_buffer(A), b_buf = whole_buffer(B);
  unsigned a_off[ACPY], b_off[BCPY];
  int a_row[ACPY];
#pragma unroll
  for (int j = 0; j < ACPY; ++j) {
    const int blk = wave + j * NW, rb = blk / KSTP;
    int m = tile_m * BM + rb * 32 + r32;
    m = m < M ? m : M - 1;
    a_row[j] = m;
    a_off[j] = piece_offset(PACKED_A, m, lda);
  }
#pragma unroll
  for (int j = 0; j < BCPY; ++j) {
    const int blk = wave + j * NW, rb = blk / KSTP;
    int n = tile_n * BN + rb * 32 + r32;
    const int n_max = PACKED_B ? (N + 15) / 16 * 16 - 1 : N - 1;   // packed weights are padded to whole blocks of 16 columns
    n = n < n_max ? n : n_max;
    b_off[j] = piece_offset(PACKED_B, n, ldb);
  }

  // c-th of the CPY pieces this lane moves per k tile (the left operand's first): memory -> register, register ->
  // LDS.  Tiles past the end are the last tile once more (a redundant copy into a buffer nobody reads any more,
  // which keeps the loop body free of branches); the steps of the last tile that lie past the end of k re-read
  // its first step and are not multiplied.
  half8_t staged[2][CPY];
  auto load_one = [&](int t, int set, int c) {
    t = t < KT ? t : KT - 1;
    if (c < ACPY) {
      const int blk = wave + c * NW, ks = blk % KSTP;
      const bool past = SHORT_LAST && t * KSTP + ks >= KSTEPS;
      if constexpr (AMap::kRowMajor) {
        staged[set][c] = buffer_load_16(a_buf, a_off[c], (unsigned)(t * KSTP + (past ? 0 : ks)) * A_STEP);
      } else {
        const half_t* src = amap(A, a_row[c], (t * KSTP + (past ? 0 : ks)) * 16 + kq, lda);
        staged[set][c] = buffer_load_16(a_buf, (unsigned)(reinterpret_cast<const char*>(src) - reinterpret_cast<const char*>(A)), 0u);
      }
    } else {
      const int blk = wave + (c - ACPY) * NW, ks = blk % KSTP;
      const bool past = SHORT_LAST && t * KSTP + ks >= KSTEPS;
      staged[set][c] = buffer_load_16(b_buf, b_off[c - ACPY], (unsigned)(t * KSTP + (past ? 0 : ks)) * B_STEP);
    }
  };
  // LDS is named outright (a generic pointer would turn the accesses into flat ones wherever the compiler cannot
  // see where `smem` comes from)
  typedef __attribute__((address_space(3))) char lds_char_t;
  typedef __attribute__((address_space(3))) half8_t lds_half8_t;
  lds_char_t* const lds = (lds_char_t*)smem;
  auto store_one = [&](int buf, int set, int c) {
    const int blk = c < ACPY ? wave + c * NW : ABLK + wave + (c - ACPY) * NW;
    *reinterpret_cast<lds_half8_t*>(lds + buf * STAGE_BYTES + blk * 1024 + lane * 16) = staged[set][c];
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // A lane's part of a 32 x 32 fragment: four groups g of four consecutive positions along one dimension (offset
  // 8 * g + 4 * (lane / 32)), at position lane % 32 of the other.  Along n unless D_ALONG_M.
  const int m_base = tile_m * BM + wm * (TM * 32);
  const int n_base = tile_n * BN + wn * (TN * 32);
  const int lane_m = D_ALONG_M ? (lane >> 5) * 4 : r32;
  const int lane_n = D_ALONG_M ? r32 : (lane >> 5) * 4;
  // Operands of the epilogue (bias, residual).  When those of the whole tile fit in 128 registers, the first row is
  // requested now and the others three k tiles before the end, so that their latency passes under the last
  // MFMAs (after the k loop a wave has nothing left to wait behind: a row requested only while the row before
  // it is finalised costs a full trip to memory).  Larger tiles keep that row-ahead scheme.
  constexpr int PRE_REGS = (int)(sizeof(typename Epi::Pre) + 3) / 4 * TN * 4 * TM;
  constexpr bool PRE_ALL = sizeof(typename Epi::Pre) > 1 && PRE_REGS <= 128 && TM > 1;
  typename Epi::Pre pre[PRE_ALL ? TM : 2][TN * 4];
  // ROWS_LDS: a finished row of fragments passes through LDS so that the epilogue takes its groups of four values
  // (four consecutive columns of a row) in row-major order, group q * 64 + lane to a lane in its q-th turn (TN * 4
  // turns): consecutive lanes then store consecutive 8-byte pieces of a row, and a store or operand load of the wave
  // covers whole cache lines.  Straight from the accumulators an instruction touches 32 rows at 16 bytes each.  (For a
  // result in fragment order that is already two runs of 256 contiguous bytes; nothing to gain there.)
  constexpr int W4 = TN * 8;                 // groups per row of the wave's tile
  constexpr int PITCH = TN * 32 + 4;         // floats between rows in LDS: 16 lanes of a write hit 64 different banks
  static_assert(!ROWS_LDS || !D_ALONG_M, "the epilogue through LDS takes accumulators with four values per lane along n");
  // (m, n) of the q-th group of four values a lane finalises in fragment row i
  auto group_m = [&](int i, int q) { return ROWS_LDS ? m_base + i * 32 + (q * 64 + lane) / W4 : m_base + i * 32 + lane_m + (D_ALONG_M ? 8 * (q % 4) : 0); };
  auto group_n = [&](int q) { return ROWS_LDS ? n_base + 4 * ((q * 64 + lane) % W4) : n_base + (q / 4) * 32 + lane_n + (D_ALONG_M ? 0 : 8 * (q % 4)); };
  auto preload_row = [&](int i, typename Epi::Pre (&dst)[TN * 4]) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        int m = group_m(i, j * 4 + g);
        int n = group_n(j * 4 + g);
        if (D_ALONG_M) {
          m = m < M ? m : (M >= 4 ? M - 4 : 0);
          n = n < N ? n : N - 1;
        } else {
          m = m < M ? m : M - 1;
          n = n < N ? n : (N >= 4 ? N - 4 : 0);
        }
        epi.preload(batch, m, n, dst[j * 4 + g]);
      }
  };
  preload_row(0, pre[0]);

  // tiles 0 and 1 on their way; tile 0 into LDS (the previous unit of this workgroup may still be reading its last
  // tiles there: barrier first); tile 2 requested into the registers tile 0 has left
#pragma unroll
  for (int c = 0; c < CPY; ++c) load_one(0, 0, c);
#pragma unroll
  for (int c = 0; c < CPY; ++c) load_one(1, 1, c);
  __syncthreads();
#pragma unroll
  for (int c = 0; c < CPY; ++c) store_one(0, 0, c);
#pragma unroll
  for (int c = 0; c < CPY; ++c) load_one(2, 0, c);
  __syncthreads();

  const lds_char_t* a_frag = lds + (wm * TM * KSTP) * 1024 + lane * 16;
  const lds_char_t* b_frag = lds + (ABLK + wn * TN * KSTP) * 1024 + lane * 16;
  half8_t fa[2][TM], fb[2][TN];
  // two running sums each (even and odd pairs of a fragment), so that consecutive v_dot2 do not wait for one another
  float ln_s1[LN_STATS ? TM : 1][2], ln_s2[LN_STATS ? TM : 1][2];
#pragma unroll
  for (int i = 0; i < (LN_STATS ? TM : 1); ++i) ln_s1[i][0] = ln_s1[i][1] = ln_s2[i][0] = ln_s2[i][1] = 0.f;
  auto read_one = [&](int buf, int ks, int rb, int r) {
    if (r < TM) fa[rb][r] = *reinterpret_cast<const lds_half8_t*>(a_frag + buf * STAGE_BYTES + (r * KSTP + ks) * 1024);
    else fb[rb][r - TM] = *reinterpret_cast<const lds_half8_t*>(b_frag + buf * STAGE_BYTES + ((r - TM) * KSTP + ks) * 1024);
  };
  constexpr int R = TM + TN, Q = TM * TN;
#pragma unroll
  for (int r = 0; r < R; ++r) read_one(0, 0, 0, r);

  // One step: the MFMAs of fragment set rb; between them the fragment reads of (read_buf, read_ks) into the other
  // set, pieces [c0, c1) of tile t + 1 from register set `set` into LDS buffer `write_buf` and pieces [l0, l1) of
  // tile t + 3 from memory into the same registers.
  auto step = [&](int rb, bool reads, int read_buf, int read_ks, int t, int set, int write_buf, int c0, int c1, int l0, int l1) {
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      if (reads) {
#pragma unroll
        for (int r = (R * q) / Q; r < (R * (q + 1)) / Q; ++r) read_one(read_buf, read_ks, rb ^ 1, r);
      }
#pragma unroll
      for (int c = c0 + ((c1 - c0) * q) / Q; c < c0 + ((c1 - c0) * (q + 1)) / Q; ++c) store_one(write_buf, set, c);
#pragma unroll
      for (int c = l0 + ((l1 - l0) * q) / Q; c < l0 + ((l1 - l0) * (q + 1)) / Q; ++c) load_one(t + 3, set, c);
      const int i = q / TN, j = q % TN;
      if constexpr (LN_STATS) {
        if (j == 0) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const half2_t h = {fa[rb][i][2 * e], fa[rb][i][2 * e + 1]};
            ln_s1[i][e & 1] = __builtin_amdgcn_fdot2(h, half2_t{(half_t)1, (half_t)1}, ln_s1[i][e & 1], false);
            ln_s2[i][e & 1] = __builtin_amdgcn_fdot2(h, h, ln_s2[i][e & 1], false);
          }
        }
      }
      acc[i][j] = D_ALONG_M ? mfma_32x32x16<BF16>(fa[rb][i], fb[rb][j], acc[i][j]) : mfma_32x32x16<BF16>(fb[rb][j], fa[rb][i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // Tile t: all steps but the last write tile t + 1 into the other buffer; before the last step the hand-over (this
  // wave's LDS writes and fragment reads have completed, then the bare barrier instruction: __syncthreads() would
  // also wait for the loads in flight); the last step reads the first fragments of tile t + 1 and requests tile
  // t + 3.  The register set (t + 1) % 2 is a compile-time argument: registers cannot be indexed at run time.
  auto run_tile = [&](int t, auto set_c, auto last_c) {
    constexpr int SET = decltype(set_c)::value ? 1 : 0;
    constexpr bool LAST = decltype(last_c)::value;        // the last tile: LAST_STEPS steps, nothing behind it
    constexpr int STEPS = LAST ? KSTEPS - (KT - 1) * KSTP : KSTP;
    const int buf = t & 1;
#pragma unroll
    for (int ks = 0; ks < STEPS; ++ks) {
      if (ks + 1 < STEPS) {
        step(ks & 1, true, buf, ks + 1, t, SET, buf ^ 1, LAST ? 0 : (CPY * ks) / (KSTP - 1), LAST ? 0 : (CPY * (ks + 1)) / (KSTP - 1), 0, 0);
      } else if (!LAST) {
        __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): LDS writes and reads of this wave are done
        __builtin_amdgcn_s_barrier();
        step(ks & 1, true, buf ^ 1, 0, t, SET, 0, 0, 0, 0, CPY);
      } else {
        step(ks & 1, false, 0, 0, t, SET, 0, 0, 0, 0, 0);
      }
    }
  };
  constexpr int PRE_AT = KT >= 3 ? KT - 3 : 0;   // the k tile in front of which the other rows' operands are requested
  auto preload_rest = [&](int t) {
    if constexpr (PRE_ALL) {
      if (t == PRE_AT) {
#pragma unroll
        for (int i = 1; i < TM; ++i) preload_row(i, pre[i]);
      }
    }
  };
  for (int t = 0; t + 1 < KT; t += 2) {
    preload_rest(t);
    run_tile(t, BoolConstant<true>(), BoolConstant<false>());
    if (t + 2 < KT) {
      preload_rest(t + 1);
      run_tile(t + 1, BoolConstant<false>(), BoolConstant<false>());
    }
  }
  preload_rest(KT - 1);
  if constexpr ((KT - 1) % 2 == 0) run_tile(KT - 1, BoolConstant<true>(), BoolConstant<true>());
  else run_tile(KT - 1, BoolConstant<false>(), BoolConstant<true>());

  // One row of fragments at a time.  The accumulators sit in the accumulation registers (a0..a255); the epilogue
  // needs its operands in ordinary vector registers, and left alone the compiler moves the whole tile over when the
  // k loop ends: as many registers again as the tile itself, paid for by spilling everything else that is live in
  // the loop.  Pinning the rows that are not yet due (an empty statement that wants them in accumulation
  // registers) keeps the move to one row at a time.
  if constexpr (LN_STATS) {
    // the two lanes that hold the two k pieces of a row put their sums together; the variance is E[x^2] - mean^2
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const float p1 = ln_s1[i][0] + ln_s1[i][1], p2 = ln_s2[i][0] + ln_s2[i][1];
      const float s1 = p1 + __shfl_xor(p1, 32, kWaveSize), s2 = p2 + __shfl_xor(p2, 32, kWaveSize);
      const float mean = s1 * (1.0f / K);
      const float var = s2 * (1.0f / K) - mean * mean;
      if (lane < 32) {
        float* dst = ln_stats + ((wm * TM + i) * 32 + lane) * 2;
        dst[0] = mean;
        dst[1] = rsqrtf((var > 0.f ? var : 0.f) + ln_eps);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if constexpr (Rows::enabled) {
      static_assert(AMap::kRowMajor, "the rows are read back as the left operand stores them: row-major or in fragment order");
      static_assert(32 % WN == 0, "the waves that share rows split them evenly");
      constexpr int RUNS = K / 8;                              // 16-byte runs of a row
      constexpr int ROWS_W = TM * 32 / WN;                     // rows of this wave
      const int per_tile = (RUNS + tiles_n - 1) / tiles_n;     // runs of this column tile: [run0, run0 + per_tile)
      const int run0 = tile_n * per_tile;
      for (int idx = lane; idx < ROWS_W * per_tile; idx += kWaveSize) {
        const int run = run0 + idx % per_tile;
        const int rw = idx / per_tile;                                              // 0 .. ROWS_W - 1
        const int row_in_tile = (wm * TM + rw / (32 / WN)) * 32 + wn * (32 / WN) + rw % (32 / WN);
        const int m = tile_m * BM + row_in_tile;
        if (run < RUNS && m < M) {
          // fragment order: [row / 16][k / 32][(k % 32 / 8) * 16 + row % 16][8 halves]
          const long at = PACKED_A ? (((long)(m >> 4) * (KTOTAL / 32) + (run >> 2)) * 512 + ((run & 3) * 16 + (m & 15)) * 8) : (long)m * lda + run * 8;
          const half8_t x = *reinterpret_cast<const half8_t*>(A + at);
          rows(m, run * 8, x, ln_stats[row_in_tile * 2], ln_stats[row_in_tile * 2 + 1]);
        }
      }
      // the accumulators stay where they are while the rows are stored (see the epilogue below)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) MONONN_PIN_ACC(acc[i][j]);
    }
  }
  typedef __attribute__((address_space(3))) float4_t lds_float4_t;
  lds_char_t* const rows_lds = lds + wave * (32 * PITCH * 4);   // this wave's 32 rows
  if constexpr (ROWS_LDS) __syncthreads();   // the other waves may still be reading the last operand tiles
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int r = i + 1; r < TM; ++r)
#pragma unroll
      for (int j = 0; j < TN; ++j) MONONN_PIN_ACC(acc[r][j]);
    if (!PRE_ALL && i + 1 < TM) preload_row(i + 1, pre[(i + 1) & 1]);
    if constexpr (ROWS_LDS) {
      // LDS serves a wave's accesses in the order they were issued: the reads below see the writes above without a
      // barrier (no other wave touches these rows); the fences keep the compiler from moving one past the other
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          *reinterpret_cast<lds_float4_t*>(rows_lds + (r32 * PITCH + j * 32 + lane_n + 8 * g) * 4) =
              float4_t{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int q = 0; q < TN * 4; ++q) {
        const float4_t f = *reinterpret_cast<const lds_float4_t*>(rows_lds + (((q * 64 + lane) / W4) * PITCH + 4 * ((q * 64 + lane) % W4)) * 4);
        const int m = group_m(i, q), n = group_n(q);
        if (m < M && n < N) {
          float v[4] = {f[0], f[1], f[2], f[3]};
          epi(batch, m, n, v, pre[PRE_ALL ? i : (i & 1)][q]);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int m = group_m(i, j * 4 + g), n = group_n(j * 4 + g);
          if (m < M && n < N) {
            float v[4] = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
            epi(batch, m, n, v, pre[PRE_ALL ? i : (i & 1)][j * 4 + g]);
          }
        }
    }
  }
}

// Correctness fallback for operand layouts / sizes the MFMA path does not take (A or B not
// contiguous along k, K not a multiple of 32): one thread per output element, fp32 accumulation.
// Strides are in elements.  Epilogue functor as above but with a single value:
//   void operator()(int batch, int m, int n, float v)
template <class T, class Epi>
__device__ __forceinline__ void gemm_naive_element(const T* A, const T* B, int K, long a_sm, long a_sk,
                                                   long b_sk, long b_sn, int batch, int m, int n, Epi& epi) {
  float acc = 0.f;
  const T* a = A + m * a_sm;
  const T* b = B + n * b_sn;
  for (int k = 0; k < K; ++k) acc += (float)a[k * a_sk] * (float)b[k * b_sk];
  epi(batch, m, n, acc);
}

// Correctness fallback for convolutions the fragment loads do not cover (padding, channel counts that break the
// 16-byte pieces): one thread per output element.  Input N,H,W,C, filter K,R,S,C, output N,P,Q,K.
template <class T, class Epi>
__device__ __forceinline__ void conv_naive_element(const T* in, const T* flt, int H, int W, int C, int R, int S, int P, int Q,
                                                   int stride_h, int stride_w, int pad_h, int pad_w, int m, int k_out, Epi& epi) {
  const int n = m / (P * Q), pq = m % (P * Q), p = pq / Q, q = pq % Q;
  float acc = 0.f;
  for (int r = 0; r < R; ++r) {
    const int h = p * stride_h + r - pad_h;
    if (h < 0 || h >= H) continue;
    for (int s = 0; s < S; ++s) {
      const int w = q * stride_w + s - pad_w;
      if (w < 0 || w >= W) continue;
      const T* x = in + (((long)n * H + h) * W + w) * C;
      const T* f = flt + (((long)k_out * R + r) * S + s) * C;
      for (int c = 0; c < C; ++c) acc += (float)x[c] * (float)f[c];
    }
  }
  epi(0, m, k_out, acc);
}

}  // namespace mononn_dev
