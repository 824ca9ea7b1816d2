// Shared device helpers for the gfx950 kernels: 64-wide wavefront reductions,
// 16-byte vector types, dtype conversion, launch-error bookkeeping.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tspipe_amd.h"

namespace ts {

constexpr int kWave = 64;  // CDNA wavefront width

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));

// Records the HIP error of a failed launch for ts_last_hip_error().
void set_last_hip_error(int code);
// Hands out (and clears) the events ts_time_next_launch() armed this thread
// with; false when there are none.
bool take_launch_events(hipEvent_t* start, hipEvent_t* stop);

inline int check_launch() {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_last_hip_error((int)e);
    return TS_ERR_LAUNCH;
  }
  return TS_OK;
}

// ---- dtype conversion (storage type <-> fp32) ---------------------------

struct bf16_t {
  uint16_t bits;
};
struct f16_t {
  _Float16 v;
};

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return __uint_as_float((uint32_t)x.bits << 16); }
__device__ __forceinline__ float to_f32(f16_t x) { return (float)x.v; }

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits) { return __uint_as_float(bits << 16); }

// Round-to-nearest-even fp32 -> bf16 (what torch's cast does); the compiler
// emits gfx950's v_cvt_pk_bf16_f32 for this conversion.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  const __bf16 b = (__bf16)f;
  uint16_t u;
  __builtin_memcpy(&u, &b, 2);
  return u;
}

template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) {
  bf16_t r;
  r.bits = f32_to_bf16_bits(x);
  return r;
}
template <>
__device__ __forceinline__ f16_t from_f32<f16_t>(float x) {
  f16_t r;
  r.v = (_Float16)x;
  return r;
}

// 2^x on the hardware transcendental unit (v_exp_f32, 1 ulp).  Results below
// the normal range flush to zero, which is what a soft-max term that small
// contributes anyway; the library exp2f spends several extra instructions on
// rescaling them.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---- 16-byte vectors of a storage type -------------------------------------

template <typename T>
struct Vec16 {
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

template <typename T>
__device__ __forceinline__ Vec16<T> load16(const T* p) {
  const u32x4 raw = *reinterpret_cast<const u32x4*>(p);
  Vec16<T> r;
  __builtin_memcpy(&r, &raw, 16);
  return r;
}

template <typename T>
__device__ __forceinline__ Vec16<T> load16_stream(const T* p) {
  const u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  Vec16<T> r;
  __builtin_memcpy(&r, &raw, 16);
  return r;
}

template <typename T>
__device__ __forceinline__ void store16(T* p, const Vec16<T>& v) {
  u32x4 raw;
  __builtin_memcpy(&raw, &v, 16);
  *reinterpret_cast<u32x4*>(p) = raw;
}

// Non-temporal store, for data that is written once and read only by a later
// kernel.  Whether it pays is measured per kernel: the KD gradient rows and
// the BatchNorm outputs gain from it; a pure zero-fill loses (the same bytes
// take 1.6x as long as with plain stores).
template <typename T>
__device__ __forceinline__ void store16_stream(T* p, const Vec16<T>& v) {
  u32x4 raw;
  __builtin_memcpy(&raw, &v, 16);
  __builtin_nontemporal_store(raw, reinterpret_cast<u32x4*>(p));
}

// ---- wavefront / block reductions -----------------------------------------

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a block of NWAVES wavefronts; every thread gets the result.
// `lds` must hold NWAVES floats and may be reused after the call returns.
template <int NWAVES>
__device__ __forceinline__ float block_sum(float v, float* lds) {
  v = wave_sum(v);
  if (NWAVES == 1) return v;
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) lds[w] = v;
  __syncthreads();
  float r = 0.f;
#pragma unroll
  for (int i = 0; i < NWAVES; ++i) r += lds[i];
  return r;
}

// This thread's share of sum(v[0..n)) when NT threads of one workgroup walk the
// array together, in a fixed order.  One workgroup has to get through the whole
// array, so the walk is bound by memory latency: 16-byte loads, eight of them
// in flight per thread (65536 values are two round trips; element by element
// they were 64, and the final sum of a 65536-row loss took 18 us instead of 5).
template <int NT>
__device__ __forceinline__ float thread_share_of_sum(const float* __restrict__ v, int64_t n) {
  constexpr int kInFlight = 8;
  float acc = 0.f;
  int64_t done = 0;
  if (((uintptr_t)v & 15u) == 0) {
    const int64_t n4 = n / 4;
    const f32x4* v4 = reinterpret_cast<const f32x4*>(v);
    f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
    for (int64_t i0 = threadIdx.x; i0 < n4; i0 += (int64_t)NT * kInFlight) {
      f32x4 a[kInFlight];
#pragma unroll
      for (int j = 0; j < kInFlight; ++j) {
        const int64_t i = i0 + (int64_t)j * NT;
        a[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (i < n4) a[j] = v4[i];
      }
#pragma unroll
      for (int j = 0; j < kInFlight; ++j) s4 += a[j];
    }
    acc = (s4[0] + s4[1]) + (s4[2] + s4[3]);
    done = n4 * 4;
  }
  for (int64_t i = done + threadIdx.x; i < n; i += NT) acc += v[i];
  return acc;
}

// Number of non-zero mask bytes, counted by the calling workgroup (every
// thread gets the result; `lds` holds NT / 64 floats).  The mask of a batch is
// a few kilobytes, so this is an L2-resident read and one block reduction --
// cheaper than a counting launch in front when only the workgroups of the
// selected rows need the number.
template <int NT>
__device__ __forceinline__ float mask_count_block(const uint8_t* __restrict__ mask, int64_t n, float* lds) {
  int c = 0;
  const int64_t n8 = ((uintptr_t)mask & 7u) == 0 ? n / 8 : 0;
  const uint64_t* m8 = reinterpret_cast<const uint64_t*>(mask);
  constexpr int kInFlight = 4;  // loads per thread and trip: one workgroup walks the whole mask
  for (int64_t i0 = threadIdx.x; i0 < n8; i0 += (int64_t)NT * kInFlight) {
    uint64_t w[kInFlight];
#pragma unroll
    for (int j = 0; j < kInFlight; ++j) {
      const int64_t i = i0 + (int64_t)j * NT;
      w[j] = i < n8 ? m8[i] : 0;
    }
#pragma unroll
    for (int j = 0; j < kInFlight; ++j) {
      uint64_t v = w[j];
      // a byte counts when any of its bits is set
      v |= v >> 4;
      v |= v >> 2;
      v |= v >> 1;
      c += __popcll(v & 0x0101010101010101ull);
    }
  }
  for (int64_t i = n8 * 8 + threadIdx.x; i < n; i += NT) c += mask[i] != 0;
  // per-thread counts stay far below 2^24 for any n the launchers accept: the float sum is exact
  return block_sum<NT / kWave>((float)c, lds);
}

}  // namespace ts
