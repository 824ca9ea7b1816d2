// Multi-tensor EMA and multi-segment copy: one launch each over a chunk
// table in device memory, one workgroup per table entry.  Both are pure
// streaming kernels (no reuse), so the only things that matter are 16-byte
// coalesced accesses, enough independent loads in flight per wavefront, and
// a grid far larger than the 256 CUs.
#include "common.h"

namespace ts {

constexpr int kEmaBlock = 256;
constexpr int kEmaUnroll = 4;  // 16-byte loads in flight per thread and operand

// out = fl(fl(t*m) + fl(s*c)).  Contraction is switched off for this
// expression: an FMA would skip one rounding and differ from the reference's
// separate mul / mul / add kernels in about a quarter of the elements.
__device__ __forceinline__ float ema1(float t, float s, float m, float c) {
#pragma clang fp contract(off)
  const float a = t * m;
  const float b = s * c;
  return a + b;
}

__global__ __launch_bounds__(kEmaBlock) void ema_multi_kernel(const ts_ema_chunk* __restrict__ table,
                                                              float m, float c) {
  // Uniform per workgroup: the compiler turns these into scalar loads.
  const ts_ema_chunk ch = table[blockIdx.x];
  const uint32_t tid = threadIdx.x;
  const uint32_t n = ch.n;

  if (ch.flags & 1u) {
    const f32x4* __restrict__ t4 = reinterpret_cast<const f32x4*>(ch.t);
    const f32x4* __restrict__ s4 = reinterpret_cast<const f32x4*>(ch.s);
    f32x4* __restrict__ o4 = reinterpret_cast<f32x4*>(ch.out);
    const uint32_t n4 = n >> 2;
    for (uint32_t base = 0; base < n4; base += kEmaBlock * kEmaUnroll) {
      f32x4 a[kEmaUnroll], b[kEmaUnroll];
#pragma unroll
      for (int u = 0; u < kEmaUnroll; ++u) {
        const uint32_t i = base + u * kEmaBlock + tid;
        if (i < n4) {
          a[u] = __builtin_nontemporal_load(t4 + i);
          b[u] = __builtin_nontemporal_load(s4 + i);
        }
      }
#pragma unroll
      for (int u = 0; u < kEmaUnroll; ++u) {
        const uint32_t i = base + u * kEmaBlock + tid;
        if (i < n4) {
          f32x4 r;
          r.x = ema1(a[u].x, b[u].x, m, c);
          r.y = ema1(a[u].y, b[u].y, m, c);
          r.z = ema1(a[u].z, b[u].z, m, c);
          r.w = ema1(a[u].w, b[u].w, m, c);
          __builtin_nontemporal_store(r, o4 + i);
        }
      }
    }
    const uint32_t rem = n & 3u;
    if (tid < rem) {
      const uint32_t i = (n4 << 2) + tid;
      ch.out[i] = ema1(ch.t[i], ch.s[i], m, c);
    }
  } else {
    // Views whose storage offset breaks 16-byte alignment: 4-byte accesses,
    // still coalesced across the wavefront.
    for (uint32_t i = tid; i < n; i += kEmaBlock) ch.out[i] = ema1(ch.t[i], ch.s[i], m, c);
  }
}

constexpr int kCopyBlock = 256;
constexpr int kCopyUnroll = 4;

__global__ __launch_bounds__(kCopyBlock) void copy_segments_kernel(
    const ts_copy_chunk* __restrict__ table) {
  const ts_copy_chunk ch = table[blockIdx.x];
  const uint32_t tid = threadIdx.x;
  const uint64_t bytes = ch.bytes;

  if (ch.flags & 1u) {
    const u32x4* __restrict__ s = reinterpret_cast<const u32x4*>(ch.src);
    u32x4* __restrict__ d = reinterpret_cast<u32x4*>(ch.dst);
    const uint64_t n16 = bytes >> 4;
    for (uint64_t base = 0; base < n16; base += (uint64_t)kCopyBlock * kCopyUnroll) {
      u32x4 v[kCopyUnroll];
#pragma unroll
      for (int u = 0; u < kCopyUnroll; ++u) {
        const uint64_t i = base + (uint64_t)u * kCopyBlock + tid;
        if (i < n16) v[u] = __builtin_nontemporal_load(s + i);
      }
#pragma unroll
      for (int u = 0; u < kCopyUnroll; ++u) {
        const uint64_t i = base + (uint64_t)u * kCopyBlock + tid;
        if (i < n16) __builtin_nontemporal_store(v[u], d + i);
      }
    }
    const uint32_t rem = (uint32_t)(bytes & 15u);
    if (tid < rem) {
      const uint64_t i = (n16 << 4) + tid;
      reinterpret_cast<uint8_t*>(ch.dst)[i] = reinterpret_cast<const uint8_t*>(ch.src)[i];
    }
  } else {
    const uint8_t* __restrict__ s = reinterpret_cast<const uint8_t*>(ch.src);
    uint8_t* __restrict__ d = reinterpret_cast<uint8_t*>(ch.dst);
    const bool a4 = ((((uintptr_t)s) | ((uintptr_t)d)) & 3u) == 0;
    if (a4) {
      const uint64_t n4 = bytes >> 2;
      const uint32_t* s4 = reinterpret_cast<const uint32_t*>(s);
      uint32_t* d4 = reinterpret_cast<uint32_t*>(d);
      for (uint64_t i = tid; i < n4; i += kCopyBlock) d4[i] = s4[i];
      const uint32_t rem = (uint32_t)(bytes & 3u);
      if (tid < rem) d[(n4 << 2) + tid] = s[(n4 << 2) + tid];
    } else {
      for (uint64_t i = tid; i < bytes; i += kCopyBlock) d[i] = s[i];
    }
  }
}

}  // namespace ts

extern "C" {

int ts_ema_multi(const ts_ema_chunk* table_dev, int64_t n_chunks, float m32, float c32,
                 ts_stream_t stream) {
  if (n_chunks < 0) return TS_ERR_ARG;
  if (n_chunks == 0) return TS_OK;
  if (!table_dev) return TS_ERR_ARG;
  if (n_chunks > 0x7fffffffLL) return TS_ERR_RANGE;
  hipLaunchKernelGGL(ts::ema_multi_kernel, dim3((unsigned)n_chunks), dim3(ts::kEmaBlock), 0,
                     (hipStream_t)stream, table_dev, m32, c32);
  return ts::check_launch();
}

int ts_copy_segments(const ts_copy_chunk* table_dev, int64_t n_chunks, ts_stream_t stream) {
  if (n_chunks < 0) return TS_ERR_ARG;
  if (n_chunks == 0) return TS_OK;
  if (!table_dev) return TS_ERR_ARG;
  if (n_chunks > 0x7fffffffLL) return TS_ERR_RANGE;
  hipLaunchKernelGGL(ts::copy_segments_kernel, dim3((unsigned)n_chunks), dim3(ts::kCopyBlock), 0,
                     (hipStream_t)stream, table_dev);
  return ts::check_launch();
}

}  // extern "C"
