// Multi-tensor EMA and multi-segment copy: one launch each over a chunk
// table in device memory.  Both are pure streaming kernels (no reuse), so the
// only things that matter are 16-byte coalesced accesses and a grid far
// larger than the 256 CUs, made of short-lived workgroups.
//
// Measured on MI355X (86.6M-element EMA): a thread that issues its loads once
// and exits, in a grid of tens of thousands of workgroups, sustains ~6.4 TB/s;
// the same work as a loop inside fewer, longer-lived workgroups drops to
// 5.0-5.8 TB/s.  So a table entry (chunk) is cut into sub-blocks, one
// workgroup each: blockIdx = chunk * subs + sub.
#include "common.h"
#include <hip/hip_ext.h>

namespace ts {

// Keeps every field of a table entry in one round of scalar loads: left to
// itself the compiler fetches the length first and the pointers only behind
// the early exit, a second dependent round in front of the vector loads.
#if defined(__HIP_DEVICE_COMPILE__)
#define TS_PIN_SCALARS(...) asm volatile("" : : __VA_ARGS__)
#else
#define TS_PIN_SCALARS(...) (void)0
#endif

// Which (chunk, sub-block) a workgroup is.  The launchers use a two-dimensional
// grid (x = sub-block, y = chunk: the same dispatch order as chunk * subs + sub)
// whenever the chunk count fits gridDim.y, which spares every workgroup an
// integer division in front of its first load.
__device__ __forceinline__ void chunk_and_sub(uint32_t subs, uint32_t& chunk, uint32_t& sub) {
  if (gridDim.x == subs) {  // two-dimensional launch (also right for a single chunk)
    chunk = blockIdx.y;
    sub = blockIdx.x;
  } else {
    chunk = blockIdx.x / subs;
    sub = blockIdx.x % subs;
  }
}

inline dim3 chunk_grid(int64_t n_chunks, int64_t subs) {
  return n_chunks <= 65535 ? dim3((unsigned)subs, (unsigned)n_chunks) : dim3((unsigned)(n_chunks * subs));
}

// A grid dimension times the workgroup size has to stay below 2^32 threads.
inline bool chunk_grid_fits(int64_t n_chunks, int64_t subs, int block) {
  const int64_t limit = 0xffffffffLL / block;
  return subs <= limit && (n_chunks <= 65535 || n_chunks <= limit / subs);
}

// The table hands out plain 64-bit addresses, which the compiler can only
// treat as generic: it would use flat_load / flat_store, instructions that are
// booked on the LDS counter as well.  All of them are device memory, so the
// vector paths say so and get global_load / global_store.
#define TS_GLOBAL __attribute__((address_space(1)))
typedef TS_GLOBAL const f32x4* gc_f32x4_ptr;
typedef TS_GLOBAL f32x4* g_f32x4_ptr;
typedef TS_GLOBAL const u32x4* gc_u32x4_ptr;
typedef TS_GLOBAL u32x4* g_u32x4_ptr;

constexpr int kEmaBlock = 256;
constexpr int kSubElems = kEmaBlock * 4;  // one 16-byte vector per thread and operand

// out = fl(fl(t*m) + fl(s*c)).  Contraction is switched off for this
// expression: an FMA would skip one rounding and differ from the reference's
// separate mul / mul / add kernels in about a quarter of the elements.
__device__ __forceinline__ float ema1(float t, float s, float m, float c) {
#pragma clang fp contract(off)
  const float a = t * m;
  const float b = s * c;
  return a + b;
}

// CLONE: the student values are also written to `out + clone_offset`, which
// fuses the pipeline's clone of the student parameters into the same pass
// (16 B per parameter instead of 8 + 12 for a separate copy).
template <bool CLONE>
__global__ __launch_bounds__(kEmaBlock) void ema_multi_kernel(const ts_ema_chunk* __restrict__ table,
                                                              uint32_t subs, float m, float c,
                                                              int64_t clone_offset) {
  // Uniform per workgroup: the compiler turns these into scalar loads.
  uint32_t chunk, sub;
  chunk_and_sub(subs, chunk, sub);
  const ts_ema_chunk ch = table[chunk];
  TS_PIN_SCALARS("s"(ch.t), "s"(ch.s), "s"(ch.out), "s"(ch.n), "s"(ch.flags));
  const uint32_t begin = sub * kSubElems;
  if (begin >= ch.n) return;  // short chunk (tensor tail or small tensor)
  const uint32_t n = (ch.n - begin < (uint32_t)kSubElems) ? ch.n - begin : (uint32_t)kSubElems;
  const float* __restrict__ tp = ch.t + begin;
  const float* __restrict__ sp = ch.s + begin;
  float* __restrict__ op = ch.out + begin;
  float* __restrict__ cp = reinterpret_cast<float*>(reinterpret_cast<char*>(op) + clone_offset);
  const uint32_t tid = threadIdx.x;

  // the vector path also needs the clone destination on a 16-byte boundary
  if ((ch.flags & 1u) && (!CLONE || (clone_offset & 15) == 0)) {
    const uint32_t n4 = n >> 2;
    if (tid < n4) {
      const f32x4 a = __builtin_nontemporal_load((gc_f32x4_ptr)tp + tid);
      const f32x4 b = __builtin_nontemporal_load((gc_f32x4_ptr)sp + tid);
      f32x4 r;
      r.x = ema1(a.x, b.x, m, c);
      r.y = ema1(a.y, b.y, m, c);
      r.z = ema1(a.z, b.z, m, c);
      r.w = ema1(a.w, b.w, m, c);
      __builtin_nontemporal_store(r, (g_f32x4_ptr)op + tid);
      if (CLONE) __builtin_nontemporal_store(b, (g_f32x4_ptr)cp + tid);
    }
    const uint32_t rem = n & 3u;
    if (tid < rem) {
      const uint32_t i = (n4 << 2) + tid;
      const float sv = sp[i];
      op[i] = ema1(tp[i], sv, m, c);
      if (CLONE) cp[i] = sv;
    }
  } else {
    // Views whose storage offset breaks 16-byte alignment: 4-byte accesses,
    // still coalesced across the wavefront.
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t i = u * kEmaBlock + tid;
      if (i < n) {
        const float sv = sp[i];
        op[i] = ema1(tp[i], sv, m, c);
        if (CLONE) cp[i] = sv;
      }
    }
  }
}

// The same update for parameter lists kept in a 2-byte floating type.  The
// eager ops the reference runs on such tensors form each product and the sum
// in fp32 and round every result to the type: out = r(r(t*m) + r(s*c)).
constexpr int kSubElems2 = kEmaBlock * 8;  // one 16-byte vector per thread and operand

// Every fp32 intermediate is pinned in a register before it is narrowed:
// otherwise the compiler folds the widening, the fp32 operation and the
// narrowing into one mixed-precision instruction that rounds once, which
// differs from the two roundings of the eager ops whenever the fp32 result
// lands on a tie of the narrow type.
__device__ __forceinline__ float ema_pin(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+v"(x));
#endif
  return x;
}

template <typename T>
__device__ __forceinline__ T ema1_t(T t, T s, float m, float c) {
#pragma clang fp contract(off)
  const float a = to_f32(from_f32<T>(ema_pin(to_f32(t) * m)));
  const float b = to_f32(from_f32<T>(ema_pin(to_f32(s) * c)));
  return from_f32<T>(ema_pin(a + b));
}

template <typename T>
__global__ __launch_bounds__(kEmaBlock) void ema_multi_kernel_2byte(const ts_ema_chunk* __restrict__ table,
                                                                    uint32_t subs, float m, float c) {
  uint32_t chunk, sub;
  chunk_and_sub(subs, chunk, sub);
  const ts_ema_chunk ch = table[chunk];
  TS_PIN_SCALARS("s"(ch.t), "s"(ch.s), "s"(ch.out), "s"(ch.n), "s"(ch.flags));
  const uint32_t begin = sub * kSubElems2;
  if (begin >= ch.n) return;
  const uint32_t n = (ch.n - begin < (uint32_t)kSubElems2) ? ch.n - begin : (uint32_t)kSubElems2;
  const T* __restrict__ tp = reinterpret_cast<const T*>(ch.t) + begin;
  const T* __restrict__ sp = reinterpret_cast<const T*>(ch.s) + begin;
  T* __restrict__ op = reinterpret_cast<T*>(ch.out) + begin;
  const uint32_t tid = threadIdx.x;
  if (ch.flags & 1u) {
    const uint32_t n8 = n >> 3;
    if (tid < n8) {
      const u32x4 ra = __builtin_nontemporal_load((gc_u32x4_ptr)tp + tid);
      const u32x4 rb = __builtin_nontemporal_load((gc_u32x4_ptr)sp + tid);
      T a[8], b[8], r[8];
      __builtin_memcpy(a, &ra, 16);
      __builtin_memcpy(b, &rb, 16);
#pragma unroll
      for (int e = 0; e < 8; ++e) r[e] = ema1_t<T>(a[e], b[e], m, c);
      u32x4 rr;
      __builtin_memcpy(&rr, r, 16);
      __builtin_nontemporal_store(rr, (g_u32x4_ptr)op + tid);
    }
    const uint32_t rem = n & 7u;
    if (tid < rem) {
      const uint32_t i = (n8 << 3) + tid;
      op[i] = ema1_t<T>(tp[i], sp[i], m, c);
    }
  } else {
    // storage offsets that break 16-byte alignment: 2-byte accesses, coalesced
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const uint32_t i = u * kEmaBlock + tid;
      if (i < n) op[i] = ema1_t<T>(tp[i], sp[i], m, c);
    }
  }
}

constexpr int kCopyBlock = 256;
constexpr int kSubBytes = kCopyBlock * 16;

// Sub-block `sub` (kSubBytes bytes) of one table entry; shared by the table
// kernel and by the few-segments kernel below.
__device__ __forceinline__ void copy_sub_block(const ts_copy_chunk& ch, uint32_t sub);

__global__ __launch_bounds__(kCopyBlock) void copy_segments_kernel(const ts_copy_chunk* __restrict__ table,
                                                                   uint32_t subs) {
  uint32_t chunk, sub;
  chunk_and_sub(subs, chunk, sub);
  const ts_copy_chunk ch = table[chunk];
  TS_PIN_SCALARS("s"(ch.src), "s"(ch.dst), "s"(ch.bytes), "s"(ch.flags));
  copy_sub_block(ch, sub);
}

// A handful of segments, described in the kernel arguments themselves: no
// table in device memory, so no upload in front of the launch.  A gather of
// four micro-batch outputs of a few kilobytes costs its caller the launch and
// little else this way; through a planned, uploaded table it was 38 us of host
// time against 5 for torch.cat.  gridDim = (sub-blocks of the longest segment,
// segments).
constexpr int kCopyFewMax = 16;
struct CopyFew {
  ts_copy_chunk c[kCopyFewMax];
};

__global__ __launch_bounds__(kCopyBlock) void copy_few_kernel(const CopyFew f) {
  const ts_copy_chunk ch = f.c[blockIdx.y];
  copy_sub_block(ch, blockIdx.x);
}

__device__ __forceinline__ void copy_sub_block(const ts_copy_chunk& ch, uint32_t sub) {
  const uint64_t begin = (uint64_t)sub * kSubBytes;
  if (begin >= ch.bytes) return;
  const uint32_t bytes =
      (ch.bytes - begin < (uint64_t)kSubBytes) ? (uint32_t)(ch.bytes - begin) : (uint32_t)kSubBytes;
  const uint8_t* __restrict__ s = reinterpret_cast<const uint8_t*>(ch.src) + begin;
  uint8_t* __restrict__ d = reinterpret_cast<uint8_t*>(ch.dst) + begin;
  const uint32_t tid = threadIdx.x;

  if (ch.flags & 1u) {
    const uint32_t n16 = bytes >> 4;
    if (tid < n16) {
      const u32x4 v = __builtin_nontemporal_load((gc_u32x4_ptr)s + tid);
      __builtin_nontemporal_store(v, (g_u32x4_ptr)d + tid);
    }
    const uint32_t rem = bytes & 15u;
    if (tid < rem) d[(n16 << 4) + tid] = s[(n16 << 4) + tid];
  } else if (((((uintptr_t)s) | ((uintptr_t)d)) & 3u) == 0) {
    const uint32_t n4 = bytes >> 2;
    const uint32_t* s4 = reinterpret_cast<const uint32_t*>(s);
    uint32_t* d4 = reinterpret_cast<uint32_t*>(d);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t i = u * kCopyBlock + tid;
      if (i < n4) d4[i] = s4[i];
    }
    const uint32_t rem = bytes & 3u;
    if (tid < rem) d[(n4 << 2) + tid] = s[(n4 << 2) + tid];
  } else {
    for (uint32_t i = tid; i < bytes; i += kCopyBlock) d[i] = s[i];
  }
}

}  // namespace ts

// A launch that, when the thread is armed with timing events, stamps the
// kernel's own begin and end into them (hipExtLaunchKernel semantics).
#define TS_LAUNCH_TIMED(kernel, grid, block, stream, ...)                                  \
  do {                                                                                     \
    hipEvent_t ev0_, ev1_;                                                                 \
    if (ts::take_launch_events(&ev0_, &ev1_))                                              \
      hipExtLaunchKernelGGL(kernel, grid, block, 0, stream, ev0_, ev1_, 0, __VA_ARGS__);   \
    else                                                                                   \
      hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__);                     \
  } while (0)

extern "C" {

int ts_ema_multi(const ts_ema_chunk* table_dev, int64_t n_chunks, int64_t chunk_elems, float m32,
                 float c32, ts_stream_t stream) {
  if (n_chunks < 0 || chunk_elems <= 0 || chunk_elems % ts::kSubElems != 0) return TS_ERR_ARG;
  if (n_chunks == 0) return TS_OK;
  if (!table_dev) return TS_ERR_ARG;
  const int64_t subs = chunk_elems / ts::kSubElems;
  if (!ts::chunk_grid_fits(n_chunks, subs, ts::kEmaBlock)) return TS_ERR_RANGE;
  TS_LAUNCH_TIMED(ts::ema_multi_kernel<false>, ts::chunk_grid(n_chunks, subs), dim3(ts::kEmaBlock),
                  (hipStream_t)stream, table_dev, (uint32_t)subs, m32, c32, (int64_t)0);
  return ts::check_launch();
}

int ts_ema_multi_dtype(const ts_ema_chunk* table_dev, int64_t n_chunks, int64_t chunk_elems, float m32,
                       float c32, int dtype, ts_stream_t stream) {
  if (dtype == TS_F32) return ts_ema_multi(table_dev, n_chunks, chunk_elems, m32, c32, stream);
  if (dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if (n_chunks < 0 || chunk_elems <= 0 || chunk_elems % ts::kSubElems2 != 0) return TS_ERR_ARG;
  if (n_chunks == 0) return TS_OK;
  if (!table_dev) return TS_ERR_ARG;
  const int64_t subs = chunk_elems / ts::kSubElems2;
  if (!ts::chunk_grid_fits(n_chunks, subs, ts::kEmaBlock)) return TS_ERR_RANGE;
  const dim3 grid = ts::chunk_grid(n_chunks, subs);
  if (dtype == TS_BF16)
    TS_LAUNCH_TIMED(ts::ema_multi_kernel_2byte<ts::bf16_t>, grid, dim3(ts::kEmaBlock), (hipStream_t)stream,
                    table_dev, (uint32_t)subs, m32, c32);
  else
    TS_LAUNCH_TIMED(ts::ema_multi_kernel_2byte<ts::f16_t>, grid, dim3(ts::kEmaBlock), (hipStream_t)stream,
                    table_dev, (uint32_t)subs, m32, c32);
  return ts::check_launch();
}

int ts_ema_clone_multi(const ts_ema_chunk* table_dev, int64_t n_chunks, int64_t chunk_elems, float m32,
                       float c32, int64_t clone_offset_bytes, ts_stream_t stream) {
  if (n_chunks < 0 || chunk_elems <= 0 || chunk_elems % ts::kSubElems != 0) return TS_ERR_ARG;
  if (clone_offset_bytes == 0) return TS_ERR_ARG;  // the clone cannot alias the EMA output
  if (clone_offset_bytes & 3) return TS_ERR_ALIGN;
  if (n_chunks == 0) return TS_OK;
  if (!table_dev) return TS_ERR_ARG;
  const int64_t subs = chunk_elems / ts::kSubElems;
  if (!ts::chunk_grid_fits(n_chunks, subs, ts::kEmaBlock)) return TS_ERR_RANGE;
  TS_LAUNCH_TIMED(ts::ema_multi_kernel<true>, ts::chunk_grid(n_chunks, subs), dim3(ts::kEmaBlock),
                  (hipStream_t)stream, table_dev, (uint32_t)subs, m32, c32, clone_offset_bytes);
  return ts::check_launch();
}

int ts_copy_few(const void* const* src, void* const* dst, const int64_t* bytes, int n_segments,
                ts_stream_t stream) {
  if (n_segments < 0 || n_segments > ts::kCopyFewMax) return TS_ERR_RANGE;
  if (n_segments == 0) return TS_OK;
  if (!src || !dst || !bytes) return TS_ERR_ARG;
  ts::CopyFew f;
  int live = 0;
  int64_t longest = 0;
  for (int i = 0; i < n_segments; ++i) {
    if (bytes[i] < 0) return TS_ERR_ARG;
    if (bytes[i] == 0) continue;
    if (!src[i] || !dst[i]) return TS_ERR_ARG;
    ts_copy_chunk& c = f.c[live++];
    c.src = src[i];
    c.dst = dst[i];
    c.bytes = (uint64_t)bytes[i];
    c.flags = ((((uintptr_t)src[i] | (uintptr_t)dst[i]) & 15u) == 0) ? 1u : 0u;
    if (bytes[i] > longest) longest = bytes[i];
  }
  if (live == 0) return TS_OK;
  for (int i = live; i < ts::kCopyFewMax; ++i) f.c[i] = ts_copy_chunk{nullptr, nullptr, 0, 0};
  const int64_t subs = (longest + ts::kSubBytes - 1) / ts::kSubBytes;
  if (subs * ts::kCopyBlock > 0xffffffffLL) return TS_ERR_RANGE;
  TS_LAUNCH_TIMED(ts::copy_few_kernel, dim3((unsigned)subs, (unsigned)live), dim3(ts::kCopyBlock), (hipStream_t)stream,
                  f);
  return ts::check_launch();
}

int ts_copy_segments(const ts_copy_chunk* table_dev, int64_t n_chunks, int64_t chunk_bytes,
                     ts_stream_t stream) {
  if (n_chunks < 0 || chunk_bytes <= 0 || chunk_bytes % ts::kSubBytes != 0) return TS_ERR_ARG;
  if (n_chunks == 0) return TS_OK;
  if (!table_dev) return TS_ERR_ARG;
  const int64_t subs = chunk_bytes / ts::kSubBytes;
  if (!ts::chunk_grid_fits(n_chunks, subs, ts::kCopyBlock)) return TS_ERR_RANGE;
  TS_LAUNCH_TIMED(ts::copy_segments_kernel, ts::chunk_grid(n_chunks, subs), dim3(ts::kCopyBlock),
                     (hipStream_t)stream, table_dev, (uint32_t)subs);
  return ts::check_launch();
}

}  // extern "C"
