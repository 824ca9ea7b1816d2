// Host-side planners: turn tensor lists into the chunk tables that the EMA
// and multi-segment copy kernels walk, one table entry per workgroup.
// Pure CPU code (no HIP calls), so it can be tested without a GPU.
#include <stdint.h>

#include "../../include/tspipe_amd.h"

namespace {

inline bool aligned(const void* p, uintptr_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// Upper bound on table entries the auto chunk size aims for: enough
// workgroups to cover 256 CUs many times over, few enough that the table
// upload (32 B per entry) stays around 100 KB.
constexpr int64_t kTargetChunks = 4096;

}  // namespace

extern "C" {

int64_t ts_ema_auto_chunk(int64_t total_elems) {
  if (total_elems <= 0) return 4096;
  int64_t c = round_up((total_elems + kTargetChunks - 1) / kTargetChunks, 4096);
  if (c > (int64_t)1 << 30) c = (int64_t)1 << 30;
  return c;
}

int64_t ts_ema_plan_dtype(const void* const* t, const void* const* s, void* const* out,
                          const int64_t* numel, int64_t n_tensors, int64_t chunk_elems, int dtype,
                          ts_ema_chunk* table, int64_t capacity) {
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  const int64_t esize = dtype == TS_F32 ? 4 : 2;
  // elements in one workgroup's share: 256 threads x 16 bytes
  const int64_t sub = 4096 / esize;
  if (n_tensors < 0 || (n_tensors > 0 && (!t || !s || !out || !numel))) return TS_ERR_ARG;
  if (chunk_elems < 0 || chunk_elems % sub != 0 || chunk_elems > ((int64_t)1 << 30))
    return TS_ERR_ARG;
  if (chunk_elems == 0) {
    int64_t total = 0;
    for (int64_t i = 0; i < n_tensors; ++i) {
      if (numel[i] < 0) return TS_ERR_ARG;
      total += numel[i];
    }
    chunk_elems = ts_ema_auto_chunk(total);
  }
  int64_t count = 0;
  for (int64_t i = 0; i < n_tensors; ++i) {
    const int64_t n = numel[i];
    if (n < 0) return TS_ERR_ARG;
    if (n == 0) continue;
    if (!t[i] || !s[i] || !out[i]) return TS_ERR_ARG;
    if (!aligned(t[i], esize) || !aligned(s[i], esize) || !aligned(out[i], esize)) return TS_ERR_ALIGN;
    // chunk_elems * esize is a multiple of 16, so every chunk of a tensor
    // shares the 16-byte alignment of the tensor's base pointers.
    const uint32_t flags = (aligned(t[i], 16) && aligned(s[i], 16) && aligned(out[i], 16)) ? 1u : 0u;
    for (int64_t off = 0; off < n; off += chunk_elems) {
      if (table) {
        if (count >= capacity) return TS_ERR_CAPACITY;
        ts_ema_chunk& c = table[count];
        c.t = (const float*)((const char*)t[i] + off * esize);
        c.s = (const float*)((const char*)s[i] + off * esize);
        c.out = (float*)((char*)out[i] + off * esize);
        c.n = (uint32_t)((n - off < chunk_elems) ? (n - off) : chunk_elems);
        c.flags = flags;
      }
      ++count;
    }
  }
  return count;
}

int64_t ts_ema_plan(const void* const* t, const void* const* s, void* const* out,
                    const int64_t* numel, int64_t n_tensors, int64_t chunk_elems,
                    ts_ema_chunk* table, int64_t capacity) {
  return ts_ema_plan_dtype(t, s, out, numel, n_tensors, chunk_elems, TS_F32, table, capacity);
}

int64_t ts_copy_auto_chunk(int64_t total_bytes) {
  if (total_bytes <= 0) return 16384;
  int64_t c = round_up((total_bytes + kTargetChunks - 1) / kTargetChunks, 16384);
  if (c > (int64_t)1 << 31) c = (int64_t)1 << 31;
  return c;
}

int64_t ts_copy_plan(const void* const* src, void* const* dst, const int64_t* bytes,
                     int64_t n_segments, int64_t chunk_bytes, ts_copy_chunk* table,
                     int64_t capacity) {
  if (n_segments < 0 || (n_segments > 0 && (!src || !dst || !bytes))) return TS_ERR_ARG;
  if (chunk_bytes < 0 || chunk_bytes % 4096 != 0) return TS_ERR_ARG;
  if (chunk_bytes == 0) {
    int64_t total = 0;
    for (int64_t i = 0; i < n_segments; ++i) {
      if (bytes[i] < 0) return TS_ERR_ARG;
      total += bytes[i];
    }
    chunk_bytes = ts_copy_auto_chunk(total);
  }
  int64_t count = 0;
  for (int64_t i = 0; i < n_segments; ++i) {
    const int64_t n = bytes[i];
    if (n < 0) return TS_ERR_ARG;
    if (n == 0) continue;
    if (!src[i] || !dst[i]) return TS_ERR_ARG;
    const uint64_t flags = (aligned(src[i], 16) && aligned(dst[i], 16)) ? 1u : 0u;
    for (int64_t off = 0; off < n; off += chunk_bytes) {
      if (table) {
        if (count >= capacity) return TS_ERR_CAPACITY;
        ts_copy_chunk& c = table[count];
        c.src = (const char*)src[i] + off;
        c.dst = (char*)dst[i] + off;
        c.bytes = (uint64_t)((n - off < chunk_bytes) ? (n - off) : chunk_bytes);
        c.flags = flags;
      }
      ++count;
    }
  }
  return count;
}

}  // extern "C"
